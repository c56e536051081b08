"""Rotary position encoding: the inverse frequencies (with the scaling rules a
checkpoint may ask for) and the cos/sin tables.

The reference builds cos/sin for every position up to
``max_position_embeddings`` once, in 32-bit, and looks rows up by position
(tokasaurus/model/llama.py:559-570,576-577); the generator itself is delegated
there to an installed package.  Definition used here: inv_freq_j = theta^(-2j/d);
``llama3`` scaling leaves wavelengths shorter than orig/high_freq_factor alone,
divides those longer than orig/low_freq_factor by ``factor`` and blends linearly
in between; ``linear`` divides all by ``factor``.
"""

from __future__ import annotations

import math

import torch

from tokasaurus_amd.kernels import ops
from tokasaurus_amd.parts.base import POSITION_ENCODINGS, PositionEncoding


def inverse_frequencies(head_dim: int, theta: float, scaling: dict | None) -> torch.Tensor:
    """[d/2] float32 on the host (a handful of numbers computed once at set-up)."""
    exponent = torch.arange(0, head_dim, 2, dtype=torch.int64).to(torch.float32) / head_dim
    inv_freq = 1.0 / (theta**exponent)
    if scaling is None or scaling["rope_type"] == "default":
        return inv_freq
    kind = scaling["rope_type"]
    factor = float(scaling["factor"])
    if kind == "linear":
        return inv_freq / factor
    if kind == "llama3":
        low = float(scaling["low_freq_factor"])
        high = float(scaling["high_freq_factor"])
        orig = float(scaling["original_max_position_embeddings"])
        wavelen = 2 * math.pi / inv_freq
        long_wave = wavelen > orig / low
        short_wave = wavelen < orig / high
        smooth = (orig / wavelen - low) / (high - low)
        blended = (1 - smooth) * inv_freq / factor + smooth * inv_freq
        out = torch.where(long_wave, inv_freq / factor, inv_freq)
        return torch.where(~long_wave & ~short_wave, blended, out)
    raise ValueError(f"unknown rope scaling {kind!r}")


@POSITION_ENCODINGS.register("rotary")
class RotaryEncoding(PositionEncoding):
    """cos/sin tables [max_positions, d/2] in 32-bit on the device; lane j of a
    head pairs with lane j + d/2."""

    def __init__(self, head_dim: int, theta: float, max_positions: int, scaling: dict | None = None):
        if head_dim % 2:
            raise ValueError(f"rotary encoding needs an even head size, got {head_dim}")
        self.head_dim = head_dim
        self.theta = float(theta)
        self.max_positions = int(max_positions)
        self.scaling = scaling
        self.cos: torch.Tensor | None = None
        self.sin: torch.Tensor | None = None

    def prepare(self, device: torch.device) -> None:
        if self.cos is not None:
            return
        inv_freq = inverse_frequencies(self.head_dim, self.theta, self.scaling).to(device)
        self.cos, self.sin = ops.rope_table(inv_freq, self.max_positions)


def interleaved_frequencies(dims: int, base: float, scaling: dict | None) -> torch.Tensor:
    """f_i = base^(-2i/dims) for i < dims/2, computed in 64-bit on the host and rounded once to
    32-bit.  ``scaling`` (``factor``, ``low``, ``high``, ``original``) rescales by wavelength
    l = 2 pi / f: f stays where l < original/high, becomes f/factor where l > original/low, and
    between the two is (1 - s) f/factor + s f with s = (original/l - low) / (high - low)."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            factor, low, high = float(scaling["factor"]), float(scaling["low"]), float(scaling["high"])
            original = float(scaling["original"])
            wavelength = 2.0 * math.pi / f
            if wavelength > original / low:
                f = f / factor
            elif not wavelength < original / high:
                s = (original / wavelength - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return torch.tensor(out, dtype=torch.float64).to(torch.float32)


def ramp_frequencies(dims: int, base: float, ramp: dict) -> tuple[torch.Tensor, float]:
    """Frequencies blended between f_i = base^(-2i/dims) and f_i / factor by a ramp over the pair's
    index (``ramp``: ``factor``, ``original``, ``fast``, ``slow``), and the factor that goes on cosine and
    sine.  With index(t) = dims ln(original / (2 pi t)) / (2 ln base), the pair whose wavelength makes t
    turns over ``original`` positions: lo = max(floor(index(fast)), 0), hi = min(ceil(index(slow)),
    dims - 1), r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1); the frequency is
    f_i / factor * r_i + f_i (1 - r_i) and the factor 0.1 ln(factor) + 1.  64-bit on the host, rounded once."""
    factor, original = float(ramp["factor"]), float(ramp["original"])

    def index(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(float(base)))

    lo = max(math.floor(index(float(ramp["fast"]))), 0)
    hi = min(math.ceil(index(float(ramp["slow"]))), dims - 1)
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        r = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / factor * r + f * (1.0 - r))
    return torch.tensor(out, dtype=torch.float64).to(torch.float32), 0.1 * math.log(factor) + 1.0


@POSITION_ENCODINGS.register("rotary_interleaved")
class InterleavedRotary(PositionEncoding):
    """A rotation of neighbouring elements (2i, 2i+1) of the leading ``dims`` elements of a head
    by the angle position * f_i.  It keeps the frequencies only: the kernel that rotates
    multiplies and takes sine and cosine in 32-bit itself, so positions have no upper end."""

    pair_halves = False  # which elements form a pair: neighbours (2i, 2i+1), or (i, i + dims/2)

    def __init__(self, dims: int, base: float, scaling: dict | None = None, ramp: dict | None = None):
        """``scaling``: rescaling by wavelength bands (``interleaved_frequencies``); ``ramp``: a blend by
        the pair's index with a factor on cosine and sine (``ramp_frequencies``); at most one of them."""
        if dims % 2 or dims <= 0:
            raise ValueError(f"a rotation of pairs needs an even number of elements, got {dims}")
        if scaling and ramp:
            raise ValueError("a rotation is rescaled by bands of wavelength or by a ramp, not both")
        self.dims = int(dims)
        self.base = float(base)
        self.scaling = dict(scaling) if scaling else None
        self.ramp = dict(ramp) if ramp else None
        self.magnitude = 1.0  # what cosine and sine are multiplied by
        self.freq: torch.Tensor | None = None

    def prepare(self, device: torch.device) -> None:
        if self.freq is None:
            if self.ramp:
                freq, self.magnitude = ramp_frequencies(self.dims, self.base, self.ramp)
                self.freq = freq.to(device)
            else:
                self.freq = interleaved_frequencies(self.dims, self.base, self.scaling).to(device)


@POSITION_ENCODINGS.register("rotary_halves")
class HalvesRotary(InterleavedRotary):
    """The same angles, position * f_i with f_i = base^(-2i/dims), for the pairs (i, i + dims/2) of
    the leading ``dims`` elements of a head; computed in the kernel like its parent's."""

    pair_halves = True
