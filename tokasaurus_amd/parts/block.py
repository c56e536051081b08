"""Arrangements of norms, mixer and feed-forward around the residual stream.

``pre_norm`` is the reference's block (tokasaurus/model/llama.py:342-359 with
:227-230,284 and :323-325,336): each half norms its input, transforms it and adds
the result to the stream.  In the last block of a step only the rows whose
logits are wanted go on after the mixer (llama.py:268-278).
"""

from __future__ import annotations

import inspect

import torch

from tokasaurus_amd.kernels import ops
from tokasaurus_amd.parts.base import (
    BLOCKS,
    CONNECTORS,
    FEED_FORWARDS,
    MIXERS,
    NORMS,
    Block,
    CacheView,
    Connector,
    Normed,
    Part,
    Prepared,
    PartSpec,
    StepContext,
    TensorSpec,
)
from tokasaurus_amd.parts.base import AVERAGE_WEIGHT
from tokasaurus_amd.parts.linear import Linear, Placer
from tokasaurus_amd.parts.short_conv import ShortConvResidual


def build_with_shared(registry, spec: PartSpec, shared: dict):
    """Build a part; hand it the model-wide ``shared`` dict if its constructor takes one."""
    ctor = registry._entries.get(spec.kind)
    if ctor is not None and "shared" in inspect.signature(ctor).parameters:
        return registry.build(spec, shared=shared)
    return registry.build(spec)


def stream_and_prepared(out) -> tuple[torch.Tensor, Prepared | None]:
    """A part returns the stream alone, or the stream with what it prepared for the next norm."""
    return out if isinstance(out, tuple) else (out, None)


@BLOCKS.register("pre_norm")
class PreNormBlock(Block):
    fuses_norm = True

    def __init__(
        self,
        mixer_norm: PartSpec,
        mixer: PartSpec,
        ff_norm: PartSpec,
        feed_forward: PartSpec,
        shared: dict | None = None,
    ):
        shared = shared if shared is not None else {}
        self.mixer_norm = build_with_shared(NORMS, mixer_norm, shared)
        self.mixer = build_with_shared(MIXERS, mixer, shared)
        self.ff_norm = build_with_shared(NORMS, ff_norm, shared)
        self.feed_forward = build_with_shared(FEED_FORWARDS, feed_forward, shared)

    def children(self) -> list[Part]:
        return [self.mixer_norm, self.mixer, self.ff_norm, self.feed_forward]

    def tensor_specs(self) -> list[TensorSpec]:
        return [s for c in self.children() for s in c.tensor_specs()]

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        for c in self.children():
            c.load(tensors, placer)

    def entry_norm(self):
        return self.mixer_norm

    def forward(
        self,
        x: torch.Tensor,
        ctx: StepContext,
        cache: CacheView | None,
        state: torch.Tensor | None,
        rows: torch.Tensor | None,
        prepared: Prepared | None = None,
        next_norm=None,
    ):
        residual = x if rows is None else ops.gather_rows(x, rows)
        if self.mixer.fuses_norm:
            out = self.mixer.forward(Normed(x, self.mixer_norm, prepared), residual, ctx, cache, state, rows,
                                     emit_norm=self.ff_norm)
        else:
            out = self.mixer.forward(Normed(x, self.mixer_norm, prepared).materialize(), residual, ctx, cache, state, rows)
        x, prepared = stream_and_prepared(out)
        if self.feed_forward.fuses_norm:
            return self.feed_forward.forward(Normed(x, self.ff_norm, prepared), x, emit_norm=next_norm)
        return self.feed_forward.forward(Normed(x, self.ff_norm, prepared).materialize(), x)


class NormPair(Part):
    """The two norms a block with side-by-side branches begins with: both read the same
    stream, so one pass computes the statistic once and writes both rows."""

    def __init__(self, first, second):
        self.first, self.second = first, second

    def children(self) -> list[Part]:
        return [n for n in (self.first, self.second) if n is not None]

    def fused(self) -> bool:
        return self.second is None or self.first.same_rule(self.second)

    def forward_pair(self, x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor | None]:
        if not self.fused():
            return self.first.forward(x), self.second.forward(x)
        n = self.first
        _, h1, h2 = ops.residual_norm(x, weights=(n.weight, self.second.weight if self.second is not None else None),
                                      unit_offset=n.unit_offset, eps=n.eps, out_dtype=n.out_dtype)
        return h1, h2


class PendingSum:
    """A block's residual sum that has not been made: ``x + mult * (a + b)`` with ``x`` the block's input rows
    (the wanted rows only, for a step's last block) and the branches' 32-bit sums (either may be None)."""

    def __init__(self, x: torch.Tensor, branches: tuple, mult: float):
        self.x, self.branches, self.mult = x, branches, float(mult)


@BLOCKS.register("parallel_residual")
class ParallelResidualBlock(Block):
    """Mixer and feed-forward side by side on a 32-bit residual stream:
        x <- x + mult * (mixer(norm1(x)) + ff(norm2(x)))
    both norms of the same x; ``feed_forward`` (and its norm) may be absent.  With ``shared_norm`` there is one
    norm and both sublayers read its rows (``ff_norm`` is then absent).  ``input_conv`` (``{"taps": n, "name":
    checkpoint name}``): what the mixer reads is first replaced by ``h + conv(h)``, a short causal convolution over
    time on every channel whose last inputs are part of a request's state (the feed-forward reads h as it is).  The stream is
    32-bit whatever the storage type; the branches hand over their last products' 32-bit sums,
    and one kernel adds them to the stream and writes the rows of the norms that read the new
    stream (the next block's pair, or the head's norm).  The norms are ``stream_rmsnorm``s; the
    mixer must have ``mix`` and the feed-forward ``transform``."""

    fuses_norm = True

    def __init__(self, mixer_norm: PartSpec, mixer: PartSpec, ff_norm: PartSpec | None = None,
                 feed_forward: PartSpec | None = None, residual_mult: float = 1.0, shared: dict | None = None,
                 shared_norm: bool = False, input_conv: dict | None = None):
        shared = shared if shared is not None else {}
        self.shared_norm = bool(shared_norm)
        if self.shared_norm and ff_norm is not None:
            raise ValueError("sublayers that share one norm have no second one")
        if not self.shared_norm and (ff_norm is None) != (feed_forward is None):
            raise ValueError("a feed-forward and its norm come together")
        self.mixer_norm = build_with_shared(NORMS, mixer_norm, shared)
        self.mixer = build_with_shared(MIXERS, mixer, shared)
        self.ff_norm = build_with_shared(NORMS, ff_norm, shared) if ff_norm is not None else None
        self.feed_forward = build_with_shared(FEED_FORWARDS, feed_forward, shared) if feed_forward is not None else None
        self.residual_mult = float(residual_mult)
        self.entry = NormPair(self.mixer_norm, self.ff_norm)
        self.input_conv = None
        if input_conv:
            self.input_conv = ShortConvResidual(self.mixer_norm.size, int(input_conv["taps"]), input_conv["name"])

    def children(self) -> list[Part]:
        return [c for c in (self.mixer_norm, self.input_conv, self.mixer, self.ff_norm, self.feed_forward) if c is not None]

    def state_needs(self):
        conv = self.input_conv.state_need() if self.input_conv is not None else None
        return ([conv] if conv is not None else []) + super().state_needs()

    def tensor_specs(self) -> list[TensorSpec]:
        return [s for c in self.children() for s in c.tensor_specs()]

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        for c in self.children():
            c.load(tensors, placer)

    def entry_norm(self):
        return self.entry

    can_defer_sum = True

    def forward(self, x, ctx: StepContext, cache, state, rows, prepared: Prepared | None = None, next_norm=None,
                defer_sum: bool = False):
        """``defer_sum``: the stream is not updated; returns ``PendingSum`` (the block's input rows, its branches and
        the multiplier) for whoever runs next on the stream and can add them in its own pass."""
        if x.dtype != torch.float32:
            raise TypeError("a parallel_residual block runs on a 32-bit stream (an embedding with stream_f32)")
        if prepared is not None and prepared.norm is self.entry and prepared.normed is not None:
            h1, h2 = prepared.normed
        else:
            h1, h2 = self.entry.forward_pair(x)
        if self.shared_norm:
            h2 = h1
        hm = h1
        if self.input_conv is not None:
            tails = None
            if self.input_conv.state_need() is not None:
                # the convolution's last inputs come first among the block's states
                tails, rest = (state[0], state[1:]) if isinstance(state, list) else (state, [])
                state = None if not rest else (rest[0] if len(rest) == 1 else rest)
            hm = self.input_conv.forward(h1, ctx, tails)
        a = self.mixer.mix(hm, ctx, cache, state, rows, out_f32=True)
        if rows is not None:
            x = ops.gather_rows(x, rows)
            h2 = ops.gather_rows(h2, rows) if h2 is not None else None
        b = self.feed_forward.transform(h2, out_f32=True) if self.feed_forward is not None else None
        if defer_sum:
            return PendingSum(x, (a, b), self.residual_mult)
        # the norms that read the new stream: the next block's pair or a single norm (the head's)
        first = second = None
        if isinstance(next_norm, NormPair) and next_norm.fused():
            first, second = next_norm.first, next_norm.second
        elif getattr(next_norm, "same_rule", None) is not None:
            first = next_norm
        x, g1, g2 = ops.residual_norm(
            x, (a, b), self.residual_mult,
            weights=(first.weight if first is not None else None, second.weight if second is not None else None),
            unit_offset=first.unit_offset if first is not None else False, eps=first.eps if first is not None else 0.0,
            out_dtype=first.out_dtype if first is not None else torch.float32)
        tap = ctx.extras.get("stream_tap")
        if tap is not None:  # a list that collects the stream after every block (tests, debugging)
            tap.append(x.clone())
        if first is None:
            return x
        return x, Prepared(None, next_norm, (g1, g2) if isinstance(next_norm, NormPair) else g1)


@BLOCKS.register("sandwich_norm")
class SandwichNormBlock(Block):
    """A norm in front of and behind every sublayer, on a 32-bit residual stream:
        x <- x + post1(mixer(norm1(x)));  x <- x + post2(ff(norm2(x)))
    ``feed_forward`` (with its two norms) may be absent.  The branches hand over their last
    products' 32-bit sums; one kernel norms a branch, adds it to the stream and writes the rows
    of the norm that reads the new stream (this block's second, the next block's first, or the
    head's).  The norms are ``stream_rmsnorm``s; the mixer must have ``mix`` and the
    feed-forward ``transform``."""

    fuses_norm = True

    def __init__(self, mixer_norm: PartSpec, mixer: PartSpec, mixer_post_norm: PartSpec, ff_norm: PartSpec | None = None,
                 feed_forward: PartSpec | None = None, ff_post_norm: PartSpec | None = None, shared: dict | None = None):
        shared = shared if shared is not None else {}
        if len({ff_norm is None, feed_forward is None, ff_post_norm is None}) != 1:
            raise ValueError("a feed-forward and its two norms come together")
        self.mixer_norm = build_with_shared(NORMS, mixer_norm, shared)
        self.mixer = build_with_shared(MIXERS, mixer, shared)
        self.mixer_post_norm = build_with_shared(NORMS, mixer_post_norm, shared)
        self.ff_norm = build_with_shared(NORMS, ff_norm, shared) if ff_norm is not None else None
        self.feed_forward = build_with_shared(FEED_FORWARDS, feed_forward, shared) if feed_forward is not None else None
        self.ff_post_norm = build_with_shared(NORMS, ff_post_norm, shared) if ff_post_norm is not None else None
        for n in (self.mixer_norm, self.mixer_post_norm, self.ff_norm, self.ff_post_norm):
            if n is not None and (getattr(n, "same_rule", None) is None or n.unit_offset):
                raise ValueError("a sandwich_norm block takes stream_rmsnorm norms with plain weights")

    def children(self) -> list[Part]:
        return [c for c in (self.mixer_norm, self.mixer, self.mixer_post_norm, self.ff_norm, self.feed_forward, self.ff_post_norm)
                if c is not None]

    def tensor_specs(self) -> list[TensorSpec]:
        return [s for c in self.children() for s in c.tensor_specs()]

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        for c in self.children():
            c.load(tensors, placer)

    def entry_norm(self):
        return self.mixer_norm

    @staticmethod
    def _add(x, branch, post, reader):
        """Norm the branch, add it, and write the rows of ``reader`` (a plain-weight stream norm or None)."""
        ok = reader is not None and getattr(reader, "same_rule", None) is not None and not reader.unit_offset
        return ops.post_norm_residual(x, branch, post.weight, post.eps, reader.weight if ok else None,
                                      reader.eps if ok else 0.0, reader.out_dtype if ok else torch.float32)

    def forward(self, x, ctx: StepContext, cache, state, rows, prepared: Prepared | None = None, next_norm=None):
        if x.dtype != torch.float32:
            raise TypeError("a sandwich_norm block runs on a 32-bit stream (an embedding with stream_f32)")
        if prepared is not None and prepared.norm is self.mixer_norm and prepared.normed is not None:
            h = prepared.normed
        else:
            h = self.mixer_norm.forward(x)
        a = self.mixer.mix(h, ctx, cache, state, rows, out_f32=True)
        if rows is not None:
            x = ops.gather_rows(x, rows)
        tap = ctx.extras.get("stream_tap")
        reader = self.ff_norm if self.feed_forward is not None else next_norm
        x, h = self._add(x, a, self.mixer_post_norm, reader)
        if self.feed_forward is not None:
            b = self.feed_forward.transform(h, out_f32=True)
            reader = next_norm
            x, h = self._add(x, b, self.ff_post_norm, reader)
        if tap is not None:  # a list that collects the stream after every block (tests, debugging)
            tap.append(x.clone())
        if h is None:
            return x
        return x, Prepared(None, reader, h)


@BLOCKS.register("post_norm")
class PostNormBlock(Block):
    """A norm behind every sublayer and none in front, on a 32-bit residual stream:
        x <- x + post1(mixer(x));  x <- x + post2(ff(x))
    ``feed_forward`` (with its norm) may be absent.  The sublayers read the stream itself, rounded once to
    the storage type.  The branches hand over their last products' 32-bit sums; one kernel norms a
    branch, adds it to the stream and writes the rows of whoever reads the new stream: the rounded stream
    for this block's feed-forward or the next block of this kind, the normed rows for a norm (the
    head's).  The post norms are ``stream_rmsnorm``s with plain weights; the mixer must have ``mix`` and
    the feed-forward ``transform``."""

    fuses_norm = True

    def __init__(self, mixer: PartSpec, mixer_post_norm: PartSpec, feed_forward: PartSpec | None = None,
                 ff_post_norm: PartSpec | None = None, shared: dict | None = None):
        shared = shared if shared is not None else {}
        if (feed_forward is None) != (ff_post_norm is None):
            raise ValueError("a feed-forward and the norm behind it come together")
        self.entry = build_with_shared(NORMS, PartSpec("stream_cast"), shared)
        self.mixer = build_with_shared(MIXERS, mixer, shared)
        self.mixer_post_norm = build_with_shared(NORMS, mixer_post_norm, shared)
        self.feed_forward = build_with_shared(FEED_FORWARDS, feed_forward, shared) if feed_forward is not None else None
        self.ff_post_norm = build_with_shared(NORMS, ff_post_norm, shared) if ff_post_norm is not None else None
        for n in (self.mixer_post_norm, self.ff_post_norm):
            if n is not None and (getattr(n, "same_rule", None) is None or n.unit_offset):
                raise ValueError("a post_norm block takes stream_rmsnorm norms with plain weights")

    def children(self) -> list[Part]:
        return [c for c in (self.entry, self.mixer, self.mixer_post_norm, self.feed_forward, self.ff_post_norm) if c is not None]

    def tensor_specs(self) -> list[TensorSpec]:
        return [s for c in self.children() for s in c.tensor_specs()]

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        for c in self.children():
            c.load(tensors, placer)

    def entry_norm(self):
        return self.entry

    def _add(self, x, branch, post, reader):
        """Norm the branch, add it, and write the rows of ``reader``: the rounded stream for a reader that
        only rounds, the normed rows for a plain-weight stream norm, nothing for any other."""
        if getattr(reader, "plain_rows", False):
            return ops.post_norm_residual(x, branch, post.weight, post.eps, out_dtype=self.entry.out_dtype, plain_rows=True)
        return SandwichNormBlock._add(x, branch, post, reader)

    def forward(self, x, ctx: StepContext, cache, state, rows, prepared: Prepared | None = None, next_norm=None):
        if x.dtype != torch.float32:
            raise TypeError("a post_norm block runs on a 32-bit stream (an embedding that writes one)")
        if prepared is not None and prepared.normed is not None and getattr(prepared.norm, "plain_rows", False):
            h = prepared.normed  # the rounded stream is the same whoever asked for it
        else:
            h = self.entry.forward(x)
        a = self.mixer.mix(h, ctx, cache, state, rows, out_f32=True)
        if rows is not None:
            x = ops.gather_rows(x, rows)
        tap = ctx.extras.get("stream_tap")
        reader = self.entry if self.feed_forward is not None else next_norm
        x, h = self._add(x, a, self.mixer_post_norm, reader)
        if self.feed_forward is not None:
            b = self.feed_forward.transform(h, out_f32=True)
            reader = next_norm
            x, h = self._add(x, b, self.ff_post_norm, reader)
        if tap is not None:  # a list that collects the stream after every block (tests, debugging)
            tap.append(x.clone())
        if h is None or reader is None:
            return x
        return x, Prepared(None, reader, h)


@CONNECTORS.register("embedding_mix")
class EmbeddingMix(Connector):
    """x <- W [x; x0]: the stream and the embedding's output side by side through one matrix
    [width, 2 width] (the stream's columns first).  Both are 32-bit streams; they are rounded
    once to the storage type for the product, whose 32-bit sums are the new stream."""

    def __init__(self, hidden_size: int, name: str):
        self.hidden_size = hidden_size
        self.proj = Linear(2 * hidden_size, [name], [hidden_size])

    def tensor_specs(self) -> list[TensorSpec]:
        return self.proj.tensor_specs()

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        self.proj.load(tensors, placer)

    def forward(self, x: torch.Tensor, x0: torch.Tensor) -> torch.Tensor:
        return self.proj(ops.concat_cast(x, x0, self.proj.weight.dtype), out_f32=True)


@CONNECTORS.register("depth_average")
class DepthAverage(Connector):
    """x <- sum_j w[j] X_j over the embedding's output X_0 and the results X_1 .. X_n of every block that has run
    so far (each block's result before any such average): what goes on to the next block, or to the head.  One
    weight vector of n + 1 numbers, kept in 32-bit; the sum is 32-bit in ascending j.  A connector of this kind
    runs behind a run entry (``models.spec.RunEntry.after``) and is handed the model's streams so far instead of
    the stream and the embedding's output; where the next reader begins with an RMS norm of the stream, the same
    pass writes that norm's rows."""

    takes_history = True
    adds_pending_sum = True  # a block in front may hand over its branches unsummed (``PendingSum``)

    def __init__(self, streams: int, name: str):
        self.streams, self.name = int(streams), name
        self.weight: torch.Tensor | None = None

    def tensor_specs(self) -> list[TensorSpec]:
        return [TensorSpec(self.name, (self.streams,), AVERAGE_WEIGHT)]

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        self.weight = placer.place(("vector_f32", self.name), lambda: tensors[self.name].to(torch.float32).contiguous().to(placer.device))

    def forward_history(self, hist: torch.Tensor, count: int, last: torch.Tensor | None, rows: torch.Tensor | None,
                        out: torch.Tensor | None, next_norm=None, pending: "PendingSum | None" = None):
        """``hist`` [streams, tokens, H]: X_0 .. X_(count - 1); ``last``: X_count where it has only the wanted
        ``rows``.  ``pending``: the newest of these is still the block's input and becomes its result here.
        Returns the new stream (in ``out`` when given), or (stream, ``Prepared``) for ``next_norm``."""
        if count + (1 if last is not None else 0) != self.streams:
            raise RuntimeError(f"a depth average over {self.streams} streams was handed {count + (1 if last is not None else 0)}")
        reader = next_norm.first if isinstance(next_norm, NormPair) and next_norm.second is None else next_norm
        if getattr(reader, "same_rule", None) is None:
            reader = None
        x, normed = ops.depth_average(hist, count, self.weight, last=last, rows=rows, out=out,
                                      norm_weight=reader.weight if reader is not None else None,
                                      unit_offset=reader.unit_offset if reader is not None else False,
                                      eps=reader.eps if reader is not None else 0.0,
                                      out_dtype=reader.out_dtype if reader is not None else torch.float32,
                                      branches=pending.branches if pending is not None else (None, None),
                                      mult=pending.mult if pending is not None else 1.0)
        if reader is None:
            return x
        return x, Prepared(None, next_norm, (normed, None) if isinstance(next_norm, NormPair) else normed)
