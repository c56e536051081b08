"""A plain, slow Sakevik on whole sequences, one function per mechanism, written from the
equations alone.  It shares no code with the engine: tensors by their checkpoint names, the
configuration as the dict that config.json holds, everything in the dtype of the weights it is
given (float64 for an oracle).

Notation: T tokens, W the width, H query heads, G key heads, d the query/key size of a head,
dv its value size, r the size of the key/value latent, dr the rotated part of a latent layer's head.
"""

from __future__ import annotations

import math

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z**3)))


# --------------------------------------------------------------------------- embedding


def bigram_rows(tokens: list[int], bigram: dict) -> list[int]:
    """Row of the bigram table for every token: a hash of (previous, current), the table's last
    row for a sequence's first token."""
    n = int(bigram["buckets"])
    rows = []
    for i, t in enumerate(tokens):
        rows.append(n if i == 0 else (tokens[i - 1] * int(bigram["mul_prev"]) + t * int(bigram["mul_cur"])) % n)
    return rows


def embed(tokens: list[int], w: dict, cfg: dict) -> torch.Tensor:
    e = cfg["embedding"]
    x = w["embed"][tokens] * float(e["scale"])
    if e.get("bigram"):
        x = x + w["bigram"][bigram_rows(tokens, e["bigram"])]
    return x


# --------------------------------------------------------------------------- rotations


def plain_frequencies(dims: int, base: float) -> torch.Tensor:
    return torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64)


def yarn_frequencies(dims: int, base: float, scaling: dict) -> tuple[torch.Tensor, float]:
    """Frequencies blended between f and f / factor by a ramp over the pair's index, and the
    number that cosine and sine are multiplied by."""
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def index_of(turns: float) -> float:  # the (real) pair index whose wavelength makes `turns` turns over `original`
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(index_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(index_of(float(scaling["slow"]))), dims - 1)
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / factor * ramp + f * (1.0 - ramp))
    return torch.tensor(out, dtype=torch.float64), 0.1 * math.log(factor) + 1.0


def turn_pairs(x: torch.Tensor, angles: torch.Tensor, layout: str, magnitude: float = 1.0) -> torch.Tensor:
    """x [T, heads, n] whole; angles [T, n/2]; pair m is (m, m + n/2) for 'halves' and (2m, 2m+1) for
    'interleaved'; (u, v) -> (u cos - v sin, v cos + u sin), cosine and sine times ``magnitude``."""
    c = (torch.cos(angles) * magnitude).to(x.dtype)[:, None, :]
    s = (torch.sin(angles) * magnitude).to(x.dtype)[:, None, :]
    n = x.shape[-1]
    out = torch.empty_like(x)
    if layout == "halves":
        u, v = x[..., : n // 2], x[..., n // 2 :]
        out[..., : n // 2], out[..., n // 2 :] = u * c - v * s, v * c + u * s
    else:
        u, v = x[..., 0::2], x[..., 1::2]
        out[..., 0::2], out[..., 1::2] = u * c - v * s, v * c + u * s
    return out


def rotate_leading(x, positions, rot: dict, layout: str):
    """The leading rot.dims elements of every head turned by position * frequency; the rest passes."""
    dims = int(rot["dims"])
    if rot.get("scaling"):
        f, mag = yarn_frequencies(dims, float(rot["base"]), rot["scaling"])
    else:
        f, mag = plain_frequencies(dims, float(rot["base"])), 1.0
    a = positions.to(torch.float64)[:, None] * f[None, :]
    out = x.clone()
    out[..., :dims] = turn_pairs(x[..., :dims], a, layout, mag)
    return out


def rotate_values(v, positions, base: float, layout: str, sign: float = 1.0):
    """Every element of a value head turned: pair m by sign * position * base^(-2m/dv)."""
    f = plain_frequencies(v.shape[-1], base)
    return turn_pairs(v, sign * positions.to(torch.float64)[:, None] * f[None, :], layout)


def window_mask(T: int, size: int | None) -> torch.Tensor:
    """[T, T] True where query i sees key j: 0 <= i - j < size (no size: every earlier key)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = j <= i
    if size:
        seen &= (i - j) < int(size)
    return seen


# --------------------------------------------------------------------------- mixers


def min_gru(h, w, p, mixer):
    """A gated recurrence whose gates read the current token only."""
    z = torch.sigmoid(h @ w[f"{p}.z"].T + w[f"{p}.z.b"])
    u = h @ w[f"{p}.x"].T + w[f"{p}.x.b"]
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    S = torch.zeros(int(mixer["width"]), dtype=h.dtype)
    rows = []
    for t in range(h.shape[0]):
        S = (1.0 - z[t]) * S + z[t] * cand[t]
        rows.append(S)
    S_all = torch.stack(rows)
    g = h @ w[f"{p}.g"].T
    return (S_all * (g * torch.sigmoid(g))) @ w[f"{p}.o"].T


def sigmoid_attention(h, w, p, mixer, positions, eps):
    """Grouped-query attention whose weights are sigmoids of the biased scores (not normalised
    over the keys), with norms of queries and keys per head, values that are rotated by their own
    position and turned back by the query's, and a gate per head."""
    H, G, d, dv = int(mixer["heads"]), int(mixer["kv_heads"]), int(mixer["dim"]), int(mixer["vdim"])
    T = h.shape[0]
    q = (h @ w[f"{p}.q"].T + w[f"{p}.q.b"]).view(T, H, d)
    k = (h @ w[f"{p}.k"].T + w[f"{p}.k.b"]).view(T, G, d)
    v = (h @ w[f"{p}.v"].T + w[f"{p}.v.b"]).view(T, G, dv)
    q = rms(q, eps) * w[f"{p}.q.norm"]
    k = rms(k, eps) * w[f"{p}.k.norm"]
    rot = mixer["rot"]
    q = rotate_leading(q, positions, rot, "halves")
    k = rotate_leading(k, positions, rot, "halves")
    v = rotate_values(v, positions, float(rot["base"]), "halves")
    each = H // G
    k = k.repeat_interleave(each, dim=1)
    v = v.repeat_interleave(each, dim=1)
    s = torch.einsum("ihd,jhd->hij", q, k) * float(mixer["scale"]) + w[f"{p}.pb"][:, None, None]
    seen = window_mask(T, (mixer.get("mask") or {}).get("size"))
    weight = torch.sigmoid(s) * seen.to(s.dtype)
    o = torch.einsum("hij,jhe->ihe", weight, v)
    o = rotate_values(o, positions, float(rot["base"]), "halves", sign=-1.0)
    gate = torch.sigmoid(h @ w[f"{p}.g"].T)  # [T, H]
    o = o * gate[:, :, None]
    return o.reshape(T, H * dv) @ w[f"{p}.o"].T + w[f"{p}.o.b"]


def latent_attention(h, w, p, mixer, positions, eps):
    """Attention whose keys and values are expansions of one normed latent a token, beside a
    rotated key part that all heads share; ordinary softmax over a window."""
    H, d, dr, dv, r = int(mixer["heads"]), int(mixer["dim"]), int(mixer["rot_dim"]), int(mixer["vdim"]), int(mixer["kv_rank"])
    T = h.shape[0]
    q = (h @ w[f"{p}.q"].T).view(T, H, d + dr)
    low = h @ w[f"{p}.dkv"].T
    c = rms(low[:, :r], eps) * w[f"{p}.dkv.norm"]
    k_rot = low[:, None, r:]  # [T, 1, dr]
    rot = mixer["rot"]
    q_rot = rotate_leading(q[..., d:], positions, rot, "interleaved")
    k_rot = rotate_leading(k_rot, positions, rot, "interleaved")
    k = (c @ w[f"{p}.uk"].T).view(T, H, d)
    v = (c @ w[f"{p}.uv"].T).view(T, H, dv)
    s = (torch.einsum("ihd,jhd->hij", q[..., :d], k) + torch.einsum("ihd,jd->hij", q_rot, k_rot[:, 0])) * float(mixer["scale"])
    seen = window_mask(T, (mixer.get("mask") or {}).get("size"))
    s = s.masked_fill(~seen, -math.inf)
    o = torch.einsum("hij,jhe->ihe", torch.softmax(s, dim=-1), v)
    return o.reshape(T, H * dv) @ w[f"{p}.o"].T


MIXERS = {"mingru": lambda h, w, p, m, pos, eps: min_gru(h, w, p, m), "attention": sigmoid_attention,
          "latent_attention": latent_attention}

# --------------------------------------------------------------------------- feed-forward


def clamped_glu(h, w, p, mlp):
    limit = float(mlp["limit"])
    g = torch.clamp(h @ w[f"{p}.gate"].T, max=limit)
    u = torch.clamp(h @ w[f"{p}.up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[f"{p}.down"].T


# --------------------------------------------------------------------------- the model


def forward(tokens: list[int], w: dict, cfg: dict, streams: list | None = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence; ``streams`` collects the stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = embed(tokens, w, cfg)
    positions = torch.arange(len(tokens))
    for i, layer in enumerate(cfg["layers"]):
        a = MIXERS[layer["type"]](x, w, f"l{i}.mix", layer["mixer"], positions, eps)
        x = x + rms(a, eps) * w[f"l{i}.norm1"]
        if layer.get("mlp") is not None:
            b = clamped_glu(x, w, f"l{i}.mlp", layer["mlp"])
            x = x + rms(b, eps) * w[f"l{i}.norm2"]
        if streams is not None:
            streams.append(x.clone())
    x = rms(x, eps) * w["final.norm"]
    return (x @ w["head"].T) * float(cfg.get("logit_scale", 1.0))
