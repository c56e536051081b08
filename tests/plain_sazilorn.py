"""A plain, slow Sazilorn on whole sequences, one function per mechanism, written from the
equations alone.  It shares no code with the engine: tensors by their checkpoint names, the
configuration as the dict that config.json holds, everything in the dtype of the weights it is
given (float64 for an oracle).

Notation: T tokens, W the width, H query heads, G key heads, d the query/key size of a head,
dv its value size.
"""

from __future__ import annotations

import math

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z**3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


# --------------------------------------------------------------------------- embedding


def embed(tokens: list[int], w: dict) -> torch.Tensor:
    """The token's row plus the learned row of its position."""
    return w["embed"][tokens] + w["pos"][: len(tokens)]


# --------------------------------------------------------------------------- around the sublayers


def offset_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm whose weight is stored around zero."""
    return rms(x, eps) * (1.0 + weight)


def short_convolution(h: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """conv(h)_t = sum_j taps[:, j] * h_(t - n + 1 + j), zeros before the start; h [T, W], taps [W, n]."""
    T, n = h.shape[0], taps.shape[1]
    out = torch.zeros_like(h)
    for t in range(T):
        for j in range(n):
            s = t - n + 1 + j
            if s >= 0:
                out[t] += taps[:, j] * h[s]
    return out


def depth_average(history: list[torch.Tensor], weights: torch.Tensor) -> torch.Tensor:
    """sum_j weights[j] * history[j] over the embedding's output and every layer's result so far."""
    assert len(history) == weights.shape[0]
    out = torch.zeros_like(history[0])
    for j, x in enumerate(history):
        out = out + weights[j] * x
    return out


# --------------------------------------------------------------------------- attention


def distance_bucket(n: int, buckets: int, far: float) -> int:
    """Distances below half the buckets have one each; the others share the rest on a logarithmic scale up to ``far``."""
    half = buckets // 2
    if n < half:
        return n
    return min(buckets - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (buckets - half))))


def softmax_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, softcap: float | None = None,
                      rel: torch.Tensor | None = None, far: float = 0.0) -> torch.Tensor:
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv]: causal softmax attention, query head h over
    key head h // (H / G); scores times ``scale``, then soft-capped, then plus rel[bucket(i - j), h]."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros((T, H, v.shape[2]), dtype=q.dtype)
    if rel is not None:
        by_distance = [distance_bucket(n, rel.shape[0], far) for n in range(T)]
        idx = torch.tensor([[by_distance[i - j] if j <= i else 0 for j in range(T)] for i in range(T)])
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if softcap is not None:
            s = softcap * torch.tanh(s / softcap)
        if rel is not None:
            s = s + rel[:, h][idx]
        mask = torch.ones((T, T), dtype=torch.bool).tril()
        s = s.masked_fill(~mask, float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def attention_mixer(h: torch.Tensor, w: dict, p: str, m: dict, eps: float) -> torch.Tensor:
    """Grouped attention with norms over the whole query and key projections and a bias by distance."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = rms(h @ w[f"{p}.q"].T, eps) * w[f"{p}.q.norm"]
    k = rms(h @ w[f"{p}.k"].T, eps) * w[f"{p}.k.norm"]
    v = h @ w[f"{p}.v"].T
    o = softmax_attention(q.view(T, H, d), k.view(T, G, d), v.view(T, G, dv), float(m["scale"]),
                          rel=w[f"{p}.rel"], far=float(m["bias_max"]))
    return o.reshape(T, H * dv) @ w[f"{p}.o"].T


# --------------------------------------------------------------------------- linear attention


def decayed_outer_products(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor) -> torch.Tensor:
    """S_t = diag(decay_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, from S = 0.
    q, k, decay [T, H, d] (decay per row of the state), v [T, H, dv] -> [T, H, dv]."""
    T, H, d = q.shape
    S = torch.zeros((H, d, v.shape[2]), dtype=q.dtype)
    out = torch.zeros((T, H, v.shape[2]), dtype=q.dtype)
    for t in range(T):
        S = decay[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return out


def lightning_mixer(h: torch.Tensor, w: dict, p: str, m: dict, eps: float) -> torch.Tensor:
    """Linear attention with one constant decay a head; the heads' results normed together and gated."""
    T = h.shape[0]
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = silu(h @ w[f"{p}.q"].T).view(T, H, d)
    k = silu(h @ w[f"{p}.k"].T).view(T, H, d)
    v = silu(h @ w[f"{p}.v"].T).view(T, H, dv)
    decay = torch.tensor([float(a) for a in m["decay"]], dtype=h.dtype)[None, :, None].expand(T, H, d)
    o = decayed_outer_products(q, k, v, decay).reshape(T, H * dv)
    o = rms(o, eps) * w[f"{p}.norm"] * torch.sigmoid(h @ w[f"{p}.g"].T)
    return o @ w[f"{p}.o"].T


def hgrn2_mixer(h: torch.Tensor, w: dict, p: str, m: dict, eps: float) -> torch.Tensor:
    """Linear attention whose forget gate (bounded below) decays the state and whose complement is the key."""
    T = h.shape[0]
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = silu(h @ w[f"{p}.q"].T).view(T, H, d)
    v = (h @ w[f"{p}.v"].T).view(T, H, dv)
    low = w[f"{p}.lower"]
    f = (low + (1.0 - low) * torch.sigmoid(h @ w[f"{p}.f"].T + w[f"{p}.f.b"])).view(T, H, d)
    o = decayed_outer_products(q, 1.0 - f, v, f)
    o = rms(o, eps) * w[f"{p}.norm"]  # head by head over dv, one weight for all heads
    return o.reshape(T, H * dv) @ w[f"{p}.o"].T


def parallel_mixer(h: torch.Tensor, w: dict, p: str, m: dict, eps: float) -> torch.Tensor:
    """Soft-capped gated attention and lightning attention side by side, each with a factor."""
    T = h.shape[0]
    a, lp = m["left"], f"{p}.left"
    H, G, d, dv = int(a["heads"]), int(a["kv_heads"]), int(a["dim"]), int(a["vdim"])
    q = (h @ w[f"{lp}.q"].T).view(T, H, d)
    k = (h @ w[f"{lp}.k"].T).view(T, G, d)
    v = (h @ w[f"{lp}.v"].T).view(T, G, dv)
    o = softmax_attention(q, k, v, float(a["scale"]), softcap=float(a["softcap"])).reshape(T, H * dv)
    left = (o * torch.sigmoid(h @ w[f"{lp}.g"].T)) @ w[f"{lp}.o"].T
    right = lightning_mixer(h, w, f"{p}.right", m["right"], eps)
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right


# --------------------------------------------------------------------------- feed-forward


def gated_ff(h: torch.Tensor, w: dict, p: str, act) -> torch.Tensor:
    return (act(h @ w[f"{p}.gate"].T) * (h @ w[f"{p}.up"].T)) @ w[f"{p}.down"].T


def route(h: torch.Tensor, w: dict, p: str, r: dict) -> tuple[torch.Tensor, torch.Tensor]:
    """The chosen experts [T, top] and their weights: softmax scores, the choice by score plus correction,
    the weights the chosen scores over their sum, times the router's scale."""
    s = torch.softmax(h @ w[f"{p}.router"].T, dim=-1)
    choice = s + w[f"{p}.correction"]
    ids = torch.topk(choice, int(r["top"]), dim=-1).indices
    g = torch.gather(s, 1, ids)
    return ids, g / (g.sum(-1, keepdim=True) + 1e-20) * float(r["scale"])


def experts_ff(h: torch.Tensor, w: dict, p: str, mlp: dict) -> torch.Tensor:
    ids, weights = route(h, w, p, mlp["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, g in zip(ids[t].tolist(), weights[t]):
            out[t] += g * gated_ff(h[t : t + 1], w, f"{p}.e{e}", silu)[0]
    if mlp.get("shared"):
        out = out + gated_ff(h, w, f"{p}.shared", silu)
    return out


def feed_forward(h: torch.Tensor, w: dict, p: str, mlp: dict | None) -> torch.Tensor | None:
    if mlp is None:
        return None
    if mlp["kind"] == "dense":
        return gated_ff(h, w, p, gelu_tanh)
    return experts_ff(h, w, p, mlp)


# --------------------------------------------------------------------------- the model


MIXERS = {"attention": attention_mixer, "hgrn2": hgrn2_mixer, "parallel": parallel_mixer}


def forward(tokens: list[int], w: dict, cfg: dict, streams: list | None = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence; ``streams`` collects the stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = embed(tokens, w)
    history = [x]
    for i, layer in enumerate(cfg["layers"]):
        h = offset_norm(x, w[f"l{i}.norm1"], eps)
        hm = h + short_convolution(h, w[f"l{i}.canon1"]) if cfg.get("canon") else h
        mixed = MIXERS[layer["type"]](hm, w, f"l{i}.mix", layer["mixer"], eps)
        ff = feed_forward(h, w, f"l{i}.mlp", layer.get("mlp"))
        history.append(x + (mixed if ff is None else mixed + ff))
        x = depth_average(history, w[f"l{i}.dwa"])
        if streams is not None:
            streams.append(x)
    return offset_norm(x, w["final.norm"], eps) @ w["head"].T
