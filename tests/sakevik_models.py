"""Small Sakevik configurations of the tests' own, their model folders, and the plain model's rows for
them.  The configurations differ from one another in every size and option: attention with one, several
and as many kv heads as heads, a rotation of a few elements and of the whole head, value heads smaller
than, equal to and larger than key heads, windows of 1, of a page, of odd sizes, beyond every test's
length and none; latent attention with and without the ramp between frequency scales, rotated parts of 2
elements and of as many as the unrotated part, latents that are no multiples of 8; recurrences of widths
off every multiple; layers with and without a feed-forward; with and without the table of token pairs;
sizes as large as the matrix-core attention takes, and sizes that fit nothing.
"""

from __future__ import annotations

import json
from pathlib import Path

import torch
from safetensors import safe_open
from safetensors.torch import save_file

import plain_sakevik
from tokasaurus_amd.weights import write_random_model


def attention_layer(heads, kv_heads, dim, vdim, scale, rot_dims, base, window=None, mlp=None, scaling=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": {"base": base, "dims": rot_dims}}
    if scaling is not None:
        mixer["rot"]["scaling"] = scaling
    if window is not None:
        mixer["mask"] = {"size": window}
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def latent_layer(heads, dim, rot_dim, vdim, kv_rank, scale, base, window=None, scaling=None, rot_dims=None, mlp=None):
    rot = {"base": base, "dims": rot_dim if rot_dims is None else rot_dims}
    if scaling is not None:
        rot["scaling"] = scaling
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale, "rot": rot}
    if window is not None:
        mixer["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


def gru_layer(width, mlp=None):
    return {"type": "mingru", "mixer": {"width": width}, "mlp": mlp}


def dense(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def model(vocab, width, layers, eps=1e-5, scale=1.0, bigram=(37, 5, 3), logit_scale=None):
    cfg = {"architecture": "Sakevik", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "embedding": {"scale": scale}, "layers": layers}
    if bigram is not None:
        cfg["embedding"]["bigram"] = {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}
    if logit_scale is not None:
        cfg["logit_scale"] = logit_scale
    return cfg


RAMP = {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}

# every mechanism in one model
MIXED = model(160, 96, [
    attention_layer(4, 2, 32, 16, 0.2, 16, 100.0, window=40, mlp=dense(144, 1.5)),
    gru_layer(72),
    latent_layer(3, 24, 8, 48, 48, 0.2, 1000.0, window=50, scaling=RAMP, mlp=dense(64, 3.0)),
    attention_layer(6, 1, 16, 32, 0.3, 16, 30.0, mlp=dense(120, 0.7)),
    gru_layer(128, mlp=dense(96, 2.5)),
], scale=9.0, logit_scale=0.5)
# sizes that fit nothing: a width that is no multiple of 4, heads no multiple of 8, value heads no multiple of 16, a
# latent of odd size, a recurrence of 50 channels; no table of pairs, no logit scale, a window of one page and one of 1
AWKWARD = model(131, 90, [
    gru_layer(50, mlp=dense(75, 1.0)),
    attention_layer(5, 1, 20, 6, 0.25, 4, 50.0, window=16),
    latent_layer(5, 12, 6, 10, 17, 0.3, 77.0, window=33, rot_dims=4, mlp=dense(33, 5.0)),
    attention_layer(3, 3, 24, 24, 0.2, 24, 10000.0, window=1, mlp=dense(40, 2.0)),
    latent_layer(1, 40, 2, 8, 24, 0.2, 20.0, scaling={"factor": 2.0, "original": 16, "fast": 4.0, "slow": 1.0}),
], eps=1e-4, bigram=None)
# heads of the sizes of large models: the largest cached key the matrix-core kernel takes (192 + 64), heads of 128,
# windows longer than any request of the tests; a table of pairs with one bucket
LARGE_HEADS = model(120, 128, [
    latent_layer(4, 128, 64, 128, 192, 0.07, 1000000.0, window=1000, scaling={"factor": 4.0, "original": 512, "fast": 32.0, "slow": 1.0},
                 mlp=dense(256, 2.0)),
    attention_layer(8, 2, 128, 128, 0.09, 64, 500000.0, window=2000, mlp=dense(256, 2.0)),
    gru_layer(512),
    attention_layer(16, 1, 64, 64, 0.12, 32, 10000.0, window=24),
], scale=11.3, bigram=(1, 7, 11), logit_scale=3.0)
# no attention at all (no cache group), and no recurrence at all (no state but the token before)
ONLY_GRU = model(64, 48, [gru_layer(40, mlp=dense(64, 2.0)), gru_layer(24)], scale=7.0, bigram=(11, 1, 1))
ONLY_ATTENTION = model(70, 64, [
    attention_layer(2, 2, 16, 16, 0.25, 8, 40.0, window=7, mlp=dense(48, 2.0)),
    latent_layer(2, 16, 16, 16, 32, 0.2, 300.0, window=9),
], scale=8.0, bigram=(4093, 1000003, 999983))
CONFIGS = {"mixed": MIXED, "awkward": AWKWARD, "large_heads": LARGE_HEADS, "only_gru": ONLY_GRU, "only_attention": ONLY_ATTENTION}


def make_folder(folder: Path, config: dict, seed: int, edits: dict | None = None) -> Path:
    """Random weights with the parts scaled so that each mechanism matters to the logits: projections
    of order one a row, biases of the projections' own size, a table of pairs as large as the
    embedding.  ``edits``: name suffix -> function of the tensor, applied last."""
    write_random_model(folder, config, seed)
    path = folder / "model.safetensors"
    tensors = {}
    with safe_open(str(path), framework="pt") as f:
        for name in f.keys():
            t = f.get_tensor(name).float()
            if t.dim() == 2:
                t = t * (1.0 / (0.02 * t.shape[1] ** 0.5))  # N(0, 1/in): outputs of order one
            if name.endswith(".b"):
                t = t * 25.0  # N(0, 1/4)
            if name == "bigram":
                t = t * 6.0
            for suffix, fn in (edits or {}).items():
                if name.endswith(suffix):
                    t = fn(t)
            tensors[name] = t.to(torch.bfloat16)
    save_file(tensors, str(path))
    return folder


def load_plain(folder: Path, dtype=torch.float64):
    config = json.loads((Path(folder) / "config.json").read_text())
    w = {}
    with safe_open(str(Path(folder) / "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            w[name] = f.get_tensor(name).to(dtype)
    return config, w


def plain_rows(folder: Path, requests: dict[str, list[int]]) -> dict[str, torch.Tensor]:
    config, w = load_plain(folder)
    return {rid: plain_sakevik.forward(toks, w, config).float() for rid, toks in requests.items()}


def row_error(row: torch.Tensor, ref: torch.Tensor) -> float:
    return float((row - ref).pow(2).mean().sqrt() / ref.pow(2).mean().sqrt().clamp_min(1e-9))


def compare_rows(got: dict, plain: dict[str, torch.Tensor], tol: float) -> float:
    """Every collected row against the plain row: the root mean square of the difference over the
    vocabulary, relative to that of the plain row.  Names the first wrong (request, position)."""
    worst = 0.0
    for (rid, pos), row in sorted(got.items()):
        err = row_error(row, plain[rid][pos])
        assert err <= tol, f"request {rid} position {pos}: relative error {err:.3e} (allowed {tol:.1e})"
        worst = max(worst, err)
    return worst


# relative error of a row of logits: summation order in 32-bit; roundings to 8 bits of mantissa in bfloat16
TOL = {"float32": 3e-4, "bfloat16": 6e-2}
