"""Small Sazilorn configurations of the tests' own, their model folders, and the plain model's rows for
them.  The configurations differ from one another in every size and option: attention with one, several and
as many kv heads as heads, tables of biases of few and many buckets that end near and far; linear attention
with key sizes off every multiple of sixteen; pairs whose two sides differ in every size; convolutions of one,
two and many taps and none; dense, routed and absent feed-forwards, with and without a shared expert; a model
without any attention (no cache group) and one without any recurrence.
"""

from __future__ import annotations

import json
from pathlib import Path

import torch
from safetensors import safe_open
from safetensors.torch import save_file

import plain_sazilorn
from tokasaurus_amd.weights import write_random_model


def attention_layer(heads, kv_heads, dim, vdim, scale, bias_max, buckets, mlp=None):
    return {"type": "attention", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "bias_max": bias_max,
                      "bias_buckets": buckets}}


def hgrn2_layer(heads, dim, vdim, mlp=None):
    return {"type": "hgrn2", "mixer": {"heads": heads, "dim": dim, "vdim": vdim}, "mlp": mlp}


def parallel_layer(left, right, left_scale, right_scale, mlp=None):
    """left: (heads, kv_heads, dim, vdim, scale, softcap); right: (heads, dim, vdim, decays)."""
    return {"type": "parallel", "mlp": mlp, "mixer": {
        "left": dict(zip(("heads", "kv_heads", "dim", "vdim", "scale", "softcap"), left)),
        "right": dict(zip(("heads", "dim", "vdim", "decay"), right)), "left_scale": left_scale, "right_scale": right_scale}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top, scale, shared=None):
    out = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": scale}}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


def model(vocab, width, layers, eps=1e-5, taps=4, max_positions=1024):
    cfg = {"architecture": "Sazilorn", "vocab": vocab, "width": width, "max_positions": max_positions, "norm": {"eps": eps},
           "layers": layers}
    if taps:
        cfg["canon"] = {"taps": taps}
    return cfg


# every mechanism in one model
MIXED = model(160, 96, [
    hgrn2_layer(3, 16, 32, mlp=dense(144)),
    attention_layer(4, 2, 32, 16, 0.2, 100, 12, mlp=moe(40, 6, 2, 2.0, shared=56)),
    parallel_layer((4, 2, 16, 32, 0.3, 5.0), (3, 16, 16, [0.5, 0.9, 0.995]), 0.7, 1.3, mlp=dense(64)),
    attention_layer(6, 1, 16, 32, 0.3, 20, 8),
    parallel_layer((2, 1, 32, 16, 0.2, 50.0), (1, 32, 48, [0.97]), 1.0, 0.25, mlp=moe(24, 5, 1, 0.5)),
])
# sizes that fit nothing: a width that is no multiple of 4, heads no multiple of 8 or 16, an odd number of experts, all of
# them chosen, two taps, a table of two buckets
AWKWARD = model(131, 90, [
    parallel_layer((3, 3, 24, 8, 0.25, 2.0), (5, 12, 6, [0.1, 0.3, 0.6, 0.9, 1.0]), 0.5, 2.0, mlp=moe(33, 3, 3, 1.0, shared=20)),
    hgrn2_layer(1, 50, 10, mlp=dense(75)),
    attention_layer(5, 1, 20, 6, 0.25, 7, 2),
    hgrn2_layer(5, 6, 20),
], eps=1e-4, taps=2)
# heads of the sizes of large models, a table of many buckets that ends beyond every test's length, one tap (no state of
# the convolution's)
LARGE_HEADS = model(120, 128, [
    attention_layer(8, 2, 128, 128, 0.09, 4000, 64, mlp=dense(256)),
    parallel_layer((16, 1, 64, 32, 0.12, 20.0), (2, 128, 128, [0.99, 0.9995]), 0.9, 0.4, mlp=dense(128)),
    hgrn2_layer(2, 128, 64, mlp=moe(64, 16, 4, 1.5, shared=64)),
], taps=1)
# no attention at all (no cache group, no pages), and no recurrence and no convolution at all (no state in any slot)
ONLY_LINEAR = model(64, 48, [hgrn2_layer(2, 8, 24, mlp=dense(64)), hgrn2_layer(4, 16, 8)], taps=7)
ONLY_ATTENTION = model(70, 64, [
    attention_layer(2, 2, 16, 16, 0.25, 33, 6, mlp=dense(48)),
    attention_layer(4, 1, 8, 24, 0.4, 500, 20, mlp=moe(16, 4, 2, 1.0)),
], taps=0)
CONFIGS = {"mixed": MIXED, "awkward": AWKWARD, "large_heads": LARGE_HEADS, "only_linear": ONLY_LINEAR, "only_attention": ONLY_ATTENTION}


def make_folder(folder: Path, config: dict, seed: int, edits: dict | None = None, steady_choice: bool = False) -> Path:
    """Random weights with the parts scaled so that each mechanism matters to the logits: projections of order one a
    row, rows of positions as large as the tokens' rows, biases and forget-gate biases of the projections' own size,
    routers whose scores differ clearly.  ``edits``: name suffix -> function of the tensor, applied last.
    ``steady_choice``: the corrections lie 1.5 apart in a shuffled order, so that the choice of experts (not their
    weights) is the same for every token and no comparison in bfloat16 rests on which of two nearly equal scores is
    larger; the 32-bit runs use the data-dependent choice."""
    write_random_model(folder, config, seed)
    path = folder / "model.safetensors"
    tensors = {}
    with safe_open(str(path), framework="pt") as f:
        for name in f.keys():
            t = f.get_tensor(name).float()
            if t.dim() == 2 and not name.endswith((".rel", "canon1")):
                t = t * (1.0 / (0.02 * t.shape[1] ** 0.5))  # N(0, 1/in): outputs of order one
            if name in ("embed", "pos"):
                t = t * (t.shape[1] ** 0.5)
            if name.endswith(".f.b"):
                t = t * 50.0
            if name.endswith(".router"):
                t = t * 2.0
            if name.endswith(".correction"):
                t = t * 4.0
                if steady_choice:
                    t = 1.5 * torch.argsort(torch.argsort(t)).float() - 0.75 * t.numel()
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
    return {rid: plain_sazilorn.forward(toks, w, config).float() for rid, toks in requests.items()}


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
# in bfloat16 a router's choice between two experts of nearly equal score can fall the other way than in the
# plain model: the bfloat16 runs use folders with a steady choice
STEADY = {"float32": False, "bfloat16": True}
