"""The plain Sakevik against properties that follow from its equations, the configuration reader and
the spec (no GPU)."""

from __future__ import annotations

import math

import pytest
import torch

import plain_sakevik as ps
from sakevik_models import AWKWARD, CONFIGS, MIXED, attention_layer, dense, gru_layer, latent_layer, model
from tokasaurus_amd.config.model_config import ConfigError
from tokasaurus_amd.config.sakevik_config import SakevikConfig
from tokasaurus_amd.models.registry import architecture_of, build_model
from tokasaurus_amd.parts.position import ramp_frequencies
from tokasaurus_amd.weights.random_init import draw_tensors


def weights_for(config, seed=0):
    arch = architecture_of(config)
    m = build_model(arch, arch.config_from_dict(config))
    w = {k: v.double() for k, v in draw_tensors(m.tensor_specs(), seed).items()}
    return {k: (v * (1.0 / (0.02 * v.shape[1] ** 0.5)) if v.dim() == 2 else v) for k, v in w.items()}


def test_bigram_rows():
    b = {"buckets": 7, "mul_prev": 3, "mul_cur": 5}
    assert ps.bigram_rows([4, 2, 6], b) == [7, (4 * 3 + 2 * 5) % 7, (2 * 3 + 6 * 5) % 7]
    assert ps.bigram_rows([9], b) == [7]


def test_the_recurrence_is_causal_and_carries_far():
    cfg = model(50, 32, [gru_layer(24)])
    w = weights_for(cfg)
    a = [3, 9, 1] + [5] * 20
    b = [4, 9, 1] + [5] * 20
    la, lb = ps.forward(a, w, cfg), ps.forward(b, w, cfg)
    assert float((la[0] - lb[0]).abs().max()) > 1e-3
    assert float((la[-1] - lb[-1]).abs().max()) > 0  # the first token still shows 20 tokens on
    c = a[:10] + [7] + a[11:]
    assert torch.equal(ps.forward(c, w, cfg)[:10], la[:10])


def test_candidate_is_continuous_and_positive():
    u = torch.tensor([-1e-9, 0.0, 1e-9], dtype=torch.float64)
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    assert float((cand - 0.5).abs().max()) < 1e-8


@pytest.mark.parametrize("kind", ["attention", "latent"])
def test_a_window_hides_exactly_the_keys_beyond_it(kind):
    W = 5
    layer = (attention_layer(2, 1, 8, 8, 0.3, 4, 20.0, window=W) if kind == "attention"
             else latent_layer(2, 8, 4, 8, 16, 0.3, 20.0, window=W))
    cfg = model(40, 16, [layer], bigram=None)
    w = weights_for(cfg)
    toks = list(range(1, 21))
    base = ps.forward(toks, w, cfg)
    for back in (W - 1, W):
        changed = list(toks)
        changed[19 - back] = 33
        diff = float((ps.forward(changed, w, cfg)[19] - base[19]).abs().max())
        assert (diff > 1e-6) == (back < W)


def test_turned_values_depend_on_distance_only():
    """Values turned by their position and turned back by the query's: the layer's output for a pair of
    tokens depends on how far apart they stand, not on where (without the table of pairs, and with
    rotations only: no other part of the model knows positions)."""
    cfg = model(40, 16, [attention_layer(2, 1, 8, 8, 0.3, 8, 20.0, window=3)], bigram=None)
    w = weights_for(cfg)
    seq = [5, 9, 9, 9, 9, 9, 9]
    out = ps.forward(seq, w, cfg)
    assert float((out[4] - out[6]).abs().max()) < 1e-9  # both see three 9s
    assert float((out[1] - out[6]).abs().max()) > 1e-6


def test_sigmoid_weights_are_not_normalised():
    """With one visible key (a window of 1) a softmax would give weight 1 whatever the score; here the
    bias on the scores changes the result."""
    cfg = model(40, 16, [attention_layer(1, 1, 8, 8, 0.3, 4, 20.0, window=1)], bigram=None)
    w = weights_for(cfg)
    a = ps.forward([3, 4, 5], w, cfg)
    w2 = dict(w)
    w2["l0.mix.pb"] = w["l0.mix.pb"] + 2.0
    # (the norm behind the mixer would hide a common factor of a single head: compare the mixer itself)
    h = ps.embed([3, 4, 5], w, cfg)
    pos = torch.arange(3)
    m = cfg["layers"][0]["mixer"]
    o1 = ps.sigmoid_attention(h, w, "l0.mix", m, pos, 1e-5) - w["l0.mix.o.b"]
    o2 = ps.sigmoid_attention(h, w2, "l0.mix", m, pos, 1e-5) - w["l0.mix.o.b"]
    assert float((o1 - o2).abs().max()) > 1e-3 and a.shape == (3, 40)


def test_latent_form_of_the_scores():
    """q_h . (W_uk,h c) = (W_uk,h^T q_h) . c: the form single tokens take in the engine."""
    torch.manual_seed(0)
    H, d, r = 3, 8, 12
    q, c, uk = torch.randn(H, d, dtype=torch.float64), torch.randn(r, dtype=torch.float64), torch.randn(H * d, r, dtype=torch.float64)
    k = (uk @ c).view(H, d)
    direct = (q * k).sum(-1)
    latent = torch.einsum("hd,hdr,r->h", q, uk.view(H, d, r), c)
    assert torch.allclose(direct, latent)


def test_ramp_frequencies():
    f, mag = ramp_frequencies(16, 1000.0, {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0})
    g, mag2 = ps.yarn_frequencies(16, 1000.0, {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0})
    assert torch.allclose(f.double(), g, rtol=1e-6) and abs(mag - mag2) < 1e-12 and abs(mag - (0.1 * math.log(8.0) + 1)) < 1e-12
    plain = ps.plain_frequencies(16, 1000.0)
    assert abs(float(g[0]) - float(plain[0])) < 1e-12  # the fastest pair keeps its frequency
    assert abs(float(g[-1]) - float(plain[-1]) / 8.0) < 1e-12  # the slowest is divided by the factor
    assert all(float(plain[i]) / 8.0 - 1e-12 <= float(g[i]) <= float(plain[i]) + 1e-12 for i in range(8))


def test_clamps():
    cfg = model(20, 8, [gru_layer(8, mlp=dense(8, 0.5))])
    w = weights_for(cfg)
    h = torch.randn(4, 8, dtype=torch.float64) * 10
    g = torch.clamp(h @ w["l0.mlp.gate"].T, max=0.5)
    u = torch.clamp(h @ w["l0.mlp.up"].T, -0.5, 0.5)
    ref = (g * torch.sigmoid(1.702 * g) * (u + 1)) @ w["l0.mlp.down"].T
    assert torch.allclose(ps.clamped_glu(h, w, "l0.mlp", cfg["layers"][0]["mlp"]), ref)
    assert float(u.abs().max()) == 0.5 and float(g.max()) == 0.5 and float(g.min()) < -0.5


def test_configuration_reader():
    cfg = SakevikConfig.from_dict(MIXED)
    assert cfg.vocab == 160 and cfg.width == 96 and cfg.logit_scale == 0.5 and cfg.embedding_scale == 9.0
    assert cfg.bigram.buckets == 37 and [l.kind for l in cfg.layers] == ["attention", "mingru", "latent_attention", "attention", "mingru"]
    assert cfg.layers[0].mixer.window == 40 and cfg.layers[3].mixer.window == 0 and cfg.layers[1].ff is None
    assert cfg.layers[2].mixer.rot.scaling == (8.0, 64.0, 16.0, 2.0)
    awk = SakevikConfig.from_dict(AWKWARD)
    assert awk.bigram is None and awk.logit_scale == 1.0 and awk.layers[4].mixer.window == 0
    bad = model(10, 8, [{"type": "conv", "mixer": {}, "mlp": None}])
    with pytest.raises(ConfigError):
        SakevikConfig.from_dict(bad)
    for path in (("layers", 0, "mixer", "heads"), ("norm",), ("embedding",), ("layers", 1, "mixer", "width")):
        broken = __import__("json").loads(__import__("json").dumps(MIXED))
        d = broken
        for key in path[:-1]:
            d = d[key]
        del d[path[-1]]
        with pytest.raises(ConfigError):
            SakevikConfig.from_dict(broken)


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_the_spec_names_the_checkpoint_tensors(name):
    config = CONFIGS[name]
    arch = architecture_of(config)
    assert arch.name == "sakevik"
    m = build_model(arch, arch.config_from_dict(config))
    names = {s.name: s.shape for s in m.tensor_specs()}
    assert names["embed"] == (config["vocab"], config["width"]) and "final.norm" in names and "head" in names
    assert ("bigram" in names) == ("bigram" in config["embedding"])
    for i, layer in enumerate(config["layers"]):
        assert (f"l{i}.norm2" in names) == (layer["mlp"] is not None) and f"l{i}.norm1" in names
        if layer["type"] == "latent_attention":
            mx = layer["mixer"]
            assert names[f"l{i}.mix.dkv"] == (mx["kv_rank"] + mx["rot_dim"], config["width"])
            assert names[f"l{i}.mix.q"] == (mx["heads"] * (mx["dim"] + mx["rot_dim"]), config["width"])
    needs = m.cache_needs()
    for need, layer in zip(needs, config["layers"]):
        assert (need is None) == (layer["type"] == "mingru")
        if need is not None:
            assert need.window == (layer["mixer"].get("mask") or {}).get("size", 0)
    assert (m.embedding_state_need() is not None) == ("bigram" in config["embedding"])
    # the plain model runs on exactly these tensors
    w = {k: v.double() for k, v in draw_tensors(m.tensor_specs(), 1).items()}
    assert ps.forward([1, 2, 3, 4], w, config).shape == (4, config["vocab"])
