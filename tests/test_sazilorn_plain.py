"""The plain Sazilorn against properties that follow from its equations, the configuration reader and
the spec (no GPU)."""

from __future__ import annotations

import math

import pytest
import torch

import plain_sazilorn as pz
from sazilorn_models import AWKWARD, CONFIGS, MIXED, attention_layer, dense, hgrn2_layer, model, moe, parallel_layer
from tokasaurus_amd.config.model_config import ConfigError
from tokasaurus_amd.config.sazilorn_config import SazilornConfig
from tokasaurus_amd.kernels.ops import distance_buckets
from tokasaurus_amd.models.registry import architecture_of, build_model
from tokasaurus_amd.weights.random_init import draw_tensors


def weights_for(config, seed=0):
    arch = architecture_of(config)
    m = build_model(arch, arch.config_from_dict(config))
    w = {k: v.double() for k, v in draw_tensors(m.tensor_specs(), seed).items()}
    return {k: (v * (1.0 / (0.02 * v.shape[1] ** 0.5)) if (v.dim() == 2 and not k.endswith(("canon1", ".rel"))) else v)
            for k, v in w.items()}


def test_positions_enter_through_the_embedding():
    cfg = model(30, 16, [hgrn2_layer(1, 4, 4)], taps=0)
    w = weights_for(cfg)
    x = pz.embed([3, 3, 3], w)
    assert torch.equal(x[1] - x[0], w["pos"][1] - w["pos"][0]) and not torch.equal(x[0], x[1])


def test_distance_buckets():
    # every short distance has a bucket of its own; the others climb on a logarithmic scale and end in the last bucket
    for buckets, far in ((14, 200), (2, 7), (8, 20), (64, 4000), (12, 100)):
        got = [pz.distance_bucket(n, buckets, far) for n in range(far + 50)]
        half = buckets // 2
        assert got[:half] == list(range(half)) and got[half] == half
        assert all(a <= b for a, b in zip(got, got[1:])) and max(got) == buckets - 1 and got[far] == buckets - 1
        assert got[: far + 1] == distance_buckets(buckets, far)  # the engine's table, written apart from the plain function
    # a boundary between two logarithmic buckets: bucket 4 + k starts where n / 4 reaches 16^(k / 4) = 2^k
    assert [pz.distance_bucket(n, 8, 64) for n in (7, 8, 15, 16, 31, 32, 63)] == [4, 5, 5, 6, 6, 7, 7]


def test_short_convolution_is_causal_and_ends_at_the_sequence_s_start():
    torch.manual_seed(0)
    h, taps = torch.randn(6, 3, dtype=torch.float64), torch.randn(3, 4, dtype=torch.float64)
    out = pz.short_convolution(h, taps)
    assert torch.allclose(out[0], taps[:, 3] * h[0])  # only the last tap meets the first token
    assert torch.allclose(out[5], sum(taps[:, j] * h[2 + j] for j in range(4)))
    h2 = h.clone()
    h2[4] += 1.0
    assert torch.equal(pz.short_convolution(h2, taps)[:4], out[:4])


def test_depth_average_weighs_every_stream():
    xs = [torch.full((2, 3), float(i + 1), dtype=torch.float64) for i in range(3)]
    out = pz.depth_average(xs, torch.tensor([0.5, -1.0, 2.0], dtype=torch.float64))
    assert torch.equal(out, torch.full((2, 3), 0.5 - 2.0 + 6.0, dtype=torch.float64))


def test_a_block_s_result_is_kept_before_the_average():
    # with weights (0, .., 0, 1) the average hands on the last block's result: the model is then a plain stack
    cfg = model(40, 16, [hgrn2_layer(2, 4, 4, mlp=dense(8)), hgrn2_layer(1, 8, 8)], taps=2)
    w = weights_for(cfg)
    for i in range(2):
        w[f"l{i}.dwa"] = torch.tensor([0.0] * (i + 1) + [1.0], dtype=torch.float64)
    streams: list = []
    pz.forward([1, 2, 3, 4], w, cfg, streams)
    eps = cfg["norm"]["eps"]
    x = pz.embed([1, 2, 3, 4], w)
    for i, layer in enumerate(cfg["layers"]):
        h = pz.offset_norm(x, w[f"l{i}.norm1"], eps)
        y = pz.hgrn2_mixer(h + pz.short_convolution(h, w[f"l{i}.canon1"]), w, f"l{i}.mix", layer["mixer"], eps)
        if layer["mlp"]:
            y = y + pz.gated_ff(h, w, f"l{i}.mlp", pz.gelu_tanh)
        x = x + y
        assert torch.allclose(streams[i], x)


def test_linear_attention_as_a_sum_over_the_past():
    # o_t = sum_{s <= t} (q_t . (prod_{s < r <= t} a_r) k_s) v_s
    torch.manual_seed(1)
    T, H, d, dv = 7, 2, 3, 4
    q, k, v = (torch.randn(T, H, n, dtype=torch.float64) for n in (d, d, dv))
    a = torch.rand(T, H, d, dtype=torch.float64)
    o = pz.decayed_outer_products(q, k, v, a)
    for t in range(T):
        want = torch.zeros(H, dv, dtype=torch.float64)
        for s in range(t + 1):
            decay = torch.ones(H, d, dtype=torch.float64)
            for r in range(s + 1, t + 1):
                decay = decay * a[r]
            want += (q[t] * decay * k[s]).sum(-1, keepdim=True) * v[s]
        assert torch.allclose(o[t], want)


def test_hgrn2_forget_gate_stays_above_its_lower_bound_and_carries_far():
    cfg = model(50, 32, [hgrn2_layer(2, 8, 8)], taps=0)
    w = weights_for(cfg)
    w["l0.mix.lower"] = torch.full_like(w["l0.mix.lower"], 0.999)  # hardly forgets
    a = [3, 9, 1] + [5] * 200
    b = [4, 9, 1] + [5] * 200
    la, lb = pz.forward(a, w, cfg), pz.forward(b, w, cfg)
    assert float((la[-1] - lb[-1]).abs().max()) > 1e-6  # the first token still shows 200 tokens on
    c = a[:10] + [7] + a[11:]
    assert torch.equal(pz.forward(c, w, cfg)[:10], la[:10])  # causal


def test_soft_cap_bounds_the_scores_and_the_bias_depends_on_distance_only():
    torch.manual_seed(2)
    T, H, d = 9, 2, 4
    q, k, v = (torch.randn(T, H, d, dtype=torch.float64) for _ in range(3))
    big = pz.softmax_attention(q * 1e4, k, v, 1.0, softcap=2.0)
    # capped scores lie in [-2, 2]: no key's weight falls below exp(-4) / T
    assert torch.isfinite(big).all()
    w_min = math.exp(-4.0) / T
    only = torch.zeros_like(v)
    only[0] = 1.0
    assert float(pz.softmax_attention(q * 1e4, k, only, 1.0, softcap=2.0)[-1].min()) >= w_min - 1e-12
    # a bias that favours distance 3 alone: every query from position 3 on returns the value three back
    rel = torch.full((8, H), -1e4, dtype=torch.float64)
    rel[3] = 0.0
    out = pz.softmax_attention(q * 0, k, v, 1.0, rel=rel, far=20.0)
    assert torch.allclose(out[3:], v[:-3])


def test_router_weights_sum_to_the_scale_and_the_correction_moves_the_choice_only():
    cfg = model(40, 16, [hgrn2_layer(1, 4, 4, mlp=moe(8, 5, 2, 1.75, shared=8))], taps=0)
    w = weights_for(cfg)
    h = torch.randn(6, 16, dtype=torch.float64)
    r = cfg["layers"][0]["mlp"]["router"]
    ids, wts = pz.route(h, w, "l0.mlp", r)
    assert torch.allclose(wts.sum(-1), torch.full((6,), 1.75, dtype=torch.float64))
    w2 = dict(w)
    w2["l0.mlp.correction"] = torch.tensor([0.0, 0.0, 0.0, 0.0, 9.0], dtype=torch.float64)
    ids2, wts2 = pz.route(h, w2, "l0.mlp", r)
    assert bool((ids2[:, 0] == 4).all())
    s = torch.softmax(h @ w["l0.mlp.router"].T, -1)
    picked = torch.gather(s, 1, ids2)
    assert torch.allclose(wts2, picked / picked.sum(-1, keepdim=True) * 1.75)  # the weights know nothing of the correction


def test_configuration_reader():
    for name, cfg in CONFIGS.items():
        c = SazilornConfig.from_dict(cfg)
        assert len(c.layers) == len(cfg["layers"]) and c.width == cfg["width"] and c.taps == cfg.get("canon", {}).get("taps", 0)
    c = SazilornConfig.from_dict(MIXED)
    assert c.layers[1].mixer.bias_max == 100 and c.layers[1].ff.shared_ff == 56 and c.layers[4].ff.shared_ff is None
    assert c.layers[2].mixer.right.decay == (0.5, 0.9, 0.995) and c.layers[2].mixer.left.softcap == 5.0
    # the table's rows come from the checkpoint's shapes where the file does not say them
    bare = attention_layer(2, 1, 8, 8, 0.3, 50, None)
    del bare["mixer"]["bias_buckets"]
    c = SazilornConfig.from_dict(model(20, 16, [bare]))
    assert c.layers[0].mixer.bias_buckets is None
    assert c.with_tensor_shapes({"l0.mix.rel": (10, 2)}).layers[0].mixer.bias_buckets == 10
    for broken in (
        {**MIXED, "layers": [{**MIXED["layers"][0], "type": "mamba"}]},
        {k: v for k, v in MIXED.items() if k != "max_positions"},
        model(20, 16, [parallel_layer((2, 1, 8, 8, 0.3, 5.0), (2, 8, 8, [0.5]), 1.0, 1.0)]),
        model(20, 16, [attention_layer(3, 2, 8, 8, 0.3, 50, 8)]),
        model(20, 16, [hgrn2_layer(1, 4, 4, mlp=moe(8, 2, 3, 1.0))]),
        model(20, 16, [hgrn2_layer(1, 4, 4, mlp={"kind": "conv", "ff": 3})]),
    ):
        with pytest.raises(ConfigError):
            SazilornConfig.from_dict(broken)


def test_spec_names_every_tensor_once_and_plans_caches_and_states():
    arch = architecture_of(AWKWARD)
    assert arch.name == "sazilorn"
    m = build_model(arch, arch.config_from_dict(AWKWARD))
    names = [s.name for s in m.tensor_specs()]
    assert len(names) == len(set(names))
    for want in ("embed", "pos", "l0.canon1", "l0.dwa", "l0.mix.left.g", "l0.mix.right.norm", "l0.mlp.e2.down", "l0.mlp.shared.up",
                 "l1.mix.f.b", "l1.mix.lower", "l2.mix.rel", "l2.mix.q.norm", "final.norm", "head"):
        assert want in names
    assert "l0.mlp.shared.sg" not in names and "l2.mlp.gate" not in names
    shapes = {s.name: s.shape for s in m.tensor_specs()}
    assert shapes["l3.dwa"] == (5,) and shapes["l2.mix.rel"] == (2, 5) and shapes["l0.canon1"] == (90, 2)
    caches, states = m.cache_needs(), m.state_needs()
    assert caches[1] is None and caches[3] is None and caches[0].num_kv_heads == 3 and caches[2].value_size == 6
    # the pair keeps the convolution's last input and the recurrence's matrices; an attention layer the former only
    assert [s.shape for s in states[0]] == [(90,), (5 * 6 * 12,)] and states[2].shape == (90,)
    # one tap: the convolution keeps nothing
    one = model(20, 16, [attention_layer(2, 1, 8, 8, 0.3, 50, 8)], taps=1)
    arch1 = architecture_of(one)
    assert build_model(arch1, arch1.config_from_dict(one)).state_needs() == [None]
