"""Sazilorn through the engine against the plain model: every mechanism alone, prompts against
token-by-token decoding, portions down to two tokens and one, unequal requests in one batch on pages
and slots that are used again, keys at page borders, far back and at both sides of the borders between
buckets of distances, first tokens, long decoding, and greedy generation through ``Engine.generate``."""

from __future__ import annotations

import json

import pytest
import torch

import plain_sazilorn as pz
from replay_helpers import mixed_trace, portions, run_steps, tail_one_by_one, whole
from sazilorn_models import (CONFIGS, MIXED, STEADY, TOL, attention_layer, compare_rows, dense, hgrn2_layer, load_plain, make_folder,
                             model, moe, parallel_layer, plain_rows)
from tiny_models import random_tokens
from tokasaurus_amd.engine.runner import ModelRunner
from tokasaurus_amd.kernels import ops

pytestmark = pytest.mark.gpu
PAGE = 16


@pytest.fixture(scope="module")
def sazilorn_folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("sazilorn")
    return {(name, steady): make_folder(root / f"{name}{int(steady)}", cfg, seed=5 + i, steady_choice=steady)
            for i, (name, cfg) in enumerate(sorted(CONFIGS.items())) for steady in (False, True)}


def runner_for(folder, dtype, tokens=512, slots=4, **kw):
    return ModelRunner.from_folder(str(folder), dtype, page_size=PAGE, num_pages=tokens // PAGE, max_slots=slots, **kw)


def step_arrays(lens, slots):
    starts = [0]
    for n in lens:
        starts.append(starts[-1] + n)
    req = [r for r, n in enumerate(lens) for _ in range(n)]
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device="cuda")  # noqa: E731
    return i32(starts), i32(req), i32(slots)


# ---------------------------------------------------------------------------------- kernels alone


@pytest.mark.parametrize("heads, dk, dv, lens", [(2, 16, 16, [1, 1, 1]), (3, 12, 6, [3, 40, 1, 9]), (1, 128, 64, [70, 7]),
                                                 (2, 50, 20, [33]), (1, 200, 8, [5, 18]), (1, 300, 8, [9, 3]), (1, 512, 4, [6]),
                                                 (3, 50, 6, [1, 1]), (1, 300, 8, [1]), (2, 128, 40, [1, 1, 1, 1])])
@pytest.mark.parametrize("form", ["constant", "forget"])
def test_linear_attention_kernel(heads, dk, dv, lens, form):
    """The recurrence on random sums, from random states in shuffled slots, against the plain loop; then the same
    tokens cut in two steps: the same bits."""
    torch.manual_seed(dk + dv)
    n, H = sum(lens), heads
    proj = torch.randn(n, 2 * H * dk + H * dv + 5, dtype=torch.float32)
    slots = list(range(len(lens)))[::-1]
    state0 = torch.randn(len(lens) + 1, H * dv * dk, dtype=torch.float32) * 0.3
    decay = torch.rand(H) if form == "constant" else None
    bias, low = (torch.randn(H * dk), torch.rand(H * dk)) if form == "forget" else (None, None)
    q_start, _, slot_t = step_arrays(lens, slots)
    dev = lambda t: None if t is None else t.cuda()  # noqa: E731
    state = state0.clone().cuda()
    o = ops.linear_attention(proj.cuda(), 0, H * dk, 2 * H * dk, state, q_start, slot_t, H, dk, dv, decay=dev(decay),
                             forget_bias=dev(bias), forget_low=dev(low))
    p64 = proj.double()
    at = 0
    for r, ln in enumerate(lens):
        rows = p64[at : at + ln]
        q = pz.silu(rows[:, : H * dk]).view(ln, H, dk)
        if form == "constant":
            k = pz.silu(rows[:, H * dk : 2 * H * dk]).view(ln, H, dk)
            v = pz.silu(rows[:, 2 * H * dk : 2 * H * dk + H * dv]).view(ln, H, dv)
            a = decay.double()[None, :, None].expand(ln, H, dk)
        else:
            f = (low.double() + (1 - low.double()) * torch.sigmoid(rows[:, H * dk : 2 * H * dk] + bias.double())).view(ln, H, dk)
            a, k = f, 1.0 - f
            v = rows[:, 2 * H * dk : 2 * H * dk + H * dv].view(ln, H, dv)
        S = state0[slots[r]].double().view(H, dv, dk).transpose(1, 2).clone()  # kept transposed: [H][dv][dk]
        for t in range(ln):
            S = a[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
            want = torch.einsum("hdv,hd->hv", S, q[t]).reshape(-1)
            assert torch.allclose(o[at + t].cpu().double(), want, atol=2e-4, rtol=2e-4), (r, t)
        assert torch.allclose(state[slots[r]].cpu().double().view(H, dv, dk), S.transpose(1, 2), atol=2e-4, rtol=2e-4)
        at += ln
    assert torch.equal(state[len(lens)].cpu(), state0[len(lens)])  # a slot of no request stays as it was
    if max(lens) == 1:
        # the form for steps of single tokens (activations in the recurrence's own kernel): the same bits
        state1 = state0.clone().cuda()
        o1 = ops.linear_attention(proj.cuda(), 0, H * dk, 2 * H * dk, state1, q_start, slot_t, H, dk, dv, decay=dev(decay),
                                  forget_bias=dev(bias), forget_low=dev(low), longest=1)
        assert torch.equal(o1, o) and torch.equal(state1, state)
    # the same tokens in two steps, cut inside every request that has two tokens or more
    cut = [max(1, ln // 3) if ln > 1 else 1 for ln in lens]
    state2 = state0.clone().cuda()
    first = torch.cat([proj[sum(lens[:r]) : sum(lens[:r]) + cut[r]] for r in range(len(lens))])
    qs1, _, _ = step_arrays(cut, slots)
    o1 = ops.linear_attention(first.cuda(), 0, H * dk, 2 * H * dk, state2, qs1, slot_t, H, dk, dv, decay=dev(decay),
                              forget_bias=dev(bias), forget_low=dev(low))
    rest = [ln - c for ln, c in zip(lens, cut)]
    keep = [r for r in range(len(lens)) if rest[r] > 0]
    if keep:
        second = torch.cat([proj[sum(lens[:r]) + cut[r] : sum(lens[: r + 1])] for r in keep])
        qs2, _, sl2 = step_arrays([rest[r] for r in keep], [slots[r] for r in keep])
        o2 = ops.linear_attention(second.cuda(), 0, H * dk, 2 * H * dk, state2, qs2, sl2, H, dk, dv, decay=dev(decay),
                                  forget_bias=dev(bias), forget_low=dev(low))
    a1 = a2 = 0
    for r, ln in enumerate(lens):
        base = sum(lens[:r])
        assert torch.equal(o1[a1 : a1 + cut[r]], o[base : base + cut[r]])
        a1 += cut[r]
        if rest[r]:
            assert torch.equal(o2[a2 : a2 + rest[r]], o[base + cut[r] : base + ln])
            a2 += rest[r]
    assert torch.equal(state2, state)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width, taps, lens", [(24, 3, [1, 1, 1]), (70, 4, [3, 40, 1, 9]), (300, 2, [5, 2]), (64, 1, [7]), (33, 9, [4, 1, 30])])
def test_short_convolution_kernel(dtype, width, taps, lens):
    """h + conv(h) from tails of earlier steps in shuffled slots; then the tails it leaves feed the next step: a
    sequence cut in two gives the rows of the whole one (single tokens move their tails in the same kernel)."""
    torch.manual_seed(width + taps)
    n = sum(lens)
    h = torch.randn(2 * n, width).to(dtype)
    w = torch.randn(width, taps)
    slots = list(range(len(lens)))[::-1]
    tails = torch.zeros(len(lens) + 1, max(taps - 1, 1) * width, dtype=torch.float32).cuda()
    # every request twice as long, in two steps of its length each
    seqs = [h[2 * sum(lens[:r]) : 2 * sum(lens[: r + 1])] for r in range(len(lens))]
    want = [s.double() + pz.short_convolution(s.double(), w.double()) for s in seqs]
    for half in (0, 1):
        rows = torch.cat([s[half * ln : (half + 1) * ln] for s, ln in zip(seqs, lens)]).cuda()
        q_start, req, slot_t = step_arrays(lens, slots)
        out = ops.short_conv(rows, w.t().contiguous().cuda(), tails if taps > 1 else None, q_start, req, slot_t, single_tokens=max(lens) == 1)
        at = 0
        for r, ln in enumerate(lens):
            ref = want[r][half * ln : (half + 1) * ln]
            tol = 1e-5 if dtype == torch.float32 else 2e-2
            assert torch.allclose(out[at : at + ln].cpu().double(), ref, atol=tol, rtol=tol), (half, r)
            at += ln


@pytest.mark.parametrize("width", [70, 256, 1028])
def test_depth_average_kernel(width):
    """The weighted sum over the streams so far, with and without a last stream that has only the wanted rows, the
    norm's rows from the same pass, and a block's branches added to the newest stream on the way."""
    torch.manual_seed(3)
    hist = torch.randn(5, 9, width).cuda()
    w = torch.randn(4).cuda()
    nw = torch.randn(width).cuda() * 0.1
    out, normed = ops.depth_average(hist, 4, w, norm_weight=nw, unit_offset=True, eps=1e-5, out_dtype=torch.float32)
    want = sum(w[j].double().cpu() * hist[j].double().cpu() for j in range(4))
    assert torch.allclose(out.cpu().double(), want, atol=1e-5)
    assert torch.allclose(normed.cpu().double(), pz.offset_norm(want, nw.cpu().double(), 1e-5), atol=1e-5)
    rows = torch.tensor([8, 0, 3], dtype=torch.int32).cuda()
    last = torch.randn(3, width).cuda()
    out, normed = ops.depth_average(hist, 3, w, last=last, rows=rows, out_dtype=torch.bfloat16)
    want = sum(w[j].double().cpu() * hist[j].double().cpu()[[8, 0, 3]] for j in range(3)) + w[3].double().cpu() * last.double().cpu()
    assert normed is None and torch.allclose(out.cpu().double(), want, atol=1e-5)
    # branches: the newest stream becomes itself + mult * (a + b), in place, before it is weighed
    a, b = torch.randn(9, width).cuda(), torch.randn(9, width).cuda()
    h2 = hist.clone()
    out, _ = ops.depth_average(h2, 4, w, branches=(a, b), mult=0.5)
    newest = hist[3].double().cpu() + 0.5 * (a.double().cpu() + b.double().cpu())
    want = sum(w[j].double().cpu() * hist[j].double().cpu() for j in range(3)) + w[3].double().cpu() * newest
    assert torch.allclose(out.cpu().double(), want, atol=1e-5) and torch.allclose(h2[3].cpu().double(), newest, atol=1e-6)
    assert torch.equal(h2[:3], hist[:3]) and torch.equal(h2[4], hist[4])
    l2 = last.clone()
    out, _ = ops.depth_average(hist, 3, w, last=l2, rows=rows, branches=(a[:3].contiguous(), None), mult=2.0)
    newest = last.double().cpu() + 2.0 * a[:3].double().cpu()
    want = sum(w[j].double().cpu() * hist[j].double().cpu()[[8, 0, 3]] for j in range(3)) + w[3].double().cpu() * newest
    assert torch.allclose(out.cpu().double(), want, atol=1e-5) and torch.allclose(l2.cpu().double(), newest, atol=1e-6)


def test_router_with_normalised_weights():
    torch.manual_seed(4)
    h, wr = torch.randn(7, 40), torch.randn(6, 40) * 0.3
    corr = torch.randn(6) * 0.2
    ids, wts, gate = ops.expert_route(h.cuda(), wr.cuda(), corr.cuda(), 1, 1, 3, normalize_scale=1.75, unit_gate=True)
    want_ids, want_w = pz.route(h.double(), {"p.router": wr.double(), "p.correction": corr.double()}, "p", {"top": 3, "scale": 1.75})
    assert torch.equal(ids.cpu().long(), want_ids) and torch.allclose(wts.cpu().double(), want_w, atol=1e-6)
    assert torch.equal(gate.cpu(), torch.ones(7))


def test_gelu_gate_and_sigmoid_gate_kernels():
    torch.manual_seed(5)
    gu = torch.randn(5, 2 * 37) * 3
    want = pz.gelu_tanh(gu[:, :37].double()) * gu[:, 37:].double()
    assert torch.allclose(ops.gelu_glu(gu.cuda()).cpu().double(), want, atol=1e-5)
    x, g = torch.randn(4, 50), torch.randn(4, 80)
    out = torch.zeros(4, 90).cuda()
    ops.sigmoid_gate(x.cuda(), g.cuda()[:, 10:60], scale=0.7, out=out[:, 40:])
    assert torch.allclose(out[:, 40:].cpu().double(), x.double() * torch.sigmoid(g[:, 10:60].double()) * 0.7, atol=1e-6)
    assert float(out[:, :40].abs().max()) == 0.0


@pytest.mark.parametrize("groups, size", [(1, 1024), (1, 300), (3, 20), (2, 512), (1, 4100)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_behind_the_recurrence(groups, size, dtype):
    """Every group's numbers over their root mean square, times the shared weight, the gate's sigmoid and a factor,
    into columns of a wider buffer: a wavefront a group for small groups, a workgroup for large ones."""
    torch.manual_seed(size)
    n = 5
    o, w = torch.randn(n, groups * size), torch.randn(size)
    gate = torch.randn(n, groups * size + 8)
    out = torch.zeros(n, groups * size + 16, dtype=dtype).cuda()
    for g in (None, gate):
        view = out[:, 16:]
        ops.group_norm_gate(o.cuda(), w.cuda(), 1e-5, groups, dtype, gate=None if g is None else g.cuda()[:, 8:], scale=0.7, out=view)
        want = pz.rms(o.double().view(n, groups, size), 1e-5) * w.double()
        if g is not None:
            want = want * torch.sigmoid(g[:, 8:].double().view(n, groups, size))
        tol = 1e-5 if dtype == torch.float32 else 2e-2
        assert torch.allclose(view.cpu().double(), want.reshape(n, -1) * 0.7, atol=tol, rtol=tol)
    assert float(out[:, :16].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gate_per_element_with_16_byte_loads(dtype):
    torch.manual_seed(6)
    x, g = torch.randn(6, 128).to(dtype), torch.randn(6, 256 + 64).to(dtype)
    out = torch.zeros(6, 128 + 64, dtype=dtype).cuda()
    ops.sigmoid_gate(x.cuda(), g.cuda()[:, 64:192], scale=1.5, out=out[:, :128])
    want = x.double() * torch.sigmoid(g[:, 64:192].double()) * 1.5
    tol = 1e-6 if dtype == torch.float32 else 2e-2
    assert torch.allclose(out[:, :128].cpu().double(), want, atol=tol, rtol=tol) and float(out[:, 128:].abs().max()) == 0.0


# ---------------------------------------------------------------------------------- one mechanism a model


SINGLE_LAYERS = {
    "attention_bias": attention_layer(4, 2, 16, 16, 0.3, 60, 10),
    "attention_bias_many_heads_a_key": attention_layer(16, 1, 32, 48, 0.2, 300, 16, mlp=dense(40)),
    "attention_bias_odd_sizes": attention_layer(3, 3, 20, 6, 0.3, 9, 4),  # sizes the matrix-core kernel does not take
    "attention_bias_large_heads": attention_layer(2, 1, 128, 128, 0.09, 150, 32),
    "hgrn2": hgrn2_layer(2, 16, 16),
    "hgrn2_odd_sizes": hgrn2_layer(3, 10, 7, mlp=dense(20)),
    "hgrn2_large_heads": hgrn2_layer(2, 128, 128),
    "pair": parallel_layer((4, 2, 16, 16, 0.3, 3.0), (2, 16, 16, [0.8, 0.99]), 0.6, 1.4),
    "pair_odd_sizes": parallel_layer((3, 1, 24, 40, 0.2, 1.0), (3, 6, 10, [0.2, 0.5, 1.0]), 2.0, 0.3, mlp=dense(30)),
    "pair_large_heads": parallel_layer((4, 1, 128, 64, 0.1, 40.0), (1, 128, 128, [0.999]), 1.0, 1.0),
    "experts": hgrn2_layer(1, 8, 8, mlp=moe(24, 7, 2, 1.5, shared=16)),
    "experts_one_chosen_no_shared": attention_layer(2, 1, 16, 16, 0.3, 40, 8, mlp=moe(10, 3, 1, 0.5)),
    "dense_gelu": hgrn2_layer(1, 8, 8, mlp=dense(100)),
}


@pytest.mark.parametrize("name", sorted(SINGLE_LAYERS))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_layer_alone(tmp_path, name, dtype):
    """A model of one layer: whole, token by token and in portions of two and three tokens; with and without
    the convolution in front of the mixer."""
    for taps in (3, 0):
        config = model(61, 64, [SINGLE_LAYERS[name]], taps=taps)
        folder = make_folder(tmp_path / f"one{taps}", config, seed=3, steady_choice=STEADY[dtype])
        reqs = {"a": random_tokens(50, 61, 1), "b": random_tokens(19, 61, 2)}
        plain = plain_rows(folder, reqs)
        runner = runner_for(folder, dtype, tokens=128)
        for rid, toks in reqs.items():
            compare_rows(run_steps(runner, whole(rid, toks)), plain, TOL[dtype])
        compare_rows(run_steps(runner, tail_one_by_one("a", reqs["a"], tail=30)), plain, TOL[dtype])
        compare_rows(run_steps(runner, portions("a", reqs["a"], [2, 3])), plain, TOL[dtype])
        compare_rows(run_steps(runner, mixed_trace(reqs, 1, max_live=2)), plain, TOL[dtype])


def test_the_stream_after_every_layer(sazilorn_folders):
    """The stream that every layer hands on (after the average over the streams so far) against the plain model's."""
    from tokasaurus_amd.engine.batch import StepEntry, layout, to_device

    folder = sazilorn_folders["mixed", False]
    cfg, w = load_plain(folder)
    tokens = random_tokens(37, MIXED["vocab"], 6)
    want: list = []
    pz.forward(tokens, w, cfg, want)
    runner = runner_for(folder, "float32")
    planned = runner.plan([StepEntry("tap", tokens, [])])
    runner.storage.reset_slots(runner.manager.take_fresh_slots())
    hb = layout(planned, runner.model.spec.vocab_size, len(runner.groups), runner.manager.slot_tables)
    ctx, _, tables = to_device(hb, runner.model.dtype, runner.model.device, runner.storage.last_token)
    ctx.extras["kv_bound"] = runner.kv_bound(ctx.max_kv_len)
    tap: list = []
    ctx.extras["model_tap"] = tap
    runner.model.forward(ctx, runner.cache_views(tables), runner.storage.states, None)
    runner.release("tap")
    assert len(tap) == len(want)
    for got, ref in zip(tap, want):
        assert float((got.cpu().double() - ref).abs().max()) < 2e-4 * max(1.0, float(ref.abs().max()))


# ---------------------------------------------------------------------------------- cuttings, batches, reuse


@pytest.mark.parametrize("name", sorted(CONFIGS))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_every_cutting_gives_the_plain_rows(sazilorn_folders, name, dtype):
    """Whole prompts, a tail decoded token by token (through recorded steps), portions of changing sizes down to
    two tokens and one, and unequal requests mixed in one batch on a pool so small that pages and slots are used
    again."""
    folder, vocab = sazilorn_folders[name, STEADY[dtype]], CONFIGS[name]["vocab"]
    reqs = {f"r{i}": random_tokens(n, vocab, 50 + i) for i, n in enumerate((70, 3, 41, 1, 97, 26))}
    plain = plain_rows(folder, reqs)
    runner = runner_for(folder, dtype, tokens=256)
    tol = TOL[dtype]
    for rid, toks in reqs.items():
        compare_rows(run_steps(runner, whole(rid, toks)), plain, tol)
    compare_rows(run_steps(runner, tail_one_by_one("r4", reqs["r4"], tail=40)), plain, tol)
    compare_rows(run_steps(runner, portions("r4", reqs["r4"], [2, 3, 16, 2, 1, 31, 5])), plain, tol)
    compare_rows(run_steps(runner, portions("r0", reqs["r0"], [15, 17, 1, 2])), plain, tol)
    for seed in (1, 2):
        compare_rows(run_steps(runner, mixed_trace(reqs, seed, max_live=4)), plain, tol)
    assert runner.manager.requests == {}
    if dtype == "float32":
        # the same position from different cuttings: the same up to the order of 32-bit sums
        a = run_steps(runner, whole("r2", reqs["r2"]))
        b = run_steps(runner, portions("r2", reqs["r2"], [2, 7]))
        for key in a:
            assert float((a[key] - b[key]).abs().max()) < 2e-4 * max(1.0, float(a[key].abs().max()))


def test_batch_rows_do_not_depend_on_their_neighbours(sazilorn_folders):
    """A request's rows beside other requests are those it has alone (32-bit: up to the order of sums)."""
    folder, vocab = sazilorn_folders["mixed", False], MIXED["vocab"]
    reqs = {f"r{i}": random_tokens(n, vocab, 70 + i) for i, n in enumerate((33, 5, 18))}
    runner = runner_for(folder, "float32", tokens=256)
    alone = {}
    for rid, toks in reqs.items():
        alone.update(run_steps(runner, whole(rid, toks)))
    together = run_steps(runner, [{"entries": [(rid, toks, list(range(len(toks)))) for rid, toks in reqs.items()], "end": list(reqs)}])
    for key, row in together.items():
        assert float((row - alone[key]).abs().max()) < 2e-4 * max(1.0, float(row.abs().max())), key


def test_slots_and_pages_are_clean_for_their_next_holder(sazilorn_folders):
    """Two slots and few pages: a request that takes a slot after another finds zero states (the recurrences'
    matrices, the convolutions' last inputs) and its own keys only."""
    for name in ("mixed", "only_linear"):
        folder, vocab = sazilorn_folders[name, False], CONFIGS[name]["vocab"]
        reqs = {f"q{i}": random_tokens(n, vocab, 90 + i) for i, n in enumerate((40, 25, 31, 12, 37))}
        plain = plain_rows(folder, reqs)
        runner = runner_for(folder, "float32", tokens=96, slots=2)
        compare_rows(run_steps(runner, mixed_trace(reqs, 5, max_live=2)), plain, TOL["float32"])
        for rid, toks in reqs.items():
            compare_rows(run_steps(runner, tail_one_by_one(rid, toks, tail=3)), plain, TOL["float32"])


# ---------------------------------------------------------------------------------- marked keys


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_marked_key_at_both_sides_of_every_bucket_s_border(tmp_path, dtype):
    """One bucket of distances is made to stand out: its bias is 8 and every other 0, so in a model of one layer
    the last token sees (almost) only the keys whose distance falls into that bucket.  A token that appears once is
    put on the bucket's first distance, on its last, and on the distances just outside: the plain model's last row
    moves if and only if the marked key is inside.  The engine must agree with the plain model in every case, for
    every bucket (one distance a bucket, then the logarithmic ones, then all beyond the reach), in a whole prompt,
    with the last tokens decoded alone, in portions of two tokens, and with the marked key itself decoded alone."""
    B, far, n = 10, 60, 200
    by_distance = [pz.distance_bucket(d, B, far) for d in range(n)]
    for b in range(1, B):
        config = model(64, 32, [attention_layer(2, 1, 16, 16, 0.5, far, B)], taps=0)
        table = torch.zeros(B)
        table[b] = 8.0
        folder = make_folder(tmp_path / f"bucket{b}", config, seed=8 + b, edits={".rel": lambda t: table[:, None].expand_as(t).clone()})
        cfg, w = load_plain(folder)
        runner = runner_for(folder, dtype, tokens=256)
        lo, hi = by_distance.index(b), max(d for d in range(n) if by_distance[d] == b)
        moved = {}
        for back in sorted({max(lo - 1, 1), lo, hi, min(hi + 1, n - 1)}):  # (distance 0 is the last token itself)
            tokens = [t % 63 for t in random_tokens(n, 64, 100 + back)]
            unmarked = pz.forward(tokens, w, cfg)[-1]
            tokens[n - 1 - back] = 63
            plain = pz.forward(tokens, w, cfg).float()
            moved[back] = float((plain[-1] - unmarked).abs().max())
            cuts = [whole("e", tokens), tail_one_by_one("e", tokens, tail=3), portions("e", tokens, [2, 61])]
            if back < 70:
                cuts.append(tail_one_by_one("e", tokens, tail=back + 2))  # the marked key itself is decoded alone
            for steps in cuts:
                got = run_steps(runner, steps)
                compare_rows({k: v for k, v in got.items() if k[1] >= n - 3}, {"e": plain}, TOL[dtype])
        inside = min(m for back, m in moved.items() if lo <= back <= hi)
        outside = max([m for back, m in moved.items() if not lo <= back <= hi] or [0.0])
        assert inside > 20 * outside, f"bucket {b} (distances {lo} to {hi}): the mark moves the last row by {moved}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_keys_at_page_borders_and_far_back(tmp_path, dtype):
    """A table of biases that leans towards the far buckets, and one token changed at a page's border, a page and
    two pages back and hundreds of tokens back: the engine's last rows are the plain model's."""
    B, far, n = 12, 90, 300
    config = model(64, 32, [attention_layer(2, 1, 16, 16, 0.5, far, B)], taps=3)
    ramp = torch.tensor([0.6 * b for b in range(B)])
    folder = make_folder(tmp_path / "far", config, seed=8, edits={".rel": lambda t: ramp[:, None].expand_as(t).clone()})
    cfg, w = load_plain(folder)
    runner = runner_for(folder, dtype, tokens=320)
    for back in (1, 15, 16, 17, 31, 32, 250, 299):
        tokens = [t % 63 for t in random_tokens(n, 64, 100 + back)]
        tokens[n - 1 - back] = 63
        plain = pz.forward(tokens, w, cfg).float()
        for steps in (whole("e", tokens), tail_one_by_one("e", tokens, tail=3), portions("e", tokens, [2, 61])):
            got = run_steps(runner, steps)
            compare_rows({k: v for k, v in got.items() if k[1] >= n - 3}, {"e": plain}, TOL[dtype])


@pytest.mark.parametrize("kind", ["hgrn2", "pair"])
def test_a_token_far_back_shows_through_the_recurrence(tmp_path, kind):
    """A state that hardly forgets (a forget gate that no token moves and that stays near one; decays near and at
    one): the first token's mark is still in the last row 300 tokens on, in a whole prompt, token by token and
    across portions."""
    layer = hgrn2_layer(2, 16, 16) if kind == "hgrn2" else parallel_layer((2, 1, 16, 16, 0.3, 5.0), (2, 16, 16, [0.9995, 1.0]), 0.01, 2.0)
    config = model(64, 32, [layer], taps=2)
    folder = make_folder(tmp_path / "slow", config, seed=3, edits={
        ".lower": lambda t: t * 0 + 0.5, ".mix.f": lambda t: t * 0, ".f.b": lambda t: t * 0 + 4.5})
    cfg, w = load_plain(folder)
    n = 300
    tokens = [t % 63 for t in random_tokens(n, 64, 9)]
    unmarked = pz.forward(tokens, w, cfg)[-1]
    tokens[0] = 63
    plain = pz.forward(tokens, w, cfg).float()
    assert float((plain[-1] - unmarked).abs().max()) > 1e-3
    runner = runner_for(folder, "float32", tokens=448)
    for steps in (whole("e", tokens), tail_one_by_one("e", tokens, tail=250), portions("e", tokens, [2, 61, 1])):
        got = run_steps(runner, steps)
        compare_rows({k: v for k, v in got.items() if k[1] >= n - 3}, {"e": plain}, 3e-5)


def test_the_convolution_reaches_across_the_cut(tmp_path):
    """Taps of order one on a convolution of five: a row's logits depend on the four tokens before it, so a tail
    that is lost at the start of a portion shows.  Portions of one, two and three tokens against the whole."""
    config = model(64, 32, [hgrn2_layer(1, 8, 8)], taps=5)
    folder = make_folder(tmp_path / "taps", config, seed=4, edits={"canon1": lambda t: t * 2.0})
    cfg, w = load_plain(folder)
    tokens = random_tokens(40, 64, 5)
    plain = {"c": pz.forward(tokens, w, cfg).float()}
    other = list(tokens)
    other[30] = (other[30] + 1) % 64
    assert float((pz.forward(other, w, cfg)[34] - plain["c"][34]).abs().max()) > 1e-3
    runner = runner_for(folder, "float32", tokens=64)
    for sizes in ([1], [2], [3, 1, 2], [4, 5]):
        compare_rows(run_steps(runner, portions("c", tokens, sizes)), plain, TOL["float32"])


def test_first_tokens_of_a_sequence(sazilorn_folders):
    """Requests of one, two and three tokens, whole and token by token: zeros in front of the convolution, a state
    that starts at zero, one key under the bias of distance zero, the first page half empty."""
    for name in sorted(CONFIGS):
        folder, vocab = sazilorn_folders[name, False], CONFIGS[name]["vocab"]
        reqs = {f"s{n}": random_tokens(n, vocab, 30 + n) for n in (1, 2, 3, 6)}
        plain = plain_rows(folder, reqs)
        runner = runner_for(folder, "float32", tokens=64)
        for rid, toks in reqs.items():
            compare_rows(run_steps(runner, whole(rid, toks)), plain, TOL["float32"])
            compare_rows(run_steps(runner, portions(rid, toks, [1])), plain, TOL["float32"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(sazilorn_folders, dtype):
    """A short prompt and 400 tokens decoded one by one through recorded steps: distances pass every bucket of the
    tables and their reach over decoded tokens."""
    folder, vocab = sazilorn_folders["mixed", STEADY[dtype]], MIXED["vocab"]
    tokens = random_tokens(420, vocab, 77)
    plain = plain_rows(folder, {"d": tokens})
    runner = runner_for(folder, dtype, tokens=448)
    got = run_steps(runner, tail_one_by_one("d", tokens, tail=400))
    compare_rows(got, plain, TOL[dtype])
    assert all(step.captured for step in runner.recorded.values()) and runner.recorded


def test_positions_end_where_the_table_ends(tmp_path):
    """A request may hold as many tokens as the table of positions has rows, and no more."""
    config = model(40, 32, [hgrn2_layer(1, 8, 8)], max_positions=48)
    folder = make_folder(tmp_path / "short", config, seed=2)
    runner = runner_for(folder, "float32", tokens=128)
    tokens = random_tokens(48, 40, 3)
    compare_rows(run_steps(runner, whole("p", tokens)), plain_rows(folder, {"p": tokens}), TOL["float32"])
    from tokasaurus_amd.engine.batch import StepEntry

    with pytest.raises(ValueError):
        runner.step([StepEntry("q", tokens + [1], [])])


# ---------------------------------------------------------------------------------- the entry points


@pytest.mark.parametrize("name", ["mixed", "awkward", "only_linear"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_engine(sazilorn_folders, dtype, name):
    """``Engine.generate``: the scheduler cuts prompts into portions beside decoding requests; the tokens are the
    plain model's greedy tokens (in bfloat16: each token is, for the plain logits of its own history, within
    rounding of the best)."""
    from tokasaurus_amd.config.engine_config import EngineConfig
    from tokasaurus_amd.engine.engine import Engine
    from tokasaurus_amd.sampling import SamplingParams

    folder, vocab = sazilorn_folders[name, STEADY[dtype]], CONFIGS[name]["vocab"]
    prompts = [random_tokens(n, vocab, 10 + n) for n in (5, 40, 23, 1, 64)]
    engine = Engine(EngineConfig(model=str(folder), dtype=dtype, page_size=PAGE, kv_cache_num_tokens=512, max_seqs_per_forward=3,
                                 max_tokens_per_forward=24, allocator_sanity_checks=True))
    done = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    cfg, w = load_plain(folder)
    for prompt, c in zip(prompts, done):
        assert len(c.tokens) == 12 and c.finish_reason == "length"
        ids = list(prompt)
        for tok in c.tokens:
            logits = pz.forward(ids, w, cfg)[-1]
            if dtype == "float32":
                assert tok == int(logits.argmax()), f"token {tok}, plain {int(logits.argmax())}"
            else:
                assert float(logits.max() - logits[tok]) < 0.05 * float(logits.std()) + 0.05
            ids.append(tok)
    assert engine.runner.manager.requests == {}


def test_command_line_and_trace_replay(sazilorn_folders, tmp_path):
    """``bin/toka`` generates from a Sazilorn folder, and ``bin/trace_run`` replays given tokens step by step: its
    logits are the plain model's."""
    import os
    import subprocess
    import sys

    import numpy as np

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder, vocab = sazilorn_folders["awkward", False], CONFIGS["awkward"]["vocab"]
    prompts = [random_tokens(9, vocab, 1), random_tokens(20, vocab, 2)]
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "toka"), f"model={folder}", "dtype=float32", f"page_size={PAGE}",
                           "kv_cache_num_tokens=256", f"prompt_ids=({json.dumps(prompts)})", "max_tokens=5", "ignore_eos=T"],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = [json.loads(l) for l in proc.stdout.splitlines() if l.strip()]
    cfg, w = load_plain(folder)
    for prompt, line in zip(prompts, lines):
        ids = list(prompt)
        for tok in line["tokens"]:
            assert tok == int(pz.forward(ids, w, cfg)[-1].argmax())
            ids.append(tok)
    a, b = random_tokens(21, vocab, 3), random_tokens(40, vocab, 4)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:17], "want": [0, 16]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[17:18], "want": [0]}, {"id": "b", "tokens": b[:33], "want": [32]}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[33:35], "want": []}, {"id": "a", "tokens": a[18:], "want": [2]}], "end": ["a"]},
        {"step": 3, "entries": [{"id": "b", "tokens": b[35:], "want": [4]}], "end": ["b"]},
    ]
    out = tmp_path / "out"
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(folder), "--dtype", "float32",
                           "--out", str(out), "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    plain = plain_rows(folder, {"a": a, "b": b})
    want = {0: [("a", 0), ("a", 16)], 1: [("a", 17), ("b", 32)], 2: [("a", 20)], 3: [("b", 39)]}
    for step, rows in want.items():
        got = torch.from_numpy(np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(len(rows), vocab).copy())
        compare_rows({key: got[i] for i, key in enumerate(rows)}, plain, TOL["float32"])


# ---------------------------------------------------------------------------------- drawn configurations


def random_config(seed: int) -> dict:
    """A model drawn from lists of comfortable and awkward sizes."""
    import random

    rng = random.Random(seed)
    width = rng.choice([32, 48, 90, 64, 100])
    layers = []
    for _ in range(rng.choice([1, 2, 3, 4])):
        kind = rng.choice(["attention", "hgrn2", "pair"])
        mlp = rng.choice([None, dense(rng.choice([24, 33, 64, 100])),
                          moe(rng.choice([8, 20, 32]), rng.choice([2, 5, 8]), rng.choice([1, 2]), rng.choice([0.5, 1.0, 2.5]),
                              shared=rng.choice([None, 8, 24]))])
        if kind == "hgrn2":
            layers.append(hgrn2_layer(rng.choice([1, 2, 5]), rng.choice([4, 16, 31, 64]), rng.choice([4, 9, 16, 64]), mlp=mlp))
        elif kind == "attention":
            kv = rng.choice([1, 2, 3])
            buckets = rng.choice([2, 4, 6, 16, 32])
            layers.append(attention_layer(kv * rng.choice([1, 2, 4, 5]), kv, rng.choice([8, 12, 16, 32, 40, 64]),
                                          rng.choice([2, 8, 16, 20, 32, 48]), rng.choice([0.1, 0.3]),
                                          rng.choice([buckets // 2 + 1, 37, 128, 1000]), buckets, mlp=mlp))
        else:
            kv = rng.choice([1, 2])
            hr = rng.choice([1, 2, 3])
            layers.append(parallel_layer((kv * rng.choice([1, 2, 3]), kv, rng.choice([8, 16, 24, 64]), rng.choice([8, 16, 32, 40]),
                                          rng.choice([0.1, 0.3]), rng.choice([1.0, 10.0, 50.0])),
                                         (hr, rng.choice([4, 16, 24, 64]), rng.choice([4, 16, 30]), [rng.choice([0.3, 0.9, 0.999, 1.0]) for _ in range(hr)]),
                                         rng.choice([0.5, 1.0]), rng.choice([0.25, 1.5]), mlp=mlp))
    return model(rng.choice([40, 97, 130]), width, layers, eps=rng.choice([1e-6, 1e-5]), taps=rng.choice([0, 1, 2, 3, 6]))


@pytest.mark.parametrize("seed", range(10))
def test_random_configurations(tmp_path, seed):
    config = random_config(seed)
    reqs = {f"r{i}": random_tokens(n, config["vocab"], 20 * seed + i) for i, n in enumerate((90, 2, 37, 130))}
    for dtype in ("float32", "bfloat16"):
        folder = make_folder(tmp_path / f"drawn{dtype}", config, seed=seed, steady_choice=STEADY[dtype])
        plain = plain_rows(folder, reqs)
        runner = runner_for(folder, dtype, tokens=320)
        for rid, toks in reqs.items():
            compare_rows(run_steps(runner, whole(rid, toks)), plain, TOL[dtype])
        compare_rows(run_steps(runner, tail_one_by_one("r3", reqs["r3"], tail=70)), plain, TOL[dtype])
        compare_rows(run_steps(runner, portions("r3", reqs["r3"], [2, 3, 16, 2, 1, 31, 5])), plain, TOL[dtype])
        compare_rows(run_steps(runner, mixed_trace(reqs, seed, max_live=3)), plain, TOL[dtype])
        assert runner.manager.requests == {}
