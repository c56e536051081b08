"""Sakevik through the engine against the plain model: every mechanism alone, prompts against
token-by-token decoding, portions down to two tokens and one, unequal requests in one batch on pages
and slots that are used again, keys just inside and just outside every window, at page borders and far
back, first tokens, long decoding, and greedy generation through ``Engine.generate``."""

from __future__ import annotations

import json

import pytest
import torch

import plain_sakevik as ps
from replay_helpers import mixed_trace, portions, run_steps, tail_one_by_one, whole
from sakevik_models import (CONFIGS, MIXED, RAMP, TOL, attention_layer, compare_rows, dense, gru_layer, latent_layer, load_plain,
                            make_folder, model, plain_rows)
from tiny_models import random_tokens
from tokasaurus_amd.engine.batch import StepEntry, layout, to_device
from tokasaurus_amd.engine.runner import ModelRunner
from tokasaurus_amd.kernels import ops

pytestmark = pytest.mark.gpu
PAGE = 16


@pytest.fixture(scope="module")
def sakevik_folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("sakevik")
    return {name: make_folder(root / name, cfg, seed=5 + i) for i, (name, cfg) in enumerate(sorted(CONFIGS.items()))}


def runner_for(folder, dtype, tokens=512, slots=4, **kw):
    return ModelRunner.from_folder(str(folder), dtype, page_size=PAGE, num_pages=tokens // PAGE, max_slots=slots, **kw)


def streams_of(runner, tokens):
    """The residual stream after every block for one whole prompt."""
    planned = runner.plan([StepEntry("tap", tokens, [])])
    runner.storage.reset_slots(runner.manager.take_fresh_slots())
    hb = layout(planned, runner.model.spec.vocab_size, len(runner.groups), runner.manager.slot_tables)
    ctx, _, tables = to_device(hb, runner.model.dtype, runner.model.device, runner.storage.last_token)
    ctx.extras["kv_bound"] = runner.kv_bound(ctx.max_kv_len)
    ctx.embedding_state = runner.storage.embedding_state
    tap: list = []
    ctx.extras["stream_tap"] = tap
    runner.model.forward(ctx, runner.cache_views(tables), runner.storage.states, None)
    runner.release("tap")
    return [t.cpu() for t in tap]


# ---------------------------------------------------------------------------------- kernels alone


@pytest.mark.parametrize("width, lens", [(24, [1, 1, 1]), (70, [3, 40, 1, 9]), (256, [300, 7]), (130, [33])])
def test_recurrence_kernel(width, lens):
    """The recurrence on random sums, from random states in shuffled slots, against the token-by-token loop;
    then the same tokens cut in two steps: the same bits."""
    torch.manual_seed(width)
    dev = "cuda"
    n = sum(lens)
    proj = torch.randn(n, 3 * width, device=dev) * 2
    state0 = torch.randn(len(lens) + 2, width, device=dev)
    slots = torch.tensor(list(range(len(lens), 0, -1)), dtype=torch.int32, device=dev)
    starts = [0]
    for l in lens:
        starts.append(starts[-1] + l)
    q_start = torch.tensor(starts, dtype=torch.int32, device=dev)
    state = state0.clone()
    bias = torch.randn(2 * width, device=dev)
    out = ops.min_gru(proj, state, q_start, slots, width, max(lens), torch.float32, bias=bias)
    p = proj.double().cpu().view(n, width, 3).permute(0, 2, 1).reshape(n, 3 * width)  # (a, u, g) a channel -> [a | u | g]
    p[:, : 2 * width] += bias.double().cpu()
    for r, l in enumerate(lens):
        S = state0[int(slots[r])].double().cpu()
        for t in range(starts[r], starts[r + 1]):
            a, u, g = p[t, :width], p[t, width : 2 * width], p[t, 2 * width :]
            z = torch.sigmoid(a)
            S = (1 - z) * S + z * torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
            assert torch.allclose(out[t].double().cpu(), S * g * torch.sigmoid(g), atol=2e-5, rtol=2e-5), (r, t)
        assert torch.allclose(state[int(slots[r])].double().cpu(), S, atol=2e-5, rtol=2e-5)
    assert torch.equal(state[0], state0[0]) and torch.equal(state[-1], state0[-1])  # slots of nobody stay
    # one request's tokens in two steps of other forms of the kernel
    if len(lens) == 1 and lens[0] > 9:
        st = state0.clone()
        one = torch.tensor([int(slots[0])], dtype=torch.int32, device=dev)
        a = ops.min_gru(proj[:9], st, torch.tensor([0, 9], dtype=torch.int32, device=dev), one, width, 9, torch.float32, bias=bias)
        b = ops.min_gru(proj[9:12], st, torch.tensor([0, 3], dtype=torch.int32, device=dev), one, width, 3, torch.float32, bias=bias)
        b = torch.cat([b, ops.min_gru(proj[12:], st, torch.tensor([0, n - 12], dtype=torch.int32, device=dev), one, width, n - 12,
                                      torch.float32, bias=bias)])
        assert torch.equal(torch.cat([a, b]), out) and torch.equal(st, state)


def test_embedding_with_pairs_and_the_token_before():
    torch.manual_seed(3)
    dev = "cuda"
    V, H, buckets = 50, 24, 7
    table = torch.randn(V, H, device=dev).bfloat16()
    pairs = torch.randn(buckets + 1, H, device=dev).bfloat16()
    prev = torch.full((5,), 11, dtype=torch.int32, device=dev)
    last = torch.tensor([0, 0, 42, 0, 0], dtype=torch.int32, device=dev)
    # request 0: positions 0..2 (a sequence's start), request 1: one token at position 9 read from the sampler's slot 2
    ids = torch.tensor([4, 5, 6, -3], dtype=torch.int32, device=dev)
    pos = torch.tensor([0, 1, 2, 9], dtype=torch.int32, device=dev)
    req = torch.tensor([0, 0, 0, 1], dtype=torch.int32, device=dev)
    q_start = torch.tensor([0, 3, 4], dtype=torch.int32, device=dev)
    slots = torch.tensor([3, 2], dtype=torch.int32, device=dev)
    x, rounded = ops.embed_bigram(ids, last, pos, req, q_start, slots, prev, table, pairs, 3.0, 5, 3)
    rows = [buckets, (4 * 5 + 5 * 3) % buckets, (5 * 5 + 6 * 3) % buckets, (11 * 5 + 42 * 3) % buckets]
    toks = [4, 5, 6, 42]
    for t in range(4):
        ref = table[toks[t]].float() * 3.0 + pairs[rows[t]].float()
        assert torch.allclose(x[t], ref, atol=1e-6, rtol=1e-6), t
    assert torch.equal(rounded, x.bfloat16())
    assert prev.tolist() == [11, 11, 42, 6, 11]


def test_stream_kernels_of_the_post_norm_block():
    torch.manual_seed(5)
    dev = "cuda"
    for rows, H in ((3, 90), (40, 256)):
        x, a = torch.randn(rows, H, device=dev), torch.randn(rows, H, device=dev) * 3
        wb = torch.rand(H, device=dev) + 0.5
        ref = x.double() + a.double() / torch.sqrt((a.double() ** 2).mean(-1, keepdim=True) + 1e-5) * wb.double()
        x1, h = ops.post_norm_residual(x.clone(), a, wb, 1e-5, out_dtype=torch.bfloat16, plain_rows=True)
        assert torch.allclose(x1.double(), ref, atol=1e-5, rtol=1e-5) and torch.equal(h, x1.bfloat16())
        x2, h2 = ops.post_norm_residual(x.clone(), a, wb, 1e-5, out_dtype=torch.float32, plain_rows=True)
        assert h2 is x2 and torch.equal(x2, x1)
        assert torch.equal(ops.cast_rows(x, torch.bfloat16), x.bfloat16()) and ops.cast_rows(x, torch.float32) is x
    gu = (torch.randn(7, 2 * 40, device=dev) * 3).bfloat16()
    g, u = gu[:, :40].float().clamp(max=1.5), gu[:, 40:].float().clamp(-1.5, 1.5)
    assert torch.allclose(ops.clamped_glu(gu, 1.5, 1.702).float(), (g * torch.sigmoid(1.702 * g) * (u + 1)), atol=2e-2, rtol=1e-2)
    gu32 = torch.randn(5, 2 * 33, device=dev) * 3
    g, u = gu32[:, :33].clamp(max=0.7), gu32[:, 33:].clamp(-0.7, 0.7)
    assert torch.allclose(ops.clamped_glu(gu32, 0.7, 1.702), g * torch.sigmoid(1.702 * g) * (u + 1), atol=1e-6, rtol=1e-5)
    v = torch.randn(3, 11, device=dev)
    assert torch.allclose(ops.scale_(v.clone(), 2.5), v * 2.5)


# ---------------------------------------------------------------------------------- one layer at a time

SINGLE_LAYERS = {
    "gru": gru_layer(40),
    "gru_with_ff": gru_layer(33, mlp=dense(50, 1.0)),
    "attention_group_of_3": attention_layer(6, 2, 32, 16, 0.2, 16, 100.0, window=20),
    "attention_whole_head_rotated_no_window": attention_layer(2, 2, 16, 16, 0.25, 16, 30.0),
    "attention_values_larger_than_keys": attention_layer(4, 1, 16, 48, 0.3, 8, 1000.0, window=33, mlp=dense(40, 2.0)),
    "attention_sizes_off_every_multiple": attention_layer(3, 1, 12, 6, 0.3, 6, 50.0, window=5),
    "attention_heads_of_128": attention_layer(4, 2, 128, 128, 0.09, 64, 500000.0, window=30),
    "attention_values_of_48": attention_layer(2, 1, 64, 48, 0.12, 32, 10000.0, window=25),
    "attention_with_ramp_on_queries_and_keys": attention_layer(4, 2, 32, 32, 0.2, 16, 500.0, window=40, scaling=RAMP),
    "latent_with_ramp": latent_layer(3, 24, 8, 40, 48, 0.2, 1000.0, window=30, scaling=RAMP),
    "latent_no_ramp_no_window": latent_layer(2, 16, 16, 16, 32, 0.25, 100.0),
    "latent_part_of_the_rotated_part_turned": latent_layer(4, 8, 8, 8, 24, 0.3, 20.0, window=12, rot_dims=4),
    "latent_odd_sizes": latent_layer(5, 12, 6, 10, 17, 0.3, 77.0, window=9),
    "latent_large": latent_layer(2, 128, 64, 128, 192, 0.07, 1000000.0, window=40,
                                 scaling={"factor": 4.0, "original": 512, "fast": 32.0, "slow": 1.0}),
    "latent_beyond_the_matrix_core_kernel": latent_layer(2, 32, 32, 32, 256, 0.1, 10000.0, window=21),
}


@pytest.mark.parametrize("name", sorted(SINGLE_LAYERS))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_layer_alone(tmp_path, name, dtype):
    """A model of one layer: the stream after it and the logits, for a whole prompt, for portions and token by token."""
    config = model(120, 64, [SINGLE_LAYERS[name]], scale=8.0)
    folder = make_folder(tmp_path / name, config, seed=21)
    tokens = random_tokens(53, config["vocab"], 5)
    cfg, w = load_plain(folder)
    streams: list = []
    logits = ps.forward(tokens, w, cfg, streams)
    runner = runner_for(folder, dtype, tokens=64)
    got = streams_of(runner, tokens)
    assert len(got) == 1 and got[0].dtype == torch.float32
    rel = (got[0].double() - streams[0]).norm(dim=-1) / streams[0].norm(dim=-1)
    assert float(rel.max()) < (5e-5 if dtype == "float32" else 6e-2), f"stream after the layer, row by row: {rel.tolist()}"
    plain = {"a": logits.float()}
    compare_rows(run_steps(runner, whole("a", tokens)), plain, TOL[dtype])
    compare_rows(run_steps(runner, portions("a", tokens, [2, 17, 1, 16, 3])), plain, TOL[dtype])
    compare_rows(run_steps(runner, tail_one_by_one("a", tokens, tail=30)), plain, TOL[dtype])


# ---------------------------------------------------------------------------------- cuttings, batches, reuse


@pytest.mark.parametrize("name", sorted(CONFIGS))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_every_cutting_gives_the_plain_rows(sakevik_folders, name, dtype):
    """Whole prompts, a tail decoded token by token (through recorded steps), portions of changing sizes
    down to two tokens and one, and unequal requests mixed in one batch on a pool so small that pages and
    slots are used again."""
    folder, vocab = sakevik_folders[name], CONFIGS[name]["vocab"]
    reqs = {f"r{i}": random_tokens(n, vocab, 50 + i) for i, n in enumerate((70, 3, 41, 1, 97, 26))}
    plain = plain_rows(folder, reqs)
    runner = runner_for(folder, dtype, tokens=256)
    tol = TOL[dtype]
    for rid, toks in reqs.items():
        compare_rows(run_steps(runner, whole(rid, toks)), plain, tol)
    compare_rows(run_steps(runner, tail_one_by_one("r4", reqs["r4"], tail=60)), plain, tol)
    compare_rows(run_steps(runner, portions("r4", reqs["r4"], [2, 3, 16, 2, 1, 31, 5])), plain, tol)
    compare_rows(run_steps(runner, portions("r0", reqs["r0"], [15, 17, 1, 2])), plain, tol)
    for seed in (1, 2):
        compare_rows(run_steps(runner, mixed_trace(reqs, seed, max_live=4)), plain, tol)
    assert runner.manager.requests == {}
    if dtype == "float32":
        a = run_steps(runner, whole("r2", reqs["r2"]))
        b = run_steps(runner, portions("r2", reqs["r2"], [2, 7]))
        assert max(float((a[k] - b[k]).abs().max()) for k in a) < 3e-4


def test_batch_rows_do_not_depend_on_their_neighbours(sakevik_folders):
    """A request alone and the same request between two others, as a prompt portion and as a single
    token: bit for bit the same logits in 32-bit."""
    folder, vocab = sakevik_folders["mixed"], MIXED["vocab"]
    a, b, c = (random_tokens(n, vocab, 90 + n) for n in (33, 50, 19))
    runner = runner_for(folder, "float32", tokens=256)
    alone = run_steps(runner, [{"entries": [("b", b[:40], list(range(40)))]}, {"entries": [("b", b[40:41], [0])], "end": ["b"]}])
    beside = run_steps(runner, [
        {"entries": [("a", a[:20], []), ("b", b[:40], list(range(40))), ("c", c[:5], [])]},
        {"entries": [("a", a[20:21], []), ("b", b[40:41], [0]), ("c", c[5:6], [])], "end": ["a", "b", "c"]}])
    for key in alone:
        assert torch.equal(alone[key], beside[key]), f"{key} differs beside other requests"


def test_slots_and_pages_are_clean_for_their_next_holder(sakevik_folders):
    """Two slots and a pool of eight pages a group serve six requests one after the other and in pairs: a
    request must not see the keys, the state or the last token of whoever held its pages and slot before."""
    for name in ("mixed", "only_gru"):
        folder, vocab = sakevik_folders[name], CONFIGS[name]["vocab"]
        reqs = {f"q{i}": random_tokens(n, vocab, 70 + i) for i, n in enumerate((60, 64, 17, 49, 30, 5))}
        plain = plain_rows(folder, reqs)
        runner = runner_for(folder, "float32", tokens=128, slots=2)
        for seed in (3, 4):
            compare_rows(run_steps(runner, mixed_trace(reqs, seed, max_live=2)), plain, TOL["float32"])


@pytest.mark.parametrize("kind", ["attention", "latent"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_keys_at_the_window_s_edge_at_page_borders_and_far_back(tmp_path, dtype, kind):
    """One key is made to stand out: its token appears once and its embedding is large, so its value (or, for
    the latent layer, its rotated key part, which eight heads meet with eight queries) is.  In a model of one layer the last token's logits then change
    if and only if that key is inside the window.  The engine must agree with the plain model with the key one
    token back, at both sides of a page's border, on the window's last place and on the first beyond it, in a
    whole prompt, decoded alone and in portions of two tokens."""
    W = 45
    layer = (attention_layer(2, 1, 16, 16, 0.5, 4, 20.0, window=W) if kind == "attention"
             else latent_layer(8, 8, 8, 16, 32, 0.5, 20.0, window=W))
    config = model(64, 32, [layer], scale=5.0, bigram=None)
    folder = make_folder(tmp_path / "marked", config, seed=8, edits={"embed": lambda t: torch.cat([t[:63], t[63:] * 8.0])})
    cfg, w = load_plain(folder)
    n = 200
    runner = runner_for(folder, dtype, tokens=256)
    for back in (1, 15, 16, 17, 31, 32, W - 2, W - 1, W, W + 1, 150):  # the marked key lies this far behind the last token
        tokens = [t % 63 for t in random_tokens(n, 64, 100 + back)]
        unmarked = ps.forward(tokens, w, cfg)[-1]
        tokens[n - 1 - back] = 63
        plain = ps.forward(tokens, w, cfg).float()
        changed = float((plain[-1] - unmarked).abs().max())
        assert (changed > 0.05) == (back < W), f"the mark {back} back moves the last row by {changed}"
        for steps in (whole("e", tokens), tail_one_by_one("e", tokens, tail=3), portions("e", tokens, [2, 61]),
                      tail_one_by_one("e", tokens, tail=W + 5)):
            got = run_steps(runner, steps)
            compare_rows({k: v for k, v in got.items() if k[1] >= n - 3}, {"e": plain}, TOL[dtype])


def test_a_token_far_back_shows_through_the_recurrence(tmp_path):
    """A gate that hardly opens keeps the state for hundreds of tokens: the first token's mark is still in the
    last row, in a whole prompt, token by token and across portions."""
    config = model(64, 32, [gru_layer(48)], scale=5.0, bigram=None)
    folder = make_folder(tmp_path / "slow", config, seed=3, edits={".z.b": lambda t: t * 0 - 5.0, ".z": lambda t: t * 0.05})
    cfg, w = load_plain(folder)
    n = 400
    tokens = [t % 63 for t in random_tokens(n, 64, 9)]
    unmarked = ps.forward(tokens, w, cfg)[-1]
    tokens[0] = 63
    plain = ps.forward(tokens, w, cfg).float()
    assert float((plain[-1] - unmarked).abs().max()) > 1e-3
    runner = runner_for(folder, "float32", tokens=448)
    for steps in (whole("e", tokens), tail_one_by_one("e", tokens, tail=350), portions("e", tokens, [2, 61, 1])):
        got = run_steps(runner, steps)
        compare_rows({k: v for k, v in got.items() if k[1] >= n - 3}, {"e": plain}, 1e-4)


def test_first_tokens_of_a_sequence(sakevik_folders):
    """Requests of one, two and three tokens, whole and token by token: the pairs' last row for the first
    token, the token before kept across steps, one key in the window, the first page half empty."""
    for name in sorted(CONFIGS):
        folder, vocab = sakevik_folders[name], CONFIGS[name]["vocab"]
        reqs = {f"s{n}": random_tokens(n, vocab, 30 + n) for n in (1, 2, 3, 6)}
        plain = plain_rows(folder, reqs)
        runner = runner_for(folder, "float32", tokens=64)
        for rid, toks in reqs.items():
            compare_rows(run_steps(runner, whole(rid, toks)), plain, TOL["float32"])
            compare_rows(run_steps(runner, portions(rid, toks, [1])), plain, TOL["float32"])


def test_the_token_before_shows_in_every_row(sakevik_folders):
    """The plain model itself: with another token in front a row changes although its own token is the
    same, so the cuttings above do tell a token before that is lost at the start of a portion."""
    folder = sakevik_folders["only_gru"]
    cfg, w = load_plain(folder)
    a = ps.embed([5, 7, 9], w, cfg)
    b = ps.embed([5, 8, 9], w, cfg)
    assert float((a[2] - b[2]).abs().max()) > 0.05 and torch.equal(a[0], b[0])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(sakevik_folders, dtype):
    """A short prompt and 400 tokens decoded one by one through recorded steps: every window passes over
    decoded tokens, pages are given back on the way."""
    folder, vocab = sakevik_folders["mixed"], MIXED["vocab"]
    tokens = random_tokens(420, vocab, 77)
    plain = plain_rows(folder, {"d": tokens})
    runner = runner_for(folder, dtype, tokens=448)
    got = run_steps(runner, tail_one_by_one("d", tokens, tail=400))
    compare_rows(got, plain, TOL[dtype])
    assert all(step.captured for step in runner.recorded.values()) and runner.recorded


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_requests_across_context_bounds(tmp_path, dtype):
    """Requests of up to 2 100 tokens: steps planned for 1 024, 2 048 and 4 096 tokens of context, windows shorter and
    longer than a chunk of keys and none, portions of hundreds of tokens after pasts of which a windowed cache has given
    most pages back, 500 tokens decoded one by one, and three requests of unequal length in one batch."""
    config = model(210, 96, [
        attention_layer(4, 2, 32, 32, 0.18, 16, 3000.0, window=180, mlp=dense(128, 2.0)),
        latent_layer(4, 32, 16, 32, 80, 0.14, 1e6, window=520, scaling={"factor": 4.0, "original": 256, "fast": 16.0, "slow": 1.0},
                     mlp=dense(128, 3.0)),
        gru_layer(160),
        latent_layer(2, 16, 8, 16, 40, 0.2, 1e4, mlp=dense(64, 2.0)),
        attention_layer(3, 3, 16, 64, 0.25, 16, 1e4, window=1300),
    ], scale=9.0, logit_scale=1.5, bigram=(211, 13, 5))
    folder = make_folder(tmp_path / "long", config, seed=3)
    n = 2100
    reqs = {"a": random_tokens(n, 210, 1), "b": random_tokens(600, 210, 2), "c": random_tokens(1200, 210, 3)}
    plain = plain_rows(folder, reqs)
    runner = runner_for(folder, dtype, tokens=4096)

    def some(got, every=9):
        return {k: v for i, (k, v) in enumerate(sorted(got.items())) if i % every == 0 or k[1] > n - 40}

    tol = TOL[dtype]
    compare_rows(some(run_steps(runner, whole("a", reqs["a"]))), plain, tol)
    compare_rows(some(run_steps(runner, portions("a", reqs["a"], [512, 3, 700, 64, 2, 600]))), plain, tol)
    compare_rows(some(run_steps(runner, tail_one_by_one("a", reqs["a"], tail=500))), plain, tol)
    a, b, c = reqs["a"], reqs["b"], reqs["c"]
    steps = [{"entries": [("a", a[:1000], [999]), ("b", b[:300], [0, 299])]},
             {"entries": [("a", a[1000:2000], [0, 999]), ("b", b[300:301], [0]), ("c", c[:1100], [1099])]},
             {"entries": [("a", a[2000:2001], [0]), ("b", b[301:600], [298]), ("c", c[1100:1101], [0])], "end": ["b"]},
             {"entries": [("a", a[2001:], [n - 2002]), ("c", c[1101:], [98])], "end": ["a", "c"]}]
    compare_rows(run_steps(runner, steps), plain, tol)
    assert runner.manager.requests == {}


@pytest.mark.parametrize("name", ["mixed", "awkward", "only_gru"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_engine(sakevik_folders, dtype, name):
    """``Engine.generate``: the scheduler cuts prompts into portions beside decoding requests; the tokens
    are the plain model's greedy tokens (in bfloat16: each token is, for the plain logits of its own
    history, within rounding of the best)."""
    from tokasaurus_amd.config.engine_config import EngineConfig
    from tokasaurus_amd.engine.engine import Engine
    from tokasaurus_amd.sampling import SamplingParams

    folder, vocab = sakevik_folders[name], CONFIGS[name]["vocab"]
    prompts = [random_tokens(n, vocab, 10 + n) for n in (5, 40, 23, 1, 64)]
    engine = Engine(EngineConfig(model=str(folder), dtype=dtype, page_size=PAGE, kv_cache_num_tokens=512, max_seqs_per_forward=3,
                                 max_tokens_per_forward=24, allocator_sanity_checks=True))
    done = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    cfg, w = load_plain(folder)
    for prompt, c in zip(prompts, done):
        assert len(c.tokens) == 12 and c.finish_reason == "length"
        ids = list(prompt)
        for tok in c.tokens:
            logits = ps.forward(ids, w, cfg)[-1]
            if dtype == "float32":
                assert tok == int(logits.argmax()), f"token {tok}, plain {int(logits.argmax())}"
            else:
                assert float(logits.max() - logits[tok]) < 0.05 * float(logits.std()) + 0.05
            ids.append(tok)
    assert engine.runner.manager.requests == {}


def test_command_line_and_trace_replay(sakevik_folders, tmp_path):
    """``bin/toka`` generates from a Sakevik folder, and ``bin/trace_run`` replays given tokens step by
    step: its logits are the plain model's."""
    import os
    import subprocess
    import sys

    import numpy as np

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder, vocab = sakevik_folders["only_attention"], CONFIGS["only_attention"]["vocab"]
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
            assert tok == int(ps.forward(ids, w, cfg)[-1].argmax())
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
        kind = rng.choice(["attention", "latent", "gru"])
        mlp = rng.choice([None, dense(rng.choice([24, 33, 64, 100]), rng.choice([0.5, 2.0, 7.0]))])
        window = rng.choice([None, 1, 2, 15, 16, 17, 40, 64, 100])
        if kind == "gru":
            layers.append(gru_layer(rng.choice([8, 31, 64, 100]), mlp=mlp))
        elif kind == "attention":
            kv = rng.choice([1, 2, 3])
            dim = rng.choice([8, 12, 16, 32, 40, 64])
            layers.append(attention_layer(kv * rng.choice([1, 2, 4, 5]), kv, dim, rng.choice([2, 8, 16, 20, 32, 48]),
                                          rng.choice([0.1, 0.3]), rng.choice([d for d in (2, 4, 8, 12, 16, 32, 64) if d <= dim]),
                                          rng.choice([10.0, 1e4, 1e6]), window=window, mlp=mlp))
        else:
            rot_dim = rng.choice([2, 4, 8, 16, 32])
            scaling = rng.choice([None, {"factor": rng.choice([2.0, 16.0]), "original": rng.choice([8, 64, 1024]),
                                         "fast": rng.choice([4.0, 32.0]), "slow": rng.choice([0.5, 1.0])}])
            layers.append(latent_layer(rng.choice([1, 2, 3, 8]), rng.choice([8, 12, 16, 32]), rot_dim, rng.choice([4, 8, 16, 24]),
                                       rng.choice([8, 17, 32, 64, 96]), rng.choice([0.1, 0.3]), rng.choice([10.0, 1e4, 1e6]),
                                       window=window, scaling=scaling, rot_dims=rng.choice([rot_dim, 2]), mlp=mlp))
    bigram = rng.choice([None, (rng.choice([1, 2, 61, 499]), rng.choice([1, 29, 12345]), rng.choice([1, 11, 999]))])
    return model(rng.choice([40, 97, 130]), width, layers, eps=rng.choice([1e-6, 1e-5]), scale=rng.choice([1.0, 6.0]),
                 bigram=bigram, logit_scale=rng.choice([None, 0.25, 3.0]))


@pytest.mark.parametrize("seed", range(12))
def test_random_configurations(tmp_path, seed):
    config = random_config(seed)
    folder = make_folder(tmp_path / "drawn", config, seed=seed)
    vocab = config["vocab"]
    reqs = {f"r{i}": random_tokens(n, vocab, 20 * seed + i) for i, n in enumerate((90, 2, 37, 130))}
    plain = plain_rows(folder, reqs)
    for dtype in ("float32", "bfloat16"):
        runner = runner_for(folder, dtype, tokens=320)
        for rid, toks in reqs.items():
            compare_rows(run_steps(runner, whole(rid, toks)), plain, TOL[dtype])
        compare_rows(run_steps(runner, tail_one_by_one("r3", reqs["r3"], tail=70)), plain, TOL[dtype])
        compare_rows(run_steps(runner, portions("r3", reqs["r3"], [2, 3, 16, 2, 1, 31, 5])), plain, TOL[dtype])
        compare_rows(run_steps(runner, mixed_trace(reqs, seed, max_live=3)), plain, TOL[dtype])
        assert runner.manager.requests == {}
