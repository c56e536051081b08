"""Grouped-query attention over the paged cache with the pieces that ``paged_attention`` does
not have, each a parameter: key and value heads of different sizes, a scale of the model's
choosing, RMS norms of the queries and of the keys over the whole projection (all heads at
once), a rotation of neighbouring elements of the leading part of a head, a sliding window, a
learned sink per query head in the softmax's denominator (or one constant score for all heads),
keys and values taken from another layer's cache (the run entry's ``cache_of``; the mixer then
has no key and value tensors), a rotation that pairs the two halves of a head's leading part
instead of neighbours, and values that are the keys themselves as projected, before the rotation
(the mixer then has no value tensor); biases on the projections; norms of queries and keys head by
head with one weight for all heads; weights that are sigmoids of the biased scores instead of a
softmax; values turned by their own position and the heads' results turned back by the query's; a
sigmoid gate per head that reads the mixer's input; a soft cap on the scaled scores; a learned bias on the
scores by (bucket of the distance, head); a sigmoid gate per element of the heads' results.

Scores, softmax weights, norms, angles and the rotation are 32-bit arithmetic in either storage
type.  One kernel norms, rotates and appends (``ops.qk_prepare``); the attention itself runs on
the matrix cores' 32-bit products (``ops.attention_tile_f32``: tiles of 16 tokens for prompt
portions, of the heads that share a kv head for single tokens) or, for sizes that kernel does
not take, on the plain 32-bit kernel (``ops.paged_attention_generic``).
"""

from __future__ import annotations

import torch

from tokasaurus_amd.kernels import ops
from tokasaurus_amd.kernels.upload import upload
from tokasaurus_amd.parts.base import (
    MIXERS,
    NORM_WEIGHT,
    POSITION_ENCODINGS,
    VECTOR,
    CacheNeed,
    CacheView,
    Mixer,
    PartSpec,
    StepContext,
    TensorSpec,
)
from tokasaurus_amd.parts.linear import Linear, Placer
from tokasaurus_amd.parts.position import InterleavedRotary


def tile_plan(ctx: StepContext, tokens_a_tile: int) -> tuple[torch.Tensor, torch.Tensor]:
    """The step's rows cut into tiles of up to ``tokens_a_tile`` neighbouring tokens of one
    request: for every tile its request and its first row.  Made once a step and shared by
    the layers; a step that is recorded keeps it for its replays."""
    key = ("tile_plan", tokens_a_tile)
    plan = ctx.extras.get(key)
    if plan is None:
        req, row0 = [], []
        for r in range(ctx.num_requests):
            a, b = ctx.host_q_start[r], ctx.host_q_start[r + 1]
            for first in range(a, b, tokens_a_tile):
                req.append(r)
                row0.append(first)
        dev = upload(req + row0, torch.int32, ctx.device)
        plan = ctx.extras[key] = (dev[: len(req)], dev[len(req):])
    return plan


@MIXERS.register("grouped_attention")
class GroupedAttention(Mixer):
    def __init__(
        self,
        hidden_size: int,
        num_heads: int,
        num_kv_heads: int,
        key_dim: int,
        value_dim: int,
        scale: float,
        names: dict[str, str],
        position: PartSpec | None = None,
        window: int = 0,
        cache_window: int | None = None,
        projection_norm: dict | None = None,
        sink_name: str | None = None,
        own_kv: bool = True,
        shared: dict | None = None,
        sink_value: float | None = None,
        values_are_keys: bool = False,
        key_chunk: int = 0,
        bias_names: dict[str, str] | None = None,
        head_norm: dict | None = None,
        score_bias_name: str | None = None,
        value_rotation: dict | None = None,
        gate_name: str | None = None,
        softcap: float | None = None,
        distance_bias: dict | None = None,
        element_gate_name: str | None = None,
    ):
        """``names``: checkpoint names of the q, k, v, o matrices (k and v only with ``own_kv``).
        ``projection_norm``: ``{"q": name, "k": name, "eps": eps}``, weights of the whole
        projections' sizes (k only with ``own_kv``).  ``window``: a query sees itself and the
        window - 1 positions before it (0: all).  ``cache_window``: how far back the cache keeps
        keys (0: all): at least ``window``, more when another layer reads this cache further
        back; by default ``window``.  ``sink_name``: one number a query head.  ``sink_value``: no
        tensor, every head's sink has this score (0: one is added to the softmax's denominator).
        ``values_are_keys``: ``names`` has no v; a token's values are its keys before the rotation.
        ``key_chunk``: in steps of few tokens a request's keys are cut at multiples of this many among
        workgroups (0: never).  ``bias_names``: checkpoint names of biases under any of q, k, v, o.
        ``head_norm``: ``{"q": name, "k": name, "eps": eps}``, RMS norms head by head with weights of one
        head's size (instead of ``projection_norm``).  ``score_bias_name``: one number a query head; the
        weight of a visible key is sigmoid(score + bias), not normalised over the keys (no softmax, no sink).
        ``value_rotation``: ``{"base": b, "pair_halves": bool}``; the value at position j is cached turned,
        pair m by j * b^(-2m/value_dim), and a head's result at position i is turned back by i.
        ``gate_name``: a matrix [heads, hidden]; head h's result is multiplied by sigmoid(gate h)_h.
        ``softcap``: a scaled score s becomes softcap * tanh(s / softcap).  ``distance_bias``: ``{"name": n, "buckets":
        B, "far": D}``, a table [B, heads] of which row bucket(i - j) is added to the score of query i and key j (after
        the scale and the soft cap): distances below B / 2 have a bucket each, the others share the rest on a
        logarithmic scale that reaches the last bucket at D.  ``element_gate_name``: a matrix [heads * value_dim,
        hidden]; the heads' results are multiplied element by element by sigmoid(gate h)."""
        self.softcap = float(softcap) if softcap else 0.0
        self.distance_bias = dict(distance_bias) if distance_bias else None
        self.element_gate_name = element_gate_name
        if score_bias_name and (self.softcap or self.distance_bias):
            raise ValueError("sigmoid weights take neither a soft cap nor a bias by distance")
        if element_gate_name and gate_name:
            raise ValueError("a gate per head or a gate per element, not both")
        self.rel: "ops.DistanceBias | None" = None
        self.key_chunk = int(key_chunk)
        bias_names = dict(bias_names or {})
        self.head_norm = dict(head_norm) if head_norm else None
        if self.head_norm and projection_norm:
            raise ValueError("queries and keys are normed over the whole projection or head by head, not both")
        self.score_bias_name = score_bias_name
        if score_bias_name and (sink_name or sink_value is not None):
            raise ValueError("sigmoid weights have no denominator for a sink to join")
        self.value_rotation = dict(value_rotation) if value_rotation else None
        if self.value_rotation and (values_are_keys or not own_kv or int(value_dim) % 2):
            raise ValueError("turned values come with a value projection of the mixer's own and an even value size")
        self.gate_name = gate_name
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are not a multiple of {num_kv_heads} kv heads")
        self.hidden_size, self.num_heads, self.num_kv_heads = hidden_size, num_heads, num_kv_heads
        self.key_dim, self.value_dim = int(key_dim), int(value_dim)
        self.scale = float(scale)
        self.window = int(window)
        self.cache_window = self.window if cache_window is None else int(cache_window)
        if self.cache_window and (not self.window or self.window > self.cache_window):
            raise ValueError(f"a window of {self.window or 'all'} keys reads further back than the {self.cache_window} the cache keeps")
        self.own_kv = bool(own_kv)
        self.projection_norm = dict(projection_norm) if projection_norm else None
        self.sink_name = sink_name
        self.sink_value = None if sink_value is None else float(sink_value)
        if sink_name and sink_value is not None:
            raise ValueError("a sink is learned (sink_name) or constant (sink_value), not both")
        self.values_are_keys = bool(values_are_keys)
        if self.values_are_keys and (self.value_dim != self.key_dim or not own_kv):
            raise ValueError("values that are the keys have the keys' size and come with keys of the mixer's own")
        kv_sizes = [num_kv_heads * key_dim] + ([] if self.values_are_keys else [num_kv_heads * value_dim])
        kv_names = [names["k"]] + ([] if self.values_are_keys else [names["v"]])
        sizes = [num_heads * key_dim] + (kv_sizes if own_kv else [])
        stacked = [names["q"]] + (kv_names if own_kv else [])
        biases = [bias_names.get("q")] + ([bias_names.get("k")] + ([] if self.values_are_keys else [bias_names.get("v")]) if own_kv else [])
        if gate_name:  # the gate reads the same input: one more part of the stacked product
            stacked, sizes, biases = stacked + [gate_name], sizes + [num_heads], biases + [None]
        if element_gate_name:
            stacked, sizes, biases = stacked + [element_gate_name], sizes + [num_heads * value_dim], biases + [None]
        self.element_gate_col = sum(sizes) - num_heads * value_dim if element_gate_name else None
        self.gate_col = sum(sizes) - num_heads if gate_name else None
        self.qkv = Linear(hidden_size, stacked, sizes, bias_names=biases)
        self.out = Linear(num_heads * value_dim, [names["o"]], [hidden_size], bias_names=[bias_names.get("o")])
        self.score_bias: torch.Tensor | None = None
        self.value_freq: torch.Tensor | None = None
        self.q_norm_weight: torch.Tensor | None = None
        self.k_norm_weight: torch.Tensor | None = None
        self.sink: torch.Tensor | None = None
        self.position = None
        if position is not None:
            shared = shared if shared is not None else {}
            self.position = shared.setdefault(("position", position), POSITION_ENCODINGS.build(position))
            if not isinstance(self.position, InterleavedRotary) or self.position.dims > key_dim:
                raise ValueError("grouped_attention rotates neighbouring elements: it takes a rotary_interleaved encoding "
                                 "of at most a key head's size")

    def tensor_specs(self) -> list[TensorSpec]:
        specs = self.qkv.tensor_specs() + self.out.tensor_specs()
        if self.projection_norm:
            specs.append(TensorSpec(self.projection_norm["q"], (self.num_heads * self.key_dim,), NORM_WEIGHT))
            if self.own_kv:
                specs.append(TensorSpec(self.projection_norm["k"], (self.num_kv_heads * self.key_dim,), NORM_WEIGHT))
        if self.head_norm:
            specs.append(TensorSpec(self.head_norm["q"], (self.key_dim,), NORM_WEIGHT))
            if self.own_kv:
                specs.append(TensorSpec(self.head_norm["k"], (self.key_dim,), NORM_WEIGHT))
        if self.sink_name:
            specs.append(TensorSpec(self.sink_name, (self.num_heads,), VECTOR))
        if self.score_bias_name:
            specs.append(TensorSpec(self.score_bias_name, (self.num_heads,), VECTOR))
        if self.distance_bias:
            specs.append(TensorSpec(self.distance_bias["name"], (int(self.distance_bias["buckets"]), self.num_heads), VECTOR))
        return specs

    @property
    def inner_size(self) -> int:
        return self.num_heads * self.value_dim

    def cache_need(self) -> CacheNeed:
        return CacheNeed(self.num_kv_heads, self.key_dim, self.cache_window,
                         0 if self.value_dim == self.key_dim else self.value_dim)

    def check_cache(self, page_size: int, dtype: torch.dtype) -> None:
        ops.check_attention_shape(dtype, self.num_heads, self.num_kv_heads, self.key_dim, page_size,
                                  value_dim=self.value_dim, generic_only=True)

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        self.qkv.load(tensors, placer)
        self.out.load(tensors, placer)

        def f32(name: str) -> torch.Tensor:
            return placer.place(("vector_f32", name), lambda: tensors[name].to(torch.float32).contiguous().to(placer.device))

        if self.projection_norm:
            self.q_norm_weight = f32(self.projection_norm["q"])
            if self.own_kv:
                self.k_norm_weight = f32(self.projection_norm["k"])
        if self.head_norm:
            self.q_norm_weight = f32(self.head_norm["q"])
            if self.own_kv:
                self.k_norm_weight = f32(self.head_norm["k"])
        if self.score_bias_name:
            self.score_bias = f32(self.score_bias_name)
        if self.distance_bias:
            buckets, far = int(self.distance_bias["buckets"]), int(self.distance_bias["far"])
            table = placer.place(("distance_buckets", buckets, far), lambda: torch.tensor(
                ops.distance_buckets(buckets, far), dtype=torch.int32).to(placer.device))
            self.rel = ops.DistanceBias(f32(self.distance_bias["name"]), table)
        if self.value_rotation:
            dv, base = self.value_dim, float(self.value_rotation["base"])
            self.value_freq = placer.place(("value_freq", dv, base), lambda: torch.tensor(
                [base ** (-2.0 * m / dv) for m in range(dv // 2)], dtype=torch.float64).to(torch.float32).to(placer.device))
        if self.sink_name:
            self.sink = f32(self.sink_name)
        elif self.sink_value is not None:
            self.sink = placer.place(("constant_f32", self.sink_value, self.num_heads), lambda: torch.full(
                (self.num_heads,), self.sink_value, dtype=torch.float32, device=placer.device))
        if self.position is not None:
            self.position.prepare(placer.device)

    def _attend(self, h: torch.Tensor, ctx: StepContext, cache: CacheView, rows: torch.Tensor | None,
                out: torch.Tensor | None = None, out_scale: float = 1.0) -> torch.Tensor:
        assert cache is not None, "grouped attention needs a cache"
        if cache.writable != self.own_kv:
            raise RuntimeError("a mixer with key and value tensors of its own writes its cache; one without reads another's")
        nq, nkv, dk, dv = self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim
        qkv = self.qkv(h)
        normed = self.projection_norm or self.head_norm
        eps = float(normed["eps"]) if normed else 0.0
        v_halves = bool(self.value_rotation and self.value_rotation.get("pair_halves"))
        ops.qk_prepare(qkv, ctx.positions, ctx.token_req, cache.block_table, self.q_norm_weight,
                       self.k_norm_weight if self.own_kv else None, eps,
                       self.position.freq if self.position is not None else None,
                       cache.keys, cache.values, nq, nkv, dk, dv, cache.page_size, write_cache=self.own_kv,
                       pair_halves=self.position is not None and self.position.pair_halves,
                       values_are_keys=self.values_are_keys, per_head=self.head_norm is not None,
                       value_freq=self.value_freq, value_pair_halves=v_halves,
                       rotation_scale=self.position.magnitude if self.position is not None else 1.0)
        gate = qkv[:, self.gate_col : self.gate_col + nq] if self.gate_col is not None else None
        after = self.value_freq is not None or gate is not None
        if ops.attention_tile_f32_fits(nq, nkv, dk, dv, cache.page_size):
            # the kernel turns the heads' results back and gates them itself where the pairs lie inside its lanes
            fused = after and (self.value_freq is None or not v_halves or ops.attention_tile_turns_halves(dv))
            gg = ops.attention_tile_heads(nq // nkv, ctx.max_q_len)
            tile_req, tile_row0 = tile_plan(ctx, 16 // gg)
            attn = ops.attention_tile_f32(qkv, cache.keys, cache.values, cache.block_table, ctx.q_start, ctx.kv_len,
                                          tile_req, tile_row0, nq, nkv, dk, dv, cache.page_size, gg,
                                          window=self.window, scale=self.scale, sink=self.sink, key_chunk=self.key_chunk,
                                          longest=ctx.extras.get("kv_bound", ctx.max_kv_len), score_bias=self.score_bias,
                                          value_freq=self.value_freq if fused else None, value_pair_halves=v_halves,
                                          gate=gate if fused else None, softcap=self.softcap, distance_bias=self.rel)
            after = after and not fused
        else:  # sizes that the matrix-core kernel does not take
            attn = ops.paged_attention_generic(qkv, cache.keys, cache.values, cache.block_table, ctx.token_req, ctx.positions,
                                               nq, nkv, dk, cache.page_size, window=self.window, scale=self.scale,
                                               value_dim=dv, sink=self.sink, score_bias=self.score_bias, softcap=self.softcap,
                                               distance_bias=self.rel)
        if after:
            # the heads' results turned back by their own positions, then each head's gate
            ops.unrotate_gate_(attn, ctx.positions, self.value_freq, v_halves, gate, nq, dv)
        if self.element_gate_col is not None:
            attn = ops.sigmoid_gate(attn, qkv[:, self.element_gate_col : self.element_gate_col + nq * dv], scale=out_scale, out=out)
        elif out is not None or out_scale != 1.0:
            raise NotImplementedError("grouped attention gives its rows with a factor, or into a view, through its gate per element only")
        return attn if rows is None else ops.gather_rows(attn, rows)

    def inner_rows(self, h, ctx, cache, state, out=None, scale: float = 1.0):
        """The heads' results in front of the output projection times ``scale``, into ``out`` (a view) when given."""
        return self._attend(h, ctx, cache, None, out=out, out_scale=scale)

    def mix(self, h, ctx, cache, state, rows, out_f32: bool = False):
        return self.out(self._attend(h, ctx, cache, rows), out_f32=out_f32)

    def forward(self, h, residual, ctx, cache, state, rows):
        return self.out(self._attend(h, ctx, cache, rows), residual=residual)
