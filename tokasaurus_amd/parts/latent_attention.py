"""Attention whose keys and values are expanded, head by head, from one small latent a token, and
only that latent is cached.

Per token: the query latent ``cq = norm(W_dq h)`` and the key/value latent ``c = norm(W_dkv h)``
(RMS norms with weights, 32-bit); ``q = W_uq cq``; per head ``k = W_uk c`` and ``v = W_uv c``;
``score = (q . k) * scale`` over every earlier token and the token itself, an ordinary softmax,
no positions; the output projection reads the heads side by side.

Two forms of the same sums, chosen request by request in every step:

* **Single tokens** never expand a cached token's keys or values.  Since ``q_h . (W_uk,h c) =
  (W_uk,h^T q_h) . c`` and ``sum_j p_j W_uv,h c_j = W_uv,h sum_j p_j c_j``, a head's query is taken
  into the latent's space (a matrix a head, ``ops.head_linear``), the attention runs with ONE
  key/value head whose keys and values are both the latent (every query head reads it: the
  arithmetic intensity of the cache is that of ``num_heads`` queries a key), and the head's
  result is taken from the latent's space to its values by ``W_uv,h``.
* **Portions of prompts** expand: in the latent's space a score costs ``kv_rank`` multiply-adds
  a head instead of ``key_dim``, which for many queries outweighs expanding every key once.  The
  latents of the portion's requests are read back from the pages (``ops.gather_keys``), one
  product gives all heads' keys and values, and they go into pages of the step's own (a block
  table that counts up) over which the ordinary attention runs.  Nothing of it is kept.

The pages hold the latent twice, once in the key layout and once in the value layout,
``2 * kv_rank`` numbers a token and layer where expanded keys and values would take
``num_heads * (key_dim + value_dim)``.

**A rotated part beside the latent** (``rot_dim`` > 0).  A query head is then ``[key_dim unrotated |
rot_dim rotated]`` in the checkpoint, and ``W_dkv h`` has ``kv_rank + rot_dim`` rows: the first are the
latent (normed), the last ONE rotated key part that all heads share (not normed); the score is the sum of
both parts' products, times ``scale``.  Here the rotated part leads: the weights' rows are permuted once
when they are placed, so that a query head is ``[rot_dim | key_dim]`` and a cached key ``[rot_dim | kv_rank]``,
the value being the key's ``kv_rank`` elements behind the rotated part.  In the latent's space a head's
query is ``[q_rot | W_uk,h^T q]`` (the matrix a head has an identity block), and the expansion of a cached
key is ``[k_rot | W_uk,h c]`` (an identity block again, exact in either storage type).  With ``q_rank`` 0
there is no query latent: ``q = W_q h``.  ``window``: a query sees itself and the window - 1 positions
before it; a portion then reads back and expands only the keys its queries see.

Scores, softmax weights and norms are 32-bit arithmetic in either storage type; the kernels are
those of ``grouped_attention`` (``ops.qk_prepare`` norms both latents and appends,
``ops.attention_tile_f32`` or, for sizes it does not take, ``ops.paged_attention_generic``).
"""

from __future__ import annotations

import numpy as np
import torch

from tokasaurus_amd.kernels import ops
from tokasaurus_amd.kernels.upload import upload
from tokasaurus_amd.parts.base import MATRIX, MIXERS, NORM_WEIGHT, POSITION_ENCODINGS, CacheNeed, CacheView, Mixer, PartSpec, StepContext, TensorSpec
from tokasaurus_amd.parts.grouped_attention import tile_plan
from tokasaurus_amd.parts.linear import Linear, Placer
from tokasaurus_amd.parts.position import InterleavedRotary


@MIXERS.register("latent_attention")
class LatentAttention(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, key_dim: int, value_dim: int, q_rank: int, kv_rank: int, scale: float,
                 norm_eps: float, names: dict[str, str], key_chunk: int = 256, rot_dim: int = 0, position: PartSpec | None = None,
                 window: int = 0, shared: dict | None = None):
        """``names``: checkpoint names under the keys dq, dkv ([rank, hidden]), dq_norm, dkv_norm
        ([rank]), uq ([heads * key_dim, q_rank]), uk ([heads * key_dim, kv_rank]), uv
        ([heads * value_dim, kv_rank]), o ([hidden, heads * value_dim]).  ``key_chunk``: in steps of
        few tokens a request's keys are cut at multiples of this many among workgroups (0: never).
        ``q_rank`` 0: no query latent; ``names`` has q ([heads * (key_dim + rot_dim), hidden]) instead of
        dq, dq_norm, uq.  ``rot_dim`` (with ``q_rank`` 0): the rotated part of a head and of dkv's rows
        (``kv_rank + rot_dim`` of them), turned by ``position`` (a rotation of pairs over at most rot_dim
        elements).  ``window``: 0 for every earlier key."""
        self.key_chunk = int(key_chunk)
        self.rot_dim, self.window = int(rot_dim), int(window)
        if self.rot_dim % 2 or self.rot_dim < 0:
            raise ValueError("the rotated part of a head has an even size")
        if q_rank and self.rot_dim:
            raise ValueError("a rotated part comes with queries projected directly (q_rank 0)")
        self.position = None
        if position is not None:
            shared = shared if shared is not None else {}
            self.position = shared.setdefault(("position", position), POSITION_ENCODINGS.build(position))
            if not isinstance(self.position, InterleavedRotary) or self.position.dims > self.rot_dim:
                raise ValueError("latent_attention turns pairs of its rotated part: a rotation of pairs over at most rot_dim elements")
        self.heads_a_call = num_heads  # query heads one call of the plain attention kernel takes (set when the cache is checked)
        self.hidden_size, self.num_heads = hidden_size, num_heads
        self.key_dim, self.value_dim, self.q_rank, self.kv_rank = int(key_dim), int(value_dim), int(q_rank), int(kv_rank)
        self.scale, self.norm_eps = float(scale), float(norm_eps)
        self.names = dict(names)
        dr = self.rot_dim
        self.query_dim, self.cached_dim = dr + self.key_dim, dr + self.kv_rank  # a head's query, a cached key
        if self.q_rank:
            self.down = Linear(hidden_size, [names["dq"], names["dkv"]], [self.q_rank, self.kv_rank])
            self.up_q = Linear(self.q_rank, [names["uq"]], [num_heads * self.key_dim])
        else:  # [q | k_rot | c] in one product, the rotated parts leading (rows permuted when placed)
            self.down = Linear(hidden_size, [names["q"], names["dkv"]], [num_heads * self.query_dim, self.cached_dim])
            self.up_q = None
        self.out = Linear(num_heads * self.value_dim, [names["o"]], [hidden_size])
        # all heads' keys and values of a cached key in one product (prompt portions)
        self.expand = Linear(self.kv_rank, [names["uk"], names["uv"]], [num_heads * self.key_dim, num_heads * self.value_dim])
        # with a rotated part the expansion reads the whole cached key: [heads * query_dim + heads * value_dim, cached_dim],
        # put together from uk, uv and identity blocks when the weights are placed
        self.expand_cached = (Linear(self.cached_dim, [f"{names['uk']}+{names['uv']}"], [num_heads * (self.query_dim + self.value_dim)])
                              if dr else None)
        self.q_norm_weight = self.c_norm_weight = None
        self.to_latent: torch.Tensor | None = None  # [heads, kv_rank, key_dim]: W_uk,h transposed
        self.from_latent: torch.Tensor | None = None  # [heads, value_dim, kv_rank]: W_uv,h

    def tensor_specs(self) -> list[TensorSpec]:
        n, H = self.names, self.num_heads
        specs = self.down.tensor_specs() + self.out.tensor_specs() + self.expand.tensor_specs() + [
            TensorSpec(n["dkv_norm"], (self.kv_rank,), NORM_WEIGHT)]
        if self.q_rank:
            specs += self.up_q.tensor_specs() + [TensorSpec(n["dq_norm"], (self.q_rank,), NORM_WEIGHT)]
        return specs

    def cache_need(self) -> CacheNeed:
        return CacheNeed(1, self.cached_dim, self.window, self.kv_rank if self.rot_dim else 0)

    def check_cache(self, page_size: int, dtype: torch.dtype) -> None:
        dc = self.cached_dim
        if ops.attention_tile_f32_fits(self.num_heads, 1, dc, self.kv_rank, page_size):
            ops.key_pages_shape(1, 1, page_size, dc, padded=True)
            ops.value_pages_shape(1, 1, page_size, self.kv_rank)
        else:
            # the plain kernel bounds the heads that share a kv head (their number times the latent's size):
            # more heads than it takes at once go in several calls
            ops.key_pages_shape(1, 1, page_size, dc, padded=True)
            ops.value_pages_shape(1, 1, page_size, self.kv_rank)
            m = self.num_heads
            while m > 1 and not ops.paged_attention_generic_fits(m, 1, dc, self.kv_rank):
                m = (m + 1) // 2
            ops.check_attention_shape(dtype, m, 1, dc, page_size, value_dim=self.kv_rank, generic_only=True)
            self.heads_a_call = m

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        n, H = self.names, self.num_heads
        d, dr, r, dv = self.key_dim, self.rot_dim, self.kv_rank, self.value_dim
        self.out.load(tensors, placer)

        def f32(name: str) -> torch.Tensor:
            return placer.place(("vector_f32", name), lambda: tensors[name].to(torch.float32).contiguous().to(placer.device))

        self.c_norm_weight = f32(n["dkv_norm"])
        if self.position is not None:
            self.position.prepare(placer.device)
        if self.q_rank:
            for lin in (self.down, self.up_q, self.expand):
                lin.load(tensors, placer)
            self.q_norm_weight = f32(n["dq_norm"])
        else:
            def rotated_first() -> torch.Tensor:
                wq = tensors[n["q"]].to(placer.dtype).view(H, d + dr, -1)
                wq = torch.cat([wq[:, d:], wq[:, :d]], dim=1).reshape(H * (d + dr), -1)
                wkv = tensors[n["dkv"]].to(placer.dtype)
                return torch.cat([wq, wkv[r:], wkv[:r]], dim=0).contiguous().to(placer.device)

            self.down.weight = placer.place(("rotated_first", n["q"], n["dkv"]), rotated_first)
            if not dr:
                self.expand.load(tensors, placer)
            else:
                def expansion() -> torch.Tensor:
                    where = tensors[n["uk"]].device
                    w = torch.zeros((H * (dr + d) + H * dv, dr + r), dtype=placer.dtype, device=where)
                    keys = w[: H * (dr + d)].view(H, dr + d, dr + r)
                    keys[:, :dr, :dr] = torch.eye(dr, dtype=placer.dtype, device=where)
                    keys[:, dr:, dr:] = tensors[n["uk"]].to(placer.dtype).view(H, d, r)
                    w[H * (dr + d) :, dr:] = tensors[n["uv"]].to(placer.dtype)
                    return w.contiguous().to(placer.device)

                self.expand_cached.weight = placer.place(("expansion_with_rotated_part", n["uk"], n["uv"]), expansion)

        def to_latent() -> torch.Tensor:
            where = tensors[n["uk"]].device
            w = torch.zeros((H, dr + r, dr + d), dtype=placer.dtype, device=where)
            w[:, :dr, :dr] = torch.eye(dr, dtype=placer.dtype, device=where)
            w[:, dr:, dr:] = tensors[n["uk"]].to(placer.dtype).view(H, d, r).transpose(1, 2)
            return w.contiguous().to(placer.device)

        self.to_latent = placer.place(("heads_transposed", dr, n["uk"]), to_latent)
        self.from_latent = placer.place(("heads", n["uv"]), lambda: tensors[n["uv"]].to(placer.dtype).view(
            H, self.value_dim, self.kv_rank).contiguous().to(placer.device))

    def _attend(self, h: torch.Tensor, ctx: StepContext, cache: CacheView, rows: torch.Tensor | None) -> torch.Tensor:
        assert cache is not None and cache.writable, "latent attention keeps its latent in a cache of its own"
        H, r = self.num_heads, self.kv_rank
        if self.q_rank:
            lat = self.down(h)  # [cq | c]
            # both latents normed (each over its whole length), the key/value latent appended as key and as value
            ops.qk_prepare(lat, ctx.positions, ctx.token_req, cache.block_table, self.q_norm_weight, self.c_norm_weight,
                           self.norm_eps, None, cache.keys, cache.values, 1, 1, r, r, cache.page_size,
                           query_dim=self.q_rank, values_are_keys=True)
            cq = lat[:, : self.q_rank]
            if lat.dtype != torch.float32 and (self.q_rank % 8 or lat.stride(0) % 8):
                cq = torch.empty((lat.shape[0], self.q_rank), dtype=lat.dtype, device=lat.device).copy_(cq)
            q = self.up_q(cq)  # [tokens, heads * key_dim]
        else:
            # [q | k_rot | c]: the latent normed, the rotated parts of every query head and of the key turned, the key
            # [k_rot | c] appended and its latent part as the value
            q = self.down(h)
            pos = self.position
            ops.qk_prepare(q, ctx.positions, ctx.token_req, cache.block_table, None, self.c_norm_weight, self.norm_eps,
                           pos.freq if pos is not None else None, cache.keys, cache.values, H, 1, self.cached_dim, r,
                           cache.page_size, query_dim=self.query_dim, values_are_keys=True, key_skip=self.rot_dim,
                           rotation_scale=pos.magnitude if pos is not None else 1.0)
        # the requests that bring portions come first in a step; their tokens are the step's first rows
        portions = int(ctx.extras.get("num_portions", 0))
        first_single = ctx.host_q_start[portions] if portions else 0
        if portions and ops.attention_tile_f32_fits(H, H, self.query_dim, self.value_dim, cache.page_size):
            o = self._over_expanded(q, ctx, cache, portions)
            if first_single < ctx.num_tokens:
                o[first_single:] = self._over_latent(q[first_single:], ctx, cache, first_single, ctx.num_requests - portions)
        else:
            o = self._over_latent(q, ctx, cache, 0, None)
        return o if rows is None else ops.gather_rows(o, rows)

    def _over_latent(self, q: torch.Tensor, ctx: StepContext, cache: CacheView, first_row: int, last_requests: int | None) -> torch.Tensor:
        """Attention in the latent's space for the step's rows from ``first_row`` on (``q`` holds those
        rows), which belong to the step's last ``last_requests`` requests, one token each (None: all
        rows of all requests)."""
        H, r, dc = self.num_heads, self.kv_rank, self.cached_dim
        ql = ops.head_linear(q, self.to_latent)  # [rows, heads * cached_dim]
        if ops.attention_tile_f32_fits(H, 1, dc, r, cache.page_size):
            gg = ops.attention_tile_heads(H, ctx.max_q_len if last_requests is None else 1)
            tile_req, tile_row0 = tile_plan(ctx, 16 // gg)
            if last_requests is not None:  # a request of one token is one tile, whatever a tile holds
                tile_req, tile_row0 = tile_req[tile_req.numel() - last_requests:], tile_row0[tile_row0.numel() - last_requests:]
            o = ops.attention_tile_f32(ql, cache.keys, cache.values, cache.block_table, ctx.q_start, ctx.kv_len,
                                       tile_req, tile_row0, H, 1, dc, r, cache.page_size, gg, scale=self.scale, window=self.window,
                                       key_chunk=self.key_chunk, longest=ctx.extras.get("kv_bound", ctx.max_kv_len),
                                       first_row=first_row)
        else:
            o = torch.empty((ql.shape[0], H * r), dtype=ql.dtype, device=ql.device)
            for h0 in range(0, H, self.heads_a_call):
                n = min(self.heads_a_call, H - h0)
                part = ops.paged_attention_generic(ql[:, h0 * dc :], cache.keys, cache.values, cache.block_table,
                                                   ctx.token_req[first_row:], ctx.positions[first_row:], n, 1, dc, cache.page_size,
                                                   window=self.window, scale=self.scale, value_dim=r)
                if n == H:
                    o = part
                else:
                    o[:, h0 * r : (h0 + n) * r] = part
        return ops.head_linear(o, self.from_latent)  # [rows, heads * value_dim]

    def _over_expanded(self, q: torch.Tensor, ctx: StepContext, cache: CacheView, portions: int) -> torch.Tensor:
        """Attention over expanded keys and values for the tokens of the step's first ``portions``
        requests; returns rows for all of the step's tokens, of which only those are written."""
        H, dk, dv, P = self.num_heads, self.query_dim, self.value_dim, cache.page_size
        plan = ctx.extras.get(("expanded_keys_plan", portions, P, self.window))
        if plan is None:  # made once a step, shared by the layers of one window
            lens = np.asarray(ctx.host_kv_len[:portions], dtype=np.int64)
            # the first key a request's queries see, moved down to its page's start: nothing before it is read
            # back (a windowed cache has given those pages up) and the expanded pages begin there
            first = np.zeros_like(lens)
            if self.window:
                q_lens = np.asarray([ctx.host_q_start[i + 1] - ctx.host_q_start[i] for i in range(portions)], dtype=np.int64)
                first = np.maximum(lens - q_lens - self.window + 1, 0) // P * P
            counts = lens - first
            pages = -(-counts // P)
            first_page = np.concatenate([[0], np.cumsum(pages)])
            total = int(counts.sum())
            req = np.repeat(np.arange(portions, dtype=np.int32), counts)
            starts = np.concatenate([[0], np.cumsum(counts)[:-1]])
            pos = (np.arange(total, dtype=np.int64) - np.repeat(starts - first, counts)).astype(np.int32)
            table = np.zeros((portions, int((first // P + pages).max())), dtype=np.int32)
            for i in range(portions):
                table[i, first[i] // P : first[i] // P + pages[i]] = first_page[i] + np.arange(pages[i])
            dev = upload(np.concatenate([req, pos, table.reshape(-1)]), torch.int32, q.device)
            n_tiles = sum(-(-(ctx.host_q_start[i + 1] - ctx.host_q_start[i]) // 16) for i in range(portions))
            plan = ctx.extras[("expanded_keys_plan", portions, P, self.window)] = (
                dev[:total], dev[total : 2 * total], dev[2 * total :].view(portions, -1), int(first_page[-1]), n_tiles)
        req_d, pos_d, table_d, n_pages, n_tiles = plan
        latents = ops.gather_keys(cache.keys, cache.block_table, req_d, pos_d, self.cached_dim, P)
        if self.expand_cached is not None:  # [k_rot | c] -> every head's [k_rot | W_uk c] and W_uv c
            kv = self.expand_cached(latents)
        else:
            kv = self.expand(latents)  # [all keys of these requests, heads * key_dim | heads * value_dim]
        # (zeros: the rest of a request's last page is read, with weight zero, and must hold numbers)
        keys = torch.zeros(ops.key_pages_shape(n_pages, H, P, dk, padded=True), dtype=q.dtype, device=q.device)
        values = torch.zeros(ops.value_pages_shape(n_pages, H, P, dv), dtype=q.dtype, device=q.device)
        ops.qk_prepare(kv, pos_d, req_d, table_d, None, None, 0.0, None, keys, values, 0, H, dk, dv, P)
        tile_req, tile_row0 = tile_plan(ctx, 16)
        return ops.attention_tile_f32(q, keys, values, table_d, ctx.q_start, ctx.kv_len, tile_req[:n_tiles], tile_row0[:n_tiles],
                                      H, H, dk, dv, P, 1, scale=self.scale, window=self.window)

    def mix(self, h, ctx, cache, state, rows, out_f32: bool = False):
        return self.out(self._attend(h, ctx, cache, rows), out_f32=out_f32)

    def forward(self, h, residual, ctx, cache, state, rows):
        return self.out(self._attend(h, ctx, cache, rows), residual=residual)
