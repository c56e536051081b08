"""Two mixers side by side on the same input: ``left_scale * left(h) + right_scale * right(h)``.

Each of the two gives its result in front of its output projection (``inner_rows``), already multiplied by
its factor, into its columns of one buffer; the two output projections are one product over that buffer with
the matrices side by side, ``[W_o left | W_o right]``, whose 32-bit sums are the weighted sum of the two
mixers' results.  At most one of the two keeps keys in pages and at most one a state in the request's slot.
"""

from __future__ import annotations

import torch

from tokasaurus_amd.kernels import ops
from tokasaurus_amd.parts.base import MIXERS, CacheNeed, Mixer, Part, PartSpec, StateNeed, TensorSpec
from tokasaurus_amd.parts.linear import Linear, Placer


@MIXERS.register("mixer_pair")
class MixerPair(Mixer):
    def __init__(self, hidden_size: int, left: PartSpec, right: PartSpec, left_scale: float = 1.0, right_scale: float = 1.0,
                 shared: dict | None = None):
        from tokasaurus_amd.parts.block import build_with_shared

        shared = shared if shared is not None else {}
        self.hidden_size = hidden_size
        self.left = build_with_shared(MIXERS, left, shared)
        self.right = build_with_shared(MIXERS, right, shared)
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)
        for m in (self.left, self.right):
            if not hasattr(m, "inner_rows") or not hasattr(m, "inner_size") or len(m.out.names) != 1 or m.out.bias_names:
                raise ValueError(f"{type(m).__name__} cannot stand in a pair: it must give its rows in front of one plain output projection")
        if sum(m.cache_need() is not None for m in (self.left, self.right)) > 1 or \
                sum(m.state_need() is not None for m in (self.left, self.right)) > 1:
            raise ValueError("of two mixers side by side at most one keeps pages and at most one a state")
        self.out = Linear(self.left.inner_size + self.right.inner_size,
                          [f"{self.left.out.names[0]}|{self.right.out.names[0]}"], [hidden_size])

    def children(self) -> list[Part]:
        return [self.left, self.right]

    def tensor_specs(self) -> list[TensorSpec]:
        return self.left.tensor_specs() + self.right.tensor_specs()

    def cache_need(self) -> CacheNeed | None:
        return self.left.cache_need() or self.right.cache_need()

    def state_need(self) -> StateNeed | None:
        return self.left.state_need() or self.right.state_need()

    def check_cache(self, page_size: int, dtype: torch.dtype) -> None:
        self.left.check_cache(page_size, dtype)
        self.right.check_cache(page_size, dtype)

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        self.left.load(tensors, placer)
        self.right.load(tensors, placer)
        a, b = self.left.out.names[0], self.right.out.names[0]
        self.out.weight = placer.place(("columns_side_by_side", a, b), lambda: torch.cat(
            [tensors[a], tensors[b]], dim=1).to(dtype=placer.dtype).contiguous().to(placer.device))

    def _inner(self, h, ctx, cache, state, rows):
        n, nl = h.shape[0], self.left.inner_size
        both = torch.empty((n, nl + self.right.inner_size), dtype=h.dtype, device=h.device)
        for m, view, scale in ((self.left, both[:, :nl], self.left_scale), (self.right, both[:, nl:], self.right_scale)):
            m.inner_rows(h, ctx, cache if m.cache_need() is not None else None, state if m.state_need() is not None else None,
                         out=view, scale=scale)
        return both if rows is None else ops.gather_rows(both, rows)

    def mix(self, h, ctx, cache, state, rows, out_f32: bool = False):
        return self.out(self._inner(h, ctx, cache, state, rows), out_f32=out_f32)

    def forward(self, h, residual, ctx, cache, state, rows):
        return self.out(self._inner(h, ctx, cache, state, rows), residual=residual)
