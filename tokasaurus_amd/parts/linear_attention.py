"""Linear attention with a decay: mixers that keep, per request, a matrix per head instead of keys and
values.  Per head ``S_t = diag(a_t) S_(t-1) + k_t v_t^T`` and ``o_t = S_t^T q_t``, from ``S = 0``.

``lightning_attention``: q, k and v are projections through silu; a_t is one constant a head (``decays``); the
heads' results side by side pass one RMS norm with a plain weight, are multiplied by sigmoid(W_g h) and projected.

``hgrn2``: q is a projection through silu and v a plain projection; a forget gate per head and row of S,
``f = low + (1 - low) * sigmoid(W_f h + b)`` with a learned lower bound ``low``, decays the state (a_t = f) and its
complement is what is written (k_t = 1 - f); every head's result passes an RMS norm over its own elements with
one weight for all heads, and the output projection follows.

Everything that reads h is one stacked product whose 32-bit sums go straight into the recurrence: activations,
gates, the state, the read-out and the norms are 32-bit arithmetic in either storage type.  The state is one
row of 32-bit numbers in the request's slot, zero when a request takes the slot; a step of any cut continues
from it with the sums of the token-by-token recurrence.

A mixer here also gives its result in front of the output projection (``inner_rows``), with a factor, into a
view that the caller names: for a mixer that runs two side by side through one stacked output product.
"""

from __future__ import annotations

import torch

from tokasaurus_amd.kernels import ops
from tokasaurus_amd.parts.base import BIAS, MIXERS, NORM_WEIGHT, UNIT_INTERVAL, Mixer, StateNeed, StepContext, TensorSpec
from tokasaurus_amd.parts.linear import Linear, Placer


class _LinearAttention(Mixer):
    """What the two forms share: the state, the output projection, and how a result leaves."""

    hidden_size: int
    num_heads: int
    key_dim: int
    value_dim: int
    out: Linear

    @property
    def inner_size(self) -> int:
        return self.num_heads * self.value_dim

    def state_need(self) -> StateNeed:
        return StateNeed((self.num_heads * self.value_dim * self.key_dim,), torch.float32)

    def inner_rows(self, h, ctx: StepContext, cache, state, out: torch.Tensor | None = None, scale: float = 1.0) -> torch.Tensor:
        raise NotImplementedError

    def mix(self, h, ctx, cache, state, rows, out_f32: bool = False):
        y = self.inner_rows(h, ctx, cache, state)
        return self.out(y if rows is None else ops.gather_rows(y, rows), out_f32=out_f32)

    def forward(self, h, residual, ctx, cache, state, rows):
        y = self.inner_rows(h, ctx, cache, state)
        return self.out(y if rows is None else ops.gather_rows(y, rows), residual=residual)


@MIXERS.register("lightning_attention")
class LightningAttention(_LinearAttention):
    def __init__(self, hidden_size: int, num_heads: int, key_dim: int, value_dim: int, decays: list[float], norm_eps: float,
                 names: dict[str, str]):
        """``decays``: one number a head.  ``names``: checkpoint names under q, k ([heads * key_dim, hidden]), v, g
        ([heads * value_dim, hidden]), norm ([heads * value_dim]) and o ([hidden, heads * value_dim])."""
        self.hidden_size, self.num_heads = hidden_size, int(num_heads)
        self.key_dim, self.value_dim = int(key_dim), int(value_dim)
        self.decays = [float(a) for a in decays]
        if len(self.decays) != self.num_heads:
            raise ValueError(f"{len(self.decays)} decays for {self.num_heads} heads")
        self.norm_eps = float(norm_eps)
        self.names = dict(names)
        qk, v = self.num_heads * self.key_dim, self.num_heads * self.value_dim
        self.inp = Linear(hidden_size, [names[x] for x in ("q", "k", "v", "g")], [qk, qk, v, v])
        self.out = Linear(v, [names["o"]], [hidden_size])
        self.decay: torch.Tensor | None = None
        self.norm_w: torch.Tensor | None = None

    def tensor_specs(self) -> list[TensorSpec]:
        return self.inp.tensor_specs() + self.out.tensor_specs() + [TensorSpec(self.names["norm"], (self.inner_size,), NORM_WEIGHT)]

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        self.inp.load(tensors, placer)
        self.out.load(tensors, placer)
        n = self.names["norm"]
        self.norm_w = placer.place(("vector_f32", n), lambda: tensors[n].to(torch.float32).contiguous().to(placer.device))
        self.decay = placer.place(("constant_f32", *self.decays), lambda: torch.tensor(
            self.decays, dtype=torch.float64).to(torch.float32).to(placer.device))

    def inner_rows(self, h, ctx, cache, state, out=None, scale: float = 1.0):
        assert state is not None, "linear attention keeps its state in the request's slot"
        H, dk, dv = self.num_heads, self.key_dim, self.value_dim
        proj = self.inp(h, out_f32=True)
        o = ops.linear_attention(proj, 0, H * dk, 2 * H * dk, state, ctx.q_start, ctx.slots, H, dk, dv, decay=self.decay, longest=ctx.max_q_len)
        gate = proj[:, 2 * H * dk + H * dv :]
        return ops.group_norm_gate(o, self.norm_w, self.norm_eps, 1, h.dtype, gate=gate, scale=scale, out=out)


@MIXERS.register("hgrn2")
class HGRN2(_LinearAttention):
    def __init__(self, hidden_size: int, num_heads: int, key_dim: int, value_dim: int, norm_eps: float, names: dict[str, str]):
        """``names``: checkpoint names under q, f ([heads * key_dim, hidden]), f_bias, lower ([heads * key_dim]), v
        ([heads * value_dim, hidden]), norm ([value_dim], shared by the heads) and o ([hidden, heads * value_dim])."""
        self.hidden_size, self.num_heads = hidden_size, int(num_heads)
        self.key_dim, self.value_dim = int(key_dim), int(value_dim)
        self.norm_eps = float(norm_eps)
        self.names = dict(names)
        qk, v = self.num_heads * self.key_dim, self.num_heads * self.value_dim
        self.inp = Linear(hidden_size, [names[x] for x in ("q", "f", "v")], [qk, qk, v])
        self.out = Linear(v, [names["o"]], [hidden_size])
        self.f_bias = self.f_low = self.norm_w = None

    def tensor_specs(self) -> list[TensorSpec]:
        qk = self.num_heads * self.key_dim
        return self.inp.tensor_specs() + self.out.tensor_specs() + [
            TensorSpec(self.names["f_bias"], (qk,), BIAS), TensorSpec(self.names["lower"], (qk,), UNIT_INTERVAL),
            TensorSpec(self.names["norm"], (self.value_dim,), NORM_WEIGHT)]

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        self.inp.load(tensors, placer)
        self.out.load(tensors, placer)

        def f32(name: str) -> torch.Tensor:
            return placer.place(("vector_f32", name), lambda: tensors[name].to(torch.float32).contiguous().to(placer.device))

        self.f_bias, self.f_low, self.norm_w = f32(self.names["f_bias"]), f32(self.names["lower"]), f32(self.names["norm"])

    def inner_rows(self, h, ctx, cache, state, out=None, scale: float = 1.0):
        assert state is not None, "linear attention keeps its state in the request's slot"
        H, dk, dv = self.num_heads, self.key_dim, self.value_dim
        proj = self.inp(h, out_f32=True)
        o = ops.linear_attention(proj, 0, H * dk, 2 * H * dk, state, ctx.q_start, ctx.slots, H, dk, dv,
                                 forget_bias=self.f_bias, forget_low=self.f_low, longest=ctx.max_q_len)
        return ops.group_norm_gate(o, self.norm_w, self.norm_eps, H, h.dtype, scale=scale, out=out)
