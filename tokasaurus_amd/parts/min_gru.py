"""A gated recurrence whose gates read only the current token (minGRU): a mixer that keeps, per
request, one number a channel instead of keys and values.

Per token and channel: ``z = sigmoid(W_z h + b_z)``, ``u = W_x h + b_x``, the candidate
``c = u + 1/2`` where ``u >= 0`` and ``sigmoid(u)`` below; ``S <- (1 - z) S + z c``; the output is
``W_o (S * silu(W_g h))``.  z, x and g are one stacked product (its rows interleaved channel by channel,
so that the recurrence reads a channel's three sums side by side) whose 32-bit sums go
straight into the recurrence, whose kernel adds the two biases: gates, candidate and state are 32-bit
arithmetic in either storage type.  The state is one row of 32-bit numbers in the request's slot, zero when a request takes the
slot; a step of any cut continues from it with the same bits as the token-by-token recurrence.
"""

from __future__ import annotations

import torch

from tokasaurus_amd.kernels import ops
from tokasaurus_amd.parts.base import BIAS, MIXERS, Mixer, StateNeed, StepContext, TensorSpec
from tokasaurus_amd.parts.linear import Linear, Placer


@MIXERS.register("min_gru")
class MinGRU(Mixer):
    def __init__(self, hidden_size: int, width: int, names: dict[str, str]):
        """``names``: checkpoint names under the keys z, x, g ([width, hidden]), z_bias, x_bias ([width])
        and o ([hidden, width])."""
        self.hidden_size, self.width = hidden_size, int(width)
        self.inp = Linear(hidden_size, [names["z"], names["x"], names["g"]], [self.width] * 3)
        self.bias_names = (names["z_bias"], names["x_bias"])
        self.bias: torch.Tensor | None = None  # [b_z | b_x], 32-bit
        self.out = Linear(self.width, [names["o"]], [hidden_size])

    def tensor_specs(self) -> list[TensorSpec]:
        return self.inp.tensor_specs() + self.out.tensor_specs() + [TensorSpec(b, (self.width,), BIAS) for b in self.bias_names]

    def state_need(self) -> StateNeed:
        return StateNeed((self.width,), torch.float32)

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        z, x, g = self.inp.names

        def interleaved() -> torch.Tensor:  # rows (z_c, x_c, g_c) for channel c = 0, 1, ..
            w = torch.stack([tensors[z], tensors[x], tensors[g]], dim=1)
            return w.reshape(3 * self.width, self.hidden_size).to(dtype=placer.dtype).contiguous().to(placer.device)

        self.inp.weight = placer.place(("rows_interleaved", z, x, g), interleaved)
        self.out.load(tensors, placer)
        self.bias = placer.place(("vector_f32", *self.bias_names), lambda: torch.cat(
            [tensors[b].to(torch.float32) for b in self.bias_names]).contiguous().to(placer.device))

    def _run(self, h: torch.Tensor, ctx: StepContext, state: torch.Tensor, rows: torch.Tensor | None) -> torch.Tensor:
        assert state is not None, "the recurrence keeps its state in the request's slot"
        proj = self.inp(h, out_f32=True)
        y = ops.min_gru(proj, state, ctx.q_start, ctx.slots, self.width, ctx.max_q_len, h.dtype, bias=self.bias)
        return y if rows is None else ops.gather_rows(y, rows)

    def mix(self, h, ctx, cache, state, rows, out_f32: bool = False):
        return self.out(self._run(h, ctx, state, rows), out_f32=out_f32)

    def forward(self, h, residual, ctx, cache, state, rows):
        return self.out(self._run(h, ctx, state, rows), residual=residual)
