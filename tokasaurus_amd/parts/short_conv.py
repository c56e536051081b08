"""A short causal convolution over time on every channel, added to its input:
``h + conv(h)`` with ``conv(h)_t = sum_j w[:, j] * h_(t - taps + 1 + j)`` and zeros before a request's
first token.  It stands between a block's entry norm and its mixer.  The last ``taps - 1`` inputs of a
request are part of its state: one row of 32-bit numbers in the request's slot, zero when a request takes
the slot; a step of any cut continues from it.  The taps are kept in 32-bit and the sums are 32-bit; the
result is rounded once to the storage type of the rows.
"""

from __future__ import annotations

import torch

from tokasaurus_amd.kernels import ops
from tokasaurus_amd.parts.base import CONV, Part, StateNeed, StepContext, TensorSpec
from tokasaurus_amd.parts.linear import Placer


class ShortConvResidual(Part):
    def __init__(self, width: int, taps: int, name: str):
        """``name``: the checkpoint's [width, taps]; the last column is the current token's."""
        self.width, self.taps, self.name = int(width), int(taps), name
        if self.taps < 1:
            raise ValueError(f"a convolution of {self.taps} taps")
        self.weight: torch.Tensor | None = None

    def tensor_specs(self) -> list[TensorSpec]:
        return [TensorSpec(self.name, (self.width, self.taps), CONV)]

    def state_need(self) -> StateNeed | None:
        return StateNeed(((self.taps - 1) * self.width,), torch.float32) if self.taps > 1 else None

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        # tap by tap, [taps, width]: neighbouring channels' weights of one tap lie together
        self.weight = placer.place(("conv_f32_by_tap", self.name), lambda: tensors[self.name].to(torch.float32).t().contiguous().to(placer.device))

    def forward(self, h: torch.Tensor, ctx: StepContext, tails: torch.Tensor | None) -> torch.Tensor:
        if self.taps > 1 and tails is None:
            raise RuntimeError("a short convolution keeps its last inputs in the request's slot: the step has no such state")
        return ops.short_conv(h, self.weight, tails, ctx.q_start, ctx.token_req, ctx.slots, single_tokens=ctx.max_q_len == 1)
