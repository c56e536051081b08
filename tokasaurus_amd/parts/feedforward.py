"""Dense gated feed-forward (tokasaurus/model/llama.py:290-339):
``x + down(silu(gate(h)) * up(h))``, no biases.  gate and up are one stacked product.
Beside it the ungated feed-forward whose activation is the square of relu."""

from __future__ import annotations

import torch

from tokasaurus_amd.kernels import ops
from tokasaurus_amd.parts.base import FEED_FORWARDS, FeedForward, Normed, TensorSpec
from tokasaurus_amd.parts.linear import Linear, Placer


@FEED_FORWARDS.register("swiglu")
class SwiGLU(FeedForward):
    fuses_norm = True

    def __init__(self, hidden_size: int, intermediate_size: int, names: dict[str, str], activation: str = "silu"):
        """``activation``: what the gate passes, "silu" or "gelu_tanh" (the tanh form of gelu)."""
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        if activation not in ("silu", "gelu_tanh"):
            raise ValueError(f"a gated feed-forward's activation is silu or gelu_tanh, not {activation!r}")
        self.glu = None if activation == "silu" else activation
        self.gate_up = Linear(hidden_size, [names["gate"], names["up"]], [intermediate_size] * 2)
        self.down = Linear(intermediate_size, [names["down"]], [hidden_size])

    def tensor_specs(self) -> list[TensorSpec]:
        return self.gate_up.tensor_specs() + self.down.tensor_specs()

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        self.gate_up.load(tensors, placer)
        self.down.load(tensors, placer)

    def forward(self, h: torch.Tensor | Normed, residual: torch.Tensor, emit_norm=None):
        return self.down.with_residual(self.gate_up(h, swiglu=True, glu=self.glu), residual, emit_norm)

    def transform(self, h: torch.Tensor, out_f32: bool = False) -> torch.Tensor:
        """The feed-forward's own output, nothing added: for blocks that combine their branches
        themselves.  ``out_f32``: the down projection's 32-bit sums leave unrounded."""
        return self.down(self.gate_up(h, swiglu=True, glu=self.glu), out_f32=out_f32)


@FEED_FORWARDS.register("squared_relu")
class SquaredReLU(FeedForward):
    """``down(max(up(h), 0)^2)``, no gate and no biases."""

    def __init__(self, hidden_size: int, intermediate_size: int, names: dict[str, str]):
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.up = Linear(hidden_size, [names["up"]], [intermediate_size])
        self.down = Linear(intermediate_size, [names["down"]], [hidden_size])

    def tensor_specs(self) -> list[TensorSpec]:
        return self.up.tensor_specs() + self.down.tensor_specs()

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        self.up.load(tensors, placer)
        self.down.load(tensors, placer)

    def forward(self, h: torch.Tensor, residual: torch.Tensor):
        return self.down(ops.squared_relu_(self.up(h)), residual=residual)

    def transform(self, h: torch.Tensor, out_f32: bool = False) -> torch.Tensor:
        return self.down(ops.squared_relu_(self.up(h)), out_f32=out_f32)


@FEED_FORWARDS.register("clamped_glu")
class ClampedGLU(FeedForward):
    """A gated feed-forward with clamps: ``g = min(gate(h), limit)``, ``u = clamp(up(h), -limit, limit)``,
    ``down(g * sigmoid(alpha * g) * (u + 1))``, no biases.  gate and up are one stacked product."""

    def __init__(self, hidden_size: int, intermediate_size: int, limit: float, names: dict[str, str], alpha: float = 1.702):
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.limit, self.alpha = float(limit), float(alpha)
        if not self.limit > 0:
            raise ValueError("the clamp's limit must be positive")
        self.gate_up = Linear(hidden_size, [names["gate"], names["up"]], [intermediate_size] * 2)
        self.down = Linear(intermediate_size, [names["down"]], [hidden_size])

    def tensor_specs(self) -> list[TensorSpec]:
        return self.gate_up.tensor_specs() + self.down.tensor_specs()

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        self.gate_up.load(tensors, placer)
        self.down.load(tensors, placer)

    def _inner(self, h: torch.Tensor) -> torch.Tensor:
        return self.gate_up(h, swiglu=True, glu=(self.limit, self.alpha))

    def forward(self, h: torch.Tensor, residual: torch.Tensor):
        return self.down(self._inner(h), residual=residual)

    def transform(self, h: torch.Tensor, out_f32: bool = False) -> torch.Tensor:
        return self.down(self._inner(h), out_f32=out_f32)
