"""A feed-forward made of many small gated experts of which every token uses a few.

The router is 32-bit arithmetic: logits ``W_router h`` over the routed experts and the identity
experts together, ``s = softmax(logits)``; the choice is made by ``s + correction`` (a learned
vector that moves the choice and not the weight); the experts form ``groups`` equal groups of
neighbours, a group's mark is its largest choice score, and only experts of the ``keep`` groups
with the largest marks can be chosen; the ``top`` largest choice scores win and the chosen experts'
``s`` are their weights, as they are or (``normalize_scale``) divided by their sum (+ 1e-20) and multiplied by a
constant.  A routed expert is ``W_down (silu(W_gate h) * (W_up h))``;
the last ``identity`` router outputs have no tensors, their output is ``h`` itself.  A shared
expert of the same form may run for every token; its output is multiplied by
``sigmoid(w_sg . h)``, one number a token, where the checkpoint has such a gate, and added.

One kernel routes (and computes the shared expert's gate); the experts' products run pair by
pair (token, chosen expert), each a function of its own token only, and are summed per token
in the order of the choice: a token's result does not depend on what else is in the batch.
"""

from __future__ import annotations

import torch

from tokasaurus_amd.kernels import ops
from tokasaurus_amd.parts.base import FEED_FORWARDS, MATRIX, SMALL_VECTOR, FeedForward, TensorSpec
from tokasaurus_amd.parts.linear import Linear, Placer


@FEED_FORWARDS.register("routed_experts")
class RoutedExperts(FeedForward):
    def __init__(self, hidden_size: int, expert_size: int, num_experts: int, top: int, names: dict[str, str],
                 identity: int = 0, groups: int = 1, keep: int = 1, shared_size: int | None = None,
                 normalize_scale: float | None = None):
        """``names``: ``router`` ([experts + identity, hidden]), ``correction`` ([experts + identity]),
        ``expert``: a pattern with ``{e}`` for the expert's number that gives the prefix of its
        ``.gate``, ``.up`` ([expert_size, hidden]) and ``.down`` ([hidden, expert_size]); with a
        shared expert also ``shared`` (the prefix of its three matrices) and, where it has a gate,
        ``shared_gate`` ([1, hidden]).  ``normalize_scale``: the chosen experts' weights are divided by their sum
        and multiplied by this number."""
        self.normalize_scale = float(normalize_scale) if normalize_scale else None
        self.hidden_size, self.expert_size = hidden_size, int(expert_size)
        self.num_experts, self.top, self.identity = int(num_experts), int(top), int(identity)
        self.groups, self.keep = int(groups), int(keep)
        self.n_all = self.num_experts + self.identity
        if self.n_all % self.groups or not 0 < self.keep <= self.groups or not 0 < self.top <= self.n_all:
            raise ValueError(f"{self.n_all} experts in {self.groups} groups, {self.keep} kept, {self.top} chosen")
        self.names = dict(names)
        self.shared_size = int(shared_size) if shared_size else None
        self.shared_gate_up = self.shared_down = None
        if self.shared_size:
            sp = names["shared"]
            self.shared_gate_up = Linear(hidden_size, [f"{sp}.gate", f"{sp}.up"], [self.shared_size] * 2)
            self.shared_down = Linear(self.shared_size, [f"{sp}.down"], [hidden_size])
        self.router = self.correction = self.w_gate_up = self.w_down = self.shared_gate = None

    def _expert(self, e: int, which: str) -> str:
        return f"{self.names['expert'].format(e=e)}.{which}"

    def tensor_specs(self) -> list[TensorSpec]:
        W, F = self.hidden_size, self.expert_size
        specs = [TensorSpec(self.names["router"], (self.n_all, W), MATRIX),
                 TensorSpec(self.names["correction"], (self.n_all,), SMALL_VECTOR)]
        for e in range(self.num_experts):
            specs += [TensorSpec(self._expert(e, "gate"), (F, W), MATRIX), TensorSpec(self._expert(e, "up"), (F, W), MATRIX),
                      TensorSpec(self._expert(e, "down"), (W, F), MATRIX)]
        if self.shared_size:
            specs += self.shared_gate_up.tensor_specs() + self.shared_down.tensor_specs()
            if self.names.get("shared_gate"):
                specs.append(TensorSpec(self.names["shared_gate"], (1, W), MATRIX))
        return specs

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        n, E = self.names, self.num_experts

        def place(key, make):
            return placer.place(key, lambda: make().contiguous().to(placer.device))

        self.router = place(("row_major", n["router"]), lambda: tensors[n["router"]].to(placer.dtype))
        self.correction = place(("vector_f32", n["correction"]), lambda: tensors[n["correction"]].to(torch.float32))
        # one tensor for all experts: [experts, gate rows | up rows, hidden] and [experts, hidden, expert_size]
        self.w_gate_up = place(("experts_gate_up", n["expert"]), lambda: torch.stack(
            [torch.cat([tensors[self._expert(e, "gate")], tensors[self._expert(e, "up")]], dim=0) for e in range(E)]).to(placer.dtype))
        self.w_down = place(("experts_down", n["expert"]), lambda: torch.stack(
            [tensors[self._expert(e, "down")] for e in range(E)]).to(placer.dtype))
        if self.shared_size:
            self.shared_gate_up.load(tensors, placer)
            self.shared_down.load(tensors, placer)
            if n.get("shared_gate"):
                self.shared_gate = place(("row_major", n["shared_gate"]), lambda: tensors[n["shared_gate"]].to(placer.dtype).reshape(-1))

    def transform(self, h: torch.Tensor, out_f32: bool = False) -> torch.Tensor:
        ids, weights, gate = ops.expert_route(h, self.router, self.correction, self.groups, self.keep, self.top, self.shared_gate,
                                              normalize_scale=self.normalize_scale,
                                              unit_gate=bool(self.shared_size) and self.shared_gate is None)
        shared = self.shared_down(self.shared_gate_up(h, swiglu=True), out_f32=True) if self.shared_size else None
        y = ops.expert_mix(h, self.w_gate_up, self.w_down, ids, weights, shared, gate)
        return y if out_f32 else y.to(h.dtype)

    def forward(self, h: torch.Tensor, residual: torch.Tensor):
        return ops.add(self.transform(h), residual.contiguous())
