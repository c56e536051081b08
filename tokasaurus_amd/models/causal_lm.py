"""A causal language model built from a ``ModelSpec``: embedding, the blocks in
run order, final norm and head (the skeleton of tokasaurus/model/llama.py:521-582,
603-667 with the architecture taken out of it)."""

from __future__ import annotations

import torch

from tokasaurus_amd.kernels import ops
from tokasaurus_amd.models.spec import ModelSpec
from tokasaurus_amd.parts.base import (BLOCKS, CONNECTORS, EMBEDDINGS, HEADS, CacheNeed, CacheView, Part, Prepared, StateNeed, StepContext,
                                       TensorSpec)
from tokasaurus_amd.parts.block import build_with_shared, stream_and_prepared
import tokasaurus_amd.parts.embedding  # noqa: F401  (registers the embedding and the head)
from tokasaurus_amd.parts.linear import Placer


def _one_or_many(needs: list):
    return None if not needs else (needs[0] if len(needs) == 1 else list(needs))


class CausalLM:
    def __init__(self, spec: ModelSpec):
        spec.validate()
        self.spec = spec
        self.shared: dict = {}
        self.embedding = build_with_shared(EMBEDDINGS, spec.embedding, self.shared)
        self.blocks = [build_with_shared(BLOCKS, b, self.shared) for b in spec.layers]
        self.head = build_with_shared(HEADS, spec.head, self.shared)
        self.connectors = [build_with_shared(CONNECTORS, c, self.shared) for c in spec.connectors]
        # an embedding that can also write the rows of the first block's entry norm is told which norm that is
        # (only one that merely rounds the stream: there is nothing of the norm to compute)
        if hasattr(self.embedding, "reader") and spec.run_order and spec.run_order[0].before is None:
            first = self.blocks[spec.run_order[0].layer]
            entry = first.entry_norm() if first.fuses_norm else None
            if getattr(entry, "plain_rows", False):
                self.embedding.reader = entry
        self.dtype: torch.dtype | None = None
        self.device: torch.device | None = None
        self.weight_bytes = 0

    # ---- tensors
    def parts(self) -> list[Part]:
        return [self.embedding, *self.connectors, *self.blocks, self.head]

    def tensor_specs(self) -> list[TensorSpec]:
        seen: dict[str, TensorSpec] = {}
        for part in self.parts():
            for s in part.tensor_specs():
                if s.name in seen and seen[s.name].shape != s.shape:
                    raise ValueError(f"tensor {s.name} is wanted with shapes {seen[s.name].shape} and {s.shape}")
                seen.setdefault(s.name, s)
        return list(seen.values())

    def load(self, tensors: dict[str, torch.Tensor], dtype: torch.dtype, device: torch.device) -> None:
        placer = Placer(dtype, device)
        for part in self.parts():
            part.load(tensors, placer)
        self.dtype, self.device = dtype, device
        self.weight_bytes = placer.bytes_placed()

    # ---- what the cache manager must provide, one item per run entry
    def cache_needs(self) -> "list[CacheNeed | None | list[CacheNeed]]":
        """What every run entry's block keeps in pages: nothing, one need, or a list of several."""
        return [_one_or_many(self.blocks[e.layer].cache_needs()) for e in self.spec.run_order]

    def state_needs(self) -> "list[StateNeed | None | list[StateNeed]]":
        return [_one_or_many(self.blocks[e.layer].state_needs()) for e in self.spec.run_order]

    def embedding_state_need(self) -> "StateNeed | None":
        """What the embedding keeps per request in its slot (``StepContext.embedding_state``), if anything."""
        return self.embedding.state_need()

    # ---- one step
    def forward(
        self,
        ctx: StepContext,
        caches: list[CacheView | None],
        states: list[torch.Tensor | None],
        want_rows: torch.Tensor | None,
        logits_out: torch.Tensor | None = None,
    ) -> torch.Tensor:
        """Run the batch of ``ctx`` and return logits [len(want_rows), vocab] in 32-bit;
        ``want_rows`` None stands for every row in order (no rows are picked out then).
        ``logits_out``: a contiguous buffer of that shape that receives the logits and is returned."""
        # (an embedding may already have made the rows of the first block's entry norm)
        x, prepared = stream_and_prepared(self.embedding.forward(ctx))
        order = self.spec.run_order
        last = len(order) - 1
        # a connector reads the embedding's output again; blocks may update the stream in place
        x0 = x.clone() if any(not getattr(c, "takes_history", False) for c in self.connectors) else None
        # connectors that read every stream so far: the embedding's output and each block's result are kept side by
        # side, [streams, tokens, H]; a block updates its input in place, so its input is a copy in the next place
        hist = None
        if any(getattr(c, "takes_history", False) for c in self.connectors) and order:
            if x.dtype != torch.float32:
                raise TypeError("connectors over the model's streams so far run on a 32-bit stream")
            hist = torch.empty((len(order) + 1, *x.shape), dtype=torch.float32, device=x.device)
            hist[0].copy_(x)
            hist[1].copy_(x)
            x = hist[1]
        for i, entry in enumerate(order):
            rows = want_rows if i == last else None
            block = self.blocks[entry.layer]
            if entry.before is not None:
                x, prepared = self.connectors[entry.before].forward(x, x0), None
                if hist is not None:
                    hist[i + 1].copy_(x)
                    x = hist[i + 1]
            reader = None  # the norm that reads the stream this entry leaves
            if i == last:
                reader = self.head.entry_norm()
            elif order[i + 1].before is None:  # (else the stream changes before the next block reads it)
                reader = self.blocks[order[i + 1].layer].entry_norm()
            after = self.connectors[entry.after] if entry.after is not None else None
            pending = None
            if block.fuses_norm and after is not None and getattr(after, "adds_pending_sum", False) and getattr(block, "can_defer_sum", False):
                # the block hands its branches over unsummed: the connector behind it adds them in its own pass
                pending = block.forward(x, ctx, caches[i], states[i], rows, prepared=prepared, next_norm=None, defer_sum=True)
                out = pending.x
            elif block.fuses_norm:
                # (a connector behind this block changes the stream before anything reads it)
                out = block.forward(x, ctx, caches[i], states[i], rows, prepared=prepared,
                                    next_norm=None if entry.after is not None else reader)
            else:
                out = block.forward(x, ctx, caches[i], states[i], rows)
            x, prepared = stream_and_prepared(out)
            if hist is not None:
                whole = rows is None
                if whole and x.data_ptr() != hist[i + 1].data_ptr():
                    hist[i + 1].copy_(x)  # (a block that did not update its input in place)
                if after is not None and getattr(after, "takes_history", False):
                    more = {"pending": pending} if pending is not None else {}
                    out = after.forward_history(hist, i + 2 if whole else i + 1, None if whole else x, rows,
                                                hist[i + 2] if (whole and i < last) else None, next_norm=reader, **more)
                    x, prepared = stream_and_prepared(out)
                elif i < last:
                    hist[i + 2].copy_(x)
                    x = hist[i + 2]
            elif entry.after is not None:
                raise RuntimeError("a connector behind a run entry reads the model's streams so far (takes_history)")
            tap = ctx.extras.get("model_tap")
            if tap is not None:  # a list that collects the stream every run entry leaves (tests, debugging)
                tap.append(x.clone())
        if last < 0 and want_rows is not None:
            x = ops.gather_rows(x, want_rows)
        if logits_out is None:
            return self.head.forward(x, prepared)
        if self.head.takes_out:
            return self.head.forward(x, prepared, out=logits_out)
        logits_out.copy_(self.head.forward(x, prepared))
        return logits_out
