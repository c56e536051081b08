"""Token embedding and the language-model head.

Embedding is a plain row gather without scaling (tokasaurus/model/llama.py:507-518).
The head norms the kept rows and multiplies by the head matrix, which is the
embedding matrix itself when the checkpoint ties them (llama.py:426-467,842-845);
logits leave in 32-bit.
"""

from __future__ import annotations

import torch

from tokasaurus_amd.kernels import ops
from tokasaurus_amd.parts.base import (EMBEDDINGS, HEADS, MATRIX, NORMS, Embedding, Head, Normed, Part, PartSpec, Prepared,
                                       StateNeed, StepContext, TensorSpec)
from tokasaurus_amd.parts.linear import Linear, Placer


@EMBEDDINGS.register("token_embedding")
class TokenEmbedding(Embedding):
    def __init__(self, vocab_size: int, hidden_size: int, name: str, scale: float | None = None, stream_f32: bool = False,
                 position_name: str | None = None, max_positions: int = 0):
        """``scale``: every row is multiplied by it.  ``stream_f32``: the rows leave in 32-bit
        whatever the table's storage type (a model that keeps its residual stream in 32-bit).
        ``position_name``: a learned table [max_positions, hidden]; the row of a token's position
        (counted from 0 in its request) is added to the token's row, unscaled."""
        self.position_name, self.max_positions = position_name, int(max_positions)
        if position_name and (not stream_f32 or self.max_positions <= 0):
            raise ValueError("learned positions go with a 32-bit stream and a table of at least one position")
        self.positions: torch.Tensor | None = None
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.name = name
        self.scale = None if scale is None else float(scale)
        self.stream_f32 = bool(stream_f32)
        if self.scale is not None and not self.stream_f32:
            raise ValueError("a scaled embedding writes a 32-bit stream (stream_f32=True)")
        self.table: torch.Tensor | None = None

    def tensor_specs(self) -> list[TensorSpec]:
        specs = [TensorSpec(self.name, (self.vocab_size, self.hidden_size), MATRIX)]
        if self.position_name:
            specs.append(TensorSpec(self.position_name, (self.max_positions, self.hidden_size), MATRIX))
        return specs

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        host = tensors[self.name]
        self.table = placer.place(
            ("row_major", self.name), lambda: host.to(dtype=placer.dtype).contiguous().to(placer.device)
        )
        if self.position_name:
            self.positions = placer.place(("row_major", self.position_name), lambda: tensors[self.position_name].to(
                dtype=placer.dtype).contiguous().to(placer.device))

    def forward(self, ctx: StepContext) -> torch.Tensor:
        if self.stream_f32:
            return ops.embed_scaled(ctx.token_ids, self.table, 1.0 if self.scale is None else self.scale, ctx.last_token,
                                    pos_table=self.positions, positions=ctx.positions if self.positions is not None else None)
        return ops.embed_gather(ctx.token_ids, self.table, ctx.last_token)


@EMBEDDINGS.register("bigram_embedding")
class BigramEmbedding(Embedding):
    """``table[token] * scale`` plus a row of a second table chosen by a hash of the token before and the
    token itself, ``(prev * mul_prev + token * mul_cur) mod buckets``; a request's first token takes the
    second table's last row (it has ``buckets + 1``).  The rows leave as a 32-bit stream.  The token before
    a step's first token is kept per request: one integer in the request's slot (``state_need``), written
    by the step that brought it.  ``reader``: set by the model to the first block's entry norm when that
    only rounds the stream; the rows then also leave rounded to the storage type."""

    def __init__(self, vocab_size: int, hidden_size: int, name: str, pairs_name: str, buckets: int, mul_prev: int, mul_cur: int,
                 scale: float = 1.0):
        self.vocab_size, self.hidden_size = vocab_size, hidden_size
        self.name, self.pairs_name = name, pairs_name
        self.buckets, self.mul_prev, self.mul_cur = int(buckets), int(mul_prev), int(mul_cur)
        if self.buckets <= 0:
            raise ValueError("a hashed table needs at least one bucket")
        self.scale = float(scale)
        self.table: torch.Tensor | None = None
        self.pairs: torch.Tensor | None = None
        self.reader = None

    def tensor_specs(self) -> list[TensorSpec]:
        return [TensorSpec(self.name, (self.vocab_size, self.hidden_size), MATRIX),
                TensorSpec(self.pairs_name, (self.buckets + 1, self.hidden_size), MATRIX)]

    def state_need(self) -> StateNeed:
        return StateNeed((1,), torch.int32)

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        def place(name: str) -> torch.Tensor:
            return placer.place(("row_major", name), lambda: tensors[name].to(dtype=placer.dtype).contiguous().to(placer.device))

        self.table, self.pairs = place(self.name), place(self.pairs_name)

    def forward(self, ctx: StepContext):
        if ctx.embedding_state is None:
            raise RuntimeError("a bigram embedding keeps the token before in the request's slot: the step has no such state")
        x, rounded = ops.embed_bigram(ctx.token_ids, ctx.last_token, ctx.positions, ctx.token_req, ctx.q_start, ctx.slots,
                                      ctx.embedding_state.view(-1), self.table, self.pairs, self.scale, self.mul_prev, self.mul_cur,
                                      want_cast=self.reader is not None)
        if self.reader is None:
            return x
        return x, Prepared(None, self.reader, rounded if rounded is not None else x)


@HEADS.register("norm_linear")
class LMHead(Head):
    def __init__(self, vocab_size: int, hidden_size: int, name: str, norm: PartSpec, softcap: float | None = None,
                 scale: float | None = None):
        """``softcap``: the logits leave as softcap * tanh(logits / softcap).  ``scale``: the logits are
        multiplied by it (before a soft cap)."""
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.softcap = float(softcap) if softcap else None
        self.scale = float(scale) if scale is not None and float(scale) != 1.0 else None
        self.norm = NORMS.build(norm)
        self.proj = Linear(hidden_size, [name], [vocab_size])

    def children(self) -> list[Part]:
        return [self.norm]

    def entry_norm(self):
        return self.norm

    def tensor_specs(self) -> list[TensorSpec]:
        return self.norm.tensor_specs() + self.proj.tensor_specs()

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        self.norm.load(tensors, placer)
        self.proj.load(tensors, placer)

    takes_out = True

    def forward(self, x: torch.Tensor, prepared: Prepared | None = None, out: torch.Tensor | None = None) -> torch.Tensor:
        logits = self.proj(Normed(x, self.norm, prepared), out_f32=True, out=out, out_scale=self.scale)
        return ops.softcap_(logits, self.softcap) if self.softcap is not None else logits
