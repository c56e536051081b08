"""RMSNorm (tokasaurus/model/llama.py:35-53): statistics in 32-bit, the
normalised value cast back to the storage type before it meets the weight."""

from __future__ import annotations

import torch

from tokasaurus_amd.kernels import ops
from tokasaurus_amd.parts.base import NORMS, NORM_OFFSET, NORM_WEIGHT, Norm, TensorSpec
from tokasaurus_amd.parts.linear import Placer


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    fusable_rms = True  # weight and eps are all a product needs to fold this norm in

    def __init__(self, size: int, eps: float, name: str):
        self.size = size
        self.eps = float(eps)
        self.name = name
        self.weight: torch.Tensor | None = None

    def tensor_specs(self) -> list[TensorSpec]:
        return [TensorSpec(self.name, (self.size,), NORM_WEIGHT)]

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        host = tensors[self.name]
        # a weight stored in 32-bit stays 32-bit; otherwise it takes the engine dtype
        dtype = torch.float32 if host.dtype == torch.float32 else placer.dtype
        self.weight = placer.place(
            ("vector", self.name), lambda: host.to(dtype=dtype).contiguous().to(placer.device)
        )

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.rmsnorm(x, self.weight, self.eps)


@NORMS.register("stream_rmsnorm")
class StreamRMSNorm(Norm):
    """RMSNorm of a residual stream that is kept in 32-bit whatever the storage type:
    ``x / sqrt(mean(x^2) + eps) * w`` computed in 32-bit and rounded once to the storage type
    that the products behind it read.  ``unit_offset``: the checkpoint stores the weight around
    zero and the norm multiplies by ``1 + w``.  The weight is kept in 32-bit.  A block that
    updates the stream may write this norm's rows in the same pass (``ops.residual_norm``)."""

    fusable_rms = False  # the few-row product's folded norm has no offset and reads storage-type rows

    def __init__(self, size: int, eps: float, name: str, unit_offset: bool = False):
        self.size = size
        self.eps = float(eps)
        self.name = name
        self.unit_offset = bool(unit_offset)
        self.weight: torch.Tensor | None = None
        self.out_dtype: torch.dtype | None = None

    def tensor_specs(self) -> list[TensorSpec]:
        return [TensorSpec(self.name, (self.size,), NORM_OFFSET if self.unit_offset else NORM_WEIGHT)]

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        host = tensors[self.name]
        self.weight = placer.place(("vector_f32", self.name), lambda: host.to(dtype=torch.float32).contiguous().to(placer.device))
        self.out_dtype = placer.dtype

    def same_rule(self, other: "Norm | None") -> bool:
        """Whether one pass can write this norm's rows and ``other``'s: the same statistic and offset."""
        return isinstance(other, StreamRMSNorm) and (other.eps, other.unit_offset, other.size) == (self.eps, self.unit_offset, self.size)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.residual_norm(x, weights=(self.weight, None), unit_offset=self.unit_offset, eps=self.eps,
                                 out_dtype=self.out_dtype)[1]


@NORMS.register("stream_cast")
class StreamCast(Norm):
    """No norm at all: the 32-bit stream rounded once to the storage type, for sublayers that read
    the stream itself (blocks that norm a sublayer's output only).  It stands where a norm would, so that
    the pass that updates the stream can write its rows like any other reader's (``plain_rows``)."""

    fusable_rms = False
    plain_rows = True

    def __init__(self):
        self.out_dtype: torch.dtype | None = None

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        self.out_dtype = placer.dtype

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.cast_rows(x, self.out_dtype)
