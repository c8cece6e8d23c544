"""RMSNorm (tokasaurus/model/llama.py:35-53): statistics in 32-bit, the
normalised value cast back to the storage type before it meets the weight."""

from __future__ import annotations

import torch

from tokasaurus_amd.kernels import ops
from tokasaurus_amd.parts.base import NORMS, NORM_WEIGHT, Norm, TensorSpec
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
