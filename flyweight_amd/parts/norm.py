"""RMS norm: y = x * rsqrt(mean(x^2) + eps) * w, sums in float32; the weight multiplies
directly (native/include/flyweight_v2_qwen_kernels.hpp:425-447 with one_centered = 0)."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import Norm, register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, spec):
        super().__init__(spec)
        self.size = int(spec["size"])
        self.eps = float(spec["eps"])
        self.one_centered = bool(spec.get("one_centered", False))

    def tensors(self) -> Dict[str, TensorDecl]:
        return {self.prefix + "weight": TensorDecl((self.size,), role="vector", init="norm")}

    def bind(self, tensors, dtype, device) -> None:
        super().bind(tensors, dtype, device)
        self.weight = tensors[self.prefix + "weight"]

    def forward(self, x: torch.Tensor, ctx, row_index: Optional[torch.Tensor] = None) -> torch.Tensor:
        return ops.rmsnorm_rows(x, self.weight, self.eps, self.dtype, row_index=row_index,
                                one_centered=self.one_centered)
