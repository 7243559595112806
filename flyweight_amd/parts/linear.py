"""A matrix product with a stored weight: out = a . W^T (+ bias).

``forward`` returns activations; ``accumulate`` adds the product to the float32 residual
stream in the kernel's epilogue, so the residual sum never leaves float32. Which kernel
runs is chosen here from the operand types and the number of rows.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops


class Linear:
    def __init__(self, weight: torch.Tensor, bias: Optional[torch.Tensor] = None):
        if weight.dim() != 2:
            raise ValueError("a linear weight is [out, in]")
        self.weight = weight.contiguous()
        self.bias = bias
        self.out_features, self.in_features = weight.shape

    def forward(self, a: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        return ops.gemm(a, self.weight, self.bias, out_dtype=out_dtype or a.dtype)

    def accumulate(self, a: torch.Tensor, residual: torch.Tensor) -> None:
        ops.gemm(a, self.weight, self.bias, accumulate_into=residual)
