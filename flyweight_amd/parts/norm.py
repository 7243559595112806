"""RMS norm: y = x * rsqrt(mean(x^2) + eps) * w, sums in float32; the weight multiplies
directly (native/include/flyweight_v2_qwen_kernels.hpp:425-447 with one_centered = 0)."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import Norm, register_norm


class Prepared:
    """What the product that last added to the residual stream left for the norm after it:
    ``activations`` bfloat16 [rows, size] = x * w of that norm and ``squares`` [tiles, 16],
    partial sums of x^2 per row, from which a product's kernel forms the row's 1/rms itself."""

    def __init__(self, norm: Norm, activations: torch.Tensor, squares: torch.Tensor):
        self.norm, self.activations, self.squares = norm, activations, squares


class LazyNorm:
    """A norm that has not run yet: the rows ``x`` (optionally gathered through ``row_index``)
    and the norm to apply. A product that can apply an RMS norm in its own kernel takes it as
    it is (``rms_parameters``, or ``prepared`` when the rows' producer already did most of it);
    anything else calls ``tensor()``, which runs the norm once."""

    def __init__(self, norm: Norm, x: torch.Tensor, ctx, row_index: Optional[torch.Tensor] = None,
                 prepared: Optional[Prepared] = None):
        self.norm, self.x, self.ctx, self.row_index = norm, x, ctx, row_index
        # only what was made for this very norm and these rows counts
        ok = prepared is not None and prepared.norm is norm and row_index is None \
            and prepared.activations.shape == x.shape
        self.prepared = prepared if ok else None
        self._tensor = None

    @property
    def rows(self) -> int:
        return self.row_index.numel() if self.row_index is not None else self.x.shape[0]

    @property
    def dtype(self) -> torch.dtype:
        return self.norm.dtype

    def rms_parameters(self):
        """(weight, eps, one_centered) if the norm is a plain RMS norm, else None."""
        return self.norm.rms_parameters() if hasattr(self.norm, "rms_parameters") else None

    def tensor(self) -> torch.Tensor:
        if self._tensor is None:
            self._tensor = self.norm.forward(self.x, self.ctx, row_index=self.row_index)
        return self._tensor


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

    def rms_parameters(self):
        return self.weight, self.eps, self.one_centered

    def forward(self, x: torch.Tensor, ctx, row_index: Optional[torch.Tensor] = None) -> torch.Tensor:
        return ops.rmsnorm_rows(x, self.weight, self.eps, self.dtype, row_index=row_index,
                                one_centered=self.one_centered)
