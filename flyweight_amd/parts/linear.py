"""A matrix product with a stored weight: out = a . W^T (+ bias).

``forward`` returns activations; ``accumulate`` adds the product to the float32 residual
stream in the kernel's epilogue, so the residual sum never leaves float32; ``swiglu`` and
``short_conv`` finish the product with that part's arithmetic. Which kernel runs is chosen
here from the operand types and the number of rows: for up to 16 rows of a bfloat16 model one
fused kernel takes the RMS norm before the product (handed over as a :class:`LazyNorm`) and
the epilogue after it, and the product that adds to the residual stream prepares the norm
that follows; otherwise the norm runs on its own and the skinny, tiled or generic
product follows.
"""

from __future__ import annotations

from typing import Optional, Union

import torch

from ..kernels import ops
from .norm import LazyNorm, Prepared

Input = Union[torch.Tensor, LazyNorm]


class Linear:
    WIDE = 32768

    def __init__(self, weight: torch.Tensor, bias: Optional[torch.Tensor] = None):
        if weight.dim() != 2:
            raise ValueError("a linear weight is [out, in]")
        self.weight = weight.contiguous()
        self.bias = bias
        self.out_features, self.in_features = weight.shape
        # The weight once more in the order in which the kernels of few rows load it (whole contiguous
        # kilobytes per wave: a decode step is bound by how fast the weights stream); the prompt kernels
        # read the row-major one. None where that layout does not apply.
        self.tiled = ops.tile_weights(self.weight)

    # ----- which path ---------------------------------------------------------------------
    def _fused(self, a: Input, features: int, epilogue: int) -> bool:
        if self.weight.dtype != torch.bfloat16 or a.dtype != torch.bfloat16:
            return False
        rows = a.rows if isinstance(a, LazyNorm) else a.shape[0]
        if not 1 <= rows <= ops.DECODE_MAX_ROWS:
            return False
        if isinstance(a, LazyNorm) and (a.rms_parameters() is None or (features >= self.WIDE and a.prepared is None)):
            return False        # very wide outputs (a vocabulary): norming once beats norming in every workgroup
        return ops.gemm_decode_fits(rows, features, self.in_features, epilogue)

    @staticmethod
    def _norm_arguments(a: Input) -> dict:
        if not isinstance(a, LazyNorm):
            return {}
        weight, eps, one_centered = a.rms_parameters()
        if a.prepared is not None:
            return {"squares": a.prepared.squares, "eps": eps}
        return {"norm_weight": weight, "eps": eps, "one_centered": one_centered, "row_index": a.row_index}

    @staticmethod
    def _rows_of(a: Input) -> torch.Tensor:
        if not isinstance(a, LazyNorm):
            return a
        return a.prepared.activations if a.prepared is not None else a.x

    @staticmethod
    def _tensor_of(a: Input) -> torch.Tensor:
        return a.tensor() if isinstance(a, LazyNorm) else a

    # From this many weights on the product that splits K over workgroups also serves a few rows: its
    # workgroups walk K from different chunks on, and a large W in row-major order then streams faster
    # than through the fused decode product (16,384 x 2,048 with SwiGLU at 8 rows: 17.6 against 19.1 us;
    # equal at one row). From operand tiles the fused product streams faster than either (gate|up at 8
    # rows 12.9 against 14.9 us, a vocabulary of 65,536 45.3 against 49.5 us); only the widest outputs
    # go to the split-K product, from nine rows on, where every workgroup's own read of all of a
    # begins to weigh (the vocabulary at 16 rows: 50.4 against 52.2 us).
    LARGE = 1 << 25
    LARGE_MIN_ROWS = 3
    LARGE_TILED = 1 << 26
    LARGE_TILED_MIN_ROWS = 9

    def _medium(self, a: Input) -> bool:
        """17..64 rows of a bfloat16 model, and fewer rows of a large weight: the product that splits
        K over workgroups, which takes prepared activations and prepares the next norm as the fused
        decode product does."""
        if self.weight.dtype != torch.bfloat16 or a.dtype != torch.bfloat16 or self.in_features % 8:
            return False
        rows = a.rows if isinstance(a, LazyNorm) else a.shape[0]
        if self.tiled is None:
            few = self.LARGE_MIN_ROWS <= rows <= ops.DECODE_MAX_ROWS and self.weight.numel() >= self.LARGE
        else:
            few = self.LARGE_TILED_MIN_ROWS <= rows <= ops.DECODE_MAX_ROWS and self.weight.numel() >= self.LARGE_TILED
        if not (few or ops.DECODE_MAX_ROWS < rows <= ops.MEDIUM_MAX_ROWS):
            return False
        return not isinstance(a, LazyNorm) or a.prepared is not None

    @staticmethod
    def _prepared_arguments(a: Input) -> dict:
        if not isinstance(a, LazyNorm):
            return {}
        return {"squares": a.prepared.squares, "eps": a.rms_parameters()[1]}

    # ----- products -----------------------------------------------------------------------
    def forward(self, a: Input, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        out_dtype = out_dtype or a.dtype
        if self._medium(a):
            return ops.gemm_medium(self._rows_of(a), self.weight, ops.EPILOGUE_STORE, bias=self.bias, out_dtype=out_dtype,
                                   w_tiled=self.tiled, **self._prepared_arguments(a))
        if self._fused(a, self.out_features, ops.EPILOGUE_STORE):
            return ops.gemm_decode(self._rows_of(a), self.weight, ops.EPILOGUE_STORE, bias=self.bias, out_dtype=out_dtype,
                                   w_tiled=self.tiled, **self._norm_arguments(a))
        return ops.gemm(self._tensor_of(a), self.weight, self.bias, out_dtype=out_dtype, w_tiled=self.tiled)

    def accumulate(self, a: torch.Tensor, residual: torch.Tensor, then=None) -> Optional[Prepared]:
        """residual += a . W^T. ``then`` names the norm that will read the residual next, if the
        caller knows it and this is the last change before it: the fused kernel then leaves that
        norm's work behind (returned; None when it did not)."""
        parameters = then.rms_parameters() if hasattr(then, "rms_parameters") else None
        if parameters is not None and (parameters[0].shape != (self.out_features,) or then.dtype != torch.bfloat16):
            parameters = None
        if self._medium(a):
            if parameters is not None:
                activations, squares = ops.gemm_medium(a, self.weight, ops.EPILOGUE_ACCUMULATE, bias=self.bias,
                                                       accumulate_into=residual, next_norm_weight=parameters[0],
                                                       next_one_centered=parameters[2], w_tiled=self.tiled)
                return Prepared(then, activations, squares)
            ops.gemm_medium(a, self.weight, ops.EPILOGUE_ACCUMULATE, bias=self.bias, accumulate_into=residual, w_tiled=self.tiled)
            return None
        if self._fused(a, self.out_features, ops.EPILOGUE_ACCUMULATE):
            if parameters is not None:
                activations, squares = ops.gemm_decode(
                    a, self.weight, ops.EPILOGUE_ACCUMULATE, bias=self.bias, accumulate_into=residual,
                    next_norm_weight=parameters[0], next_one_centered=parameters[2], w_tiled=self.tiled)
                return Prepared(then, activations, squares)
            ops.gemm_decode(a, self.weight, ops.EPILOGUE_ACCUMULATE, bias=self.bias, accumulate_into=residual, w_tiled=self.tiled)
            return None
        ops.gemm(a, self.weight, self.bias, accumulate_into=residual, w_tiled=self.tiled)
        return None

    def swiglu(self, a: Input) -> torch.Tensor:
        """The weight holds gate rows then up rows: silu(a . gate^T) * (a . up^T)."""
        if self.bias is None and self._medium(a):
            return ops.gemm_medium(self._rows_of(a), self.weight, ops.EPILOGUE_SWIGLU, w_tiled=self.tiled, **self._prepared_arguments(a))
        if self.bias is None and self._fused(a, self.out_features // 2, ops.EPILOGUE_SWIGLU):
            return ops.gemm_decode(self._rows_of(a), self.weight, ops.EPILOGUE_SWIGLU, out_dtype=torch.bfloat16,
                                   w_tiled=self.tiled, **self._norm_arguments(a))
        return ops.gemm_swiglu(self._tensor_of(a), self.weight, w_tiled=self.tiled)

    def short_conv_decode(self, a: Input, taps: torch.Tensor, conv_bias: Optional[torch.Tensor], state: torch.Tensor,
                          seg_slot: torch.Tensor, out_dtype: torch.dtype) -> Optional[torch.Tensor]:
        """For single-token segments: the weight holds B, C and x rows; returns C * conv(B * x)
        with the state shifted, or None when the fused kernel does not take the shape. (Beyond 16
        rows the product and the convolution run apart: as an epilogue of the split-K product a
        workgroup would have to own B, C and x of its channels, which leaves a third as many tiles
        and a fourfold split of K: 41 us against 15.3 + 4.8 us at 64 rows.)"""
        if not self._fused(a, self.out_features // 3, ops.EPILOGUE_CONV):
            return None
        return ops.gemm_decode(self._rows_of(a), self.weight, ops.EPILOGUE_CONV, bias=self.bias, out_dtype=out_dtype,
                               taps=taps, conv_bias=conv_bias, state=state, seg_slot=seg_slot, w_tiled=self.tiled,
                               **self._norm_arguments(a))
