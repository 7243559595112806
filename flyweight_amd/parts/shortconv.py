"""Gated short convolution (LFM2's conv mixer).

(B | C | x) = in_proj(h); bx = B * x; y = causal depthwise FIR of width L over bx along the
sequence (tap L-1 on the current token); out = out_proj(C * y). No activation. The request's
state is the last L-1 values of bx per channel, zero at the start
(native/src/v2_runtime.cpp:28269-28283; kernels native/include/flyweight_v2_native_kernels.hpp:1295-1345).
With ``bias`` each of the three linear maps carries one (in_proj after the product, conv after
the taps' sum, out_proj after the product); the reference loads none.
"""

from __future__ import annotations

from typing import Dict

import torch

from ..cache.needs import FixedState
from ..config.spec import ConfigError
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import Mixer, register_mixer
from .linear import Linear


@register_mixer("short_conv")
class ShortConv(Mixer):
    graph_safe = True
    accepts_lazy_norm = True

    def __init__(self, spec):
        super().__init__(spec)
        self.hidden = int(spec["hidden_size"])
        self.kernel_size = int(spec["kernel_size"])
        self.bias = bool(spec.get("bias", False))
        if not 2 <= self.kernel_size <= 16:
            raise ConfigError(f"short conv kernel size {self.kernel_size} outside 2..16")

    def cache_need(self):
        return FixedState((self.hidden, self.kernel_size - 1), torch.float32)

    def tensors(self) -> Dict[str, TensorDecl]:
        p, H, L = self.prefix, self.hidden, self.kernel_size
        declared = {
            p + "in_proj.weight": TensorDecl((3 * H, H)),
            p + "conv.weight": TensorDecl((H, 1, L), "vector", "conv"),      # depthwise: [channels, 1, taps]
            p + "out_proj.weight": TensorDecl((H, H)),
        }
        if self.bias:
            declared[p + "in_proj.bias"] = TensorDecl((3 * H,), "vector", "bias")
            declared[p + "conv.bias"] = TensorDecl((H,), "vector", "bias")
            declared[p + "out_proj.bias"] = TensorDecl((H,), "vector", "bias")
        return declared

    def bind(self, tensors, dtype, device) -> None:
        super().bind(tensors, dtype, device)
        p = self.prefix
        self.in_proj = Linear(tensors[p + "in_proj.weight"], tensors.get(p + "in_proj.bias") if self.bias else None)
        self.out_proj = Linear(tensors[p + "out_proj.weight"], tensors.get(p + "out_proj.bias") if self.bias else None)
        self.taps = tensors[p + "conv.weight"].reshape(self.hidden, self.kernel_size).contiguous()
        self.conv_bias = tensors[p + "conv.bias"] if self.bias else None

    def forward(self, h, residual, ctx, cache):
        if ctx.all_decode:      # single-token segments: norm, in_proj, convolution and state shift in one kernel
            gated = self.in_proj.short_conv_decode(h, self.taps, self.conv_bias, cache.state, ctx.seg_slot, self.dtype)
            if gated is not None:
                return self.out_proj.accumulate(gated, residual, then=getattr(ctx, "upcoming_norm", None))
        bcx = self.in_proj.forward(h, out_dtype=torch.float32)  # B * x and the taps' sum stay in float32
        gated = ops.shortconv(bcx, self.taps, self.conv_bias, cache.state, ctx.row_seg, ctx.seg_row0, ctx.seg_slot,
                              ctx.num_segments, out_dtype=self.dtype)
        return self.out_proj.accumulate(gated, residual, then=getattr(ctx, "upcoming_norm", None))
