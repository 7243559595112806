"""Rotary position encoding, half-split pairing: channel i of a head pairs with channel
i + rotary_dim/2, angle = position * theta^(-2i/rotary_dim); channels past ``rotary_dim``
pass through (native/include/flyweight_v2_native_kernels.hpp:993-1050). The inverse
frequencies are formed in float64 on the host; the per-step cos/sin tables are float32.
``rotary_dim = 0`` (or kind ``none``) means no position encoding at all."""

from __future__ import annotations

import torch

from ..config.spec import ConfigError
from ..kernels import ops
from .base import PositionEncoding, register_position_encoding


@register_position_encoding("rotary_neox")
class RotaryNeox(PositionEncoding):
    graph_safe = True

    def __init__(self, spec):
        super().__init__(spec)
        self.theta = float(spec["theta"])
        self.head_dim = int(spec["head_dim"])
        self.rotary_dim = int(spec.get("rotary_dim", self.head_dim))
        if self.rotary_dim % 2 or not 0 <= self.rotary_dim <= self.head_dim:
            raise ConfigError(f"rotary_dim {self.rotary_dim} must be even and at most head_dim {self.head_dim}")
        self._inv_freq = None

    def bind(self, tensors, dtype, device) -> None:
        super().bind(tensors, dtype, device)
        half = self.rotary_dim // 2
        exponents = torch.arange(half, dtype=torch.float64) * 2.0 / max(self.rotary_dim, 1)
        self._inv_freq = (self.theta ** (-exponents)).to(device)

    def tables(self, ctx):
        if self.rotary_dim == 0:
            return None, None
        return ops.rope_table(ctx.encoding_pos, self._inv_freq)


@register_position_encoding("none")
class NoPosition(PositionEncoding):
    graph_safe = True

    rotary_dim = 0

    def tables(self, ctx):
        return None, None
