"""SwiGLU feed-forward: f = W_down (silu(W_gate h) * (W_up h)), no biases
(native/src/v2_runtime.cpp:28797-28805; silu_mul native/include/flyweight_v2_qwen_kernels.hpp:1209-1223).
Gate and up are one operand of 2I rows, so h is read once."""

from __future__ import annotations

from typing import Dict

import torch

from ..config.spec import ConfigError
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import FeedForward, register_feed_forward
from .linear import Linear

_DEFAULT_NAMES = {"gate": "gate_proj", "up": "up_proj", "down": "down_proj"}


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    graph_safe = True
    accepts_lazy_norm = True

    def __init__(self, spec):
        super().__init__(spec)
        self.hidden = int(spec["hidden_size"])
        self.intermediate = int(spec["intermediate_size"])
        self.names = {**_DEFAULT_NAMES, **dict(spec.get("names", {}))}

    def _name(self, which: str) -> str:
        return f"{self.prefix}{self.names[which]}.weight"

    def tensors(self) -> Dict[str, TensorDecl]:
        return {
            self._name("gate"): TensorDecl((self.intermediate, self.hidden)),
            self._name("up"): TensorDecl((self.intermediate, self.hidden)),
            self._name("down"): TensorDecl((self.hidden, self.intermediate)),
        }

    def bind(self, tensors, dtype, device) -> None:
        super().bind(tensors, dtype, device)
        gate, up = tensors[self._name("gate")], tensors[self._name("up")]
        if gate.dtype != up.dtype:
            raise ConfigError(f"{self.prefix}: gate and up projections are stored in different precisions")
        self.gate_up = Linear(torch.cat([gate, up], dim=0))
        self.down = Linear(tensors[self._name("down")])

    def forward(self, h, residual, ctx):
        # the activation is formed from float32 sums and rounded once
        return self.down.accumulate(self.gate_up.swiglu(h), residual, then=getattr(ctx, "upcoming_norm", None))
