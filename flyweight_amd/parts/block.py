"""The arrangement of parts in a layer.

``pre_norm_residual``: x <- x + mixer(norm1(x)); x <- x + ffn(norm2(x)), the residual
stream x in float32 (native/src/v2_runtime.cpp:28077,28282,28774,29133-29136). Another
arrangement (post-norm, parallel mixer and feed-forward) is another class registered here.
"""

from __future__ import annotations

from .base import Block, build_part, register_block
from .norm import LazyNorm


@register_block("pre_norm_residual")
class PreNormResidualBlock(Block):
    def __init__(self, spec):
        self.spec = spec
        self.mixer_norm = build_part("norm", spec.mixer_norm)
        self.mixer = build_part("mixer", spec.mixer)
        self.ffn_norm = build_part("norm", spec.ffn_norm)
        self.ffn = build_part("ffn", spec.ffn)

    def parts(self):
        return (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn)

    def first_norm(self):
        return self.mixer_norm

    def cache_need(self):
        return self.mixer.cache_need()

    @property
    def graph_safe(self) -> bool:
        position = getattr(self.mixer, "position", None)
        return all(part.graph_safe for part in self.parts()) and (position is None or position.graph_safe)

    def forward(self, x, ctx, cache, prepared=None, norm_after=None):
        """``x`` [rows, hidden] float32 is updated in place."""
        # A part that can take the norm into its own first kernel gets it unevaluated. A part is
        # told which norm reads the residual after it (ctx.upcoming_norm) and may return what its
        # last product prepared for that norm; a part that returns nothing costs a plain norm.
        h = LazyNorm(self.mixer_norm, x, ctx, prepared=prepared)
        ctx.upcoming_norm = self.ffn_norm
        prepared = self.mixer.forward(h if getattr(self.mixer, "accepts_lazy_norm", False) else h.tensor(), x, ctx, cache)
        h = LazyNorm(self.ffn_norm, x, ctx, prepared=prepared)
        ctx.upcoming_norm = norm_after
        prepared = self.ffn.forward(h if getattr(self.ffn, "accepts_lazy_norm", False) else h.tensor(), x, ctx)
        ctx.upcoming_norm = None
        return prepared
