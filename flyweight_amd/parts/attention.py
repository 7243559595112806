"""Grouped-query attention over the paged cache.

q = W_q h, k = W_k h, v = W_v h; optional per-head RMS norm of q and k (one weight of
head_dim shared by all heads); position encoding on q and k; k and v appended to the
cache; scores q.k / sqrt(head_dim) over the cached keys the row may see (causal, optionally
only the last ``window``), softmax in float32, weighted sum of values; out = W_o o.
Query head i reads kv head i // (num_heads / num_kv_heads). Formulas as the reference's
LFM2 attention branch computes them (native/src/v2_runtime.cpp:28429-28478).
"""

from __future__ import annotations

from typing import Dict

import numpy as np
import torch

from ..cache.needs import PagedKV
from ..config.spec import ConfigError
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import Mixer, build_part, register_mixer
from .linear import Linear

_DEFAULT_NAMES = {"q": "q_proj", "k": "k_proj", "v": "v_proj", "o": "o_proj", "q_norm": "q_norm", "k_norm": "k_norm"}


@register_mixer("gqa_attention")
class GQAttention(Mixer):
    graph_safe = True
    accepts_lazy_norm = True
    # Up to this many rows a decode step forms queries and keys inside the attention kernel (at 8 rows
    # 18.9 us against 15.4 + 4.9 us in two kernels); with many rows the attention is bound by reading
    # the cache and the work in front of it only delays every workgroup (64 rows: 74.1 against 65.9 + 7.2 us).
    FUSED_DECODE_ROWS = 16

    def __init__(self, spec):
        super().__init__(spec)
        self.hidden = int(spec["hidden_size"])
        self.num_heads = int(spec["num_heads"])
        self.num_kv_heads = int(spec["num_kv_heads"])
        self.head_dim = int(spec["head_dim"])
        self.qk_norm = bool(spec.get("qk_norm", False))
        self.qk_norm_eps = float(spec.get("qk_norm_eps", 1e-6)) if self.qk_norm else 1.0
        self.window = spec.get("window")
        self.scale = float(spec.get("softmax_scale", self.head_dim ** -0.5))
        self.bias = bool(spec.get("bias", False))
        self.names = {**_DEFAULT_NAMES, **dict(spec.get("names", {}))}
        self.position = build_part("position", spec["position"])
        if self.num_heads % self.num_kv_heads:
            raise ConfigError(f"{self.num_heads} heads are not a multiple of {self.num_kv_heads} kv heads")
        if self.head_dim > ops.MAX_HEAD_DIM:
            raise ConfigError(f"head_dim {self.head_dim} exceeds the kernels' limit of {ops.MAX_HEAD_DIM}")
        if self.window is not None and int(self.window) <= 0:
            raise ConfigError("an attention window must be positive (or None for all keys)")

    def cache_need(self):
        return PagedKV(self.num_kv_heads, self.head_dim, None if self.window is None else int(self.window))

    def _name(self, which: str, leaf: str = "weight") -> str:
        return f"{self.prefix}{self.names[which]}.{leaf}"

    def tensors(self) -> Dict[str, TensorDecl]:
        q_width, kv_width = self.num_heads * self.head_dim, self.num_kv_heads * self.head_dim
        declared = {
            self._name("q"): TensorDecl((q_width, self.hidden)),
            self._name("k"): TensorDecl((kv_width, self.hidden)),
            self._name("v"): TensorDecl((kv_width, self.hidden)),
            self._name("o"): TensorDecl((self.hidden, q_width)),
        }
        if self.bias:
            declared[self._name("q", "bias")] = TensorDecl((q_width,), "vector", "bias")
            declared[self._name("k", "bias")] = TensorDecl((kv_width,), "vector", "bias")
            declared[self._name("v", "bias")] = TensorDecl((kv_width,), "vector", "bias")
            declared[self._name("o", "bias")] = TensorDecl((self.hidden,), "vector", "bias")
        if self.qk_norm:
            declared[self._name("q_norm")] = TensorDecl((self.head_dim,), "vector", "norm")
            declared[self._name("k_norm")] = TensorDecl((self.head_dim,), "vector", "norm")
        return declared

    def bind(self, tensors, dtype, device) -> None:
        super().bind(tensors, dtype, device)
        self.position.bind(tensors, dtype, device)
        q, k, v = (tensors[self._name(n)] for n in ("q", "k", "v"))
        if not (q.dtype == k.dtype == v.dtype):
            raise ConfigError(f"{self.prefix}: q, k and v projections are stored in different precisions")
        # one operand for the three projections: rows are q heads, then k heads, then v heads
        bias = torch.cat([tensors[self._name(n, "bias")] for n in ("q", "k", "v")]) if self.bias else None
        self.qkv = Linear(torch.cat([q, k, v], dim=0), bias)
        self.out = Linear(tensors[self._name("o")], tensors[self._name("o", "bias")] if self.bias else None)
        self.q_norm_weight = tensors[self._name("q_norm")] if self.qk_norm else None
        self.k_norm_weight = tensors[self._name("k_norm")] if self.qk_norm else None

    # The kernels on the matrix cores need index arrays of this part's own. The prompt kernel works
    # on tiles of up to 64 rows of one segment: which tiles there are, and in which order workgroups
    # take them. The split-key decode kernel shares a step's work out over the chip by the number of
    # runs of keys (four pages each) that all the rows it serves see together: a long row among
    # short ones gets more workgroups, and a recorded step adapts as its requests grow.
    RUN_OF_KEYS = ops.DECODE_SPLIT_PAGES * ops.PAGE_SIZE

    def step_arrays_key(self):
        fast = getattr(self, "dtype", None) == torch.bfloat16 and ops.attention_is_tiled(self.head_dim)
        return ("query_tiles", ops.QUERY_TILE, self.RUN_OF_KEYS) if fast else None

    def _decode_work(self, batch) -> int:
        single = batch.num_rows if batch.all_decode else batch.decode_prefix    # the rows that go to the decode kernel
        positions = np.asarray(batch.host_row_pos[:single], dtype=np.int64)
        return int(np.sum((positions + self.RUN_OF_KEYS) // self.RUN_OF_KEYS))

    def step_arrays(self, batch):
        seg_row0 = batch.host_seg_row0
        tile_seg, tile_row0 = ops.query_tiles(seg_row0)
        # Workgroups start in the order of the tiles: those that see the most keys go first, the short
        # ones fill in behind. The tiles of the leading single rows stay in front (they go to the
        # decode kernel and their tiles are skipped).
        if len(tile_seg) - batch.decode_prefix > 1 and not batch.all_decode:
            tile_seg, tile_row0 = np.asarray(tile_seg, dtype=np.int32), np.asarray(tile_row0, dtype=np.int32)
            tile_end = np.minimum(tile_row0 + ops.QUERY_TILE, np.asarray(seg_row0, dtype=np.int32)[tile_seg + 1])
            keys_seen = batch.host_row_pos[tile_end - 1].astype(np.int64)
            keys_seen[:batch.decode_prefix] = np.iinfo(np.int64).max
            order = np.argsort(-keys_seen, kind="stable")
            tile_seg, tile_row0 = tile_seg[order], tile_row0[order]
        return {"tile_seg": np.asarray(tile_seg, dtype=np.int32), "tile_row0": np.asarray(tile_row0, dtype=np.int32),
                "decode_work": np.asarray([self._decode_work(batch)], dtype=np.int32)}

    def refresh_step_arrays(self, batch, arrays) -> None:
        arrays["decode_work"][0] = self._decode_work(batch)     # the tiles of single rows never change

    def forward(self, h, residual, ctx, cache):
        qkv = self.qkv.forward(h, out_dtype=torch.float32)      # normed, rotated and rounded once, below
        cos, sin = ctx.position_tables(self.position)
        own = ctx.step_arrays(self) if self.step_arrays_key() is not None else {}
        if ctx.all_decode and ctx.num_rows <= self.FUSED_DECODE_ROWS and qkv.dtype == torch.float32 and self.step_arrays_key() is not None:
            # a few single-token segments on the matrix cores: norm, rotation, cache write and attention in one kernel
            attended = ops.attention_decode_fused(
                qkv, self.num_heads, self.num_kv_heads, self.head_dim, self.q_norm_weight, self.k_norm_weight, self.qk_norm_eps,
                cos, sin, self.position.rotary_dim, cache.k_pages, cache.v_pages, cache.block_table, ctx.row_seg, ctx.row_pos,
                self.scale, ctx.max_context, int(self.window or 0), write_kv=cache.writes,
                decode_work=own.get("decode_work"))
            return self.out.accumulate(attended, residual, then=getattr(ctx, "upcoming_norm", None))
        q = ops.qk_norm_rope_kv_write(
            qkv, self.num_heads, self.num_kv_heads, self.head_dim, self.q_norm_weight, self.k_norm_weight,
            self.qk_norm_eps, cos, sin, self.position.rotary_dim, cache.k_pages, cache.v_pages, cache.block_table,
            ctx.row_seg, ctx.row_pos, write_kv=cache.writes)
        attended = ops.attention(q, self.num_heads, self.num_kv_heads, self.head_dim, cache.k_pages, cache.v_pages,
                                 cache.block_table, ctx, self.scale, int(self.window or 0),
                                 tile_seg=own.get("tile_seg"), tile_row0=own.get("tile_row0"), decode_work=own.get("decode_work"))
        return self.out.accumulate(attended, residual, then=getattr(ctx, "upcoming_norm", None))
