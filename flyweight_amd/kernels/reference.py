"""The plain C++ references of the kernels (``csrc/reference``), on numpy arrays in host memory.

They are the oracle that needs no GPU: the tests hold them against the tests' numpy model and
hold the HIP kernels against them. Nothing of the product path imports this module. Every
function takes and returns float32 (int32 for indices); cache pages and states are updated in
place as the kernels update theirs."""

from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import numpy as np

from .build import ensure_reference_built

_lib: Optional[ctypes.CDLL] = None


class ReferenceError_(RuntimeError):
    pass


def library() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(ensure_reference_built())
        _lib.fwr_last_error.restype = ctypes.c_char_p
    return _lib


def _check(status: int) -> None:
    if status != 0:
        raise ReferenceError_(library().fwr_last_error().decode("utf-8", "replace"))


def _f(array) -> np.ndarray:
    return np.ascontiguousarray(array, dtype=np.float32)


def _i(array) -> np.ndarray:
    return np.ascontiguousarray(array, dtype=np.int32)


def _p(array: Optional[np.ndarray]) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if array is None else array.ctypes.data)


def _inplace(array: np.ndarray, name: str) -> np.ndarray:
    if array.dtype != np.float32 or not array.flags["C_CONTIGUOUS"]:
        raise ValueError(f"{name} is updated in place: it must be a contiguous float32 array")
    return array


def embed_rows(table, ids, scale: float = 1.0) -> np.ndarray:
    table, ids = _f(table), _i(ids)
    out = np.empty((ids.size, table.shape[1]), dtype=np.float32)
    _check(library().fwr_embed_rows(_p(table), _p(ids), _p(out), ids.size, table.shape[1], table.shape[0], ctypes.c_float(scale)))
    return out


def rmsnorm_rows(x, weight, eps: float, row_index=None, one_centered: bool = False) -> np.ndarray:
    x, weight = _f(x), _f(weight)
    index = None if row_index is None else _i(row_index)
    rows = x.shape[0] if index is None else index.size
    out = np.empty((rows, x.shape[1]), dtype=np.float32)
    _check(library().fwr_rmsnorm_rows(_p(x), _p(weight), _p(out), _p(index), rows, x.shape[1], ctypes.c_float(eps), int(one_centered)))
    return out


def gemm(a, w, bias=None, accumulate_into: Optional[np.ndarray] = None) -> np.ndarray:
    a, w = _f(a), _f(w)
    bias = None if bias is None else _f(bias)
    out = np.empty((a.shape[0], w.shape[0]), dtype=np.float32) if accumulate_into is None else _inplace(accumulate_into, "the residual")
    _check(library().fwr_gemm(_p(a), _p(w), _p(bias), _p(out), a.shape[0], w.shape[0], a.shape[1], int(accumulate_into is not None)))
    return out


def gemm_swiglu(a, w) -> np.ndarray:
    a, w = _f(a), _f(w)
    out = np.empty((a.shape[0], w.shape[0] // 2), dtype=np.float32)
    _check(library().fwr_gemm_swiglu(_p(a), _p(w), _p(out), a.shape[0], w.shape[0] // 2, a.shape[1]))
    return out


def swiglu(gate_up) -> np.ndarray:
    gate_up = _f(gate_up)
    out = np.empty((gate_up.shape[0], gate_up.shape[1] // 2), dtype=np.float32)
    _check(library().fwr_swiglu(_p(gate_up), _p(out), gate_up.shape[0], gate_up.shape[1] // 2))
    return out


def shortconv(bcx, taps, conv_bias, state: np.ndarray, seg_row0, seg_slot) -> np.ndarray:
    """``state`` [slots, H, L - 1] is read and updated in place."""
    bcx, taps = _f(bcx), _f(taps)
    conv_bias = None if conv_bias is None else _f(conv_bias)
    seg_row0, seg_slot = _i(seg_row0), _i(seg_slot)
    hidden, kernel = taps.shape
    out = np.empty((bcx.shape[0], hidden), dtype=np.float32)
    _check(library().fwr_shortconv(_p(bcx), _p(out), _p(taps), _p(conv_bias), _p(_inplace(state, "the state")), _p(seg_row0),
                                   _p(seg_slot), seg_slot.size, hidden, kernel, state.shape[0]))
    return out


def rope_table(positions, inv_freq) -> Tuple[np.ndarray, np.ndarray]:
    positions, inv_freq = _i(positions), np.ascontiguousarray(inv_freq, dtype=np.float64)
    cos = np.empty((positions.size, inv_freq.size), dtype=np.float32)
    sin = np.empty_like(cos)
    _check(library().fwr_rope_table(_p(positions), _p(inv_freq), _p(cos), _p(sin), positions.size, inv_freq.size))
    return cos, sin


def qk_norm_rope_kv_write(qkv, num_heads: int, num_kv_heads: int, head_dim: int, q_norm_weight, k_norm_weight, eps: float,
                          cos, sin, rotary_dim: int, k_pages: np.ndarray, v_pages: np.ndarray, block_table, row_seg, row_pos,
                          write_kv: bool = True) -> np.ndarray:
    """K pages [pages, nkv, page, hd] and V pages [pages, nkv, hd, page] are written in place."""
    qkv = _f(qkv)
    qw = None if q_norm_weight is None else _f(q_norm_weight)
    kw = None if k_norm_weight is None else _f(k_norm_weight)
    cos = None if cos is None else _f(cos)
    sin = None if sin is None else _f(sin)
    block_table, row_seg, row_pos = _i(block_table), _i(row_seg), _i(row_pos)
    q_out = np.empty((qkv.shape[0], num_heads * head_dim), dtype=np.float32)
    _check(library().fwr_qk_norm_rope_kv_write(
        _p(qkv), _p(q_out), _p(qw), _p(kw), ctypes.c_float(eps), _p(cos), _p(sin), int(rotary_dim), _p(_inplace(k_pages, "K pages")),
        _p(_inplace(v_pages, "V pages")), _p(block_table), block_table.shape[1], _p(row_seg), _p(row_pos), qkv.shape[0], num_heads,
        num_kv_heads, head_dim, k_pages.shape[2], k_pages.shape[0], int(write_kv)))
    return q_out


def attention(q, num_heads: int, num_kv_heads: int, head_dim: int, k_pages, v_pages, block_table, row_seg, row_pos,
              scale: float, window: int = 0) -> np.ndarray:
    q, k_pages, v_pages = _f(q), _f(k_pages), _f(v_pages)
    block_table, row_seg, row_pos = _i(block_table), _i(row_seg), _i(row_pos)
    out = np.empty_like(q)
    _check(library().fwr_attention(_p(q), _p(out), _p(k_pages), _p(v_pages), _p(block_table), block_table.shape[1], _p(row_seg),
                                   _p(row_pos), q.shape[0], num_heads, num_kv_heads, head_dim, ctypes.c_float(scale), int(window),
                                   k_pages.shape[2], k_pages.shape[0]))
    return out


def argmax_rows(logits) -> np.ndarray:
    logits = _f(logits)
    ids = np.empty(logits.shape[0], dtype=np.int32)
    _check(library().fwr_argmax_rows(_p(logits), _p(ids), logits.shape[0], logits.shape[1]))
    return ids


def sample_rows(logits, settings, states) -> Tuple[np.ndarray, np.ndarray]:
    """The next token of every row and the generators' states afterwards (``states`` uint64 [rows]
    is not changed): settings float32 [rows, 4] = temperature, top_k, top_p, min_p."""
    logits = _f(logits)
    settings = np.ascontiguousarray(settings, dtype=np.float32)
    moved_on = np.ascontiguousarray(states, dtype=np.uint64).copy()
    ids = np.empty(logits.shape[0], dtype=np.int32)
    _check(library().fwr_sample_rows(_p(logits), _p(settings), _p(moved_on), _p(ids), logits.shape[0], logits.shape[1]))
    return ids, moved_on


def scale_softcap(x, scale: float = 1.0, cap: float = 0.0) -> np.ndarray:
    x = _f(x).copy()
    _check(library().fwr_scale_softcap(_p(x), ctypes.c_longlong(x.size), ctypes.c_float(scale), ctypes.c_float(cap)))
    return x
