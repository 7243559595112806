"""Python face of the gfx950 kernel library: one function per kernel entry point.

Each function checks devices, dtypes and shapes on the host, then calls the flat C ABI
through ctypes on the current HIP stream. There is no CPU fallback: without the library
or without a GPU these functions raise.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import build as _build

F32, BF16 = 0, 1
PAGE_SIZE = 64          # tokens per cache page: the width of a wavefront
MAX_HEAD_DIM = 256

_lib = None


class KernelError(RuntimeError):
    pass


def library() -> ctypes.CDLL:
    """Loads (building first if nothing is built) the kernel library."""
    global _lib
    if _lib is None:
        path = _build.ensure_built()
        lib = ctypes.CDLL(path)
        lib.fw_last_error.restype = ctypes.c_char_p
        lib.fw_abi_version.restype = ctypes.c_int
        if lib.fw_abi_version() != 1:
            raise KernelError(f"{path}: kernel library ABI {lib.fw_abi_version()} != 1; rebuild it")
        _lib = lib
    return _lib


def library_path() -> str:
    library()
    return _lib._name


def _check(status: int) -> None:
    if status != 0:
        raise KernelError(library().fw_last_error().decode("utf-8", "replace"))


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    raise KernelError(f"kernels take float32 or bfloat16, not {dtype}")


def _dev(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise KernelError("kernels run on the GPU only; got a CPU tensor")
        if not t.is_contiguous():
            raise KernelError("kernels need contiguous tensors")


def _p(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _stream() -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _want(t: torch.Tensor, dtype: torch.dtype, name: str) -> None:
    if t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, found {t.dtype}")


# ---------------------------------------------------------------------------------------
def embed_rows(table: torch.Tensor, ids: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    _dev(table, ids, out)
    _want(ids, torch.int32, "ids")
    vocab, hidden = table.shape
    rows = ids.numel()
    if out is None:
        out = torch.empty((rows, hidden), dtype=torch.float32, device=table.device)
    _want(out, torch.float32, "out")
    if out.shape != (rows, hidden):
        raise KernelError(f"embed_rows: out is {tuple(out.shape)}, expected {(rows, hidden)}")
    _check(library().fw_embed_rows(_p(table), _code(table.dtype), _p(ids), _p(out), rows, hidden, vocab, _stream()))
    return out


def rmsnorm_rows(x: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
                 row_index: Optional[torch.Tensor] = None, one_centered: bool = False,
                 out: Optional[torch.Tensor] = None) -> torch.Tensor:
    _dev(x, weight, row_index, out)
    _want(x, torch.float32, "x")
    _want(weight, torch.float32, "weight")
    hidden = x.shape[-1]
    if weight.shape != (hidden,):
        raise KernelError(f"rmsnorm: weight is {tuple(weight.shape)}, row width is {hidden}")
    rows = x.numel() // hidden if row_index is None else row_index.numel()
    if row_index is not None:
        _want(row_index, torch.int32, "row_index")
    if out is None:
        out = torch.empty((rows, hidden), dtype=out_dtype, device=x.device)
    if out.shape != (rows, hidden) or out.dtype != out_dtype:
        raise KernelError("rmsnorm: out has the wrong shape or dtype")
    _check(library().fw_rmsnorm_rows(_p(x), _p(weight), _p(out), _code(out_dtype), _p(row_index), rows, hidden,
                                     ctypes.c_float(eps), int(one_centered), _stream()))
    return out


def gemm_generic(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
                 out_dtype: Optional[torch.dtype] = None, accumulate_into: Optional[torch.Tensor] = None,
                 out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """a [M, K] . w [N, K]^T (+ bias). With ``accumulate_into`` (float32 [M, N]) the
    product is added to it in place: the residual sum in float32."""
    _dev(a, w, bias, accumulate_into, out)
    M, K = a.shape
    N, K2 = w.shape
    if K != K2:
        raise KernelError(f"gemm: a is {tuple(a.shape)} but w is {tuple(w.shape)}")
    if bias is not None:
        _want(bias, torch.float32, "bias")
        if bias.shape != (N,):
            raise KernelError(f"gemm: bias is {tuple(bias.shape)}, expected {(N,)}")
    if accumulate_into is not None:
        _want(accumulate_into, torch.float32, "accumulate_into")
        if accumulate_into.shape != (M, N):
            raise KernelError(f"gemm: destination is {tuple(accumulate_into.shape)}, expected {(M, N)}")
        target, mode, code = accumulate_into, 1, F32
    else:
        out_dtype = out_dtype or a.dtype
        if out is None:
            out = torch.empty((M, N), dtype=out_dtype, device=a.device)
        if out.shape != (M, N) or out.dtype != out_dtype:
            raise KernelError("gemm: out has the wrong shape or dtype")
        target, mode, code = out, 0, _code(out_dtype)
    _check(library().fw_gemm_generic(_p(a), _code(a.dtype), _p(w), _code(w.dtype), _p(bias), _p(target), code, mode,
                                     M, N, K, _stream()))
    return target


def swiglu(gate_up: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
           out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """silu(gate) * up of [rows, gate | up]; the input may be float32 beside a bfloat16 output."""
    _dev(gate_up, out)
    out_dtype = out_dtype or gate_up.dtype
    rows, width = gate_up.shape
    if width % 2:
        raise KernelError("swiglu: the input holds gate and up halves; its width must be even")
    inter = width // 2
    if out is None:
        out = torch.empty((rows, inter), dtype=out_dtype, device=gate_up.device)
    if out.shape != (rows, inter) or out.dtype != out_dtype:
        raise KernelError("swiglu: out has the wrong shape or dtype")
    _check(library().fw_swiglu(_p(gate_up), _code(gate_up.dtype), _p(out), _code(out_dtype), rows, inter, _stream()))
    return out


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor):
    """cos and sin [rows, half] (float32) of position * inv_freq (float64)."""
    _dev(positions, inv_freq)
    _want(positions, torch.int32, "positions")
    _want(inv_freq, torch.float64, "inv_freq")
    rows, half = positions.numel(), inv_freq.numel()
    cos = torch.empty((rows, half), dtype=torch.float32, device=positions.device)
    sin = torch.empty_like(cos)
    _check(library().fw_rope_table(_p(positions), _p(inv_freq), _p(cos), _p(sin), rows, half, _stream()))
    return cos, sin


def shortconv(bcx: torch.Tensor, taps: torch.Tensor, conv_bias: Optional[torch.Tensor], state: torch.Tensor,
              row_seg: torch.Tensor, seg_row0: torch.Tensor, seg_slot: torch.Tensor, segments: int,
              out_dtype: Optional[torch.dtype] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """state [slots, H, L-1] is read and updated in place. ``bcx`` may be float32 beside a
    bfloat16 output."""
    _dev(bcx, taps, conv_bias, state, row_seg, seg_row0, seg_slot, out)
    out_dtype = out_dtype or bcx.dtype
    rows, width = bcx.shape
    hidden, kernel = taps.shape
    if width != 3 * hidden:
        raise KernelError(f"shortconv: input width {width} is not 3 x {hidden}")
    _want(taps, torch.float32, "taps")
    _want(state, torch.float32, "state")
    if state.dim() != 3 or state.shape[1:] != (hidden, kernel - 1):
        raise KernelError(f"shortconv: state is {tuple(state.shape)}, expected [slots, {hidden}, {kernel - 1}]")
    if conv_bias is not None:
        _want(conv_bias, torch.float32, "conv_bias")
        if conv_bias.shape != (hidden,):
            raise KernelError("shortconv: bias has the wrong shape")
    for name, t, n in (("row_seg", row_seg, rows), ("seg_row0", seg_row0, segments + 1), ("seg_slot", seg_slot, segments)):
        _want(t, torch.int32, name)
        if t.numel() < n:
            raise KernelError(f"shortconv: {name} holds {t.numel()} entries, needs {n}")
    if out is None:
        out = torch.empty((rows, hidden), dtype=out_dtype, device=bcx.device)
    if out.shape != (rows, hidden) or out.dtype != out_dtype:
        raise KernelError("shortconv: out has the wrong shape or dtype")
    _check(library().fw_shortconv(_p(bcx), _code(bcx.dtype), _p(out), _code(out_dtype), _p(taps), _p(conv_bias), _p(state), _p(row_seg),
                                  _p(seg_row0), _p(seg_slot), rows, segments, hidden, kernel, state.shape[0], _stream()))
    return out


def _check_pages(k_pages: torch.Tensor, v_pages: torch.Tensor, kv_heads: int, head_dim: int, dtype: torch.dtype):
    pages = k_pages.shape[0]
    if k_pages.shape != (pages, kv_heads, PAGE_SIZE, head_dim):
        raise KernelError(f"K pages are {tuple(k_pages.shape)}, expected [pages, {kv_heads}, {PAGE_SIZE}, {head_dim}]")
    if v_pages.shape != (pages, kv_heads, head_dim, PAGE_SIZE):
        raise KernelError(f"V pages are {tuple(v_pages.shape)}, expected [pages, {kv_heads}, {head_dim}, {PAGE_SIZE}]")
    if k_pages.dtype != dtype or v_pages.dtype != dtype:
        raise KernelError(f"cache pages are {k_pages.dtype}/{v_pages.dtype} but activations are {dtype}")
    return pages


def qk_norm_rope_kv_write(qkv: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
                          q_norm_weight: Optional[torch.Tensor], k_norm_weight: Optional[torch.Tensor], eps: float,
                          cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], rotary_dim: int,
                          k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                          row_seg: torch.Tensor, row_pos: torch.Tensor, write_kv: bool = True) -> torch.Tensor:
    """The output and the cache take the pages' dtype; ``qkv`` may be float32 beside bfloat16 pages."""
    _dev(qkv, q_norm_weight, k_norm_weight, cos, sin, k_pages, v_pages, block_table, row_seg, row_pos)
    rows, width = qkv.shape
    if width != (num_heads + 2 * num_kv_heads) * head_dim:
        raise KernelError(f"qk_norm_rope: qkv width {width} != ({num_heads} + 2 x {num_kv_heads}) x {head_dim}")
    pages = _check_pages(k_pages, v_pages, num_kv_heads, head_dim, k_pages.dtype)
    for w in (q_norm_weight, k_norm_weight):
        if w is not None:
            _want(w, torch.float32, "norm weight")
            if w.shape != (head_dim,):
                raise KernelError("qk_norm_rope: a head norm weight must be [head_dim]")
    if rotary_dim:
        for t in (cos, sin):
            _want(t, torch.float32, "rotation table")
            if t.shape != (rows, rotary_dim // 2):
                raise KernelError(f"qk_norm_rope: rotation table is {tuple(t.shape)}, expected {(rows, rotary_dim // 2)}")
    _want(block_table, torch.int32, "block_table")
    _want(row_seg, torch.int32, "row_seg")
    _want(row_pos, torch.int32, "row_pos")
    if block_table.dim() != 2 or row_seg.numel() < rows or row_pos.numel() < rows:
        raise KernelError("qk_norm_rope: batch index arrays are too short")
    q_out = torch.empty((rows, num_heads * head_dim), dtype=k_pages.dtype, device=qkv.device)
    _check(library().fw_qk_norm_rope_kv_write(
        _p(qkv), _code(qkv.dtype), _p(q_out), _code(k_pages.dtype), _p(q_norm_weight), _p(k_norm_weight), ctypes.c_float(eps), _p(cos), _p(sin),
        rotary_dim, _p(k_pages), _p(v_pages), _p(block_table), block_table.shape[1], _p(row_seg), _p(row_pos), rows,
        num_heads, num_kv_heads, head_dim, PAGE_SIZE, pages, int(write_kv), _stream()))
    return q_out


def attention_generic(q: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int, k_pages: torch.Tensor,
                      v_pages: torch.Tensor, block_table: torch.Tensor, row_seg: torch.Tensor, row_pos: torch.Tensor,
                      scale: float, window: int = 0) -> torch.Tensor:
    _dev(q, k_pages, v_pages, block_table, row_seg, row_pos)
    rows = q.shape[0]
    if q.shape != (rows, num_heads * head_dim):
        raise KernelError(f"attention: q is {tuple(q.shape)}, expected {(rows, num_heads * head_dim)}")
    pages = _check_pages(k_pages, v_pages, num_kv_heads, head_dim, q.dtype)
    _want(block_table, torch.int32, "block_table")
    _want(row_seg, torch.int32, "row_seg")
    _want(row_pos, torch.int32, "row_pos")
    if block_table.dim() != 2 or row_seg.numel() < rows or row_pos.numel() < rows:
        raise KernelError("attention: batch index arrays are too short")
    out = torch.empty_like(q)
    _check(library().fw_attention_generic(
        _p(q), _p(out), _code(q.dtype), _p(k_pages), _p(v_pages), _p(block_table), block_table.shape[1], _p(row_seg),
        _p(row_pos), rows, num_heads, num_kv_heads, head_dim, ctypes.c_float(scale), int(window), PAGE_SIZE, pages,
        _stream()))
    return out


def argmax_rows(logits: torch.Tensor) -> torch.Tensor:
    _dev(logits)
    _want(logits, torch.float32, "logits")
    rows, vocab = logits.shape
    ids = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    _check(library().fw_argmax_rows(_p(logits), _p(ids), rows, vocab, _stream()))
    return ids


def topk_rows(logits: torch.Tensor, k: int):
    _dev(logits)
    _want(logits, torch.float32, "logits")
    rows, vocab = logits.shape
    values = torch.empty((rows, k), dtype=torch.float32, device=logits.device)
    ids = torch.empty((rows, k), dtype=torch.int32, device=logits.device)
    _check(library().fw_topk_rows(_p(logits), _p(values), _p(ids), rows, vocab, k, _stream()))
    return values, ids


def fill_zero(t: torch.Tensor) -> None:
    _dev(t)
    _check(library().fw_fill_zero(_p(t), ctypes.c_longlong(t.numel() * t.element_size()), _stream()))


# ---- dispatch: which kernel serves a call ------------------------------------------------
def gemm(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
         out_dtype: Optional[torch.dtype] = None, accumulate_into: Optional[torch.Tensor] = None) -> torch.Tensor:
    return gemm_generic(a, w, bias, out_dtype=out_dtype, accumulate_into=accumulate_into)


def attention(q: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int, k_pages: torch.Tensor,
              v_pages: torch.Tensor, block_table: torch.Tensor, ctx, scale: float, window: int = 0) -> torch.Tensor:
    return attention_generic(q, num_heads, num_kv_heads, head_dim, k_pages, v_pages, block_table, ctx.row_seg,
                             ctx.row_pos, scale, window)
