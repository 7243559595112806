"""Python face of the gfx950 kernel library: one function per kernel entry point.

Each function checks devices, dtypes and shapes on the host, then calls the flat C ABI
through ctypes on the current HIP stream. There is no CPU fallback: without the library
or without a GPU these functions raise.
"""

from __future__ import annotations

import ctypes
import os
import time
from typing import Dict, Optional

import torch

from . import build as _build

F32, BF16 = 0, 1
PAGE_SIZE = 64          # tokens per cache page: the width of a wavefront
MAX_HEAD_DIM = 256
ABI_VERSION = 9

_lib = None


class KernelError(RuntimeError):
    pass


class _ProfiledLibrary:
    """The kernel library with every call bracketed by two events on the current stream.
    Nothing is waited for at a launch (a host that waits lets the GPU's clock drop, which would
    rescale every figure): the events are read when the report is asked for, as the reference's
    per-kernel profile does (native/src/v2_runtime.cpp:27590-27728)."""
    CAPACITY = 1 << 16

    def __init__(self, lib):
        self._library = lib
        self._pending = []          # (name, first event, second event)
        self._totals: Dict[str, Dict[str, float]] = {}
        self.overflow = 0

    def __getattr__(self, name):
        entry = getattr(self._library, name)
        if not name.startswith("fw_") or name in ("fw_last_error", "fw_abi_version") or name.endswith(("_plan", "_fits", "_tiles")):
            return entry

        def timed(*args):
            if len(self._pending) >= self.CAPACITY or torch.cuda.is_current_stream_capturing():
                self.overflow += 1
                return entry(*args)
            first, second = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            first.record()
            began = time.perf_counter()
            status = entry(*args)
            host_ms = (time.perf_counter() - began) * 1e3
            second.record()
            self._pending.append((name, first, second))
            total = self._totals.setdefault(name, {"calls": 0, "gpu_ms": 0.0, "host_launch_ms": 0.0, "max_us": 0.0})
            total["calls"] += 1
            total["host_launch_ms"] += host_ms
            return status
        return timed

    def report(self) -> Dict[str, Dict[str, float]]:
        torch.cuda.synchronize()
        for name, first, second in self._pending:
            ms = first.elapsed_time(second)
            total = self._totals[name]
            total["gpu_ms"] += ms
            total["max_us"] = max(total["max_us"], ms * 1e3)
        self._pending = []
        return {name: dict(total) for name, total in sorted(self._totals.items(), key=lambda item: -item[1]["gpu_ms"])}


_profiled: Optional[_ProfiledLibrary] = None


def kernel_profile(enable: bool = True) -> None:
    """Switches the per-kernel profile on or off (also switched on by FLYWEIGHT_KERNEL_PROFILE=1
    in the environment, as in the reference). While it is on, steps are not recorded into graphs."""
    global _profiled
    if enable and _profiled is None:
        _profiled = _ProfiledLibrary(library())
    elif not enable:
        _profiled = None


def kernel_profile_active() -> bool:
    return _profiled is not None


def kernel_profile_report() -> Dict[str, Dict[str, float]]:
    """Entry point -> calls, GPU milliseconds between its two events, host milliseconds inside
    the launching call, the longest single call in microseconds; sorted by GPU time."""
    return _profiled.report() if _profiled is not None else {}


def library():
    """Loads (building first if nothing is built) the kernel library."""
    global _lib
    if _profiled is not None:
        return _profiled
    if _lib is None:
        path = _build.ensure_built()
        lib = ctypes.CDLL(path)
        lib.fw_last_error.restype = ctypes.c_char_p
        lib.fw_abi_version.restype = ctypes.c_int
        if lib.fw_abi_version() != ABI_VERSION:
            raise KernelError(f"{path}: kernel library ABI {lib.fw_abi_version()} != {ABI_VERSION}; rebuild it")
        _lib = lib
        if os.environ.get("FLYWEIGHT_KERNEL_PROFILE", "")[:1] == "1":
            kernel_profile(True)
            return _profiled
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


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> ctypes.c_void_p:
    """The current HIP stream of the current device (asked for at every launch: a graph
    capture or a caller's stream context changes it)."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _want(t: torch.Tensor, dtype: torch.dtype, name: str) -> None:
    if t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, found {t.dtype}")


# ---------------------------------------------------------------------------------------
def embed_rows(table: torch.Tensor, ids: torch.Tensor, out: Optional[torch.Tensor] = None, scale: float = 1.0) -> torch.Tensor:
    _dev(table, ids, out)
    _want(ids, torch.int32, "ids")
    vocab, hidden = table.shape
    rows = ids.numel()
    if out is None:
        out = torch.empty((rows, hidden), dtype=torch.float32, device=table.device)
    _want(out, torch.float32, "out")
    if out.shape != (rows, hidden):
        raise KernelError(f"embed_rows: out is {tuple(out.shape)}, expected {(rows, hidden)}")
    _check(library().fw_embed_rows(_p(table), _code(table.dtype), _p(ids), _p(out), rows, hidden, vocab,
                                   ctypes.c_float(scale), _stream()))
    return out


def scale_softcap_(x: torch.Tensor, scale: float = 1.0, cap: float = 0.0) -> torch.Tensor:
    """In place on float32: x * scale, then with ``cap`` > 0 cap * tanh(x / cap)."""
    _dev(x)
    _want(x, torch.float32, "x")
    if cap < 0:
        raise KernelError("scale_softcap: the cap must not be negative")
    _check(library().fw_scale_softcap(_p(x), ctypes.c_longlong(x.numel()), ctypes.c_float(scale), ctypes.c_float(cap), _stream()))
    return x


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


def argmax_rows(logits: torch.Tensor, out: Optional[torch.Tensor] = None, also: Optional[torch.Tensor] = None,
                advance: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The id of each row's largest logit (ties: the lowest id), int32 [rows], into ``out`` if
    given and into ``also`` as well; ``advance[r]`` goes up by one (all contiguous int32 of at
    least ``rows`` elements)."""
    _dev(logits)
    _want(logits, torch.float32, "logits")
    rows, vocab = logits.shape
    ids = out if out is not None else torch.empty((rows,), dtype=torch.int32, device=logits.device)
    for name, target in (("out", out), ("also", also), ("advance", advance)):
        if target is not None:
            _dev(target)
            _want(target, torch.int32, name)
            if target.numel() < rows or not target.is_contiguous():
                raise KernelError(f"argmax_rows: {name} must be contiguous and hold {rows} ids")
    workspace = torch.empty((max(rows, 1), 64), dtype=torch.int64, device=logits.device)       # best key of each part
    _check(library().fw_argmax_rows(_p(logits), _p(ids), _p(also), _p(advance), _p(workspace), rows, vocab, _stream()))
    return ids


def sample_rows(logits: torch.Tensor, settings: torch.Tensor, states: torch.Tensor, out: Optional[torch.Tensor] = None,
                also: Optional[torch.Tensor] = None, advance: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The next token of every row, drawn on the device (fw_sample_rows): ``settings`` float32
    [rows, 4] = temperature (0: greedy), top_k (0: all), top_p, min_p; ``states`` int64 [rows], the
    rows' xorshift64* generators, moved on in place by the rows that draw. ``out`` / ``also`` /
    ``advance`` as for ``argmax_rows``."""
    _dev(logits, settings, states)
    _want(logits, torch.float32, "logits")
    _want(settings, torch.float32, "settings")
    _want(states, torch.int64, "states")
    rows, vocab = logits.shape
    if settings.numel() < 4 * rows or states.numel() < rows or not settings.is_contiguous() or not states.is_contiguous():
        raise KernelError(f"sample_rows: settings must hold [{rows}, 4] and states [{rows}], contiguous")
    ids = out if out is not None else torch.empty((rows,), dtype=torch.int32, device=logits.device)
    for name, target in (("out", out), ("also", also), ("advance", advance)):
        if target is not None:
            _dev(target)
            _want(target, torch.int32, name)
            if target.numel() < rows or not target.is_contiguous():
                raise KernelError(f"sample_rows: {name} must be contiguous and hold {rows} ids")
    _check(library().fw_sample_rows(_p(logits), _p(settings), _p(states), _p(ids), _p(also), _p(advance), rows, vocab, _stream()))
    return ids


def fill_zero(t: torch.Tensor) -> None:
    _dev(t)
    _check(library().fw_fill_zero(_p(t), ctypes.c_longlong(t.numel() * t.element_size()), _stream()))


def fill_zero_pieces(first: torch.Tensor, pieces: int, stride_bytes: int) -> None:
    """Clears ``pieces`` runs of memory the size of ``first`` (contiguous), ``stride_bytes`` apart,
    beginning with ``first`` itself: the caller vouches that all of them lie in one allocation."""
    _dev(first)
    _check(library().fw_fill_zero_pieces(_p(first), int(pieces), ctypes.c_longlong(first.numel() * first.element_size()),
                                         ctypes.c_longlong(int(stride_bytes)), _stream()))


def gather_rows(rows: torch.Tensor, index: torch.Tensor) -> torch.Tensor:
    """rows[index] for float32 rows and an int32 index on the device (the embedding kernel: a
    table of rows is a table of rows)."""
    return embed_rows(rows, index)


def _fast_gemm(a: torch.Tensor, w: torch.Tensor, bias, target: torch.Tensor, out_code: int, mode: int, N: int,
               w_tiled: Optional[torch.Tensor] = None) -> None:
    """bfloat16 operands on the matrix cores: the skinny kernel for up to 16 rows, the medium one
    (K split over workgroups) for up to 64, the tiled ones beyond (large tiles where they fill the
    chip, K cut into slices where even the small tiles are too few)."""
    M, K = a.shape
    if SKINNY_MAX_ROWS < M <= MEDIUM_MAX_ROWS or (M <= SKINNY_MAX_ROWS and w.numel() >= MEDIUM_LARGE and K % 8 == 0):
        # also a few rows of a large W (a vocabulary's head: 65,536 x 2,048 at 8 rows 52 against 61 us)
        gemm_medium_into(a, w, bias, target, out_code, mode, N, w_tiled=w_tiled)
        return
    if M <= SKINNY_MAX_ROWS:
        entry = library().fw_gemm_skinny
    elif M > BIG_MIN_ROWS and library().fw_gemm_mfma_big_tiles(mode, M, N, K) >= BIG_TILES_MIN:
        entry = library().fw_gemm_mfma_big      # enough 256 x 256 tiles to fill the chip
    elif K >= (DEEP_MIN_K if mode == 1 else DEEP_MIN_K_STORE) and _deep_columns(mode, M, N, K):
        # whole rounds of one tile per compute unit: the waves split K
        _check(library().fw_gemm_mfma_deep(_p(a), _p(w), _p(bias), _p(target), out_code, mode, M, N, K,
                                           _deep_columns(mode, M, N, K), _stream()))
        return
    elif _deep_columns_few_rows(mode, M, N, K, one_round=True):
        _check(library().fw_gemm_mfma_deep(_p(a), _p(w), _p(bias), _p(target), out_code, mode, M, N, K,
                                           _deep_columns_few_rows(mode, M, N, K), _stream()))
        return
    elif M > BIG_MIN_ROWS and _big_tiles_store_well(mode, M, N, K):
        entry = library().fw_gemm_mfma_big      # fewer large tiles than compute units, but every other way takes two rounds
    elif _deep_columns_few_rows(mode, M, N, K):
        _check(library().fw_gemm_mfma_deep(_p(a), _p(w), _p(bias), _p(target), out_code, mode, M, N, K,
                                           _deep_columns_few_rows(mode, M, N, K), _stream()))
        return
    else:
        need_bytes, need_counters = ctypes.c_size_t(0), ctypes.c_int(0)
        _check(library().fw_gemm_mfma_split_plan(mode, M, N, K, ctypes.byref(need_bytes), ctypes.byref(need_counters)))
        if need_bytes.value:                    # fewer tiles than compute units: K is cut into slices
            workspace = torch.empty(need_bytes.value // 4, dtype=torch.float32, device=a.device)
            counters = _medium_counters(a.device, need_counters.value)
            _check(library().fw_gemm_mfma_split(_p(a), _p(w), _p(bias), _p(target), out_code, mode, M, N, K, _p(workspace),
                                                ctypes.c_size_t(need_bytes.value), _p(counters), counters.numel(), _stream()))
            return
        entry = library().fw_gemm_mfma
    _check(entry(_p(a), _p(w), _p(bias), _p(target), out_code, mode, M, N, K, _stream()))


SKINNY_MAX_ROWS = 16
MEDIUM_MAX_ROWS = 64
MEDIUM_LARGE = 1 << 25    # weights from which the medium product beats the skinny one at any number of rows
BIG_TILES_MIN = 192      # 256 x 256 tiles from which the large-tile prompt product is used (256 compute units)
DEEP_MIN_K = 1024         # adding into the residual (2,048 x 2,048 x 2,048: 31 vs 39 us; x 8,192: 83 vs 118 us; 2,048 x 1,024 x 1,024: 13 vs 15 us)
DEEP_MIN_K_STORE = 4096   # storing: no old values travel during the exchange at a tile's end, a short K gains nothing
DEEP_ROUND = 256          # tiles of a round: one per compute unit
DEEP_FILL = 0.85          # least share of the rounds' places that the tiles must fill (640 narrow tiles, 0.83: 193 vs 189 us)
# adding into the residual, 2,048 features: 144 wide tiles (1,152 rows) K 8,192 72 vs 103 us, K 2,048 28 vs 35 us; 160
# narrow tiles (576 rows) 46 vs 65 us and 16.5 vs 27 us; 576 narrow (2,304 rows) 120 vs 135 us; 128 narrow tiles lose
DEEP_FILL_ADDING = 0.55


def _round_fill(tiles: int) -> float:
    """The share of the places in whole rounds over the chip that the tiles fill."""
    rounds = -(-tiles // DEEP_ROUND)
    return tiles / (rounds * DEEP_ROUND) if tiles > 0 else 0.0


def _deep_columns(mode: int, M: int, N: int, K: int) -> int:
    """The width of the tiles whose waves split K that serves this shape: the width (128 or 64
    columns) whose tiles fill their rounds over the chip better, the wider at a tie, if they fill
    enough of them; else 0. A product that adds into the residual needs less (the other kernels
    ask for the old values at the end of a tile, where nothing hides the read)."""
    fills = {columns: _round_fill(library().fw_gemm_mfma_deep_tiles(mode, M, N, K, columns)) for columns in (128, 64)}
    columns = 128 if fills[128] >= fills[64] else 64
    return columns if fills[columns] >= (DEEP_FILL_ADDING if mode == 1 else DEEP_FILL) else 0


DEEP_FEW_ROWS = 512       # up to here the tiles whose waves split K also serve a short K, if they are not too few
DEEP_FEW_TILES_WIDE = 192   # tiles of 128 columns from which those are taken, else
DEEP_FEW_TILES = 96       # tiles of 64 columns from which those are


BIG_TILES_MIN_STORE = 96      # large tiles from which a storing product takes them, if the output fills
BIG_FILL_STORE = 0.95         # at least this share of them


def _big_tiles_store_well(mode: int, M: int, N: int, K: int) -> bool:
    """A storing product that no kernel serves in one round of small tiles takes the large
    tiles from 96 of them on if they are well filled: 768 x 3,072 (K 1,024) 18.7 -> 14.9 us,
    512 x 4,608 21.1 -> 14.6 us, 1,024 x 3,072 (K 2,048) 29.5 -> 25.0 us; 2,048 x 1,024 (96 tiles
    of 192 columns, an eighth of them outside the output) would lose, 14.1 -> 17.5 us."""
    if mode != 0:
        return False
    rows, columns = ctypes.c_int(0), ctypes.c_int(0)
    tiles = library().fw_gemm_mfma_big_plan(mode, M, N, K, ctypes.byref(rows), ctypes.byref(columns))
    return tiles >= BIG_TILES_MIN_STORE and M * N >= BIG_FILL_STORE * tiles * rows.value * columns.value


def _deep_columns_few_rows(mode: int, M: int, N: int, K: int, one_round: bool = False) -> int:
    """A few hundred rows (decode steps of that many requests, short prompts) give the 128 x 128
    tiles of the register-staged product less than a round over the chip; the tiles whose waves
    split K bring their operands straight into LDS, three slabs ahead, and a workgroup alone on
    its compute unit keeps them coming. Measured against the products they replace, 8 in a row:
    storing 6,144 features at 256 rows 16.0 vs 21.0 us, at 128 rows 15.0 vs 18.6; 3,072 features at
    256 rows 15.0 vs 18.6, at 512 rows 15.9 vs 21.0 us; adding 2,048 features (K 2,048) at 512 rows
    16.2 vs 23.0 us, at 320 rows 15.7 vs 21.5 us. With a long K (8,192) the product that cuts K over
    workgroups is level with them."""
    if mode not in (0, 1) or M > DEEP_FEW_ROWS or K > (LONG_K if mode == 1 else 1 << 30):
        return 0
    wide = library().fw_gemm_mfma_deep_tiles(mode, M, N, K, 128)
    narrow = library().fw_gemm_mfma_deep_tiles(mode, M, N, K, 64)
    if mode == 0 and DEEP_FEW_TILES_WIDE <= wide <= DEEP_ROUND:
        return 128
    if DEEP_FEW_TILES <= narrow <= (1 if one_round else 2) * DEEP_ROUND:
        return 64
    return 0


BIG_MIN_ROWS = 128       # up to here a 256-row tile would be at least half empty (the head at 128 rows: 110 vs 78 us)
_MEDIUM_COUNTERS = {}


TICKET_COUNTERS = 1 << 20      # 4 MB per device


def _medium_counters(device: torch.device, count: int) -> torch.Tensor:
    """Zeroed int32 counters for the tickets of the kernels whose last workgroup finishes the
    work of the others (the medium product, decode attention), one set per device: each kernel
    leaves them at zero, and calls on one device follow each other in stream order (work on
    several streams of one device at once would need a set per stream). The set is allocated
    once and never replaced: recorded graphs hold its address."""
    have = _MEDIUM_COUNTERS.get(device.index)
    if have is None:
        if torch.cuda.is_current_stream_capturing():
            raise KernelError("the ticket counters must exist before a graph is captured (prepare_device)")
        have = _MEDIUM_COUNTERS[device.index] = torch.zeros(TICKET_COUNTERS, dtype=torch.int32, device=device)
    if count > have.numel():
        raise KernelError(f"a kernel asks for {count} ticket counters; the device's set holds {have.numel()}")
    return have


def prepare_device(device: torch.device) -> None:
    """Allocates what kernels keep between calls on this device; a model does this when its
    weights arrive, so that nothing is allocated for the first time inside a graph capture."""
    _medium_counters(torch.device(device), 0)


def tile_weights(w: torch.Tensor) -> Optional[torch.Tensor]:
    """``w`` [rows, K] bfloat16 once more in operand tiles, [ceil(rows / 16), K / 32, 4, 16, 8]: what the
    decode products read as whole contiguous kilobytes per wave (see fw_gemm_decode). None where the
    layout does not apply (K no multiple of 32, another dtype)."""
    if w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] % 32 or not w.is_cuda:
        return None
    rows, K = w.shape
    padded = (rows + 15) // 16 * 16
    if padded != rows:
        w = torch.cat([w, torch.zeros((padded - rows, K), dtype=w.dtype, device=w.device)])
    return w.view(padded // 16, 16, K // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous()


def _tiled_for(w: torch.Tensor, w_tiled: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    """``w_tiled`` if it is ``w`` in operand tiles (checked by its shape), else an error."""
    if w_tiled is None:
        return None
    rows, K = w.shape
    if (w_tiled.dtype != torch.bfloat16 or K % 32 or tuple(w_tiled.shape) != ((rows + 15) // 16, K // 32, 4, 16, 8)
            or not w_tiled.is_contiguous() or w_tiled.device != w.device):
        raise KernelError(f"weights in operand tiles for w {tuple(w.shape)} are bfloat16 [{(rows + 15) // 16}, {K // 32}, 4, 16, 8], "
                          f"found {tuple(w_tiled.shape)}")
    return w_tiled


def gemm_medium_into(a: torch.Tensor, w: torch.Tensor, bias, target: torch.Tensor, out_code: int, mode: int, N: int,
                     next_norm_weight: Optional[torch.Tensor] = None, next_one_centered: bool = False,
                     squares: Optional[torch.Tensor] = None, eps: float = 0.0, w_tiled: Optional[torch.Tensor] = None):
    """The product for 1..64 rows with K split over workgroups (fw_gemm_medium). With
    ``squares`` ``a`` holds prepared activations (x * w of an RMS norm) and the rows' 1/rms is
    formed from those sums. With ``next_norm_weight`` (accumulating product) returns what the
    norm after it needs: (activations x * w_next, sums of squares)."""
    M, K = a.shape
    need_bytes, need_counters, squares_rows = ctypes.c_size_t(0), ctypes.c_int(0), ctypes.c_int(0)
    _check(library().fw_gemm_medium_plan(M, N, K, mode, ctypes.byref(need_bytes), ctypes.byref(need_counters),
                                         ctypes.byref(squares_rows)))
    workspace = counters = next_activations = next_squares = None
    if need_bytes.value:
        workspace = torch.empty(need_bytes.value // 4, dtype=torch.float32, device=a.device)
        counters = _medium_counters(a.device, need_counters.value)
    stride = 16 if M <= DECODE_MAX_ROWS else 64
    if next_norm_weight is not None:
        next_activations = torch.empty((M, N), dtype=torch.bfloat16, device=a.device)
        next_squares = torch.empty((squares_rows.value, stride), dtype=torch.float32, device=a.device)
    if squares is not None and (squares.dtype != torch.float32 or squares.dim() != 2 or squares.shape[1] != stride
                                or not squares.is_contiguous()):
        raise KernelError(f"gemm_medium: sums of squares for {M} rows are float32 [n, {stride}]")
    w_tiled = _tiled_for(w, w_tiled)
    _check(library().fw_gemm_medium(_p(a), _p(w if w_tiled is None else w_tiled), int(w_tiled is not None), _p(bias), _p(target), out_code, mode, M, N, K, _p(workspace),
                                    ctypes.c_size_t(need_bytes.value), _p(counters),
                                    0 if counters is None else counters.numel(), _p(next_norm_weight),
                                    int(next_one_centered), _p(next_activations), _p(next_squares), _p(squares),
                                    0 if squares is None else squares.shape[0], ctypes.c_float(eps), _stream()))
    if next_norm_weight is not None:
        return next_activations, next_squares
    return None


def gemm_medium(a: torch.Tensor, w: torch.Tensor, epilogue: int, *, bias: Optional[torch.Tensor] = None,
                out_dtype: Optional[torch.dtype] = None, accumulate_into: Optional[torch.Tensor] = None,
                squares: Optional[torch.Tensor] = None, eps: float = 0.0,
                next_norm_weight: Optional[torch.Tensor] = None, next_one_centered: bool = False,
                w_tiled: Optional[torch.Tensor] = None):
    """The medium product with the fused decode product's conventions (EPILOGUE_STORE /
    ACCUMULATE / SWIGLU): returns the output, or for an accumulation with ``next_norm_weight``
    what the norm after it needs."""
    _dev(a, w, bias, accumulate_into, squares, next_norm_weight)
    _want(a, torch.bfloat16, "a")
    _want(w, torch.bfloat16, "w")
    M, K = a.shape
    kinds = 2 if epilogue == EPILOGUE_SWIGLU else 1
    if not 1 <= M <= MEDIUM_MAX_ROWS or w.shape[1] != K or w.shape[0] % kinds or K % 8 or epilogue not in (0, 1, 2):
        raise KernelError(f"gemm_medium: a is {tuple(a.shape)}, w is {tuple(w.shape)}, epilogue {epilogue}")
    N = w.shape[0] // kinds
    if bias is not None and (bias.dtype != torch.float32 or bias.shape != (w.shape[0],)):
        raise KernelError("gemm_medium: bias must be float32, one entry per row of w")
    if next_norm_weight is not None and (epilogue != EPILOGUE_ACCUMULATE or next_norm_weight.dtype != torch.float32
                                         or next_norm_weight.shape != (N,)):
        raise KernelError("gemm_medium: only the accumulating product prepares the next norm, whose weight is float32 [N]")
    if epilogue == EPILOGUE_ACCUMULATE:
        _want(accumulate_into, torch.float32, "accumulate_into")
        if accumulate_into.shape != (M, N):
            raise KernelError(f"gemm_medium: destination is {tuple(accumulate_into.shape)}, expected {(M, N)}")
        left = gemm_medium_into(a, w, bias, accumulate_into, F32, 1, N, next_norm_weight, next_one_centered, squares, eps, w_tiled=w_tiled)
        return accumulate_into if left is None else left
    out_dtype = torch.bfloat16 if epilogue == EPILOGUE_SWIGLU else (out_dtype or torch.bfloat16)
    out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    gemm_medium_into(a, w, bias, out, _code(out_dtype), epilogue, N, squares=squares, eps=eps, w_tiled=w_tiled)
    return out


def gemm_deep(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
              out_dtype: Optional[torch.dtype] = None, accumulate_into: Optional[torch.Tensor] = None,
              columns: int = 128) -> torch.Tensor:
    """a [M, K] . w [N, K]^T (+ bias) on 128 x 128 tiles whose waves split K (fw_gemm_mfma_deep),
    whatever the dispatch of ``gemm`` would choose: bfloat16 operands, K a multiple of 64."""
    _dev(a, w, bias, accumulate_into)
    _want(a, torch.bfloat16, "a")
    _want(w, torch.bfloat16, "w")
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K or (bias is not None and (bias.dtype != torch.float32 or bias.shape != (N,))):
        raise KernelError(f"gemm_deep: a is {tuple(a.shape)}, w is {tuple(w.shape)}; bias is float32 [N]")
    if accumulate_into is not None:
        _want(accumulate_into, torch.float32, "accumulate_into")
        if accumulate_into.shape != (M, N):
            raise KernelError(f"gemm_deep: destination is {tuple(accumulate_into.shape)}, expected {(M, N)}")
        target, mode = accumulate_into, 1
    else:
        target, mode = torch.empty((M, N), dtype=out_dtype or a.dtype, device=a.device), 0
    _check(library().fw_gemm_mfma_deep(_p(a), _p(w), _p(bias), _p(target), _code(target.dtype), mode, M, N, K, int(columns), _stream()))
    return target


def _fast_ok(a: torch.Tensor, w: torch.Tensor) -> bool:
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.shape[0] >= 1 and a.shape[1] % 8 == 0
            and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


# ---- dispatch: which kernel serves a call ------------------------------------------------
def gemm(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
         out_dtype: Optional[torch.dtype] = None, accumulate_into: Optional[torch.Tensor] = None,
         w_tiled: Optional[torch.Tensor] = None) -> torch.Tensor:
    """a [M, K] . w [N, K]^T (+ bias): bfloat16 operands go to the matrix-core kernels,
    everything else (float32, mixed) to the generic float32 one. ``w_tiled``: ``w`` once more in
    operand tiles (``tile_weights``), for the kernels of few rows that read it so."""
    if not _fast_ok(a, w):
        return gemm_generic(a, w, bias, out_dtype=out_dtype, accumulate_into=accumulate_into)
    _dev(a, w, bias, accumulate_into)
    M, K = a.shape
    N, K2 = w.shape
    if K != K2:
        raise KernelError(f"gemm: a is {tuple(a.shape)} but w is {tuple(w.shape)}")
    if bias is not None and (bias.dtype != torch.float32 or bias.shape != (N,)):
        raise KernelError("gemm: bias must be float32 [N]")
    if accumulate_into is not None:
        _want(accumulate_into, torch.float32, "accumulate_into")
        if accumulate_into.shape != (M, N):
            raise KernelError(f"gemm: destination is {tuple(accumulate_into.shape)}, expected {(M, N)}")
        _fast_gemm(a, w, bias, accumulate_into, F32, 1, N, w_tiled)
        return accumulate_into
    out_dtype = out_dtype or a.dtype
    out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    _fast_gemm(a, w, bias, out, _code(out_dtype), 0, N, w_tiled)
    return out


def gemm_swiglu(a: torch.Tensor, w_gate_up: torch.Tensor, w_tiled: Optional[torch.Tensor] = None) -> torch.Tensor:
    """silu(a . gate^T) * (a . up^T) with w_gate_up = [gate rows; up rows]: [M, I] in a's dtype.
    On the bfloat16 path the activation is formed from the float32 sums inside the product's
    kernel; otherwise the [M, 2I] intermediate is float32 and a second kernel forms it."""
    rows2, K = w_gate_up.shape
    if rows2 % 2:
        raise KernelError("gemm_swiglu: the operand holds gate and up rows; their number must be even")
    if _fast_ok(a, w_gate_up):
        _dev(a, w_gate_up)
        if a.shape[1] != K:
            raise KernelError(f"gemm_swiglu: a is {tuple(a.shape)} but w is {tuple(w_gate_up.shape)}")
        out = torch.empty((a.shape[0], rows2 // 2), dtype=torch.bfloat16, device=a.device)
        _fast_gemm(a, w_gate_up, None, out, BF16, 2, rows2 // 2, w_tiled)
        return out
    return swiglu(gemm_generic(a, w_gate_up, out_dtype=torch.float32), out_dtype=a.dtype)


# ---- fused products for decode steps of up to 16 rows --------------------------------------------
EPILOGUE_STORE, EPILOGUE_ACCUMULATE, EPILOGUE_SWIGLU, EPILOGUE_CONV = 0, 1, 2, 3
DECODE_MAX_ROWS = 16
LONG_K = 4096
LONG_K_TILED_ROWS = 8


def gemm_decode_fits(rows: int, features: int, k: int, epilogue: int) -> bool:
    return bool(library().fw_gemm_decode_fits(int(rows), int(features), int(k), int(epilogue)))


def gemm_decode(a: torch.Tensor, w: torch.Tensor, epilogue: int, *, bias: Optional[torch.Tensor] = None,
                norm_weight: Optional[torch.Tensor] = None, eps: float = 0.0, one_centered: bool = False,
                row_index: Optional[torch.Tensor] = None, out_dtype: Optional[torch.dtype] = None,
                accumulate_into: Optional[torch.Tensor] = None, taps: Optional[torch.Tensor] = None,
                conv_bias: Optional[torch.Tensor] = None, state: Optional[torch.Tensor] = None,
                seg_slot: Optional[torch.Tensor] = None, squares: Optional[torch.Tensor] = None,
                next_norm_weight: Optional[torch.Tensor] = None, next_one_centered: bool = False,
                w_tiled: Optional[torch.Tensor] = None):
    """One kernel for (optional RMS norm of float32 rows) -> product with bfloat16 ``w`` -> epilogue.
    With ``norm_weight`` ``a`` holds float32 rows (gathered through ``row_index`` if given), else
    bfloat16 activations. With ``next_norm_weight`` the accumulating epilogue also leaves what
    the norm after it needs, and the call returns (activations x * w_next, sums of squares);
    a later call takes those as ``a`` and ``squares`` (with ``eps``) and skips the norm's
    arithmetic. See fw_gemm_decode in fw_kernels.h for the epilogues."""
    _dev(a, w, bias, norm_weight, row_index, accumulate_into, taps, conv_bias, state, seg_slot, squares, next_norm_weight)
    _want(w, torch.bfloat16, "w")
    normed = norm_weight is not None
    if squares is not None and (normed or squares.dtype != torch.float32 or squares.dim() != 2 or squares.shape[1] != 16
                                or not squares.is_contiguous()):
        raise KernelError("gemm_decode: sums of squares are float32 [tiles, 16] and replace the norm")
    rows = row_index.numel() if (normed and row_index is not None) else a.shape[0]
    K = a.shape[1]
    tiles = {EPILOGUE_SWIGLU: 2, EPILOGUE_CONV: 3}.get(epilogue, 1)
    if w.shape[1] != K or w.shape[0] % tiles:
        raise KernelError(f"gemm_decode: a is {tuple(a.shape)} but w is {tuple(w.shape)}")
    N = w.shape[0] // tiles
    if normed:
        _want(a, torch.float32, "a")
        _want(norm_weight, torch.float32, "norm_weight")
        if norm_weight.shape != (K,):
            raise KernelError("gemm_decode: the norm weight must be [K]")
        if row_index is not None:
            _want(row_index, torch.int32, "row_index")
    else:
        _want(a, torch.bfloat16, "a")
    if bias is not None and (bias.dtype != torch.float32 or bias.shape != (w.shape[0],)):
        raise KernelError("gemm_decode: bias must be float32, one entry per row of w")
    kernel_size = 0
    if epilogue == EPILOGUE_CONV:
        _want(taps, torch.float32, "taps")
        _want(state, torch.float32, "state")
        _want(seg_slot, torch.int32, "seg_slot")
        kernel_size = taps.shape[1]
        if taps.shape != (N, kernel_size) or state.dim() != 3 or state.shape[1:] != (N, kernel_size - 1):
            raise KernelError("gemm_decode: taps must be [N, L] and state [slots, N, L - 1]")
        if seg_slot.numel() < rows or (conv_bias is not None and conv_bias.shape != (N,)):
            raise KernelError("gemm_decode: seg_slot or the convolution bias has the wrong size")
    if epilogue == EPILOGUE_ACCUMULATE:
        _want(accumulate_into, torch.float32, "accumulate_into")
        if accumulate_into.shape != (rows, N):
            raise KernelError(f"gemm_decode: destination is {tuple(accumulate_into.shape)}, expected {(rows, N)}")
        target, out_dtype = accumulate_into, torch.float32
    else:
        out_dtype = out_dtype or torch.bfloat16
        target = torch.empty((rows, N), dtype=out_dtype, device=a.device)
    next_activations = next_squares = None
    if next_norm_weight is not None and (epilogue != EPILOGUE_ACCUMULATE or next_norm_weight.dtype != torch.float32
                                         or next_norm_weight.shape != (N,)):
        raise KernelError("gemm_decode: only the accumulating product prepares the next norm, whose weight is float32 [N]")
    if epilogue == EPILOGUE_ACCUMULATE and K >= LONG_K and N <= 4096 and not (w_tiled is not None and rows <= LONG_K_TILED_ROWS):
        # few features and a long K: the kernel that splits K over workgroups streams W faster (from operand
        # tiles only beyond eight rows: 2,048 features over K 8,192 at 8 rows 11.4 against 11.0 us, at 16
        # rows 11.3 against 13.4)
        left = gemm_medium_into(a, w, bias, target, F32, 1, N, next_norm_weight, next_one_centered, w_tiled=w_tiled)
        return target if left is None else left
    if next_norm_weight is not None:
        next_activations = torch.empty((rows, N), dtype=torch.bfloat16, device=a.device)
        next_squares = torch.empty((library().fw_gemm_decode_accumulate_tiles(N), 16), dtype=torch.float32, device=a.device)
    prologue = 1 if normed else (2 if squares is not None else 0)
    w_tiled = _tiled_for(w, w_tiled)
    _check(library().fw_gemm_decode(
        prologue, _p(a), _p(norm_weight), _p(row_index), ctypes.c_float(eps), int(one_centered),
        _p(w if w_tiled is None else w_tiled), int(w_tiled is not None), _p(bias),
        _p(target), _code(out_dtype), int(epilogue), rows, N, K, _p(taps), _p(conv_bias), _p(state), _p(seg_slot),
        int(kernel_size), _p(next_norm_weight), int(next_one_centered), _p(next_activations), _p(next_squares),
        _p(squares), 0 if squares is None else squares.shape[0], _stream()))
    if next_norm_weight is not None:
        return next_activations, next_squares
    return target


DECODE_SPLIT_PAGES = 4


QUERY_TILE = 64


def query_tiles(seg_row0):
    """Cuts the rows of each segment into tiles of up to 64 that never span two segments:
    (segment of each tile, first row of each tile), as lists."""
    tile_seg, tile_row0 = [], []
    for seg in range(len(seg_row0) - 1):
        for row in range(seg_row0[seg], seg_row0[seg + 1], QUERY_TILE):
            tile_seg.append(seg)
            tile_row0.append(row)
    return tile_seg, tile_row0


def decode_splits(max_context: int, window: int = 0) -> int:
    """Into how many workgroups at most the keys that a row sees are cut: runs of 4 pages."""
    blocks = (max_context + PAGE_SIZE - 1) // PAGE_SIZE
    if window > 0:
        blocks = min(blocks, (window + PAGE_SIZE - 2) // PAGE_SIZE + 1)
    return max(1, (blocks + DECODE_SPLIT_PAGES - 1) // DECODE_SPLIT_PAGES)


def attention_prefill(q: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int, k_pages: torch.Tensor,
                      v_pages: torch.Tensor, block_table: torch.Tensor, tile_seg: torch.Tensor, tile_row0: torch.Tensor,
                      seg_row0: torch.Tensor, row_pos: torch.Tensor, scale: float, window: int = 0,
                      heads_together: int = 0, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``heads_together``: query heads of a kv group per workgroup (1, or 4 up to head_dim 64), 0: the
    kernel's choice. Only the rows of the given tiles are written (into ``out`` if given)."""
    _dev(q, k_pages, v_pages, block_table, tile_seg, tile_row0, seg_row0, row_pos)
    _want(q, torch.bfloat16, "q")
    rows = q.shape[0]
    if q.shape != (rows, num_heads * head_dim):
        raise KernelError(f"attention: q is {tuple(q.shape)}, expected {(rows, num_heads * head_dim)}")
    pages = _check_pages(k_pages, v_pages, num_kv_heads, head_dim, torch.bfloat16)
    for name, t in (("block_table", block_table), ("tile_seg", tile_seg), ("tile_row0", tile_row0),
                    ("seg_row0", seg_row0), ("row_pos", row_pos)):
        _want(t, torch.int32, name)
    if block_table.dim() != 2 or row_pos.numel() < rows or tile_seg.numel() != tile_row0.numel():
        raise KernelError("attention: batch index arrays are inconsistent")
    if out is None:
        out = torch.empty_like(q)
    elif out.shape != q.shape or out.dtype != q.dtype or not out.is_contiguous():
        raise KernelError("attention: out must be like q")
    _check(library().fw_attention_prefill(
        _p(q), _p(out), _p(k_pages), _p(v_pages), _p(block_table), block_table.shape[1], _p(tile_seg), _p(tile_row0),
        tile_seg.numel(), _p(seg_row0), _p(row_pos), rows, num_heads, num_kv_heads, head_dim, ctypes.c_float(scale),
        int(window), PAGE_SIZE, pages, int(heads_together), _stream()))
    return out


def _work(decode_work: Optional[torch.Tensor]):
    if decode_work is not None:
        _dev(decode_work)
        _want(decode_work, torch.int32, "decode_work")
        if decode_work.numel() < 1:
            raise KernelError("attention_decode: decode_work holds one int32")
    return _p(decode_work)


def attention_decode(q: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int, k_pages: torch.Tensor,
                     v_pages: torch.Tensor, block_table: torch.Tensor, row_seg: torch.Tensor, row_pos: torch.Tensor,
                     scale: float, max_context: int, window: int = 0, out: Optional[torch.Tensor] = None,
                     decode_work: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One row per request; ``max_context`` bounds position + 1 of every row (the host knows it).
    ``decode_work``: one int32 on the device, the runs of 4 pages that the rows see together (the
    sum of ceil((position + 1) / 256)): the kernel shares the work out by it (fewer, longer
    workgroups once there are more than about 512); without it, one run per workgroup."""
    _dev(q, k_pages, v_pages, block_table, row_seg, row_pos)
    _want(q, torch.bfloat16, "q")
    rows = q.shape[0]
    if q.shape != (rows, num_heads * head_dim):
        raise KernelError(f"attention: q is {tuple(q.shape)}, expected {(rows, num_heads * head_dim)}")
    pages = _check_pages(k_pages, v_pages, num_kv_heads, head_dim, torch.bfloat16)
    for name, t in (("block_table", block_table), ("row_seg", row_seg), ("row_pos", row_pos)):
        _want(t, torch.int32, name)
    if block_table.dim() != 2 or row_seg.numel() < rows or row_pos.numel() < rows:
        raise KernelError("attention: batch index arrays are too short")
    splits = decode_splits(max_context, window)
    partial = torch.empty((rows, num_heads, splits, head_dim + 4), dtype=torch.float32, device=q.device)
    if out is None:
        out = torch.empty_like(q)
    elif out.shape != q.shape or out.dtype != q.dtype or not out.is_contiguous():
        raise KernelError("attention: out must be like q")
    group = num_heads // num_kv_heads
    tickets = _medium_counters(q.device, rows * num_kv_heads * ((group + 15) // 16))
    _check(library().fw_attention_decode(
        _p(q), _p(out), _p(partial), splits, int(max_context), _work(decode_work), _p(tickets), tickets.numel(), _p(k_pages), _p(v_pages),
        _p(block_table),
        block_table.shape[1], _p(row_seg), _p(row_pos), rows, num_heads, num_kv_heads, head_dim, ctypes.c_float(scale),
        int(window), PAGE_SIZE, pages, _stream()))
    return out


def attention_decode_fused(qkv: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
                           q_norm_weight: Optional[torch.Tensor], k_norm_weight: Optional[torch.Tensor], eps: float,
                           cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], rotary_dim: int, k_pages: torch.Tensor,
                           v_pages: torch.Tensor, block_table: torch.Tensor, row_seg: torch.Tensor, row_pos: torch.Tensor,
                           scale: float, max_context: int, window: int = 0, write_kv: bool = True,
                           decode_work: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One row per request, from the step's raw projections ``qkv`` (float32 [rows, (heads + 2 kv
    heads) * head_dim]): per-head norm and rotation of queries and keys, the new keys and values
    into their pages, and the split-key attention, in one kernel. Returns bfloat16 [rows, heads *
    head_dim]; the same numbers as ``qk_norm_rope_kv_write`` followed by ``attention_decode``."""
    _dev(qkv, q_norm_weight, k_norm_weight, cos, sin, k_pages, v_pages, block_table, row_seg, row_pos)
    _want(qkv, torch.float32, "qkv")
    rows, width = qkv.shape
    if width != (num_heads + 2 * num_kv_heads) * head_dim:
        raise KernelError(f"attention_decode_fused: qkv width {width} != ({num_heads} + 2 x {num_kv_heads}) x {head_dim}")
    pages = _check_pages(k_pages, v_pages, num_kv_heads, head_dim, torch.bfloat16)
    for w in (q_norm_weight, k_norm_weight):
        if w is not None:
            _want(w, torch.float32, "norm weight")
            if w.shape != (head_dim,):
                raise KernelError("attention_decode_fused: a head norm weight must be [head_dim]")
    if rotary_dim:
        for t in (cos, sin):
            _want(t, torch.float32, "rotation table")
            if t.shape != (rows, rotary_dim // 2):
                raise KernelError(f"attention_decode_fused: rotation table is {tuple(t.shape)}, expected {(rows, rotary_dim // 2)}")
    for name, t in (("block_table", block_table), ("row_seg", row_seg), ("row_pos", row_pos)):
        _want(t, torch.int32, name)
    if block_table.dim() != 2 or row_seg.numel() < rows or row_pos.numel() < rows:
        raise KernelError("attention: batch index arrays are too short")
    splits = decode_splits(max_context, window)
    partial = torch.empty((rows, num_heads, splits, head_dim + 4), dtype=torch.float32, device=qkv.device)
    out = torch.empty((rows, num_heads * head_dim), dtype=torch.bfloat16, device=qkv.device)
    group = num_heads // num_kv_heads
    tickets = _medium_counters(qkv.device, rows * num_kv_heads * ((group + 15) // 16))
    _check(library().fw_attention_decode_fused(
        _p(qkv), _p(q_norm_weight), _p(k_norm_weight), ctypes.c_float(eps), _p(cos), _p(sin), int(rotary_dim), int(write_kv), _p(out),
        _p(partial), splits, int(max_context), _work(decode_work), _p(tickets), tickets.numel(), _p(k_pages), _p(v_pages), _p(block_table),
        block_table.shape[1], _p(row_seg), _p(row_pos), rows, num_heads, num_kv_heads, head_dim, ctypes.c_float(scale), int(window),
        PAGE_SIZE, pages, _stream()))
    return out


def attention_is_tiled(head_dim: int) -> bool:
    """Whether bfloat16 attention with this head size runs on the matrix-core kernels (which
    work on tiles of QUERY_TILE rows)."""
    return head_dim % 16 == 0 and 16 <= head_dim <= MAX_HEAD_DIM


def attention(q: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int, k_pages: torch.Tensor,
              v_pages: torch.Tensor, block_table: torch.Tensor, ctx, scale: float, window: int = 0,
              tile_seg: Optional[torch.Tensor] = None, tile_row0: Optional[torch.Tensor] = None,
              decode_work: Optional[torch.Tensor] = None) -> torch.Tensor:
    """bfloat16 with a head size in steps of 16 runs on the matrix cores: the split-key decode
    kernel for segments of one row (all of them, or those a mixed step begins with: a single row
    would hold a 64-row tile of the prompt kernel and walk its whole context alone), the tiled
    kernel for the rest (``tile_seg``, ``tile_row0``: the tiles of ``query_tiles`` in the order
    workgroups take them, those of the leading single rows in front; ``decode_work``: see
    ``attention_decode``); float32 and everything else on the generic kernel."""
    fast = q.dtype == torch.bfloat16 and attention_is_tiled(head_dim)
    if fast and ctx.all_decode:
        return attention_decode(q, num_heads, num_kv_heads, head_dim, k_pages, v_pages, block_table, ctx.row_seg,
                                ctx.row_pos, scale, ctx.max_context, window, decode_work=decode_work)
    if fast:
        if tile_seg is None or tile_row0 is None:
            raise KernelError("attention: the tiled kernel needs the step's query tiles")
        single = getattr(ctx, "decode_prefix", 0)       # leading segments of one row: rows and tiles 0 .. single - 1
        # four query heads of a kv group per workgroup pay where the rows sit behind a long context
        # (a page is read once for the four); from the start of a prompt one head per workgroup
        # gives more and shorter workgroups, which evens out the causal triangle
        rows = q.shape[0] - single
        keys = min(window, ctx.max_context) if window else ctx.max_context      # the most keys a row can see
        together = 4 if head_dim <= 64 and num_heads // num_kv_heads >= 4 and keys >= 4 * rows else 0
        if single == 0:
            return attention_prefill(q, num_heads, num_kv_heads, head_dim, k_pages, v_pages, block_table, tile_seg,
                                     tile_row0, ctx.seg_row0, ctx.row_pos, scale, window, heads_together=together)
        out = torch.empty_like(q)
        attention_decode(q[:single], num_heads, num_kv_heads, head_dim, k_pages, v_pages, block_table, ctx.row_seg,
                         ctx.row_pos, scale, ctx.max_context, window, out=out[:single], decode_work=decode_work)
        return attention_prefill(q, num_heads, num_kv_heads, head_dim, k_pages, v_pages, block_table,
                                 tile_seg[single:], tile_row0[single:], ctx.seg_row0, ctx.row_pos, scale, window,
                                 heads_together=together, out=out)
    return attention_generic(q, num_heads, num_kv_heads, head_dim, k_pages, v_pages, block_table, ctx.row_seg,
                             ctx.row_pos, scale, window)
