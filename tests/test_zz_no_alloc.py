"""The argmax entry point that allocates nothing (``fw_argmax_rows_static``), called through
ctypes as a caller outside the package would: against ``fw_argmax_rows`` on two calls in a row,
the second with a smaller input, so that what the first call left in the built-in scratch array
shows if it leaks into the second."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _library():
    from flyweight_amd.kernels.build import ensure_built
    lib = ctypes.CDLL(ensure_built())
    pointer, c_int = ctypes.c_void_p, ctypes.c_int
    lib.fw_argmax_rows.restype = c_int
    lib.fw_argmax_rows.argtypes = [pointer, pointer, pointer, pointer, pointer, c_int, c_int, pointer]
    lib.fw_argmax_rows_static.restype = c_int
    lib.fw_argmax_rows_static.argtypes = [pointer, pointer, pointer, pointer, c_int, c_int, pointer]
    lib.fw_argmax_rows_static_max_rows.restype = c_int
    lib.fw_last_error.restype = ctypes.c_char_p
    return lib


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _both(lib, logits, with_extras):
    rows, vocab = logits.shape
    device = logits.device
    outputs = []
    for static in (False, True):
        ids = torch.full((rows,), -1, dtype=torch.int32, device=device)
        also = torch.full((rows,), -1, dtype=torch.int32, device=device) if with_extras else None
        advance = torch.arange(rows, dtype=torch.int32, device=device) if with_extras else None
        extra = [ctypes.c_void_p(t.data_ptr() if t is not None else 0) for t in (also, advance)]
        if static:
            status = lib.fw_argmax_rows_static(logits.data_ptr(), ids.data_ptr(), *extra, rows, vocab, _stream())
        else:
            workspace = torch.empty((rows, 64), dtype=torch.int64, device=device)
            status = lib.fw_argmax_rows(logits.data_ptr(), ids.data_ptr(), *extra, workspace.data_ptr(), rows, vocab, _stream())
        assert status == 0, lib.fw_last_error().decode()
        torch.cuda.synchronize()
        outputs.append((ids.cpu(), None if also is None else also.cpu(), None if advance is None else advance.cpu()))
    return outputs


def test_argmax_without_allocation_equals_argmax_with_a_workspace():
    lib = _library()
    device = torch.device("cuda:0")
    generator = torch.Generator(device="cpu").manual_seed(3)
    limit = lib.fw_argmax_rows_static_max_rows()
    assert limit == 1024
    # first call: many rows, a vocabulary that is no power of two, ties (the lowest id must win)
    large = torch.randn((300, 65537), generator=generator).to(device)
    large[7, 100] = large[7, 60000] = 50.0
    large[8, :] = 0.0
    # second call, at once behind it: fewer rows, a small vocabulary (parts of the rows hold nothing)
    small = torch.randn((5, 37), generator=generator).to(device)
    small[2, 3] = small[2, 30] = 9.0
    for logits, with_extras in ((large, True), (small, False), (small, True)):
        reference, static = _both(lib, logits, with_extras)
        expected = logits.cpu().argmax(dim=1).to(torch.int32)
        assert torch.equal(static[0], reference[0])
        rows_without_ties = [r for r in range(logits.shape[0]) if (logits[r] == logits[r].max()).sum() == 1]
        assert torch.equal(static[0][rows_without_ties], expected[rows_without_ties])
        if with_extras:
            assert torch.equal(static[1], static[0]) and torch.equal(static[1], reference[1])
            assert torch.equal(static[2], torch.arange(logits.shape[0], dtype=torch.int32) + 1)
    assert _both(lib, large, False)[1][0][7] == 100 and _both(lib, large, False)[1][0][8] == 0
    assert _both(lib, small, False)[1][0][2] == 3
    # beyond the built-in scratch: refused, with the limit in the text; nothing runs
    too_many = torch.zeros((limit + 1, 8), device=device)
    ids = torch.full((limit + 1,), -1, dtype=torch.int32, device=device)
    status = lib.fw_argmax_rows_static(too_many.data_ptr(), ids.data_ptr(), None, None, limit + 1, 8, _stream())
    torch.cuda.synchronize()
    assert status == -1 and str(limit) in lib.fw_last_error().decode() and bool((ids == -1).all())
    # exactly the limit fits
    full = torch.randn((limit, 129), generator=generator).to(device)
    reference, static = _both(lib, full, False)
    assert torch.equal(static[0], reference[0]) and torch.equal(static[0], full.cpu().argmax(dim=1).to(torch.int32))
