"""Each kernel alone against a plain float64 computation, at other sizes than the engine's
tiny models use: widths and vocabularies that are no power of two, head sizes in steps of
16, odd numbers of heads and groups."""

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL = {torch.float32: 3e-6, torch.bfloat16: 1.2e-2}     # relative to the largest expected value
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops():
    from flyweight_amd.kernels import ops
    ops.library()
    return ops


def gen(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed + sum(shape))
    return torch.randn(*shape, generator=g, dtype=torch.float64) * scale


def close(found, expected, dtype, factor=1.0):
    found = found.detach().cpu().to(torch.float64)
    assert found.shape == expected.shape
    assert torch.isfinite(found).all()
    limit = TOL[dtype] * factor * max(1.0, float(expected.abs().max()))
    worst = float((found - expected).abs().max())
    assert worst <= limit, f"largest difference {worst:.3e} exceeds {limit:.3e}"


def as_dev(t, dtype):
    return t.to(dtype).to(DEV).contiguous()


def back(t):
    """What the kernel really saw after rounding to its dtype."""
    return t.detach().cpu().to(torch.float64)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed_rows(ops, dtype):
    table = as_dev(gen(301, 100), dtype)
    ids = torch.tensor([0, 300, 7, 7, 150], dtype=torch.int32, device=DEV)
    out = ops.embed_rows(table, ids)
    assert out.dtype == torch.float32 and torch.equal(out.cpu(), table.float().cpu()[ids.cpu().long()])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [100, 4100])
def test_rmsnorm_rows(ops, dtype, hidden):
    x = gen(7, hidden, scale=3).float()
    w = (1 + 0.1 * gen(hidden)).float()
    want = x.double() / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + 1e-4) * w.double()
    close(ops.rmsnorm_rows(x.to(DEV), w.to(DEV), 1e-4, dtype), want, dtype)
    index = torch.tensor([6, 0, 3], dtype=torch.int32, device=DEV)
    close(ops.rmsnorm_rows(x.to(DEV), w.to(DEV), 1e-4, dtype, row_index=index), want[[6, 0, 3]], dtype)
    centered = x.double() / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + 1e-4) * (1 + w.double())
    close(ops.rmsnorm_rows(x.to(DEV), w.to(DEV), 1e-4, dtype, one_centered=True), centered, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 70, 130), (5, 200, 96), (67, 129, 257), (130, 64, 40)])
def test_gemm(ops, dtype, M, N, K):
    a, w = as_dev(gen(M, K), dtype), as_dev(gen(N, K, seed=1, scale=K ** -0.5), dtype)
    bias = gen(N, seed=2).float().to(DEV)
    want = back(a) @ back(w).T
    close(ops.gemm(a, w), want, dtype)
    close(ops.gemm(a, w, bias, out_dtype=torch.float32), want + bias.cpu().double(), torch.float32)
    residual = gen(M, N, seed=3).float().to(DEV)
    before = residual.cpu().double()
    ops.gemm(a, w, accumulate_into=residual)
    close(residual, before + want, torch.float32)      # float32 sums of the rounded operands either way
    if dtype == torch.bfloat16:     # a 32-bit weight beside bfloat16 activations stays 32-bit
        w32 = gen(N, K, seed=1, scale=K ** -0.5).float().to(DEV)
        close(ops.gemm(a, w32, out_dtype=torch.float32), back(a) @ w32.cpu().double().T, torch.float32)


def test_gemm_rows_do_not_depend_on_the_batch(ops):
    a, w = as_dev(gen(70, 200), torch.float32), as_dev(gen(90, 200, seed=1), torch.float32)
    whole = ops.gemm(a, w)
    assert torch.equal(ops.gemm(a[13:14].contiguous(), w)[0], whole[13])
    assert torch.equal(ops.gemm(a[60:70].contiguous(), w), whole[60:70])


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu(ops, dtype):
    gu = as_dev(gen(5, 2 * 77, scale=4), dtype)
    gu[0, 0], gu[0, 1] = 80.0, -80.0        # the sigmoid must not overflow
    g, u = back(gu)[:, :77], back(gu)[:, 77:]
    out = ops.swiglu(gu)
    close(out, F.silu(g) * u, dtype)
    wide = as_dev(gen(5, 2 * 77, scale=4), torch.float32)       # float32 in, rounded once on the way out
    close(ops.swiglu(wide, out_dtype=dtype), F.silu(back(wide)[:, :77]) * back(wide)[:, 77:], dtype)


def test_rope_table(ops):
    positions = torch.tensor([0, 1, 63, 64, 4095, 131071], dtype=torch.int32, device=DEV)
    inv = (1e6 ** (-torch.arange(24, dtype=torch.float64) * 2 / 48)).to(DEV)
    cos, sin = ops.rope_table(positions, inv)
    angle = positions.cpu().double()[:, None] * inv.cpu()[None]
    assert float((cos.cpu().double() - torch.cos(angle)).abs().max()) < 1e-6
    assert float((sin.cpu().double() - torch.sin(angle)).abs().max()) < 1e-6


def conv_reference(bcx, taps, bias, state, segments):
    """Per segment: the plain left-padded convolution over [state | segment]."""
    rows, width = bcx.shape
    H, L = taps.shape
    out = torch.zeros(rows, H, dtype=torch.float64)
    new_state = state.clone()
    for first, count, slot in segments:
        part = bcx[first:first + count]
        bx = part[:, :H] * part[:, 2 * H:]
        seq = torch.cat([state[slot].T, bx], dim=0)                 # [L-1 + count, H]
        for t in range(count):
            y = (taps.T * seq[t:t + L]).sum(0)
            if bias is not None:
                y = y + bias
            out[first + t] = part[t, H:2 * H] * y
        new_state[slot] = seq[-(L - 1):].T
    return out, new_state


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,L,with_bias", [(70, 3, False), (130, 4, True), (257, 2, True), (64, 7, False)])
def test_shortconv_mixed_segments(ops, dtype, H, L, with_bias):
    # segments of 1, 2 (< L-1 for L = 4), L-1 and many rows; slots out of order
    counts = [5, 1, 2, L - 1, 40, 1]
    slots = [3, 0, 6, 2, 5, 1]
    segments, first = [], 0
    for count, slot in zip(counts, slots):
        segments.append((first, count, slot))
        first += count
    rows = first
    bcx = as_dev(gen(rows, 3 * H), dtype)
    taps = gen(H, L, seed=1).float()
    bias = gen(H, seed=2).float() if with_bias else None
    state = gen(7, H, L - 1, seed=3).float()
    want_out, want_state = conv_reference(back(bcx), taps.double(), None if bias is None else bias.double(), state.double(), segments)
    row_seg = torch.tensor([s for s, (_, c, _) in enumerate(segments) for _ in range(c)], dtype=torch.int32, device=DEV)
    seg_row0 = torch.tensor([f for f, _, _ in segments] + [rows], dtype=torch.int32, device=DEV)
    seg_slot = torch.tensor(slots, dtype=torch.int32, device=DEV)
    dev_state = state.to(DEV)
    out = ops.shortconv(bcx, taps.to(DEV), None if bias is None else bias.to(DEV), dev_state, row_seg, seg_row0, seg_slot, len(segments))
    close(out, want_out, dtype)
    close(dev_state, want_state, torch.float32, 10.0 if dtype == torch.bfloat16 else 1.0)
    # all single rows: the fused decode variant, from the state the first call left
    n = 4
    bcx1 = as_dev(gen(n, 3 * H, seed=5), dtype)
    segs1 = [(i, 1, s) for i, s in enumerate([2, 6, 0, 4])]
    want_out1, want_state1 = conv_reference(back(bcx1), taps.double(), None if bias is None else bias.double(),
                                            dev_state.cpu().double(), segs1)
    ids = torch.arange(n, dtype=torch.int32, device=DEV)
    out1 = ops.shortconv(bcx1, taps.to(DEV), None if bias is None else bias.to(DEV), dev_state, ids,
                         torch.arange(n + 1, dtype=torch.int32, device=DEV), torch.tensor([2, 6, 0, 4], dtype=torch.int32, device=DEV), n)
    close(out1, want_out1, dtype)
    close(dev_state, want_state1, torch.float32, 10.0 if dtype == torch.bfloat16 else 1.0)


def rope_reference(x, cos, sin, rotary):
    half = rotary // 2
    a, b, rest = x[..., :half], x[..., half:rotary], x[..., rotary:]
    return torch.cat([a * cos - b * sin, b * cos + a * sin, rest], dim=-1)


def scatter_setup(rows_per_seg, starts, num_pages, seed=0):
    """Block tables with scattered pages, and the per-row index arrays."""
    rng = np.random.default_rng(seed)
    pages = rng.permutation(num_pages).tolist()
    stride = max((s + n + 63) // 64 for s, n in zip(starts, rows_per_seg))
    table = np.zeros((len(starts), stride), dtype=np.int32)
    for i, (s, n) in enumerate(zip(starts, rows_per_seg)):
        for b in range((s + n + 63) // 64):
            table[i, b] = pages.pop()
    row_seg = np.concatenate([np.full(n, i) for i, n in enumerate(rows_per_seg)]).astype(np.int32)
    row_pos = np.concatenate([np.arange(s, s + n) for s, n in zip(starts, rows_per_seg)]).astype(np.int32)
    return table, row_seg, row_pos


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,hd,rotary,normed", [(4, 2, 16, 16, True), (3, 1, 48, 48, True), (6, 3, 80, 32, False),
                                                     (2, 2, 128, 128, True), (5, 5, 256, 0, True)])
def test_qk_norm_rope_kv_write(ops, dtype, nh, nkv, hd, rotary, normed):
    rows_per_seg, starts = [3, 1, 70], [0, 63, 60]
    table, row_seg, row_pos = scatter_setup(rows_per_seg, starts, num_pages=9)
    rows = sum(rows_per_seg)
    qkv = as_dev(gen(rows, (nh + 2 * nkv) * hd), dtype)
    qw, kw = (1 + 0.1 * gen(hd, seed=1)).float(), (1 + 0.1 * gen(hd, seed=2)).float()
    eps = 1e-5
    inv = (1e4 ** (-torch.arange(max(rotary // 2, 1), dtype=torch.float64) * 2 / max(rotary, 1)))
    angle = torch.tensor(row_pos, dtype=torch.float64)[:, None] * inv[None]
    cos, sin = torch.cos(angle), torch.sin(angle)
    k_pages = torch.full((9, nkv, 64, hd), 77.0, dtype=dtype, device=DEV)
    v_pages = torch.full((9, nkv, hd, 64), 77.0, dtype=dtype, device=DEV)
    d = lambda a: torch.tensor(a, device=DEV)       # noqa: E731
    q_out = ops.qk_norm_rope_kv_write(qkv, nh, nkv, hd, qw.to(DEV) if normed else None, kw.to(DEV) if normed else None, eps,
                                      cos.float().to(DEV) if rotary else None, sin.float().to(DEV) if rotary else None, rotary,
                                      k_pages, v_pages, d(table), d(row_seg), d(row_pos))
    x = back(qkv)
    q = x[:, :nh * hd].reshape(rows, nh, hd)
    k = x[:, nh * hd:(nh + nkv) * hd].reshape(rows, nkv, hd)
    v = x[:, (nh + nkv) * hd:].reshape(rows, nkv, hd)
    if normed:
        q = q / torch.sqrt((q ** 2).mean(-1, keepdim=True) + eps) * qw.double()
        k = k / torch.sqrt((k ** 2).mean(-1, keepdim=True) + eps) * kw.double()
    if rotary:
        q, k = rope_reference(q, cos[:, None], sin[:, None], rotary), rope_reference(k, cos[:, None], sin[:, None], rotary)
    close(q_out, q.reshape(rows, nh * hd), dtype)
    kp, vp = k_pages.cpu().double(), v_pages.cpu().double()
    for r in range(rows):
        page, slot = table[row_seg[r], row_pos[r] // 64], row_pos[r] % 64
        close(kp[page, :, slot, :], k[r], dtype)
        assert torch.equal(vp[page, :, :, slot], v[r])          # values are stored untouched
    written = torch.zeros(9, 64, dtype=torch.bool)
    for r in range(rows):
        written[table[row_seg[r], row_pos[r] // 64], row_pos[r] % 64] = True
    assert bool((kp.permute(0, 2, 1, 3)[~written] == 77.0).all()) and bool((vp.permute(0, 3, 1, 2)[~written] == 77.0).all())


def attention_reference(q, keys, values, pos, scale, window, group):
    out = torch.zeros_like(q)
    for head in range(q.shape[0]):
        lo = 0 if not window else max(0, pos - window + 1)
        s = (keys[lo:pos + 1, head // group] @ q[head]) * scale
        p = torch.softmax(s, dim=0)
        out[head] = p @ values[lo:pos + 1, head // group]
    return out


def paged(keys, values, table_row, num_pages, dtype, poison=float("nan")):
    """Scatter [T, nkv, hd] keys/values into pages; everything else is poison."""
    T, nkv, hd = keys.shape
    k_pages = torch.full((num_pages, nkv, 64, hd), poison, dtype=torch.float64)
    v_pages = torch.full((num_pages, nkv, hd, 64), poison, dtype=torch.float64)
    for t in range(T):
        k_pages[table_row[t // 64], :, t % 64, :] = keys[t]
        v_pages[table_row[t // 64], :, :, t % 64] = values[t]
    return k_pages.to(dtype).to(DEV), v_pages.to(dtype).to(DEV)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,hd,window", [(4, 2, 16, 0), (3, 1, 48, 0), (6, 3, 80, 0), (2, 2, 128, 0), (5, 1, 256, 0),
                                              (4, 2, 32, 70), (4, 4, 64, 64), (2, 1, 64, 1)])
def test_attention_over_scattered_pages(ops, dtype, nh, nkv, hd, window):
    # the block table of the reference's contract test: pages {9, 2, 14, 5} of a pool of 16
    # (native/tests/paged_kv_contract.cpp:89-242)
    T = 250
    table_row = [9, 2, 14, 5]
    keys, values = gen(T, nkv, hd).to(dtype).double(), gen(T, nkv, hd, seed=1).to(dtype).double()
    k_pages, v_pages = paged(keys, values, table_row, 16, dtype)
    positions = [0, 1, 62, 63, 64, 65, 127, 128, 129, 200, 249]
    q = as_dev(gen(len(positions), nh * hd, seed=2), dtype)
    scale = 1 / math.sqrt(hd)
    table = torch.tensor([table_row], dtype=torch.int32, device=DEV)
    row_seg = torch.zeros(len(positions), dtype=torch.int32, device=DEV)
    row_pos = torch.tensor(positions, dtype=torch.int32, device=DEV)
    out = ops.attention_generic(q, nh, nkv, hd, k_pages, v_pages, table, row_seg, row_pos, scale, window)
    want = torch.stack([attention_reference(back(q)[i].reshape(nh, hd), keys, values, p, scale, window, nh // nkv).reshape(-1)
                        for i, p in enumerate(positions)])
    close(out, want, dtype)


@pytest.mark.parametrize("nh,nkv,hd,window", [(4, 2, 16, 0), (32, 8, 64, 0), (3, 1, 48, 0), (5, 1, 24, 0), (8, 2, 128, 100), (2, 1, 256, 0)])
def test_where_the_pages_lie_changes_no_bit_of_any_attention_kernel(ops, nh, nkv, hd, window):
    """The paging contract of the reference (native/tests/paged_kv_contract.cpp:89-242): the
    same keys and values under the block table {9, 2, 14, 5} of a pool of 16 pages and under the
    identity table {0, 1, 2, 3} give the same result bit for bit, from every attention kernel:
    the wave-per-row one in both precisions, the tiled one (one head and four heads of a group per
    workgroup), the split-key one, and the one that also forms and writes the step's keys."""
    T = 250
    scattered, identity = [9, 2, 14, 5], [0, 1, 2, 3]
    keys, values = gen(T, nkv, hd).to(torch.bfloat16).double(), gen(T, nkv, hd, seed=1).to(torch.bfloat16).double()
    scale = 1 / math.sqrt(hd)
    d = lambda a: torch.tensor(np.asarray(a, dtype=np.int32), device=DEV)       # noqa: E731
    positions = [0, 1, 62, 63, 64, 65, 127, 128, 129, 200, 249]
    rows = len(positions)
    tiled = ops.attention_is_tiled(hd)

    def every_kernel(table_row, dtype):
        """name -> result of each kernel that takes this head size and precision, over pages
        laid out by ``table_row``; what no table names is not a number."""
        k_pages, v_pages = paged(keys, values, table_row, 16, dtype)
        table = d([table_row])
        q = as_dev(gen(rows, nh * hd, seed=2), dtype)
        found = {"generic": ops.attention_generic(q, nh, nkv, hd, k_pages, v_pages, table, d(np.zeros(rows)), d(positions), scale, window)}
        if dtype != torch.bfloat16 or not tiled:
            return found
        # a portion of the sequence: rows 120..249 of the one request, in tiles of 64
        portion = list(range(120, T))
        qp = as_dev(gen(len(portion), nh * hd, seed=3), dtype)
        tile_seg, tile_row0 = ops.query_tiles([0, len(portion)])
        for together in (1, 4) if hd <= 64 else (1,):
            found[f"tiled, {together} heads"] = ops.attention_prefill(
                qp, nh, nkv, hd, k_pages, v_pages, table, d(tile_seg), d(tile_row0), d([0, len(portion)]), d(portion), scale, window,
                heads_together=together)
        # decode: one row per request, four requests that share the one table row's pages at different lengths
        lengths = [250, 129, 64, 1]
        tables = d([table_row] * len(lengths))
        qd = as_dev(gen(len(lengths), nh * hd, seed=4), dtype)
        found["split-key"] = ops.attention_decode(qd, nh, nkv, hd, k_pages, v_pages, tables, d(np.arange(len(lengths))),
                                                  d([n - 1 for n in lengths]), scale, max_context=256, window=window)
        # the fused kernel writes the row's own key and value first: one request at position 249
        qkv = gen(1, (nh + 2 * nkv) * hd, seed=5).float().to(DEV)
        weight = (1 + 0.1 * gen(hd, seed=6)).float().to(DEV)
        inv = 1e4 ** (-torch.arange(hd // 2, dtype=torch.float64) * 2 / hd)
        angle = torch.tensor([T - 1], dtype=torch.float64)[:, None] * inv[None]
        found["fused"] = ops.attention_decode_fused(qkv, nh, nkv, hd, weight, weight, 1e-5, torch.cos(angle).float().to(DEV),
                                                    torch.sin(angle).float().to(DEV), hd, k_pages, v_pages, table, d([0]), d([T - 1]),
                                                    scale, max_context=256, window=window)
        page = table_row[(T - 1) // 64]
        found["fused: the key it wrote"] = k_pages[page, :, (T - 1) % 64, :].clone()
        found["fused: the value it wrote"] = v_pages[page, :, :, (T - 1) % 64].clone()
        return found

    for dtype in DTYPES:
        here, there = every_kernel(scattered, dtype), every_kernel(identity, dtype)
        assert here.keys() == there.keys()
        assert ("split-key" in here) == (dtype == torch.bfloat16 and tiled)
        for name in here:
            assert torch.isfinite(here[name].float()).all(), f"{name} ({dtype}) read a page that no table names"
            assert torch.equal(here[name], there[name]), f"{name} ({dtype}) depends on where the pages lie"


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_finds_one_far_key_and_the_edges_of_a_window(ops, dtype):
    """One key is made to match the query far better than all others, so the output is
    that key's value: at a far position, at both sides of every page edge, and just inside
    and just outside a window."""
    nh, nkv, hd, T = 2, 1, 64, 700
    table_row = list(range(11))
    scale = 1 / math.sqrt(hd)
    keys = gen(T, nkv, hd, scale=0.1)
    values = gen(T, nkv, hd, seed=1)
    direction = torch.zeros(hd, dtype=torch.float64); direction[5] = 1.0
    q = torch.zeros(1, nh * hd, dtype=torch.float64)
    q[0, 5] = q[0, hd + 5] = 60.0
    table = torch.tensor([table_row], dtype=torch.int32, device=DEV)
    zero = torch.zeros(1, dtype=torch.int32, device=DEV)
    pos = torch.tensor([T - 1], dtype=torch.int32, device=DEV)
    for target in (3, 63, 64, 127, 128, 640, 698, 699):
        k = keys.clone(); k[target, 0] = direction * 8
        k_pages, v_pages = paged(k.to(dtype).double(), values.to(dtype).double(), table_row, 11, dtype)
        out = ops.attention_generic(as_dev(q, dtype), nh, nkv, hd, k_pages, v_pages, table, zero, pos, scale, 0)
        close(out[0, :hd], values[target, 0].to(dtype).double(), dtype)
    window = 100            # the row at 699 sees 600..699
    for target, seen in ((600, True), (599, False), (640, True)):
        k = keys.clone(); k[target, 0] = direction * 8
        k_pages, v_pages = paged(k.to(dtype).double(), values.to(dtype).double(), table_row, 11, dtype)
        out = ops.attention_generic(as_dev(q, dtype), nh, nkv, hd, k_pages, v_pages, table, zero, pos, scale, window)
        hit = float((out[0, :hd].cpu().double() - values[target, 0].to(dtype).double()).abs().max()) < 0.05
        assert hit == seen, f"key {target} with a window of {window} at position {T - 1}"


def test_argmax(ops):
    logits = gen(5, 1000).float()
    logits[0, 17] = logits[0, 900] = 50.0               # ties go to the lowest id
    logits[1, 999] = 60.0                               # the last entry of a vocabulary that is no power of two
    logits[2, :] = -3.0                                 # all equal
    logits[3, 5] = float("nan"); logits[3, 6] = 40.0    # NaN sorts last
    ids = ops.argmax_rows(logits.to(DEV)).cpu().tolist()
    assert ids[:4] == [17, 999, 0, 6] and ids[4] == int(logits[4].argmax())
    # into a row of a record and into a second place (the next step's token ids; longer than the rows)
    record = torch.full((2, 5), -1, dtype=torch.int32, device=DEV)
    second = torch.full((8,), -1, dtype=torch.int32, device=DEV)
    counters = torch.arange(10, 18, dtype=torch.int32, device=DEV)       # a counter per row goes up by one
    assert ops.argmax_rows(logits.to(DEV), out=record[1], also=second, advance=counters).data_ptr() == record[1].data_ptr()
    assert record.cpu().tolist() == [[-1] * 5, ids] and second.cpu().tolist() == ids + [-1] * 3
    assert counters.cpu().tolist() == [11, 12, 13, 14, 15, 15, 16, 17]


def test_kernels_refuse_what_they_were_not_written_for(ops):
    from flyweight_amd.kernels.ops import KernelError
    x = torch.zeros(2, 8, device=DEV)
    with pytest.raises(KernelError, match="GPU only"):
        ops.rmsnorm_rows(torch.zeros(2, 8), torch.ones(8), 1e-5, torch.float32)
    with pytest.raises(KernelError, match="weight"):
        ops.rmsnorm_rows(x, torch.ones(9, device=DEV), 1e-5, torch.float32)
    with pytest.raises(KernelError):
        ops.gemm(x, torch.zeros(4, 9, device=DEV))
    with pytest.raises(KernelError, match="float32 or bfloat16"):
        ops.gemm(x.half(), torch.zeros(4, 8, device=DEV).half())
    with pytest.raises(KernelError, match="head_dim"):
        ops.attention_generic(torch.zeros(1, 512, device=DEV), 1, 1, 512, torch.zeros(1, 1, 64, 512, device=DEV),
                              torch.zeros(1, 1, 512, 64, device=DEV), torch.zeros(1, 1, dtype=torch.int32, device=DEV),
                              torch.zeros(1, dtype=torch.int32, device=DEV), torch.zeros(1, dtype=torch.int32, device=DEV), 1.0)
    with pytest.raises(KernelError, match="kernel size"):
        ops.shortconv(torch.zeros(1, 24, device=DEV), torch.zeros(8, 17, device=DEV), None, torch.zeros(1, 8, 16, device=DEV),
                      torch.zeros(1, dtype=torch.int32, device=DEV), torch.zeros(2, dtype=torch.int32, device=DEV),
                      torch.zeros(1, dtype=torch.int32, device=DEV), 1)


# ----- the matrix-core products ----------------------------------------------------------------
@pytest.mark.parametrize("M", [1, 8, 17, 64, 65, 128, 300])
@pytest.mark.parametrize("N,K", [(70, 64), (129, 96), (272, 136), (4100, 2056)])
def test_fast_gemm_every_epilogue(ops, M, N, K):
    a = as_dev(gen(M, K), torch.bfloat16)
    w = as_dev(gen(N, K, seed=1, scale=K ** -0.5), torch.bfloat16)
    bias = gen(N, seed=2).float().to(DEV)
    want = back(a) @ back(w).T
    close(ops.gemm(a, w, out_dtype=torch.float32), want, torch.float32, 2.0)
    close(ops.gemm(a, w, bias, out_dtype=torch.float32), want + bias.cpu().double(), torch.float32, 2.0)
    close(ops.gemm(a, w), want, torch.bfloat16, 0.4)        # one rounding of the result
    residual = gen(M, N, seed=3).float().to(DEV)
    before = residual.cpu().double()
    ops.gemm(a, w, accumulate_into=residual)
    close(residual, before + want, torch.float32, 2.0)
    if N % 2 == 0:
        half = N // 2
        act = F.silu(want[:, :half]) * want[:, half:]
        close(ops.gemm_swiglu(a, w), act, torch.bfloat16, 0.4)


@pytest.mark.parametrize("M,N,K,tiles", [(2048, 6144, 96, 256), (1500, 8200, 160, 198), (4000, 3100, 64, 208), (1800, 6000, 2080, 256),
                                         (1536, 6100, 96, 192), (2048, 3072, 96, 256), (1990, 3000, 2080, 256), (1900, 4000, 160, 240)])
def test_large_tile_prompt_product(ops, M, N, K, tiles):
    """Shapes that the large-tile kernel cuts into at least 192 tiles go to it: every epilogue,
    edges in both directions, few and many slabs. ``tiles`` tells which tile a storing or
    accumulating product takes: 256 x 256 (the second and third shape), 256 x 192 (the first,
    fourth and fifth: one round over the chip with the narrower tile), 128 x 192 (the sixth and
    seventh: 128 tiles of 256 rows, 256 of 128) and 128 x 256 (the last); the gated product keeps
    the 256 x 256 tiles."""
    assert ops.library().fw_gemm_mfma_big_tiles(0, M, N, K) == tiles and tiles >= ops.BIG_TILES_MIN
    assert not ops.library().fw_gemm_mfma_big_tiles(0, M, N, K + 8)
    a = as_dev(gen(M, K), torch.bfloat16)
    w = as_dev(gen(N, K, seed=1, scale=K ** -0.5), torch.bfloat16)
    bias = gen(N, seed=2).float().to(DEV)
    want = back(a) @ back(w).T
    close(ops.gemm(a, w, bias, out_dtype=torch.float32), want + bias.cpu().double(), torch.float32, 2.0)
    close(ops.gemm(a, w), want, torch.bfloat16, 0.4)
    residual = gen(M, N, seed=3).float().to(DEV)
    before = residual.cpu().double()
    ops.gemm(a, w, accumulate_into=residual)
    close(residual, before + want, torch.float32, 2.0)
    if N % 2 == 0 and ops.library().fw_gemm_mfma_big_tiles(2, M, N // 2, K) >= ops.BIG_TILES_MIN:
        half = N // 2
        close(ops.gemm_swiglu(a, w), F.silu(want[:, :half]) * want[:, half:], torch.bfloat16, 0.4)


@pytest.mark.parametrize("M,N,K", [(65, 2048, 2048), (128, 2048, 8192), (130, 104, 1032), (200, 3072, 2048), (300, 2500, 520),
                                   (1000, 200, 4096)])
def test_tiled_product_cuts_k_into_slices(ops, M, N, K):
    """More than 64 rows but fewer tiles than compute units: K goes to several workgroups and the
    last one of a tile to arrive adds the slices in their order. Every epilogue, edges in rows,
    features and K, twice in a row (the tickets are left at zero), and bitwise the same whichever
    workgroup came last."""
    import ctypes
    need_bytes, need_counters = ctypes.c_size_t(0), ctypes.c_int(0)
    assert ops.library().fw_gemm_mfma_split_plan(0, M, N, K, ctypes.byref(need_bytes), ctypes.byref(need_counters)) == 0
    assert need_bytes.value > 0 and need_counters.value > 0, "the shape is meant to be cut"
    a = as_dev(gen(M, K), torch.bfloat16)
    w = as_dev(gen(N, K, seed=1, scale=K ** -0.5), torch.bfloat16)
    bias = gen(N, seed=2).float().to(DEV)
    want = back(a) @ back(w).T
    first = ops.gemm(a, w, bias, out_dtype=torch.float32)
    close(first, want + bias.cpu().double(), torch.float32, 2.0)
    for _ in range(3):
        assert torch.equal(ops.gemm(a, w, bias, out_dtype=torch.float32), first)
    close(ops.gemm(a, w), want, torch.bfloat16, 0.4)
    residual = gen(M, N, seed=3).float().to(DEV)
    before = residual.cpu().double()
    ops.gemm(a, w, accumulate_into=residual)
    close(residual, before + want, torch.float32, 2.0)
    if N % 2 == 0:
        half = N // 2
        close(ops.gemm_swiglu(a, w), F.silu(want[:, :half]) * want[:, half:], torch.bfloat16, 0.4)


@pytest.mark.parametrize("columns", [128, 64])
@pytest.mark.parametrize("M,N,K", [(1, 1, 64), (128, 128, 64), (130, 70, 192), (300, 200, 448), (129, 257, 2112), (1000, 520, 8192)])
def test_tiles_whose_waves_split_k(ops, M, N, K, columns):
    """128 x 128 tiles of which every wave multiplies a quarter of each slab of K and the four
    partial tiles meet in LDS: one slab, fewer slabs than stages, many; edges in rows and
    features; store (float32, bfloat16) and accumulate; bitwise the same every time."""
    a = as_dev(gen(M, K), torch.bfloat16)
    w = as_dev(gen(N, K, seed=1, scale=K ** -0.5), torch.bfloat16)
    bias = gen(N, seed=2).float().to(DEV)
    want = back(a) @ back(w).T
    first = ops.gemm_deep(a, w, bias, out_dtype=torch.float32, columns=columns)
    close(first, want + bias.cpu().double(), torch.float32, 2.0)
    assert torch.equal(ops.gemm_deep(a, w, bias, out_dtype=torch.float32, columns=columns), first)
    close(ops.gemm_deep(a, w, columns=columns), want, torch.bfloat16, 0.4)
    residual = gen(M, N, seed=3).float().to(DEV)
    before = residual.cpu().double()
    ops.gemm_deep(a, w, accumulate_into=residual, columns=columns)
    close(residual, before + want, torch.float32, 2.0)
    with pytest.raises(ops.KernelError, match="multiple of 64"):
        ops.gemm_deep(a[:, :K - 8].contiguous(), w[:, :K - 8].contiguous())


@pytest.mark.parametrize("M,N,K,expected", [(2048, 2048, 4096, 128), (1800, 1990, 4160, 128), (2048, 1024, 2048, 64),
                                            (1152, 2048, 2048, 128), (576, 2048, 1024, 64), (2304, 2048, 1024, 64)])
def test_the_prompt_product_of_one_round_of_tiles_over_a_long_k(ops, M, N, K, expected):
    """What the dispatch sends to those tiles: about one 128 x 128 tile per compute unit and a
    long K (the w2 product of a 2,048-token prompt); for a product that adds into the residual
    also rounds that are little more than half full, on the width that fills them better."""
    columns = ops._deep_columns(1, M, N, K)
    assert columns == expected and K >= ops.DEEP_MIN_K
    assert ops._deep_columns(1, 512, 2048, 8192) == 0 and ops._deep_columns(0, 1152, 2048, 8192) == 0
    a = as_dev(gen(M, K), torch.bfloat16)
    w = as_dev(gen(N, K, seed=1, scale=K ** -0.5), torch.bfloat16)
    want = back(a) @ back(w).T
    residual = gen(M, N, seed=3).float().to(DEV)
    before = residual.cpu().double()
    ops.gemm(a, w, accumulate_into=residual)
    close(residual, before + want, torch.float32, 2.0)
    direct = before.float().to(DEV)
    ops.gemm_deep(a, w, accumulate_into=direct, columns=columns)
    assert torch.equal(direct, residual)
    close(ops.gemm(a, w, out_dtype=torch.float32), want, torch.float32, 2.0)


@pytest.mark.parametrize("M,N,K,mode,columns", [(256, 6144, 2048, 0, 64), (500, 6100, 1984, 0, 128), (130, 6144, 2048, 0, 64),
                                                   (512, 2048, 2048, 1, 64), (320, 2048, 2048, 1, 64), (300, 3072, 1024, 0, 64),
                                                   (256, 2048, 8192, 1, 0), (600, 6144, 2048, 0, 0), (256, 1024, 2048, 0, 0)])
def test_a_few_hundred_rows_go_to_the_tiles_whose_waves_split_k(ops, M, N, K, mode, columns):
    """A decode step of a few hundred requests: storing and short accumulating products take those
    tiles when they are not too few (equal, bit for bit, to the kernel called by name); a long K,
    more rows or too few tiles stay with the other products."""
    assert ops._deep_columns_few_rows(mode, M, N, K) == columns
    a = as_dev(gen(M, K), torch.bfloat16)
    w = as_dev(gen(N, K, seed=1, scale=K ** -0.5), torch.bfloat16)
    want = back(a) @ back(w).T
    if mode == 0:
        got = ops.gemm(a, w, out_dtype=torch.float32)
        close(got, want, torch.float32, 2.0)
        if columns:
            assert torch.equal(got, ops.gemm_deep(a, w, out_dtype=torch.float32, columns=columns))
    else:
        residual = gen(M, N, seed=3).float().to(DEV)
        before = residual.cpu().double()
        ops.gemm(a, w, accumulate_into=residual)
        close(residual, before + want, torch.float32, 2.0)
        if columns:
            direct = before.float().to(DEV)
            ops.gemm_deep(a, w, accumulate_into=direct, columns=columns)
            assert torch.equal(direct, residual)


def test_fast_gemm_rows_do_not_depend_on_the_batch(ops):
    a = as_dev(gen(300, 256), torch.bfloat16)
    w = as_dev(gen(200, 256, seed=1), torch.bfloat16)
    whole = ops.gemm(a, w, out_dtype=torch.float32)
    assert torch.equal(ops.gemm(a[100:230].contiguous(), w, out_dtype=torch.float32), whole[100:230])
    few = ops.gemm(a[:40].contiguous(), w, out_dtype=torch.float32)
    assert torch.equal(ops.gemm(a[7:30].contiguous(), w, out_dtype=torch.float32), few[7:30])
    fewer = ops.gemm(a[:12].contiguous(), w, out_dtype=torch.float32)
    assert torch.equal(ops.gemm(a[7:8].contiguous(), w, out_dtype=torch.float32)[0], fewer[7])
    # the kernels for few, some and many rows sum in different orders: equal up to float32 rounding
    close(few, whole[:40].cpu().double(), torch.float32, 2.0)
    close(fewer, whole[:12].cpu().double(), torch.float32, 2.0)


@pytest.mark.parametrize("M", [17, 33, 48, 64])
@pytest.mark.parametrize("N,K", [(64, 4096), (96, 520), (2048, 8192), (6144, 2048), (25000, 72)])
def test_medium_gemm_splits_k_over_workgroups(ops, M, N, K):
    """Few features and a long K: slices of K go to different workgroups and the last one to
    arrive sums them in slice order. Twice in a row (the tickets are left at zero), every
    epilogue, and bitwise the same whichever workgroup came last."""
    a = as_dev(gen(M, K), torch.bfloat16)
    w = as_dev(gen(N, K, seed=1, scale=K ** -0.5), torch.bfloat16)
    bias = gen(N, seed=2).float().to(DEV)
    want = back(a) @ back(w).T
    first = ops.gemm(a, w, bias, out_dtype=torch.float32)
    close(first, want + bias.cpu().double(), torch.float32, 2.0)
    for _ in range(3):
        assert torch.equal(ops.gemm(a, w, bias, out_dtype=torch.float32), first)
    # other rows through the same workspace: nothing of the call before may be seen again
    for seed in (7, 8):
        other = as_dev(gen(M, K, seed=seed), torch.bfloat16)
        close(ops.gemm(other, w, out_dtype=torch.float32), back(other) @ back(w).T, torch.float32, 2.0)
    close(ops.gemm(a, w), want, torch.bfloat16, 0.4)
    residual = gen(M, N, seed=3).float().to(DEV)
    before = residual.cpu().double()
    ops.gemm(a, w, accumulate_into=residual)
    close(residual, before + want, torch.float32, 2.0)
    half = N // 2
    close(ops.gemm_swiglu(a, w), F.silu(want[:, :half]) * want[:, half:], torch.bfloat16, 0.4)


# ----- attention on the matrix cores -------------------------------------------------------------
def _mfma_setup(nh, nkv, hd, lengths, num_pages, seed=0):
    """Several sequences with scattered pages; everything not written is NaN."""
    rng = np.random.default_rng(seed)
    order = rng.permutation(num_pages).tolist()
    stride = max((n + 63) // 64 for n in lengths)
    table = np.zeros((len(lengths), stride), dtype=np.int32)
    keys, values = [], []
    k_pages = torch.full((num_pages, nkv, 64, hd), float("nan"), dtype=torch.float64)
    v_pages = torch.full((num_pages, nkv, hd, 64), float("nan"), dtype=torch.float64)
    for i, n in enumerate(lengths):
        k = gen(n, nkv, hd, seed=seed + 10 * i).to(torch.bfloat16).double()
        v = gen(n, nkv, hd, seed=seed + 10 * i + 1).to(torch.bfloat16).double()
        keys.append(k); values.append(v)
        for b in range((n + 63) // 64):
            table[i, b] = order.pop()
        for t in range(n):
            k_pages[table[i, t // 64], :, t % 64, :] = k[t]
            v_pages[table[i, t // 64], :, :, t % 64] = v[t]
    return keys, values, table, k_pages.to(torch.bfloat16).to(DEV), v_pages.to(torch.bfloat16).to(DEV)


@pytest.mark.parametrize("nh,nkv,hd,window", [(4, 2, 16, 0), (3, 1, 48, 0), (6, 3, 80, 0), (32, 8, 64, 0), (2, 2, 128, 0),
                                              (16, 1, 256, 0), (4, 2, 32, 70), (4, 4, 64, 64), (2, 1, 64, 1)])
def test_attention_prefill_on_the_matrix_cores(ops, nh, nkv, hd, window):
    # segments: a whole prompt, a continuation across a page edge, single rows, a tile and one row
    lengths = [150, 200, 64, 65, 33]
    starts = [0, 120, 63, 64, 16]
    keys, values, table, k_pages, v_pages = _mfma_setup(nh, nkv, hd, lengths, num_pages=14, seed=3)
    counts = [n - s for n, s in zip(lengths, starts)]
    seg_row0 = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    row_pos = np.concatenate([np.arange(s, n) for s, n in zip(starts, lengths)]).astype(np.int32)
    row_seg = np.concatenate([np.full(c, i) for i, c in enumerate(counts)]).astype(np.int32)
    tile_seg, tile_row0 = ops.query_tiles(seg_row0.tolist())
    rows = int(seg_row0[-1])
    q = as_dev(gen(rows, nh * hd, seed=2), torch.bfloat16)
    scale = 1 / math.sqrt(hd)
    d = lambda a: torch.tensor(np.asarray(a, dtype=np.int32), device=DEV)       # noqa: E731
    out = ops.attention_prefill(q, nh, nkv, hd, k_pages, v_pages, d(table), d(tile_seg), d(tile_row0), d(seg_row0),
                                d(row_pos), scale, window)
    want = torch.stack([attention_reference(back(q)[r].reshape(nh, hd), keys[row_seg[r]], values[row_seg[r]], int(row_pos[r]),
                                            scale, window, nh // nkv).reshape(-1) for r in range(rows)])
    close(out, want, torch.bfloat16)
    # the generic kernel on the same cache agrees (it runs the same rows when the batch is float32)
    generic = ops.attention_generic(q, nh, nkv, hd, torch.nan_to_num(k_pages), torch.nan_to_num(v_pages), d(table),
                                    d(row_seg), d(row_pos), scale, window)
    close(generic, want, torch.bfloat16)


@pytest.mark.parametrize("window", [0, 50])
def test_attention_gives_the_leading_single_rows_of_a_mixed_step_to_the_decode_kernel(ops, window):
    """A step that begins with decoded tokens and goes on with portions of prompts: the single rows
    in front go through the split-key kernel, everything else (a single row further back too)
    through the tiled one, and both write one output."""
    from types import SimpleNamespace
    nh, nkv, hd = 8, 2, 64
    lengths = [131, 6, 57, 71, 300]
    starts = [130, 5, 20, 70, 290]
    keys, values, table, k_pages, v_pages = _mfma_setup(nh, nkv, hd, lengths, num_pages=16, seed=9)
    counts = [n - s for n, s in zip(lengths, starts)]
    seg_row0 = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    row_pos = np.concatenate([np.arange(s, n) for s, n in zip(starts, lengths)]).astype(np.int32)
    row_seg = np.concatenate([np.full(c, i) for i, c in enumerate(counts)]).astype(np.int32)
    tile_seg, tile_row0 = ops.query_tiles(seg_row0.tolist())
    rows = int(seg_row0[-1])
    q = as_dev(gen(rows, nh * hd, seed=8), torch.bfloat16)
    scale = 1 / math.sqrt(hd)
    d = lambda a: torch.tensor(np.asarray(a, dtype=np.int32), device=DEV)       # noqa: E731
    ctx = SimpleNamespace(all_decode=False, decode_prefix=2, max_context=max(lengths), row_seg=d(row_seg), row_pos=d(row_pos),
                          seg_row0=d(seg_row0))
    tiles = dict(tile_seg=d(tile_seg), tile_row0=d(tile_row0))
    mixed = ops.attention(q, nh, nkv, hd, k_pages, v_pages, d(table), ctx, scale, window, **tiles)
    want = torch.stack([attention_reference(back(q)[r].reshape(nh, hd), keys[row_seg[r]], values[row_seg[r]], int(row_pos[r]),
                                            scale, window, nh // nkv).reshape(-1) for r in range(rows)])
    close(mixed, want, torch.bfloat16)
    ctx.decode_prefix = 0
    tiled = ops.attention(q, nh, nkv, hd, k_pages, v_pages, d(table), ctx, scale, window, **tiles)
    assert torch.equal(mixed[2:], tiled[2:])        # the rows of the tiled kernel do not depend on who else it serves


@pytest.mark.parametrize("nh,nkv,hd,window", [(4, 1, 16, 0), (3, 1, 48, 0), (12, 2, 64, 0), (32, 8, 64, 0), (8, 2, 32, 70)])
def test_attention_prefill_takes_four_heads_of_a_group_together(ops, nh, nkv, hd, window):
    """One workgroup reads a page once for four query heads of the kv group: whole runs of four,
    a group of three (one head idle), a group of six (a run of four and one of two), head sizes
    below the kernel's, a window. Against the reference and bitwise against one head at a time."""
    lengths = [150, 200, 64, 65, 33]
    starts = [0, 120, 63, 64, 16]
    keys, values, table, k_pages, v_pages = _mfma_setup(nh, nkv, hd, lengths, num_pages=14, seed=5)
    counts = [n - s for n, s in zip(lengths, starts)]
    seg_row0 = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    row_pos = np.concatenate([np.arange(s, n) for s, n in zip(starts, lengths)]).astype(np.int32)
    row_seg = np.concatenate([np.full(c, i) for i, c in enumerate(counts)]).astype(np.int32)
    tile_seg, tile_row0 = ops.query_tiles(seg_row0.tolist())
    rows = int(seg_row0[-1])
    q = as_dev(gen(rows, nh * hd, seed=4), torch.bfloat16)
    scale = 1 / math.sqrt(hd)
    d = lambda a: torch.tensor(np.asarray(a, dtype=np.int32), device=DEV)       # noqa: E731
    run = lambda together: ops.attention_prefill(q, nh, nkv, hd, k_pages, v_pages, d(table), d(tile_seg), d(tile_row0),  # noqa: E731
                                                 d(seg_row0), d(row_pos), scale, window, heads_together=together)
    four = run(4)
    want = torch.stack([attention_reference(back(q)[r].reshape(nh, hd), keys[row_seg[r]], values[row_seg[r]], int(row_pos[r]),
                                            scale, window, nh // nkv).reshape(-1) for r in range(rows)])
    close(four, want, torch.bfloat16)
    assert torch.equal(four, run(1))
    with pytest.raises(ops.KernelError, match="heads together"):
        run(2)


@pytest.mark.parametrize("nh,nkv,hd,window", [(4, 2, 16, 0), (3, 1, 48, 0), (6, 3, 80, 0), (32, 8, 64, 0), (2, 2, 128, 0),
                                              (20, 1, 256, 0), (4, 2, 32, 300), (4, 4, 64, 64), (2, 1, 64, 1)])
def test_attention_decode_on_the_matrix_cores(ops, nh, nkv, hd, window):
    lengths = [1, 64, 65, 256, 257, 700, 1000]
    keys, values, table, k_pages, v_pages = _mfma_setup(nh, nkv, hd, lengths, num_pages=40, seed=5)
    rows = len(lengths)
    q = as_dev(gen(rows, nh * hd, seed=2), torch.bfloat16)
    scale = 1 / math.sqrt(hd)
    d = lambda a: torch.tensor(np.asarray(a, dtype=np.int32), device=DEV)       # noqa: E731
    positions = [n - 1 for n in lengths]
    out = ops.attention_decode(q, nh, nkv, hd, k_pages, v_pages, d(table), d(np.arange(rows)), d(positions), scale,
                               max_context=max(lengths), window=window)
    want = torch.stack([attention_reference(back(q)[r].reshape(nh, hd), keys[r], values[r], positions[r], scale, window,
                                            nh // nkv).reshape(-1) for r in range(rows)])
    close(out, want, torch.bfloat16)
    # a larger bound on the context changes the grid, not the result
    again = ops.attention_decode(q, nh, nkv, hd, k_pages, v_pages, d(table), d(np.arange(rows)), d(positions), scale,
                                 max_context=1024, window=window)
    assert torch.equal(again, out)
    # however the work is shared out, the result is the reference's: one run of pages per workgroup, a few, all
    for work in (1, 40, 700, 5000, 1 << 20):
        shared = ops.attention_decode(q, nh, nkv, hd, k_pages, v_pages, d(table), d(np.arange(rows)), d(positions), scale,
                                      max_context=1024, window=window, decode_work=d([work]))
        close(shared, want, torch.bfloat16)
    # a row's result does not depend on the rest of the batch
    alone = ops.attention_decode(q[5:6].contiguous(), nh, nkv, hd, k_pages, v_pages, d(table[5:6]), d([0]), d([positions[5]]),
                                 scale, max_context=lengths[5], window=window)
    assert torch.equal(alone[0], out[5])
    from flyweight_amd.kernels.ops import KernelError
    with pytest.raises(KernelError, match="do not cover|exceeds the block table"):
        ops.library()
        import ctypes
        partial = torch.empty(rows * nh * (hd + 4), device=DEV)
        status = ops.library().fw_attention_decode(
            ctypes.c_void_p(q.data_ptr()), ctypes.c_void_p(out.data_ptr()), ctypes.c_void_p(partial.data_ptr()), 1, 100000,
            None, None, 0, ctypes.c_void_p(k_pages.data_ptr()), ctypes.c_void_p(v_pages.data_ptr()), ctypes.c_void_p(d(table).data_ptr()),
            table.shape[1], ctypes.c_void_p(d(np.arange(rows)).data_ptr()), ctypes.c_void_p(d(positions).data_ptr()), rows, nh,
            nkv, hd, ctypes.c_float(scale), 0, 64, 40, None)
        ops._check(status)


def test_matrix_core_attention_finds_one_far_key_and_the_edges_of_a_window(ops):
    """The same single-dominant-key cases as for the generic kernel, for both fast kernels."""
    nh, nkv, hd, T = 8, 2, 64, 700
    scale = 1 / math.sqrt(hd)
    table = np.arange(11, dtype=np.int32)[None]
    base_keys = gen(T, nkv, hd, scale=0.1)
    values = gen(T, nkv, hd, seed=1).to(torch.bfloat16).double()
    direction = torch.zeros(hd, dtype=torch.float64); direction[5] = 1.0
    q = torch.zeros(1, nh * hd, dtype=torch.float64)
    q[0, 5::hd] = 60.0
    d = lambda a: torch.tensor(np.asarray(a, dtype=np.int32), device=DEV)       # noqa: E731

    def run(target, window):
        k = base_keys.clone(); k[target, :] = direction * 8
        k_pages = torch.full((11, nkv, 64, hd), float("nan"), dtype=torch.float64)
        v_pages = torch.full((11, nkv, hd, 64), float("nan"), dtype=torch.float64)
        for t in range(T):
            k_pages[t // 64, :, t % 64, :] = k[t]
            v_pages[t // 64, :, :, t % 64] = values[t]
        k_pages, v_pages = k_pages.to(torch.bfloat16).to(DEV), v_pages.to(torch.bfloat16).to(DEV)
        qd = as_dev(q, torch.bfloat16)
        dec = ops.attention_decode(qd, nh, nkv, hd, k_pages, v_pages, d(table), d([0]), d([T - 1]), scale, T, window)
        pre = ops.attention_prefill(qd, nh, nkv, hd, k_pages, v_pages, d(table), d([0]), d([0]), d([0, 1]), d([T - 1]), scale, window)
        return dec[0].cpu().double().reshape(nh, hd), pre[0].cpu().double().reshape(nh, hd)

    for target in (3, 63, 64, 127, 128, 255, 256, 640, 698, 699):
        for found in run(target, 0):
            for head in range(nh):
                assert float((found[head] - values[target, head // 4]).abs().max()) < 0.05, f"key {target}"
    for target, seen in ((600, True), (599, False), (640, True)):
        for found in run(target, 100):
            hit = float((found[0] - values[target, 0]).abs().max()) < 0.05
            assert hit == seen, f"key {target} with a window of 100 at position {T - 1}"


# ----- the fused decode product -----------------------------------------------------------------
def _normed(x, weight, eps, one_centered=False):
    w = 1 + weight if one_centered else weight
    return x / torch.sqrt((x ** 2).mean(-1, keepdim=True) + eps) * w


def _kernel_norm(ops, x, norm_w, eps, index=None, one_centered=False):
    """The normed rows exactly as the fused kernel forms them (x * w rounded to bfloat16, times
    the row's 1/rms): its product with an identity matrix. They are checked against the float64
    norm to one bfloat16 rounding; the products are then checked against THESE rows, so that a
    value the kernel rounds the other way than float64 would does not pass for an error of the
    product."""
    K = x.shape[1]
    identity = torch.eye(K, dtype=torch.bfloat16, device=DEV)
    h = ops.gemm_decode(x.to(DEV), identity, ops.EPILOGUE_STORE, norm_weight=norm_w.to(DEV), eps=eps, one_centered=one_centered,
                        row_index=None if index is None else index.to(DEV), out_dtype=torch.float32).cpu().double()
    exact = _normed(x.double(), norm_w.double(), eps, one_centered)
    exact = exact if index is None else exact[index.long()]
    assert float(((h - exact).abs() / exact.abs().clamp_min(1e-3)).max()) <= 2.0 ** -8        # bfloat16: 8 bits of mantissa
    return h


@pytest.mark.parametrize("M", [1, 5, 8, 9, 16])
@pytest.mark.parametrize("N,K", [(72, 64), (200, 96), (4096, 512), (4104, 136), (16400, 256), (2048, 4096)])
def test_fused_decode_product(ops, M, N, K):
    """Norm prologue or plain activations, every epilogue, outputs narrower and wider than one
    tile per compute unit, K that is no multiple of the chunk."""
    x = gen(M + 3, K, scale=2).float()
    norm_w = (1 + 0.1 * gen(K, seed=1)).float()
    w = as_dev(gen(N, K, seed=2, scale=K ** -0.5), torch.bfloat16)
    bias = gen(N, seed=3).float()
    eps = 1e-5
    index = torch.tensor(list(range(M + 2, 2, -1)), dtype=torch.int32)      # rows gathered in reverse
    h = _kernel_norm(ops, x, norm_w, eps, index)         # what the kernel keeps in LDS
    want = h @ back(w).T
    assert ops.gemm_decode_fits(M, N, K, ops.EPILOGUE_STORE)
    got = ops.gemm_decode(x.to(DEV), w, ops.EPILOGUE_STORE, norm_weight=norm_w.to(DEV), eps=eps, row_index=index.to(DEV),
                          out_dtype=torch.float32)
    close(got, want, torch.float32, 2.0)
    got = ops.gemm_decode(x.to(DEV), w, ops.EPILOGUE_STORE, norm_weight=norm_w.to(DEV), eps=eps, row_index=index.to(DEV),
                          bias=bias.to(DEV), out_dtype=torch.bfloat16)
    close(got, want + bias.double(), torch.bfloat16, 0.4)
    centered = _kernel_norm(ops, x[:M].contiguous(), norm_w, eps, one_centered=True) @ back(w).T
    got = ops.gemm_decode(x[:M].contiguous().to(DEV), w, ops.EPILOGUE_STORE, norm_weight=norm_w.to(DEV), eps=eps, one_centered=True,
                          out_dtype=torch.float32)
    close(got, centered, torch.float32, 2.0)
    # plain bfloat16 activations; adding into the residual stream
    a = as_dev(gen(M, K, seed=4), torch.bfloat16)
    plain = back(a) @ back(w).T
    close(ops.gemm_decode(a, w, ops.EPILOGUE_STORE, out_dtype=torch.float32), plain, torch.float32, 2.0)
    residual = gen(M, N, seed=5).float().to(DEV)
    before = residual.cpu().double()
    ops.gemm_decode(a, w, ops.EPILOGUE_ACCUMULATE, accumulate_into=residual, bias=bias.to(DEV))
    close(residual, before + plain + bias.double(), torch.float32, 2.0)
    # the same product from the skinny kernel agrees to float32 rounding
    close(ops.gemm(a, w, out_dtype=torch.float32), plain, torch.float32, 2.0)
    if N % 2 == 0:
        half = N // 2
        close(ops.gemm_decode(a, w, ops.EPILOGUE_SWIGLU), F.silu(plain[:, :half]) * plain[:, half:], torch.bfloat16, 0.4)
        got = ops.gemm_decode(x.to(DEV), w, ops.EPILOGUE_SWIGLU, norm_weight=norm_w.to(DEV), eps=eps, row_index=index.to(DEV))
        close(got, F.silu(want[:, :half]) * want[:, half:], torch.bfloat16, 0.4)


@pytest.mark.parametrize("M", [1, 7, 16])
@pytest.mark.parametrize("H,L,with_bias", [(72, 3, False), (136, 4, True), (4096, 2, True)])
def test_fused_decode_product_with_the_convolution_epilogue(ops, M, H, L, with_bias):
    K = 256 if H > 1000 else H
    x = gen(M, K, scale=2).float()
    norm_w = (1 + 0.1 * gen(K, seed=1)).float()
    w = as_dev(gen(3 * H, K, seed=2, scale=K ** -0.5), torch.bfloat16)
    in_bias = gen(3 * H, seed=3).float() if with_bias else None
    taps = gen(H, L, seed=4).float()
    conv_bias = gen(H, seed=5).float() if with_bias else None
    state = gen(M + 2, H, L - 1, seed=6).float()
    slots = torch.tensor(list(range(M + 1, 1, -1)), dtype=torch.int32)
    eps = 1e-6
    h = _kernel_norm(ops, x, norm_w, eps)
    bcx = h @ back(w).T + (in_bias.double() if with_bias else 0)
    segments = [(i, 1, int(slots[i])) for i in range(M)]
    want_out, want_state = conv_reference(bcx, taps.double(), None if conv_bias is None else conv_bias.double(), state.double(), segments)
    dev_state = state.to(DEV)
    d = lambda t: None if t is None else t.to(DEV)      # noqa: E731
    got = ops.gemm_decode(x.to(DEV), w, ops.EPILOGUE_CONV, norm_weight=norm_w.to(DEV), eps=eps, bias=d(in_bias), taps=taps.to(DEV),
                          conv_bias=d(conv_bias), state=dev_state, seg_slot=slots.to(DEV), out_dtype=torch.bfloat16)
    close(got, want_out, torch.bfloat16, 0.6)
    close(dev_state, want_state, torch.float32, 4.0)
    # and from bfloat16 activations, float32 out
    a = as_dev(gen(M, K, seed=7), torch.bfloat16)
    bcx = back(a) @ back(w).T + (in_bias.double() if with_bias else 0)
    want_out, want_state2 = conv_reference(bcx, taps.double(), None if conv_bias is None else conv_bias.double(), want_state, segments)
    got = ops.gemm_decode(a, w, ops.EPILOGUE_CONV, bias=d(in_bias), taps=taps.to(DEV), conv_bias=d(conv_bias), state=dev_state,
                          seg_slot=slots.to(DEV), out_dtype=torch.float32)
    close(got, want_out, torch.float32, 4.0)
    close(dev_state, want_state2, torch.float32, 4.0)


@pytest.mark.parametrize("M", [1, 6, 16])
@pytest.mark.parametrize("H,N,one_centered,K", [(72, 80, False, 136), (200, 96, True, 136), (4104, 144, False, 136),
                                                 (2048, 6144, True, 136), (2048, 96, False, 8192), (104, 96, True, 4104)])
def test_fused_decode_product_prepares_the_next_norm(ops, M, H, N, one_centered, K):
    """The product that adds to the residual stream leaves x * w of the norm after it and sums
    of squares per tile; the next product takes both instead of norming itself. Checked: what
    is left, and the next product (every epilogue that may follow) against a plain norm. With a
    long K the accumulating product is the one that splits K over workgroups."""
    a = as_dev(gen(M, K, seed=1), torch.bfloat16)
    w_out = as_dev(gen(H, K, seed=2, scale=K ** -0.5), torch.bfloat16)
    residual = gen(M, H, seed=3, scale=2).float().to(DEV)
    norm_w = (0.1 * gen(H, seed=4) + (0 if one_centered else 1)).float()
    eps = 1e-5
    x_new = residual.cpu().double() + back(a) @ back(w_out).T
    activations, squares = ops.gemm_decode(a, w_out, ops.EPILOGUE_ACCUMULATE, accumulate_into=residual,
                                           next_norm_weight=norm_w.to(DEV), next_one_centered=one_centered)
    close(residual, x_new, torch.float32, 2.0)
    x_kernel = residual.cpu().double()               # the float32 values the kernel squared and scaled
    scale = norm_w.double() + (1 if one_centered else 0)
    assert activations.dtype == torch.bfloat16 and squares.shape[1] == 16
    assert torch.equal(activations.cpu(), (x_kernel.float() * scale.float()).to(torch.bfloat16))
    total = squares.cpu().double().sum(0)
    assert float((total[:M] - (x_kernel ** 2).sum(-1)).abs().max()) <= 1e-5 * float((x_kernel ** 2).sum(-1).max())
    assert float(total[M:].abs().max()) == 0.0 if M < 16 else True
    # the following product: rows as the kernel forms them are activations * 1/rms
    inv = 1.0 / torch.sqrt((x_kernel ** 2).mean(-1, keepdim=True) + eps)
    h = activations.cpu().double() * inv
    w = as_dev(gen(N, H, seed=5, scale=H ** -0.5), torch.bfloat16)
    want = h @ back(w).T
    got = ops.gemm_decode(activations, w, ops.EPILOGUE_STORE, squares=squares, eps=eps, out_dtype=torch.float32)
    close(got, want, torch.float32, 2.0)
    fused = ops.gemm_decode(residual, w, ops.EPILOGUE_STORE, norm_weight=norm_w.to(DEV), eps=eps, one_centered=one_centered,
                            out_dtype=torch.float32)
    close(got, fused.cpu().double(), torch.float32, 2.0)        # the norm done in the product's own prologue agrees
    half = N // 2
    got = ops.gemm_decode(activations, w, ops.EPILOGUE_SWIGLU, squares=squares, eps=eps)
    close(got, F.silu(want[:, :half]) * want[:, half:], torch.bfloat16, 0.4)
    if N % 3 == 0:
        C, L = N // 3, 3
        taps, state = gen(C, L, seed=6).float(), gen(M, C, L - 1, seed=7).float()
        slots = torch.arange(M - 1, -1, -1, dtype=torch.int32)
        segments = [(i, 1, int(slots[i])) for i in range(M)]
        want_out, want_state = conv_reference(want, taps.double(), None, state.double(), segments)
        dev_state = state.to(DEV)
        got = ops.gemm_decode(activations, w, ops.EPILOGUE_CONV, squares=squares, eps=eps, taps=taps.to(DEV), state=dev_state,
                              seg_slot=slots.to(DEV), out_dtype=torch.float32)
        close(got, want_out, torch.float32, 4.0)
        close(dev_state, want_state, torch.float32, 4.0)


@pytest.mark.parametrize("M", [17, 40, 64])
@pytest.mark.parametrize("H,N,K,one_centered", [(72, 80, 136, False), (2048, 6144, 8192, True), (4104, 144, 64, False)])
def test_medium_product_prepares_and_takes_the_next_norm(ops, M, H, N, K, one_centered):
    """The same hand-over as in the fused decode product, for 17..64 rows: the accumulating
    product leaves x * w and sums of squares (rows 64 wide), the next product takes them."""
    a = as_dev(gen(M, K, seed=1), torch.bfloat16)
    w_out = as_dev(gen(H, K, seed=2, scale=K ** -0.5), torch.bfloat16)
    residual = gen(M, H, seed=3, scale=2).float().to(DEV)
    norm_w = (0.1 * gen(H, seed=4) + (0 if one_centered else 1)).float()
    eps = 1e-5
    x_new = residual.cpu().double() + back(a) @ back(w_out).T
    activations, squares = ops.gemm_medium(a, w_out, ops.EPILOGUE_ACCUMULATE, accumulate_into=residual,
                                           next_norm_weight=norm_w.to(DEV), next_one_centered=one_centered)
    close(residual, x_new, torch.float32, 2.0)
    x_kernel = residual.cpu().double()
    scale = norm_w.double() + (1 if one_centered else 0)
    assert squares.shape[1] == 64
    assert torch.equal(activations.cpu(), (x_kernel.float() * scale.float()).to(torch.bfloat16))
    total = squares.cpu().double().sum(0)
    assert float((total[:M] - (x_kernel ** 2).sum(-1)).abs().max()) <= 1e-5 * float((x_kernel ** 2).sum(-1).max())
    inv = 1.0 / torch.sqrt((x_kernel ** 2).mean(-1, keepdim=True) + eps)
    h = activations.cpu().double() * inv
    w = as_dev(gen(N, H, seed=5, scale=H ** -0.5), torch.bfloat16)
    bias = gen(N, seed=6).float().to(DEV)
    want = h @ back(w).T
    got = ops.gemm_medium(activations, w, ops.EPILOGUE_STORE, squares=squares, eps=eps, out_dtype=torch.float32, bias=bias)
    close(got, want + bias.cpu().double(), torch.float32, 2.0)
    # against a plain norm kernel followed by the plain product: one more rounding (the norm's output)
    normed = ops.rmsnorm_rows(residual, norm_w.to(DEV), eps, torch.bfloat16, one_centered=one_centered)
    close(ops.gemm(normed, w, out_dtype=torch.float32), want, torch.bfloat16, 1.0)
    half = N // 2
    got = ops.gemm_medium(activations, w, ops.EPILOGUE_SWIGLU, squares=squares, eps=eps)
    close(got, F.silu(want[:, :half]) * want[:, half:], torch.bfloat16, 0.4)
    other = gen(M, N, seed=7).float().to(DEV)
    before = other.cpu().double()
    ops.gemm_medium(activations, w, ops.EPILOGUE_ACCUMULATE, accumulate_into=other, squares=squares, eps=eps)
    close(other, before + want, torch.float32, 2.0)


def test_fused_decode_product_limits(ops):
    from flyweight_amd.kernels.ops import KernelError
    assert not ops.gemm_decode_fits(17, 64, 64, ops.EPILOGUE_STORE) and not ops.gemm_decode_fits(4, 64, 68, ops.EPILOGUE_STORE)
    assert ops.gemm_decode_fits(16, 64, 8192, ops.EPILOGUE_STORE) and ops.gemm_decode_fits(1, 64, 8, ops.EPILOGUE_ACCUMULATE)
    a = torch.zeros(17, 64, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(KernelError, match="1..16 rows"):
        ops.gemm_decode(a, torch.zeros(32, 64, dtype=torch.bfloat16, device=DEV), ops.EPILOGUE_STORE)
    # 16 rows and a long K
    a = as_dev(gen(16, 8192), torch.bfloat16)
    w = as_dev(gen(136, 8192, seed=1, scale=0.01), torch.bfloat16)
    residual = torch.zeros(16, 136, device=DEV)
    ops.gemm_decode(a, w, ops.EPILOGUE_ACCUMULATE, accumulate_into=residual)
    close(residual, back(a) @ back(w).T, torch.float32, 2.0)


# ----- weights in operand tiles ---------------------------------------------------------------------
@pytest.mark.parametrize("M", [1, 8, 16, 17, 40, 64])
@pytest.mark.parametrize("N,K", [(72, 64), (200, 96), (1000, 544), (4096, 512), (16400, 256), (2048, 4096), (40, 8192)])
def test_weights_in_operand_tiles_change_no_bit_of_the_products_of_few_rows(ops, monkeypatch, M, N, K):
    """The decode products read W either row-major or once more in tiles of 16 rows x 32 columns
    laid out as a wave loads them (``ops.tile_weights``): the same numbers from other addresses, so
    every epilogue gives bit for bit what it gives from the row-major matrix. Feature counts that
    are no multiple of 16 (the tiles' rows are padded with zeros), narrow and wide outputs, a K
    long enough for the product that cuts it over workgroups, gate|up and B|C|x operands."""
    # (which kernel adds a long K into few features depends on the layout, and two kernels sum in two
    # orders: here both layouts go to the fused product, whatever the rows)
    monkeypatch.setattr(ops, "LONG_K", 1 << 30)
    g = torch.Generator().manual_seed(N + K + M)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16).to(DEV)
    bias = torch.randn(N, generator=g).float().to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16).to(DEV)
    tiled = ops.tile_weights(w)
    assert tiled.shape == ((N + 15) // 16, K // 32, 4, 16, 8)
    # tile (i, j) holds rows 16 i .., columns 32 j .., a lane's eight columns together
    i, j, r, c = (N - 1) // 16, K // 32 - 1, (N - 1) % 16, 19
    assert tiled[i, j, c // 8, r, c % 8] == w[N - 1, 32 * j + c]
    assert ops.tile_weights(torch.zeros(8, 40, dtype=torch.bfloat16, device=DEV)) is None       # K no multiple of 32
    assert ops.tile_weights(w.float()) is None
    product = ops.gemm_decode if M <= 16 else ops.gemm_medium
    residual = torch.randn(M, N, generator=g).float().to(DEV)
    for epilogue, kwargs in ((ops.EPILOGUE_STORE, dict(bias=bias, out_dtype=torch.float32)),
                             (ops.EPILOGUE_STORE, dict(out_dtype=torch.bfloat16)),
                             (ops.EPILOGUE_ACCUMULATE, dict(bias=bias))):
        results = []
        for layout in (None, tiled):
            if epilogue == ops.EPILOGUE_ACCUMULATE:
                kwargs["accumulate_into"] = residual.clone()
            results.append(product(a, w, epilogue, w_tiled=layout, **kwargs))
        assert torch.equal(results[0], results[1]), f"epilogue {epilogue} {kwargs.get('out_dtype')}"
    # with the next norm prepared, and taken by a product on tiles again
    norm_w = (1 + 0.1 * torch.randn(N, generator=g)).float().to(DEV)
    prepared = [product(a, w, ops.EPILOGUE_ACCUMULATE, accumulate_into=residual.clone(), next_norm_weight=norm_w, w_tiled=layout)
                for layout in (None, tiled)]
    # (the sums of squares hold a column per row of a; columns behind the last row are not specified)
    assert torch.equal(prepared[0][0], prepared[1][0]) and torch.equal(prepared[0][1][:, :M], prepared[1][1][:, :M])
    if N % 32 == 0:
        w_next = (torch.randn(96, N, generator=g) / math.sqrt(N)).to(torch.bfloat16).to(DEV)
        taken = [product(prepared[0][0], w_next, ops.EPILOGUE_STORE, squares=prepared[0][1], eps=1e-5, out_dtype=torch.float32, w_tiled=layout)
                 for layout in (None, ops.tile_weights(w_next))]
        assert torch.equal(taken[0], taken[1])
    # gate | up, and B | C | x with the convolution behind them (up to 16 rows)
    if N % 2 == 0:
        gated = [product(a, w, ops.EPILOGUE_SWIGLU, w_tiled=layout) for layout in (None, tiled)]
        assert torch.equal(gated[0], gated[1])
    if N % 3 == 0 and M <= 16:
        H = N // 3
        taps = (torch.randn(H, 3, generator=g) * 0.5).float().to(DEV)
        state = torch.randn(M + 2, H, 2, generator=g).float().to(DEV)
        slots = torch.randperm(M + 2, generator=g)[:M].to(torch.int32).to(DEV)
        outs, states = [], []
        for layout in (None, tiled):
            mine = state.clone()
            outs.append(ops.gemm_decode(a, w, ops.EPILOGUE_CONV, taps=taps, state=mine, seg_slot=slots, out_dtype=torch.bfloat16, w_tiled=layout))
            states.append(mine)
        assert torch.equal(outs[0], outs[1]) and torch.equal(states[0], states[1])
    with pytest.raises(ops.KernelError, match="operand tiles"):
        product(a, w, ops.EPILOGUE_STORE, w_tiled=tiled[:-1].contiguous() if tiled.shape[0] > 1 else tiled.reshape(-1))
