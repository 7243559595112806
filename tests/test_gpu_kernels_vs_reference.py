"""Every HIP kernel against its plain C++ reference (csrc/reference), on the same inputs after
rounding to the kernel's storage type, at sizes other than the engine's tiny models: widths
and vocabularies that are no power of two, odd head counts, scattered pages, mixed segments."""

import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]
TOL = {torch.float32: 1e-5, torch.bfloat16: 1.5e-2}


@pytest.fixture(scope="module")
def ops():
    from flyweight_amd.kernels import ops
    ops.library()
    return ops


@pytest.fixture(scope="module")
def ref():
    from flyweight_amd.kernels import reference
    reference.library()
    return reference


def rounded(array, dtype):
    """(device tensor in ``dtype``, float32 numpy of exactly those values)."""
    t = torch.as_tensor(array, dtype=torch.float32).to(dtype)
    return t.to(DEV).contiguous(), t.float().numpy()


def ints(array):
    return torch.as_tensor(np.asarray(array, dtype=np.int32), device=DEV)


def close(found, expected, dtype, factor=1.0):
    found = found.detach().float().cpu().numpy()
    assert found.shape == expected.shape and np.isfinite(found).all()
    limit = TOL[dtype] * factor * max(1.0, float(np.abs(expected).max()))
    assert float(np.abs(found - expected).max()) <= limit, f"{float(np.abs(found - expected).max()):.3e} > {limit:.3e}"


RNG = np.random.default_rng(12)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rows_kernels(ops, ref, dtype):
    table, table_h = rounded(RNG.normal(size=(301, 100)), dtype)
    ids = [0, 300, 7, 7, 150]
    assert np.array_equal(ops.embed_rows(table, ints(ids), scale=0.5).cpu().numpy(), ref.embed_rows(table_h, ids, 0.5))
    x = RNG.normal(size=(9, 1100)).astype(np.float32) * 3
    w = (1 + 0.2 * RNG.normal(size=1100)).astype(np.float32)
    xd, wd = torch.tensor(x, device=DEV), torch.tensor(w, device=DEV)
    close(ops.rmsnorm_rows(xd, wd, 1e-5, dtype), ref.rmsnorm_rows(x, w, 1e-5), dtype)
    close(ops.rmsnorm_rows(xd, wd, 1e-6, dtype, row_index=ints([8, 2, 2])), ref.rmsnorm_rows(x, w, 1e-6, row_index=[8, 2, 2]), dtype)
    gate_up = RNG.normal(size=(6, 2 * 330)).astype(np.float32) * 2
    close(ops.swiglu(torch.tensor(gate_up, device=DEV), out_dtype=dtype), ref.swiglu(gate_up), dtype)
    logits = RNG.normal(size=(5, 3001)).astype(np.float32)
    close(ops.scale_softcap_(torch.tensor(logits, device=DEV), 0.7, 1.5), ref.scale_softcap(logits, 0.7, 1.5), torch.float32)
    logits[0, 40] = logits[0, 2900] = 9.0
    logits[1, :] = -1.0
    ld = torch.tensor(logits, device=DEV)
    assert ops.argmax_rows(ld).cpu().tolist() == ref.argmax_rows(logits).tolist()


def test_sampler_draws_the_reference_samplers_tokens(ops, ref):
    """The device sampler against the C++ one (whole row sorted, every sum in order): the same
    tokens and the same generator states over random rows and settings, drawn three times in a
    row; also into the places a following decode step reads (ids, positions)."""
    from test_reference_kernels import sampling_cases
    drawn = 0
    for logits, settings, states in sampling_cases(60, seed=5):
        rows = len(logits)
        device_logits, device_settings = torch.tensor(logits, device=DEV), torch.tensor(settings, device=DEV)
        device_states = torch.tensor(states.view(np.int64), device=DEV)
        also = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
        positions = torch.arange(rows, dtype=torch.int32, device=DEV)
        for draw in range(3):
            want_ids, states = ref.sample_rows(logits, settings, states)
            got = ops.sample_rows(device_logits, device_settings, device_states, also=also, advance=positions)
            assert got.cpu().tolist() == want_ids.tolist() == also.cpu().tolist()
            assert np.array_equal(device_states.cpu().numpy().view(np.uint64), states)
            assert positions.cpu().tolist() == [r + draw + 1 for r in range(rows)]
            drawn += rows
    assert drawn > 500
    # a vocabulary like a model's, rows that are greedy beside rows that draw
    logits = (RNG.normal(size=(6, 65536)) * 3).astype(np.float32)
    settings = np.array([[0, 0, 1, 0], [0.8, 40, 0.95, 0.05], [1.0, 0, 0.9, 0], [0.7, 1024, 1.0, 0.01], [2.0, 5000, 0.99, 0], [1.0, 0, 1.0, 0]],
                        dtype=np.float32)
    states = np.arange(1, 7, dtype=np.uint64) * np.uint64(0x9E3779B97F4A7C15)
    want_ids, want_states = ref.sample_rows(logits, settings, states)
    device_states = torch.tensor(states.view(np.int64), device=DEV)
    got = ops.sample_rows(torch.tensor(logits, device=DEV), torch.tensor(settings, device=DEV), device_states)
    assert got.cpu().tolist() == want_ids.tolist() and got.cpu().tolist()[0] == int(logits[0].argmax())
    assert np.array_equal(device_states.cpu().numpy().view(np.uint64), want_states) and want_states[0] == states[0]
    # flat rows over the whole vocabulary (no top_k): the list is searched, not walked
    # (where min_p alone ends the list; a row of one value and a row of two, which no bin of the value divides)
    flat = (RNG.normal(size=(8, 65536)) * 0.02).astype(np.float32)
    flat[5, :] = 1.5
    flat[6, :] = np.where(RNG.random(65536) < 0.5, 0.25, -0.25)
    flat[7, 30000:] = -np.inf
    flat_settings = np.array([[0.8, 0, 1, 0], [0.8, 0, 0.9, 0], [1.0, 0, 0.95, 0.05], [0.7, 5000, 0.9, 0.5], [1.0, 0, 1.0, 0.9],
                              [0.8, 0, 0.9, 0], [1.0, 0, 0.7, 0.5], [0.9, 40000, 0.99, 0]], dtype=np.float32)
    flat_states = np.arange(11, 19, dtype=np.uint64) * np.uint64(0x9E3779B97F4A7C15)
    for draw in range(4):
        want_ids, want_states = ref.sample_rows(flat, flat_settings, flat_states)
        device_states = torch.tensor(flat_states.view(np.int64), device=DEV)
        got = ops.sample_rows(torch.tensor(flat, device=DEV), torch.tensor(flat_settings, device=DEV), device_states)
        assert got.cpu().tolist() == want_ids.tolist()
        assert np.array_equal(device_states.cpu().numpy().view(np.uint64), want_states)
        flat_states = want_states
    # a larger vocabulary that is no multiple of four (rows read element by element, a coarser fixed point)
    wide = (RNG.normal(size=(4, 150001)) * 2).astype(np.float32)
    wide_settings = np.array([[1.0, 0, 1, 0], [0.9, 0, 0.8, 0], [1.2, 20000, 0.95, 0.001], [0.6, 0, 0.99, 0.02]], dtype=np.float32)
    wide_states = np.arange(21, 25, dtype=np.uint64) * np.uint64(0x9E3779B97F4A7C15)
    for draw in range(3):
        want_ids, want_states = ref.sample_rows(wide, wide_settings, wide_states)
        device_states = torch.tensor(wide_states.view(np.int64), device=DEV)
        got = ops.sample_rows(torch.tensor(wide, device=DEV), torch.tensor(wide_settings, device=DEV), device_states)
        assert got.cpu().tolist() == want_ids.tolist()
        assert np.array_equal(device_states.cpu().numpy().view(np.uint64), want_states)
        wide_states = want_states


# rows that pick every product kernel: the fused decode product (<= 16), the split-K one (17..64),
# the tiled prompt kernels (beyond), and the plain float32 kernel
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 72, 200), (7, 200, 264), (16, 1000, 136), (33, 136, 520), (64, 96, 1032), (150, 200, 264)])
def test_products_with_every_epilogue(ops, ref, dtype, M, N, K):
    a, a_h = rounded(RNG.normal(size=(M, K)), dtype)
    w, w_h = rounded(RNG.normal(size=(N, K)) / math.sqrt(K), dtype)
    bias = RNG.normal(size=N).astype(np.float32)
    factor = 1.0 if dtype == torch.float32 else 2.0
    close(ops.gemm(a, w, torch.tensor(bias, device=DEV), out_dtype=torch.float32), ref.gemm(a_h, w_h, bias), dtype, factor)
    residual = RNG.normal(size=(M, N)).astype(np.float32)
    target = torch.tensor(residual, device=DEV)
    ops.gemm(a, w, accumulate_into=target)
    close(target, ref.gemm(a_h, w_h, accumulate_into=residual.copy()), dtype, factor)
    if N % 2 == 0:
        close(ops.gemm_swiglu(a, w), ref.gemm_swiglu(a_h, w_h), dtype, factor)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,kernel,bias", [(72, 3, False), (200, 4, True), (40, 7, True)])
def test_short_convolution_over_mixed_segments(ops, ref, dtype, hidden, kernel, bias):
    counts = [5, 1, 1, 40, 2]
    slots = [3, 0, 4, 1, 2]
    seg_row0 = np.concatenate([[0], np.cumsum(counts)])
    rows = int(seg_row0[-1])
    bcx = RNG.normal(size=(rows, 3 * hidden)).astype(np.float32)
    taps = RNG.normal(size=(hidden, kernel)).astype(np.float32) * 0.5
    conv_bias = RNG.normal(size=hidden).astype(np.float32) if bias else None
    state = RNG.normal(size=(6, hidden, kernel - 1)).astype(np.float32)
    row_seg = np.concatenate([np.full(c, i) for i, c in enumerate(counts)])
    state_d = torch.tensor(state, device=DEV)
    out = ops.shortconv(torch.tensor(bcx, device=DEV), torch.tensor(taps, device=DEV), None if conv_bias is None else torch.tensor(conv_bias, device=DEV),
                        state_d, ints(row_seg), ints(seg_row0), ints(slots), len(counts), out_dtype=dtype)
    want_state = state.copy()
    want = ref.shortconv(bcx, taps, conv_bias, want_state, seg_row0, slots)
    close(out, want, dtype)
    close(state_d, want_state, torch.float32)
    assert np.array_equal(state_d[5].cpu().numpy(), state[5])       # a slot of nobody's is not touched


def scattered_cache(lengths, nkv, hd, num_pages, seed):
    rng = np.random.default_rng(seed)
    order = rng.permutation(num_pages).tolist()
    tables = [[order.pop() for _ in range((n + 63) // 64)] for n in lengths]
    stride = max(len(t) for t in tables)
    return np.array([t + [0] * (stride - len(t)) for t in tables], dtype=np.int32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,hd,rotary,window", [(6, 2, 48, 48, 0), (5, 5, 16, 8, 0), (8, 1, 64, 64, 90), (3, 1, 112, 0, 0)])
def test_norm_rotation_cache_write_and_attention_over_mixed_segments(ops, ref, dtype, nh, nkv, hd, rotary, window):
    """Three requests behind contexts of different lengths: a portion of a prompt, a decoded token,
    a portion that crosses a page edge. The kernels write the new keys and values into scattered
    pages and attend over them; the references do the same on copies."""
    starts, counts = [70, 130, 0], [40, 1, 75]
    lengths = [s + c for s, c in zip(starts, counts)]
    table = scattered_cache(lengths, nkv, hd, 9, seed=hd)
    rows = sum(counts)
    row_seg = np.concatenate([np.full(c, i) for i, c in enumerate(counts)])
    row_pos = np.concatenate([np.arange(s, s + c) for s, c in zip(starts, counts)])
    seg_row0 = np.concatenate([[0], np.cumsum(counts)])
    # the contexts so far, already in the pages (rounded to the cache's type)
    k_h = np.zeros((9, nkv, 64, hd), dtype=np.float32)
    v_h = np.zeros((9, nkv, hd, 64), dtype=np.float32)
    for seg, start in enumerate(starts):
        for t in range(start):
            page = table[seg, t // 64]
            k_h[page, :, t % 64, :] = RNG.normal(size=(nkv, hd))
            v_h[page, :, :, t % 64] = RNG.normal(size=(nkv, hd))
    k_d, k_h = rounded(k_h, dtype)
    v_d, v_h = rounded(v_h, dtype)
    qkv = RNG.normal(size=(rows, (nh + 2 * nkv) * hd)).astype(np.float32)
    qw, kw = (1 + 0.3 * RNG.normal(size=hd)).astype(np.float32), (1 + 0.3 * RNG.normal(size=hd)).astype(np.float32)
    inv_freq = 1000.0 ** (-(np.arange(rotary // 2, dtype=np.float64) * 2.0 / max(rotary, 1)))
    cos_h, sin_h = ref.rope_table(row_pos, inv_freq) if rotary else (None, None)
    if rotary:
        cos_d, sin_d = ops.rope_table(ints(row_pos), torch.tensor(inv_freq, device=DEV))
        close(cos_d, cos_h, torch.float32), close(sin_d, sin_h, torch.float32)
    else:
        cos_d = sin_d = None
    q_d = ops.qk_norm_rope_kv_write(torch.tensor(qkv, device=DEV), nh, nkv, hd, torch.tensor(qw, device=DEV), torch.tensor(kw, device=DEV),
                                    1e-5, cos_d, sin_d, rotary, k_d, v_d, ints(table), ints(row_seg), ints(row_pos))
    q_h = ref.qk_norm_rope_kv_write(qkv, nh, nkv, hd, qw, kw, 1e-5, cos_h, sin_h, rotary, k_h, v_h, table, row_seg, row_pos)
    close(q_d, q_h, dtype)
    close(k_d, k_h, dtype), close(v_d, v_h, dtype)
    # attention on what the kernel itself stored, so that only attention is compared
    q_seen, k_seen, v_seen = q_d.float().cpu().numpy(), k_d.float().cpu().numpy(), v_d.float().cpu().numpy()
    scale = 1 / math.sqrt(hd)
    want = ref.attention(q_seen, nh, nkv, hd, k_seen, v_seen, table, row_seg, row_pos, scale, window)
    generic = ops.attention_generic(q_d, nh, nkv, hd, k_d, v_d, ints(table), ints(row_seg), ints(row_pos), scale, window)
    close(generic, want, dtype)
    if dtype == torch.bfloat16:
        tile_seg, tile_row0 = ops.query_tiles(seg_row0.tolist())
        tiled = ops.attention_prefill(q_d, nh, nkv, hd, k_d, v_d, ints(table), ints(tile_seg), ints(tile_row0), ints(seg_row0),
                                      ints(row_pos), scale, window)
        close(tiled, want, dtype)
        # one row per request through the split-key decode kernel: the last row of each segment
        last = [int(seg_row0[i + 1]) - 1 for i in range(3)]
        decoded = ops.attention_decode(q_d[last].contiguous(), nh, nkv, hd, k_d, v_d, ints(table), ints([0, 1, 2]), ints(row_pos[last]),
                                       scale, max(lengths), window)
        close(decoded, want[last], dtype)


@pytest.mark.parametrize("nh,nkv,hd,rotary,window,normed", [(32, 8, 64, 64, 0, True), (6, 2, 48, 48, 0, True), (5, 5, 16, 8, 0, True),
                                                            (8, 1, 64, 64, 90, True), (3, 1, 112, 0, 0, False), (40, 2, 32, 32, 0, True)])
def test_decode_attention_with_norm_rotation_and_cache_write_in_front(ops, ref, nh, nkv, hd, rotary, window, normed):
    """One new token for each of five requests behind contexts that end at different places of a
    page (its first key, its last, a page of its own): the fused kernel against the two kernels it
    replaces, bit for bit (outputs and pages), and against the C++ reference."""
    contexts = [0, 63, 64, 200, 449]
    rows = len(contexts)
    table = scattered_cache([c + 1 for c in contexts], nkv, hd, 16, seed=hd + nh)
    k_h = np.zeros((16, nkv, 64, hd), dtype=np.float32)
    v_h = np.zeros((16, nkv, hd, 64), dtype=np.float32)
    for seg, length in enumerate(contexts):
        for t in range(length):
            page = table[seg, t // 64]
            k_h[page, :, t % 64, :] = RNG.normal(size=(nkv, hd))
            v_h[page, :, :, t % 64] = RNG.normal(size=(nkv, hd))
    k_two, k_h = rounded(k_h, torch.bfloat16)
    v_two, v_h = rounded(v_h, torch.bfloat16)
    k_one, v_one = k_two.clone(), v_two.clone()
    qkv = RNG.normal(size=(rows, (nh + 2 * nkv) * hd)).astype(np.float32)
    qw = (1 + 0.3 * RNG.normal(size=hd)).astype(np.float32) if normed else None
    kw = (1 + 0.3 * RNG.normal(size=hd)).astype(np.float32) if normed else None
    dev = lambda a: None if a is None else torch.tensor(a, device=DEV)       # noqa: E731
    inv_freq = 1000.0 ** (-(np.arange(rotary // 2, dtype=np.float64) * 2.0 / max(rotary, 1)))
    positions, segments = ints(contexts), ints(range(rows))
    cos, sin = ops.rope_table(positions, torch.tensor(inv_freq, device=DEV)) if rotary else (None, None)
    scale = 1 / math.sqrt(hd)
    q = ops.qk_norm_rope_kv_write(dev(qkv), nh, nkv, hd, dev(qw), dev(kw), 1e-5, cos, sin, rotary, k_two, v_two, ints(table), segments, positions)
    two = ops.attention_decode(q, nh, nkv, hd, k_two, v_two, ints(table), segments, positions, scale, 512, window)
    one = ops.attention_decode_fused(dev(qkv), nh, nkv, hd, dev(qw), dev(kw), 1e-5, cos, sin, rotary, k_one, v_one, ints(table), segments,
                                     positions, scale, 512, window)
    assert torch.equal(one, two) and torch.equal(k_one, k_two) and torch.equal(v_one, v_two)
    # a layer that reads another's cache forms its queries and leaves the cache alone
    k_other, v_other = k_one.clone(), v_one.clone()
    again = ops.attention_decode_fused(dev(qkv * 1.0), nh, nkv, hd, dev(qw), dev(kw), 1e-5, cos, sin, rotary, k_other, v_other, ints(table),
                                       segments, positions, scale, 512, window, write_kv=False)
    assert torch.equal(again, two) and torch.equal(k_other, k_one) and torch.equal(v_other, v_one)
    # and the C++ reference of the whole
    cos_h, sin_h = ref.rope_table(contexts, inv_freq) if rotary else (None, None)
    q_h = ref.qk_norm_rope_kv_write(qkv, nh, nkv, hd, qw, kw, 1e-5, cos_h, sin_h, rotary, k_h, v_h, table, range(rows), contexts)
    want = ref.attention(q_h, nh, nkv, hd, k_h, v_h, table, range(rows), contexts, scale, window)
    close(one, want, torch.bfloat16, 2.0)


@pytest.mark.parametrize("M,hidden,K,kernel,bias", [(16, 136, 264, 3, False), (1, 72, 1032, 4, True), (8, 200, 520, 2, True), (13, 2048, 2048, 3, False)])
def test_products_with_the_short_convolution_behind_them(ops, ref, M, hidden, K, kernel, bias):
    """in_proj with the gated convolution and the state shift in its epilogue, for single-token
    rows of requests in scattered slots (the fused decode product, up to 16 rows), against the
    references of the product and of the convolution."""
    a, a_h = rounded(RNG.normal(size=(M, K)), torch.bfloat16)
    w, w_h = rounded(RNG.normal(size=(3 * hidden, K)) / math.sqrt(K), torch.bfloat16)
    in_bias = RNG.normal(size=3 * hidden).astype(np.float32) * 0.1 if bias else None
    conv_bias = RNG.normal(size=hidden).astype(np.float32) * 0.1 if bias else None
    taps = RNG.normal(size=(hidden, kernel)).astype(np.float32) * 0.5
    slots = RNG.permutation(M + 3)[:M]
    state = RNG.normal(size=(M + 3, hidden, kernel - 1)).astype(np.float32)
    want_state = state.copy()
    want = ref.shortconv(ref.gemm(a_h, w_h, in_bias), taps, conv_bias, want_state, np.arange(M + 1), slots)
    dev = lambda x: None if x is None else torch.tensor(x, device=DEV)      # noqa: E731
    for kernel_call in (ops.gemm_decode,):
        state_d = dev(state)
        out = kernel_call(a, w, ops.EPILOGUE_CONV, bias=dev(in_bias), out_dtype=torch.bfloat16, taps=dev(taps), conv_bias=dev(conv_bias),
                          state=state_d, seg_slot=ints(slots))
        close(out, want, torch.bfloat16, 2.0)
        close(state_d, want_state, torch.bfloat16, 2.0)         # B * x comes from bfloat16 operands
        untouched = [s for s in range(M + 3) if s not in slots.tolist()]
        assert np.array_equal(state_d[untouched].cpu().numpy(), state[untouched])
