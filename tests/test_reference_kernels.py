"""The plain C++ references of the kernels (csrc/reference, no GPU) against the plain numpy
model: each operation alone, and a whole tiny model put together from them over a paged cache
and state slots, fed in portions with pages that are scattered, against the whole-sequence
evaluation. The GPU tests then hold the HIP kernels against these same functions."""

import math

import numpy as np
import pytest

import plain_lfm2 as plain
from flyweight_amd.kernels import reference as ref
from helpers import CONFIGS, make_model, random_tokens

RNG = np.random.default_rng(5)


def close(found, expected, tolerance=2e-6):
    expected = np.asarray(expected, dtype=np.float64)
    assert found.shape == expected.shape
    assert np.abs(found - expected).max() <= tolerance * max(1.0, np.abs(expected).max())


def test_rows_products_and_activations():
    x = RNG.normal(size=(7, 50)).astype(np.float32)
    w = RNG.normal(size=50).astype(np.float32)
    close(ref.rmsnorm_rows(x, w, 1e-5), plain.rms_norm(x.astype(np.float64), w, 1e-5))
    close(ref.rmsnorm_rows(x, w, 1e-5, row_index=[4, 0]), plain.rms_norm(x[[4, 0]].astype(np.float64), w, 1e-5))
    close(ref.rmsnorm_rows(x, w, 1e-3, one_centered=True), plain.rms_norm(x.astype(np.float64), 1.0 + w, 1e-3))
    table = RNG.normal(size=(11, 6)).astype(np.float32)
    close(ref.embed_rows(table, [3, 3, 10, 0], scale=1.5), 1.5 * table[[3, 3, 10, 0]].astype(np.float64))
    with pytest.raises(ref.ReferenceError_, match="outside the table"):
        ref.embed_rows(table, [11])
    a, m, bias = (RNG.normal(size=s).astype(np.float32) for s in ((5, 33), (9, 33), (9,)))
    close(ref.gemm(a, m, bias), a.astype(np.float64) @ m.astype(np.float64).T + bias)
    residual = RNG.normal(size=(5, 9)).astype(np.float32)
    before = residual.astype(np.float64)
    assert ref.gemm(a, m, accumulate_into=residual) is residual
    close(residual, before + a.astype(np.float64) @ m.astype(np.float64).T)
    gate_up = RNG.normal(size=(14, 33)).astype(np.float32)
    both = a.astype(np.float64) @ gate_up.astype(np.float64).T
    close(ref.gemm_swiglu(a, gate_up), plain.silu(both[:, :7]) * both[:, 7:])
    close(ref.swiglu(both), plain.silu(both[:, :7]) * both[:, 7:])
    assert np.isfinite(ref.swiglu(np.array([[-700.0, 700.0, 1.0, 1.0]]))).all()
    close(ref.scale_softcap(both, 0.5, 3.0), 3.0 * np.tanh(0.5 * both / 3.0))
    close(ref.scale_softcap(both, 2.0), 2.0 * both)


def test_short_convolution_over_segments_and_state():
    H, L, T = 6, 4, 23
    bcx = RNG.normal(size=(T, 3 * H)).astype(np.float32)
    taps, bias = RNG.normal(size=(H, L)).astype(np.float32), RNG.normal(size=H).astype(np.float32)
    bx = bcx[:, :H].astype(np.float64) * bcx[:, 2 * H:]
    want = bcx[:, H:2 * H] * (plain.causal_depthwise_conv(bx, taps.astype(np.float64)) + bias)
    for cuts in ([T], [1] * T, [2, 2, 7, 1, 11], [3, 20]):
        state = np.full((3, H, L - 1), np.nan, dtype=np.float32)
        state[1] = 0.0
        pieces, at = [], 0
        for n in cuts:      # one segment per call, in slot 1
            pieces.append(ref.shortconv(bcx[at:at + n], taps, bias, state, [0, n], [1]))
            at += n
        close(np.concatenate(pieces), want, 1e-5)
        close(state[1], bx[-(L - 1):].T, 1e-6)          # the state is the last L - 1 columns of B * x
        assert np.isnan(state[[0, 2]]).all()            # other slots are not touched
    # two segments of different requests in one call
    state = np.zeros((2, H, L - 1), dtype=np.float32)
    out = ref.shortconv(bcx, taps, None, state, [0, 9, T], [1, 0])
    alone = bcx[9:, H:2 * H] * plain.causal_depthwise_conv(bx[9:], taps.astype(np.float64))
    close(out[9:], alone, 1e-5)


def _paged(num_pages, nkv, hd, page=64):
    return (np.full((num_pages, nkv, page, hd), np.nan, dtype=np.float32), np.full((num_pages, nkv, hd, page), np.nan, dtype=np.float32))


@pytest.mark.parametrize("nh,nkv,hd,window,rotary", [(4, 2, 16, 0, 16), (3, 1, 32, 0, 32), (6, 3, 8, 70, 4), (2, 2, 16, 0, 0)])
def test_norm_rotation_cache_write_and_paged_attention(nh, nkv, hd, window, rotary):
    T, theta, eps = 150, 100.0, 1e-5
    config = {"hidden_size": nh * hd, "num_attention_heads": nh, "num_key_value_heads": nkv, "norm_eps": eps, "rope_theta": theta}
    w = {"a.q_proj.weight": np.eye(nh * hd), "a.k_proj.weight": np.eye(nkv * hd, nh * hd), "a.v_proj.weight": np.eye(nkv * hd, nh * hd),
         "a.q_layernorm.weight": 1 + 0.3 * RNG.normal(size=hd), "a.k_layernorm.weight": 1 + 0.3 * RNG.normal(size=hd)}
    qkv = RNG.normal(size=(T, (nh + 2 * nkv) * hd)).astype(np.float32)
    q_raw, k_raw, v_raw = qkv[:, :nh * hd], qkv[:, nh * hd:(nh + nkv) * hd], qkv[:, (nh + nkv) * hd:]
    # the plain model's q, k: norm, then rotation of the first `rotary` channels
    half = rotary // 2
    inv_freq = theta ** (-(np.arange(half, dtype=np.float64) * 2.0 / max(rotary, 1)))
    cos_p, sin_p = (np.cos(np.arange(T)[:, None] * inv_freq), np.sin(np.arange(T)[:, None] * inv_freq))
    q_want = plain.rope_half_split(plain.rms_norm(q_raw.astype(np.float64).reshape(T, nh, hd), w["a.q_layernorm.weight"], eps), cos_p, sin_p) \
        if rotary else plain.rms_norm(q_raw.astype(np.float64).reshape(T, nh, hd), w["a.q_layernorm.weight"], eps)
    k_want = plain.rope_half_split(plain.rms_norm(k_raw.astype(np.float64).reshape(T, nkv, hd), w["a.k_layernorm.weight"], eps), cos_p, sin_p) \
        if rotary else plain.rms_norm(k_raw.astype(np.float64).reshape(T, nkv, hd), w["a.k_layernorm.weight"], eps)
    want = plain.causal_attention(q_want, k_want, v_raw.astype(np.float64).reshape(T, nkv, hd), 1 / math.sqrt(hd), window or None)
    # the reference over scattered pages, the sequence fed in portions
    k_pages, v_pages = _paged(7, nkv, hd)
    table = np.array([[5, 2, 6]], dtype=np.int32)
    found, at = [], 0
    for n in (40, 1, 1, 60, 48):
        positions = np.arange(at, at + n)
        cos, sin = ref.rope_table(positions, inv_freq) if rotary else (None, None)
        q = ref.qk_norm_rope_kv_write(qkv[at:at + n], nh, nkv, hd, w["a.q_layernorm.weight"], w["a.k_layernorm.weight"], eps, cos, sin,
                                      rotary, k_pages, v_pages, table, np.zeros(n), positions)
        close(q.reshape(n, nh, hd), q_want[at:at + n], 1e-5)
        found.append(ref.attention(q, nh, nkv, hd, k_pages, v_pages, table, np.zeros(n), positions, 1 / math.sqrt(hd), window))
        at += n
    close(np.concatenate(found).reshape(T, nh, hd), want, 1e-5)
    close(k_pages[5, :, :, :].transpose(1, 0, 2), k_want[:64], 1e-5)             # page 5 holds tokens 0..63, a key's channels together
    close(v_pages[2].transpose(2, 0, 1), v_raw.reshape(T, nkv, hd)[64:128], 1e-6)     # V keeps a channel's tokens together
    assert np.isnan(k_pages[[0, 1, 3, 4]]).all()                                     # no other page was written
    # a layer that reads another's cache does not write
    copy = k_pages.copy()
    ref.qk_norm_rope_kv_write(qkv[:5] * 3, nh, nkv, hd, None, None, eps, None, None, 0, k_pages, v_pages, table, np.zeros(5), np.arange(5),
                              write_kv=False)
    assert np.array_equal(copy, k_pages, equal_nan=True)


def test_argmax_order():
    logits = RNG.normal(size=(4, 300)).astype(np.float32)
    logits[0, 17] = logits[0, 250] = 50.0
    logits[1, :] = 1.0
    logits[2, 5] = np.nan
    assert ref.argmax_rows(logits).tolist() == [17, 0, int(np.nanargmax(logits[2])), int(logits[3].argmax())]
    assert ref.argmax_rows(logits[:, :1]).tolist() == [0, 0, 0, 0]


def sampling_cases(count, seed=0):
    """Rows of logits with sampling settings and generator states that meet every branch of the
    sampler: flat and peaked rows, ties, NaN and -inf, top_k from 1 to beyond the vocabulary."""
    rng = np.random.default_rng(seed)
    for trial in range(count):
        vocab = int(rng.choice([5, 130, 1000, 1024, 1025, 4099]))
        rows = int(rng.integers(1, 7))
        logits = (rng.standard_normal((rows, vocab)) * [0.01, 1.0, 4.0, 12.0][trial % 4]).astype(np.float32)
        if trial % 5 == 0:
            logits[:, : max(1, vocab // 3)] = np.round(logits[:, : max(1, vocab // 3)])     # ties, and both zeros
        if trial % 7 == 0:
            logits[0, rng.integers(0, vocab)] = np.nan
        if trial % 11 == 0:
            logits[-1, rng.integers(0, vocab)] = -np.inf
        settings = np.zeros((rows, 4), dtype=np.float32)
        for r in range(rows):
            settings[r] = (rng.choice([0.0, 0.3, 0.8, 1.0, 2.0]), rng.choice([0, 1, 2, 40, 256, 1024, 1500, vocab, vocab + 5]),
                           rng.choice([1.0, 0.95, 0.5, 0.05]), rng.choice([0.0, 0.05, 0.5, 1.0]))
        states = rng.integers(0, 2 ** 63 - 1, size=rows).astype(np.uint64)
        states[0] = 0
        yield logits, settings, states


def test_sampler_against_the_plain_one_and_the_host_rules():
    """The C++ sampler, the plain implementation's and the package's host rules draw the same
    tokens and leave the generators in the same states, over random rows and settings."""
    import plain_lfm2
    from flyweight_amd.sampling import SamplingConfig, XorShift64Star
    from host_sampling import draw_from_candidates, host_candidates
    drawn = 0
    for logits, settings, states in sampling_cases(40):
        ids, moved_on = ref.sample_rows(logits, settings, states)
        for r in range(len(logits)):
            temperature, top_k, top_p, min_p = (float(v) for v in settings[r])
            top_k = int(top_k)
            if not np.isnan(logits[r]).any():       # (the plain sampler says nothing about NaN; the engine's rule is: last)
                plain_rng = plain_lfm2.XorShift64Star(int(states[r]))
                assert ids[r] == plain_lfm2.sample(logits[r], temperature, top_k, top_p, min_p, plain_rng)
                # the generator moves on once per drawn token, also when top_k leaves one candidate
                assert plain_rng.state == int(moved_on[r]) and (plain_rng.state != int(states[r])) == (temperature > 0)
            host_rng = XorShift64Star(int(states[r]))
            values, order = host_candidates(logits[r], top_k if 0 < top_k < logits.shape[1] else 0)
            config = SamplingConfig(temperature=temperature, top_k=top_k, top_p=top_p, min_p=min_p)
            assert ids[r] == draw_from_candidates(values, order, config, host_rng)
            assert int(moved_on[r]) == host_rng.state
            drawn += int(moved_on[r]) != int(states[r])
    assert drawn > 40


def reference_forward(config, w, steps, num_pages=8):
    """A whole LFM2 from the C++ references alone: ``steps`` is a list of batches
    [(request, tokens)]; returns request -> logits of every token fed. Pages are handed out from
    the back, so that block tables are scattered; slots are handed out as requests appear."""
    H, nh, nkv = config["hidden_size"], config["num_attention_heads"], config["num_key_value_heads"]
    hd, eps, L = H // nh, config["norm_eps"], config["conv_L_cache"]
    attention = plain.attention_layers(config)
    f = {name: tensor.astype(np.float32) for name, tensor in w.items()}
    pages = {i: _paged(num_pages, nkv, hd) for i, a in enumerate(attention) if a}
    states = {i: np.zeros((4, H, L - 1), dtype=np.float32) for i, a in enumerate(attention) if not a}
    free_pages, tables, lengths, slots = list(range(num_pages)), {}, {}, {}
    inv_freq = config["rope_theta"] ** (-(np.arange(hd // 2, dtype=np.float64) * 2.0 / hd))
    logits = {}
    for batch in steps:
        tokens, row_seg, row_pos, seg_row0 = [], [], [], [0]
        for seg, (request, new) in enumerate(batch):
            if request not in slots:
                slots[request], lengths[request], tables[request] = len(slots), 0, []
            start = lengths[request]
            while len(tables[request]) * 64 < start + len(new):
                tables[request].append(free_pages.pop())
            tokens += list(new)
            row_seg += [seg] * len(new)
            row_pos += list(range(start, start + len(new)))
            seg_row0.append(seg_row0[-1] + len(new))
            lengths[request] = start + len(new)
        stride = max(len(tables[r]) for r, _ in batch)
        table = np.array([tables[r] + [0] * (stride - len(tables[r])) for r, _ in batch], dtype=np.int32)
        seg_slot = [slots[r] for r, _ in batch]
        x = ref.embed_rows(f["model.embed_tokens.weight"], tokens)
        cos, sin = ref.rope_table(row_pos, inv_freq)
        for i, is_attention in enumerate(attention):
            p = f"model.layers.{i}."
            h = ref.rmsnorm_rows(x, f[p + "operator_norm.weight"], eps)
            if is_attention:
                qkv = ref.gemm(h, np.concatenate([f[p + f"self_attn.{n}_proj.weight"] for n in "qkv"]))
                q = ref.qk_norm_rope_kv_write(qkv, nh, nkv, hd, f[p + "self_attn.q_layernorm.weight"], f[p + "self_attn.k_layernorm.weight"],
                                              eps, cos, sin, hd, *pages[i], table, row_seg, row_pos)
                mixed = ref.attention(q, nh, nkv, hd, *pages[i], table, row_seg, row_pos, 1 / math.sqrt(hd))
                ref.gemm(mixed, f[p + "self_attn.out_proj.weight"], accumulate_into=x)
            else:
                bias = config.get("conv_bias", False)
                bcx = ref.gemm(h, f[p + "conv.in_proj.weight"], f[p + "conv.in_proj.bias"] if bias else None)
                gated = ref.shortconv(bcx, f[p + "conv.conv.weight"].reshape(H, L), f[p + "conv.conv.bias"] if bias else None,
                                      states[i], seg_row0, seg_slot)
                ref.gemm(gated, f[p + "conv.out_proj.weight"], f[p + "conv.out_proj.bias"] if bias else None, accumulate_into=x)
            h = ref.rmsnorm_rows(x, f[p + "ffn_norm.weight"], eps)
            hidden = ref.gemm_swiglu(h, np.concatenate([f[p + "feed_forward.w1.weight"], f[p + "feed_forward.w3.weight"]]))
            ref.gemm(hidden, f[p + "feed_forward.w2.weight"], accumulate_into=x)
        tied = config.get("tie_word_embeddings", True)
        out = ref.gemm(ref.rmsnorm_rows(x, f["model.embedding_norm.weight"], eps), f["model.embed_tokens.weight" if tied else "lm_head.weight"])
        for seg, (request, new) in enumerate(batch):
            logits.setdefault(request, []).append(out[seg_row0[seg]:seg_row0[seg + 1]])
    return {request: np.concatenate(parts) for request, parts in logits.items()}


@pytest.mark.parametrize("name", ["A", "B"])
def test_a_whole_model_from_the_references_equals_the_plain_model(tmp_path, name):
    folder = make_model(str(tmp_path / name), name, seed=8)
    config, w = plain.read_folder(folder)
    a, b = random_tokens(config["vocab_size"], 100, 1), random_tokens(config["vocab_size"], 70, 2)
    steps = [[("a", a[:40])], [("a", a[40:41]), ("b", b[:30])], [("b", b[30:32]), ("a", a[41:50])], [("a", a[50:]), ("b", b[32:])]]
    found = reference_forward(config, w, steps)
    for request, tokens in (("a", a), ("b", b)):
        want = plain.forward(config, w, tokens)
        assert np.abs(found[request] - want).max() <= 2e-5 * np.abs(want).max()
    # greedy through the references: the plain model's tokens
    prompt = a[:9]
    tokens = list(prompt)
    for _ in range(4):
        tokens.append(int(ref.argmax_rows(reference_forward(config, w, [[("g", tokens)]])["g"][-1:])[0]))
    assert tokens[9:] == plain.greedy(config, w, prompt, 4)
