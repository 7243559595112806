"""Pins the plain implementation (tests/plain_lfm2.py) by what fixes it beside the
reference's text: special cases that reduce to a library routine, invariants, and the
reference's own recurrences, each chosen so that a plausible mistake fails it."""

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import plain_lfm2 as plain
from helpers import CONFIGS, make_model, random_tokens

RNG = np.random.default_rng(0)


def test_rms_norm():
    x = RNG.normal(size=(5, 24)) * 3
    w = RNG.normal(size=24)
    eps = 1e-3
    y = plain.rms_norm(x, np.ones(24), eps)
    n = x.shape[-1]
    sq = (x * x).sum(-1)
    np.testing.assert_allclose((y * y).sum(-1), n * sq / (sq + n * eps), rtol=1e-12)
    np.testing.assert_allclose(plain.rms_norm(x, w, eps), x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * w, rtol=1e-12)
    # the weight multiplies directly (not 1 + w): a zero weight gives zero
    assert np.abs(plain.rms_norm(x, np.zeros(24), eps)).max() == 0.0
    # scale invariance up to eps; eps inside the root (a large eps shrinks the output)
    np.testing.assert_allclose(plain.rms_norm(1e4 * x, w, 1e-12), plain.rms_norm(x, w, 1e-12), rtol=1e-6)
    assert np.abs(plain.rms_norm(x, w, 100.0)).max() < np.abs(plain.rms_norm(x, w, eps)).max() / 3


def test_short_conv_is_a_left_padded_depthwise_convolution():
    T, H, L = 11, 6, 4
    bx, taps = RNG.normal(size=(T, H)), RNG.normal(size=(H, L))
    y = plain.causal_depthwise_conv(bx, taps)
    lib = F.conv1d(torch.tensor(bx.T[None]), torch.tensor(taps[:, None, :]), groups=H, padding=L - 1)[0, :, :T].T.numpy()
    np.testing.assert_allclose(y, lib, rtol=1e-12, atol=1e-12)
    for c in range(H):      # np.convolve flips its kernel
        np.testing.assert_allclose(y[:, c], np.convolve(bx[:, c], taps[c, ::-1])[:T], rtol=1e-12, atol=1e-12)
    # the last tap multiplies the current token
    identity = np.zeros((H, L)); identity[:, -1] = 1.0
    np.testing.assert_allclose(plain.causal_depthwise_conv(bx, identity), bx)
    oldest = np.zeros((H, L)); oldest[:, 0] = 1.0
    np.testing.assert_allclose(plain.causal_depthwise_conv(bx, oldest)[L - 1:], bx[:T - L + 1])
    assert np.abs(plain.causal_depthwise_conv(bx, oldest)[:L - 1]).max() == 0.0     # zero before the start


def test_short_conv_equals_the_reference_ring_recurrence():
    # native/include/flyweight_v2_native_kernels.hpp:1302-1319: state = last L-1 values of bx, oldest first
    T, H, L = 9, 5, 3
    bx, taps = RNG.normal(size=(T, H)), RNG.normal(size=(H, L))
    state = np.zeros((H, L - 1))
    rows = []
    for t in range(T):
        value = taps[:, L - 1] * bx[t]
        for i in range(L - 1):
            value = value + taps[:, i] * state[:, i]
        state = np.concatenate([state[:, 1:], bx[t][:, None]], axis=1)
        rows.append(value)
    np.testing.assert_allclose(plain.causal_depthwise_conv(bx, taps), np.stack(rows), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(state, bx[-(L - 1):].T)      # the state is the last L-1 columns of bx


def _conv_weights(H, L, bias):
    w = {"p.in_proj.weight": RNG.normal(size=(3 * H, H)), "p.conv.weight": RNG.normal(size=(H, 1, L)),
         "p.out_proj.weight": RNG.normal(size=(H, H))}
    if bias:
        w.update({"p.in_proj.bias": RNG.normal(size=3 * H), "p.conv.bias": RNG.normal(size=H), "p.out_proj.bias": RNG.normal(size=H)})
    return w


def test_in_proj_thirds_are_b_c_x():
    H, L, T = 8, 3, 6
    config = {"hidden_size": H, "conv_bias": False}
    w = _conv_weights(H, L, False)
    h = RNG.normal(size=(T, H))
    out = plain.short_conv_mixer(h, w, "p.", config)
    swapped = dict(w)
    m = w["p.in_proj.weight"]
    swapped["p.in_proj.weight"] = np.concatenate([m[2 * H:], m[H:2 * H], m[:H]])       # B <-> x: B*x is unchanged
    np.testing.assert_allclose(plain.short_conv_mixer(h, swapped, "p.", config), out, rtol=1e-12)
    gate_off = dict(w)
    gate_off["p.in_proj.weight"] = np.concatenate([m[:H], np.zeros((H, H)), m[2 * H:]])  # C = 0 silences the mixer
    assert np.abs(plain.short_conv_mixer(h, gate_off, "p.", config)).max() == 0.0
    other = dict(w)
    other["p.in_proj.weight"] = np.concatenate([np.zeros((H, H)), m[H:]])               # so does B = 0
    assert np.abs(plain.short_conv_mixer(h, other, "p.", config)).max() == 0.0
    # C gates after the convolution: with identity taps the mixer is out_proj(C * B * x)
    ident = dict(w); taps = np.zeros((H, 1, L)); taps[:, 0, -1] = 1.0; ident["p.conv.weight"] = taps
    bcx = h @ m.T
    np.testing.assert_allclose(plain.short_conv_mixer(h, ident, "p.", config),
                               (bcx[:, H:2 * H] * bcx[:, :H] * bcx[:, 2 * H:]) @ w["p.out_proj.weight"].T, rtol=1e-12)


def test_conv_biases_sit_after_each_linear_map():
    H, L, T = 4, 4, 5
    w = _conv_weights(H, L, True)
    h = RNG.normal(size=(T, H))
    out = plain.short_conv_mixer(h, w, "p.", {"hidden_size": H, "conv_bias": True})
    bcx = h @ w["p.in_proj.weight"].T + w["p.in_proj.bias"]
    y = plain.causal_depthwise_conv(bcx[:, :H] * bcx[:, 2 * H:], w["p.conv.weight"].reshape(H, L)) + w["p.conv.bias"]
    np.testing.assert_allclose(out, (bcx[:, H:2 * H] * y) @ w["p.out_proj.weight"].T + w["p.out_proj.bias"], rtol=1e-12)
    lib = F.conv1d(torch.tensor((bcx[:, :H] * bcx[:, 2 * H:]).T[None]), torch.tensor(w["p.conv.weight"]),
                   bias=torch.tensor(w["p.conv.bias"]), groups=H, padding=L - 1)[0, :, :T].T.numpy()
    np.testing.assert_allclose(y, lib, rtol=1e-12)


def test_rope():
    hd, theta = 16, 100.0
    x = RNG.normal(size=(7, 3, hd))
    cos, sin = plain.rope_angles(np.arange(7), hd, theta)
    np.testing.assert_allclose(np.arctan2(sin[3], cos[3]) % (2 * np.pi), (3 * theta ** (-np.arange(8) * 2 / hd)) % (2 * np.pi), rtol=1e-9)
    rotated = plain.rope_half_split(x, cos, sin)
    np.testing.assert_allclose(rotated[0], x[0])                                        # position 0: identity
    np.testing.assert_allclose((rotated ** 2).sum(-1), (x ** 2).sum(-1), rtol=1e-12)    # a rotation
    # half-split pairing: a one-hot channel 0 leaks into channel hd/2, not channel 1
    onehot = np.zeros((1, 1, hd)); onehot[0, 0, 0] = 1.0
    c1, s1 = plain.rope_angles(np.array([1]), hd, theta)
    r = plain.rope_half_split(onehot, c1, s1)[0, 0]
    assert abs(r[0] - math.cos(1.0)) < 1e-12 and abs(r[hd // 2] - math.sin(1.0)) < 1e-12 and r[1] == 0.0
    # scores depend on distances only
    q, k = RNG.normal(size=(1, 1, hd)), RNG.normal(size=(1, 1, hd))
    def score(p, t):
        cp, sp = plain.rope_angles(np.array([p]), hd, theta)
        ct, st = plain.rope_angles(np.array([t]), hd, theta)
        return float((plain.rope_half_split(q, cp, sp) * plain.rope_half_split(k, ct, st)).sum())
    assert abs(score(9, 4) - score(105, 100)) < 1e-9 and abs(score(9, 4) - score(4, 9)) > 1e-3
    # a partial rotation leaves the tail alone
    cp, sp = plain.rope_angles(np.arange(7), 8, theta)
    np.testing.assert_allclose(plain.rope_half_split(x, cp, sp)[..., 8:], x[..., 8:])


def test_attention_special_cases_and_library_agreement():
    T, nh, nkv, hd = 9, 6, 2, 8
    q, k, v = RNG.normal(size=(T, nh, hd)), RNG.normal(size=(T, nkv, hd)), RNG.normal(size=(T, nkv, hd))
    scale = 1 / math.sqrt(hd)
    out = plain.causal_attention(q, k, v, scale)
    group = nh // nkv
    np.testing.assert_allclose(out[0], np.repeat(v[0], group, axis=0))                  # one key: the value itself
    same = plain.causal_attention(q, np.repeat(k[:1], T, axis=0), v, scale)
    np.testing.assert_allclose(same[4, 0], v[:5, 0].mean(0), rtol=1e-12)                # equal keys: the mean
    tq, tk, tv = (torch.tensor(a).transpose(0, 1)[None] for a in (q, k, v))
    lib = F.scaled_dot_product_attention(tq, tk.repeat_interleave(group, 1), tv.repeat_interleave(group, 1), is_causal=True)
    np.testing.assert_allclose(out, lib[0].transpose(0, 1).numpy(), rtol=1e-10, atol=1e-12)
    # causality: a later token changes nothing earlier
    k2, v2 = k.copy(), v.copy(); k2[6] += 1.0; v2[6] -= 2.0
    np.testing.assert_allclose(plain.causal_attention(q, k2, v2, scale)[:6], out[:6])
    # a window of w keys: the row sees exactly its last w
    windowed = plain.causal_attention(q, k, v, scale, window=3)
    np.testing.assert_allclose(windowed[:3], out[:3])
    np.testing.assert_allclose(windowed[7], plain.causal_attention(q[5:8], k[5:8], v[5:8], scale)[2], rtol=1e-12)


def test_swiglu_and_its_tails():
    h = RNG.normal(size=(4, 6))
    w = {"f.w1.weight": RNG.normal(size=(10, 6)), "f.w3.weight": RNG.normal(size=(10, 6)), "f.w2.weight": RNG.normal(size=(6, 10))}
    th = torch.tensor(h)
    lib = (F.silu(th @ torch.tensor(w["f.w1.weight"]).T) * (th @ torch.tensor(w["f.w3.weight"]).T)) @ torch.tensor(w["f.w2.weight"]).T
    np.testing.assert_allclose(plain.swiglu(h, w, "f."), lib.numpy(), rtol=1e-12)
    assert np.isfinite(plain.silu(np.array([-700.0, 700.0]))).all()


@pytest.mark.parametrize("name", ["A", "B"])
def test_block_order_head_and_whole_model_invariants(tmp_path, name):
    folder = make_model(str(tmp_path / name), name, seed=3)
    config, w = plain.read_folder(folder)
    assert plain.feed_forward_width(config) == w["model.layers.0.feed_forward.w1.weight"].shape[0]
    tokens = random_tokens(config["vocab_size"], 40, 1)
    logits = plain.forward(config, w, tokens)
    assert logits.shape == (40, config["vocab_size"])
    # causality of the whole model
    changed = list(tokens); changed[30] = (changed[30] + 1) % config["vocab_size"]
    again = plain.forward(config, w, changed)
    np.testing.assert_allclose(again[:30], logits[:30], rtol=1e-12)
    assert np.abs(again[30:] - logits[30:]).max() > 1e-3
    # silencing every mixer's and feed-forward's last map makes the blocks the identity
    silent = dict(w)
    for key in w:
        if key.endswith(("out_proj.weight", "out_proj.bias", "feed_forward.w2.weight")):
            silent[key] = np.zeros_like(w[key])
    tied = config.get("tie_word_embeddings", True)
    head = w["model.embed_tokens.weight"] if tied else w["lm_head.weight"]
    bare = plain.rms_norm(w["model.embed_tokens.weight"][tokens], w["model.embedding_norm.weight"], config["norm_eps"]) @ head.T
    np.testing.assert_allclose(plain.forward(config, silent, tokens), bare, rtol=1e-12)
    if not tied:        # an untied model ignores the embedding table at the head
        other = dict(w); other["lm_head.weight"] = w["lm_head.weight"] * 2
        np.testing.assert_allclose(plain.forward(config, other, tokens), 2 * logits, rtol=1e-12)
    # each part matters at this weight scale: removing it changes the logits visibly
    for suffix in ("conv.conv.weight", "self_attn.v_proj.weight", "feed_forward.w3.weight"):
        cut = {k: (np.zeros_like(v) if k.endswith(suffix) else v) for k, v in w.items()}
        assert np.abs(plain.forward(config, cut, tokens) - logits).max() > 0.05 * np.abs(logits).max()


def test_greedy_ties_go_to_the_lowest_id(tmp_path):
    assert plain.most_likely(np.array([1.0, 3.0, 3.0, 2.0])) == 1
    assert plain.most_likely(np.array([-np.inf, -np.inf])) == 0
    # through the whole model: with a tied head a copy of the winner's embedding row has the
    # winner's logit exactly; whichever of the two ids is lower must be generated
    folder = make_model(str(tmp_path / "A"), "A", seed=3)
    config, w = plain.read_folder(folder)
    prompt = random_tokens(config["vocab_size"], 9, 2)
    winner = plain.greedy(config, w, prompt, 1)[0]
    free = [t for t in range(config["vocab_size"]) if t not in prompt and t != winner]
    above, below = max(free), min(free)
    assert below < winner < above
    table = w["model.embed_tokens.weight"]
    for copy, expected in ((above, winner), (below, below)):
        changed = dict(w)
        changed["model.embed_tokens.weight"] = table.copy()
        changed["model.embed_tokens.weight"][copy] = table[winner]
        logits = plain.forward(config, changed, prompt)[-1]
        assert logits[copy] == logits[winner] == logits.max()
        assert plain.greedy(config, changed, prompt, 1) == [expected]


# ----- the attention mixer's own choices: what is normed, when, with which eps and scale ------
def _attention_setup(nh=4, nkv=2, hd=8, T=6, eps=1e-5, theta=100.0):
    H = nh * hd
    config = {"hidden_size": H, "num_attention_heads": nh, "num_key_value_heads": nkv, "norm_eps": eps, "rope_theta": theta}
    w = {"a.q_proj.weight": RNG.normal(size=(nh * hd, H)), "a.k_proj.weight": RNG.normal(size=(nkv * hd, H)),
         "a.v_proj.weight": RNG.normal(size=(nkv * hd, H)), "a.out_proj.weight": np.eye(H),
         "a.q_layernorm.weight": 1.0 + 0.3 * RNG.normal(size=hd), "a.k_layernorm.weight": 1.0 + 0.3 * RNG.normal(size=hd)}
    return config, w, RNG.normal(size=(T, H))


def test_qk_norm_comes_before_the_rotation():
    """A norm weight that is one-hot on channel 0 leaves a vector along channel 0; the rotation
    then spreads it over channels 0 and hd/2 at every position but the first. Rotating first and
    norming after would leave channel 0 alone everywhere."""
    config, w, h = _attention_setup()
    hd = 8
    for name in ("a.q_layernorm.weight", "a.k_layernorm.weight"):
        w[name] = np.zeros(hd)
        w[name][0] = 1.0
    q, k, _ = plain.attention_qkv(h, w, "a.", config, np.arange(6))
    raw = (h @ w["a.q_proj.weight"].T).reshape(6, 4, hd)
    length = raw[..., 0] / np.sqrt((raw ** 2).mean(-1) + config["norm_eps"])      # channel 0 after the norm
    for p in range(6):
        others = [c for c in range(hd) if c not in (0, hd // 2)]
        assert np.abs(q[p][:, others]).max() == 0.0 and np.abs(k[p][:, others]).max() == 0.0
        # channel 0's pair turns by the angle p / theta^0 = p
        np.testing.assert_allclose(q[p][:, 0], length[p] * math.cos(p), rtol=1e-12, atol=1e-15)
        np.testing.assert_allclose(q[p][:, hd // 2], length[p] * math.sin(p), rtol=1e-12, atol=1e-15)
    assert np.abs(q[0][:, hd // 2]).max() == 0.0 and np.abs(q[1][:, hd // 2]).min() > 0.0


def test_qk_norm_is_per_head_with_one_weight_for_all_heads():
    config, w, h = _attention_setup()
    nh, nkv, hd, group = 4, 2, 8, 2
    out = plain.attention_mixer(h, w, "a.", config).reshape(6, nh, hd)       # out_proj is the identity
    # swapping the two query heads of kv group 0 swaps their outputs: one norm weight serves both
    rows = w["a.q_proj.weight"].reshape(nh, hd, -1)
    swapped = dict(w)
    swapped["a.q_proj.weight"] = rows[[1, 0, 2, 3]].reshape(nh * hd, -1)
    np.testing.assert_allclose(plain.attention_mixer(h, swapped, "a.", config).reshape(6, nh, hd), out[:, [1, 0, 2, 3]], rtol=1e-12)
    # the norm is over a head's channels alone: making one head's projection 50 times larger leaves
    # the other heads exactly alone, and that head itself nearly so (eps is all that notices)
    louder = dict(w)
    scaled = rows.copy()
    scaled[2] *= 50.0
    louder["a.q_proj.weight"] = scaled.reshape(nh * hd, -1)
    loud = plain.attention_mixer(h, louder, "a.", config).reshape(6, nh, hd)
    np.testing.assert_allclose(loud[:, [0, 1, 3]], out[:, [0, 1, 3]], rtol=1e-12)
    np.testing.assert_allclose(loud[:, 2], out[:, 2], rtol=1e-4)
    # v is not normed: doubling v_proj doubles the output
    double = dict(w)
    double["a.v_proj.weight"] = 2 * w["a.v_proj.weight"]
    np.testing.assert_allclose(plain.attention_mixer(h, double, "a.", config).reshape(6, nh, hd), 2 * out, rtol=1e-12)


def test_qk_norm_uses_the_models_eps_inside_the_root():
    """mean(x^2) + eps under the root, per head: a huge eps shrinks q and k, the scores vanish and
    every row attends evenly, so the output becomes the running mean of v."""
    config, w, h = _attention_setup(eps=1e12)
    nh, nkv, hd = 4, 2, 8
    out = plain.attention_mixer(h, w, "a.", config).reshape(6, nh, hd)
    v = (h @ w["a.v_proj.weight"].T).reshape(6, nkv, hd)
    running = np.cumsum(v, axis=0) / np.arange(1, 7)[:, None, None]
    np.testing.assert_allclose(out, np.repeat(running, nh // nkv, axis=1), rtol=1e-6, atol=1e-9)
    config["norm_eps"] = 1e-5
    assert np.abs(plain.attention_mixer(h, w, "a.", config).reshape(6, nh, hd) - np.repeat(running, 2, axis=1)).max() > 0.1
    # and it is the norm's eps as rms_norm has it: q of the mixer is rms_norm of the projection
    q, _, _ = plain.attention_qkv(h, w, "a.", config, np.zeros(6))            # position 0: no rotation
    raw = (h @ w["a.q_proj.weight"].T).reshape(6, nh, hd)
    np.testing.assert_allclose(q, raw / np.sqrt((raw ** 2).mean(-1, keepdims=True) + 1e-5) * w["a.q_layernorm.weight"], rtol=1e-12)


@pytest.mark.parametrize("hd", [8, 32])
def test_the_mixer_scales_scores_by_one_over_root_head_dim(hd):
    """The library's attention divides by sqrt(head_dim) when no scale is given: fed the mixer's
    own q, k and v it must give the mixer's output, for two head sizes."""
    config, w, h = _attention_setup(nh=4, nkv=2, hd=hd, T=7)
    q, k, v = plain.attention_qkv(h, w, "a.", config, np.arange(7))
    tq, tk, tv = (torch.tensor(a).transpose(0, 1)[None] for a in (q, k, v))
    lib = F.scaled_dot_product_attention(tq, tk.repeat_interleave(2, 1), tv.repeat_interleave(2, 1), is_causal=True)
    np.testing.assert_allclose(plain.attention_mixer(h, w, "a.", config), lib[0].transpose(0, 1).reshape(7, 4 * hd).numpy(),
                               rtol=1e-10, atol=1e-12)


def test_attention_by_blocks_and_the_tail_of_a_sequence_equal_the_row_by_row_model(tmp_path):
    """The long-context tests compare with ``forward_tail``: attention by blocks of rows, and
    behind the last attention layer only the rows that the wanted ones depend on. Both must give
    what the row-by-row functions give: blocks that end inside the sequence, a first row in
    mid-sequence, groups of heads, and both tiny models whole (in B two convolution layers
    follow the last attention layer and reach six rows back)."""
    T, nh, nkv, hd = 150, 6, 2, 16
    q, k, v = RNG.standard_normal((T, nh, hd)), RNG.standard_normal((T, nkv, hd)), RNG.standard_normal((T, nkv, hd))
    whole = plain.causal_attention(q, k, v, 0.3)
    for first_row, block in ((0, 64), (0, 150), (97, 16), (149, 512)):
        rows = plain.causal_attention_rows(q[first_row:], k, v, 0.3, first_row, block=block)
        np.testing.assert_allclose(rows, whole[first_row:], rtol=1e-11, atol=1e-13)
    for name in ("A", "B"):
        folder = make_model(str(tmp_path / name), name, seed=5)
        config, w = plain.read_folder(folder)
        tokens = random_tokens(config["vocab_size"], 90, 2)
        logits = plain.forward(config, w, tokens)
        for last in (1, 17, 90):
            np.testing.assert_allclose(plain.forward_tail(config, w, tokens, last), logits[-last:], rtol=1e-9, atol=1e-11)
