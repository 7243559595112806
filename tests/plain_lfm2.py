"""A plain, slow LFM2 in float64 numpy: whole sequences, no cache, one function per part.

Written from the reference's formulas (each function cites where the reference computes
the same thing); it shares no code with ``flyweight_amd``: it reads config.json and the
safetensors file on its own. The reference is read, not run. Paths are relative to the
reference's root.
"""

from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import numpy as np


# ----- model folder ------------------------------------------------------------------------
def read_folder(folder: str):
    """config.json as a dict and every tensor as float64 (through the safetensors package,
    not the engine's own reader)."""
    import torch
    from safetensors.torch import load_file

    with open(os.path.join(folder, "config.json"), "r", encoding="utf-8") as handle:
        config = json.load(handle)
    weights = {name: tensor.to(torch.float64).numpy()
               for name, tensor in load_file(os.path.join(folder, "model.safetensors")).items()}
    return config, weights


def feed_forward_width(config: dict) -> int:
    """Effective SwiGLU width. The reference reads it off the gate tensor
    (native/src/v2_runtime.cpp:3527-3534); from config.json it is two thirds of
    intermediate_size, times the multiplier, rounded up to the multiple, when
    block_auto_adjust_ff_dim is set."""
    width = config["intermediate_size"]
    if config.get("block_auto_adjust_ff_dim", False):
        width = int(2 * width / 3)
        if config.get("block_ffn_dim_multiplier") is not None:
            width = int(config["block_ffn_dim_multiplier"] * width)
        multiple = config["block_multiple_of"]
        width = multiple * ((width + multiple - 1) // multiple)
    return width


def attention_layers(config: dict) -> List[bool]:
    layers = config["num_hidden_layers"]
    if config.get("layer_types") is not None:
        return [kind in ("full_attention", "attn", "attention") for kind in config["layer_types"]]
    chosen = set(config["full_attn_idxs"])
    return [i in chosen for i in range(layers)]


# ----- parts -------------------------------------------------------------------------------
def rms_norm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """y = x * rsqrt(mean(x^2) + eps) * w over the last axis; the weight multiplies
    directly. native/include/flyweight_v2_qwen_kernels.hpp:425-447;
    oracle tests/lfm2_gguf_fixture.py:249-250."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * weight


def rope_angles(positions: np.ndarray, rotary_dim: int, theta: float):
    """angle[p, i] = p / theta^(2i / rotary_dim), i < rotary_dim / 2.
    native/include/flyweight_v2_native_kernels.hpp:993-1008."""
    half = rotary_dim // 2
    inv_freq = theta ** (-(np.arange(half, dtype=np.float64) * 2.0 / rotary_dim))
    angle = np.asarray(positions, dtype=np.float64)[:, None] * inv_freq[None, :]
    return np.cos(angle), np.sin(angle)


def rope_half_split(x: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
    """x [T, heads, head_dim]; channel i pairs with i + half:
    out[i] = a cos - b sin, out[i + half] = b cos + a sin.
    native/include/flyweight_v2_native_kernels.hpp:1033-1047; oracle tests/lfm2_gguf_fixture.py:252-257."""
    half = cos.shape[-1]
    a, b, rest = x[..., :half], x[..., half:2 * half], x[..., 2 * half:]
    c, s = cos[:, None, :], sin[:, None, :]
    return np.concatenate([a * c - b * s, b * c + a * s, rest], axis=-1)


def causal_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float,
                     window: Optional[int] = None) -> np.ndarray:
    """q [T, nh, hd], k and v [T, nkv, hd] -> [T, nh, hd]. Row t sees keys s <= t (and
    s > t - window); query head i reads kv head i // (nh / nkv); softmax with the maximum
    subtracted. native/include/flyweight_v2_qwen_kernels.hpp:12570-12585 (scores),
    :12664-12704 (softmax and values); causal rule native/include/flyweight_v2_native_kernels.hpp:4150-4176;
    oracle tests/lfm2_gguf_fixture.py:284-288."""
    T, nh, hd = q.shape
    group = nh // k.shape[1]
    out = np.zeros_like(q)
    for t in range(T):
        lo = 0 if window is None else max(0, t - window + 1)
        for head in range(nh):
            kv = head // group
            scores = (k[lo:t + 1, kv] @ q[t, head]) * scale
            p = np.exp(scores - scores.max())
            out[t, head] = (p / p.sum()) @ v[lo:t + 1, kv]
    return out


def attention_qkv(h: np.ndarray, w: Dict[str, np.ndarray], prefix: str, config: dict, positions: np.ndarray):
    """Queries, keys and values as the attention reads them: projections; then, per head, the
    RMS norm of q and of k over the head's channels, one weight of head_dim for all heads, with
    the model's one eps (native/include/flyweight_v2_native_kernels.hpp:1015-1032); then the
    rotation of the normed vectors (:1033-1047); v as projected. The head size is
    hidden / heads (native/src/v2_runtime.cpp:4222)."""
    T = h.shape[0]
    nh, nkv = config["num_attention_heads"], config["num_key_value_heads"]
    hd = config["hidden_size"] // nh
    eps = config["norm_eps"]
    q = (h @ w[prefix + "q_proj.weight"].T).reshape(T, nh, hd)
    k = (h @ w[prefix + "k_proj.weight"].T).reshape(T, nkv, hd)
    v = (h @ w[prefix + "v_proj.weight"].T).reshape(T, nkv, hd)
    q = rms_norm(q, w[prefix + "q_layernorm.weight"], eps)
    k = rms_norm(k, w[prefix + "k_layernorm.weight"], eps)
    cos, sin = rope_angles(positions, hd, config["rope_theta"])
    return rope_half_split(q, cos, sin), rope_half_split(k, cos, sin), v


def attention_mixer(h: np.ndarray, w: Dict[str, np.ndarray], prefix: str, config: dict) -> np.ndarray:
    """native/src/v2_runtime.cpp:28429-28478: q, k, v projections; per-head RMS norm of q
    and k; rotation; causal softmax attention with scores scaled by 1 / sqrt(head_dim);
    output projection."""
    T = h.shape[0]
    q, k, v = attention_qkv(h, w, prefix, config, np.arange(T))
    out = causal_attention(q, k, v, 1.0 / math.sqrt(q.shape[-1]))
    return out.reshape(T, -1) @ w[prefix + "out_proj.weight"].T


def causal_depthwise_conv(bx: np.ndarray, taps: np.ndarray) -> np.ndarray:
    """bx [T, H], taps [H, L] oldest first: y_t = sum_j taps[:, j] * bx_{t-(L-1)+j}, zero
    before the start. native/include/flyweight_v2_native_kernels.hpp:1302-1319 (the ring starts
    zeroed, native/src/v2_runtime.cpp:20437-20440)."""
    T, H = bx.shape
    L = taps.shape[1]
    padded = np.concatenate([np.zeros((L - 1, H)), bx], axis=0)
    y = np.zeros((T, H))
    for j in range(L):
        y += taps[None, :, j] * padded[j:j + T]
    return y


def short_conv_mixer(h: np.ndarray, w: Dict[str, np.ndarray], prefix: str, config: dict) -> np.ndarray:
    """native/src/v2_runtime.cpp:28269-28283; oracle tests/lfm2_gguf_fixture.py:290-296:
    in_proj -> (B, C, x); bx = B * x; depthwise causal conv; C * y; out_proj. The optional
    biases sit after each linear map (the reference's only biased conv adds its bias after
    the taps, native/include/flyweight_v2_native_kernels.hpp:1370)."""
    H = config["hidden_size"]
    bias = config.get("conv_bias", False)
    bcx = h @ w[prefix + "in_proj.weight"].T
    if bias:
        bcx = bcx + w[prefix + "in_proj.bias"]
    B, C, x = bcx[:, :H], bcx[:, H:2 * H], bcx[:, 2 * H:]
    taps = w[prefix + "conv.weight"].reshape(H, -1)
    y = causal_depthwise_conv(B * x, taps)
    if bias:
        y = y + w[prefix + "conv.bias"]
    out = (C * y) @ w[prefix + "out_proj.weight"].T
    if bias:
        out = out + w[prefix + "out_proj.bias"]
    return out


def silu(x: np.ndarray) -> np.ndarray:
    return x / (1.0 + np.exp(-x))


def swiglu(h: np.ndarray, w: Dict[str, np.ndarray], prefix: str) -> np.ndarray:
    """down(silu(gate h) * (up h)); native/src/v2_runtime.cpp:28797-28805;
    oracle tests/lfm2_gguf_fixture.py:310-311."""
    gate = h @ w[prefix + "w1.weight"].T
    up = h @ w[prefix + "w3.weight"].T
    return (silu(gate) * up) @ w[prefix + "w2.weight"].T


# ----- the whole model ---------------------------------------------------------------------
def forward(config: dict, w: Dict[str, np.ndarray], tokens: Sequence[int]) -> np.ndarray:
    """Logits [T, vocab] for a whole sequence. Block: x += mixer(norm(x)); x += ffn(norm(x))
    (native/src/v2_runtime.cpp:28077,28282,28774,29133-29136); final norm then the head, which
    is the embedding table when tied (:29176,4189-4191)."""
    eps = config["norm_eps"]
    x = w["model.embed_tokens.weight"][np.asarray(tokens, dtype=np.int64)]
    for index, is_attention in enumerate(attention_layers(config)):
        base = f"model.layers.{index}."
        h = rms_norm(x, w[base + "operator_norm.weight"], eps)
        if is_attention:
            x = x + attention_mixer(h, w, base + "self_attn.", config)
        else:
            x = x + short_conv_mixer(h, w, base + "conv.", config)
        h = rms_norm(x, w[base + "ffn_norm.weight"], eps)
        x = x + swiglu(h, w, base + "feed_forward.")
    h = rms_norm(x, w["model.embedding_norm.weight"], eps)
    tied = config.get("tie_word_embeddings", config.get("tie_embedding", True))
    head = w["model.embed_tokens.weight"] if tied else w["lm_head.weight"]
    return h @ head.T


# ----- long sequences: the same formulas, by blocks, and only the rows that are compared -----
def causal_attention_rows(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float, first_row: int,
                          block: int = 512) -> np.ndarray:
    """``causal_attention`` for the rows from ``first_row`` on only (q holds those rows alone:
    [T - first_row, nh, hd]; k and v all T), a block of rows against all their keys at a time
    instead of row by row. Same formulas and citations as ``causal_attention``; the test of the
    plain model holds the two against each other. (The sums run in float64 through torch's
    threaded routines: tens of thousands of keys per row, thousands of rows.)"""
    import torch
    R, nh, hd = q.shape
    T, nkv = k.shape[0], k.shape[1]
    assert first_row + R == T
    group = nh // nkv
    out = np.zeros_like(q)
    keys, values = torch.from_numpy(np.ascontiguousarray(k)), torch.from_numpy(np.ascontiguousarray(v))
    for start in range(0, R, block):
        rows = min(block, R - start)
        last_key = first_row + start + rows             # keys below this index are seen by some row of the block
        position = torch.arange(first_row + start, first_row + start + rows)[:, None]
        hidden = torch.arange(last_key)[None, :] > position        # [rows, keys]: the future
        for kv in range(nkv):
            queries = torch.from_numpy(np.ascontiguousarray(q[start:start + rows, kv * group:(kv + 1) * group]))   # [rows, group, hd]
            scores = torch.einsum("rgd,sd->rgs", queries, keys[:last_key, kv]) * scale
            scores.masked_fill_(hidden[:, None, :], float("-inf"))
            p = torch.softmax(scores, dim=-1)
            out[start:start + rows, kv * group:(kv + 1) * group] = torch.einsum("rgs,sd->rgd", p, values[:last_key, kv]).numpy()
    return out


def forward_tail(config: dict, w: Dict[str, np.ndarray], tokens: Sequence[int], last: int) -> np.ndarray:
    """Logits of the last ``last`` positions of a long sequence, [last, vocab]: ``forward``, with
    attention by blocks and, from the last attention layer on, only the rows that the wanted ones
    depend on (each short convolution behind it reaches L - 1 rows further back)."""
    eps = config["norm_eps"]
    T = len(tokens)
    kinds = attention_layers(config)
    taps = config["conv_L_cache"]
    last_attention = max((i for i, a in enumerate(kinds) if a), default=-1)
    convs_behind = sum(1 for a in kinds[last_attention + 1:] if not a)
    first = max(0, T - last - convs_behind * (taps - 1)) if last_attention >= 0 else 0      # the rows kept from that layer on
    x = w["model.embed_tokens.weight"][np.asarray(tokens, dtype=np.int64)]
    kept_from = 0
    for index, is_attention in enumerate(kinds):
        base = f"model.layers.{index}."
        h = rms_norm(x, w[base + "operator_norm.weight"], eps)
        if is_attention:
            prefix = base + "self_attn."
            q, k, v = attention_qkv(h, w, prefix, config, np.arange(T))
            rows_from = first if index == last_attention else 0
            out = causal_attention_rows(q[rows_from:], k, v, 1.0 / math.sqrt(q.shape[-1]), rows_from)
            if index == last_attention:
                x, kept_from = x[first:], first
            x = x + out.reshape(out.shape[0], -1) @ w[prefix + "out_proj.weight"].T
        else:
            # behind the last attention layer the kept rows begin in mid-sequence: the first L - 1 of them
            # see zeros where their forerunners were, and are among the rows dropped at the end
            x = x + short_conv_mixer(h, w, base + "conv.", config)
        h = rms_norm(x, w[base + "ffn_norm.weight"], eps)
        x = x + swiglu(h, w, base + "feed_forward.")
    assert T - kept_from >= last
    h = rms_norm(x[-last:], w["model.embedding_norm.weight"], eps)
    tied = config.get("tie_word_embeddings", config.get("tie_embedding", True))
    head = w["model.embed_tokens.weight"] if tied else w["lm_head.weight"]
    return h @ head.T


def most_likely(logits: np.ndarray) -> int:
    """The largest logit's id; among equal ones the lowest id wins
    (native/include/flyweight_v2_qwen_kernels.hpp:2391-2405: the key orders by value, then by
    0xffffffff - id)."""
    best = 0
    for index in range(1, len(logits)):
        if logits[index] > logits[best]:
            best = index
    return best


def greedy(config: dict, w: Dict[str, np.ndarray], prompt: Sequence[int], count: int) -> List[int]:
    """Greedy continuation."""
    tokens = list(prompt)
    produced = []
    for _ in range(count):
        logits = forward(config, w, tokens)[-1]
        token = most_likely(logits)
        produced.append(token)
        tokens.append(token)
    return produced


# ----- sampling ----------------------------------------------------------------------------
class XorShift64Star:
    """native/src/v2_runtime.cpp:29307-29314: state 0 becomes 0x9e3779b97f4a7c15;
    x ^= x >> 12; x ^= x << 25; x ^= x >> 27; u = ((x * 2685821657736338717) >> 11) / 2^53."""

    MASK = (1 << 64) - 1

    def __init__(self, seed: int):
        self.state = seed & self.MASK

    def uniform(self) -> float:
        x = self.state or 0x9E3779B97F4A7C15
        x ^= x >> 12
        x ^= (x << 25) & self.MASK
        x ^= x >> 27
        self.state = x
        return ((x * 2685821657736338717 & self.MASK) >> 11) / 9007199254740992.0


def sample(logits: np.ndarray, temperature: float, top_k: int, top_p: float, min_p: float,
           rng: XorShift64Star) -> int:
    """native/src/v2_runtime.cpp:29500-29566 (candidates sorted by value descending, id
    ascending; top_k of them, 0 = all), :29686-29743 (greedy when temperature is 0;
    p ~ exp((l - l_max) / T) in float64; top_p keeps the prefix whose cumulative share
    reaches top_p; min_p keeps candidates with p >= min_p * p_0; draw threshold = u * kept
    total, first candidate whose cumulative reaches it)."""
    order = sorted(range(len(logits)), key=lambda i: (-float(logits[i]), i))
    if top_k > 0:
        order = order[:top_k]
    if not temperature > 0:
        return order[0]
    values = np.array([float(logits[i]) for i in order], dtype=np.float64) / temperature
    p = np.exp(values - values[0])
    total = p.sum()
    keep = len(p)
    if top_p < 1.0:
        cumulative = 0.0
        for i in range(len(p)):
            cumulative += p[i] / total
            if cumulative >= top_p:
                keep = i + 1
                break
    if min_p > 0.0:
        floor = min_p * p[0]
        kept = 1
        while kept < keep and p[kept] >= floor:
            kept += 1
        keep = kept
    threshold = rng.uniform() * p[:keep].sum()
    cumulative = 0.0
    for i in range(keep):
        cumulative += p[i]
        if threshold <= cumulative:
            return order[i]
    return order[keep - 1]
