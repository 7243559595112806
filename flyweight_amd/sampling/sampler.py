"""Choosing the next token from a row of logits.

Greedy is an argmax on the device with ties to the lowest id. Otherwise the ``top_k`` best
candidates (value descending, id ascending) come from the device when ``top_k <= 256`` and
from a full download and a host sort when not; probabilities exp((l - l_max) / T) are
formed in float64, ``top_p`` keeps the prefix whose cumulative share reaches it, ``min_p``
keeps candidates at least that fraction of the best, and the draw walks the sorted list
until the cumulative mass reaches u * kept mass (native/src/v2_runtime.cpp:29500-29566,
29686-29743). Each request owns an xorshift64* generator (:29307-29314), so what else is
in the batch cannot change its draws.
"""

from __future__ import annotations

import math
import time
from typing import List, Optional, Sequence

import numpy as np
import torch

from ..kernels import ops
from .config import MAX_DEVICE_TOP_K, SamplingConfig

_MASK = (1 << 64) - 1
_GOLDEN = 0x9E3779B97F4A7C15


class XorShift64Star:
    def __init__(self, seed: int):
        self.state = int(seed) & _MASK

    def uniform(self) -> float:
        x = self.state or _GOLDEN
        x ^= x >> 12
        x ^= (x << 25) & _MASK
        x ^= x >> 27
        self.state = x
        return (((x * 2685821657736338717) & _MASK) >> 11) * (1.0 / 9007199254740992.0)


def make_rng(seed: Optional[int], request_number: int) -> XorShift64Star:
    """A seeded request draws a reproducible stream; an unseeded one mixes the clock with
    its number (native/src/v2_runtime.cpp:32593-32596)."""
    if seed is None:
        seed = (time.time_ns() ^ ((request_number + 1) * _GOLDEN)) & _MASK
    return XorShift64Star(seed)


def draw_from_candidates(values: Sequence[float], ids: Sequence[int], config: SamplingConfig,
                         rng: XorShift64Star) -> int:
    """``values`` sorted descending (ties by ascending id), ``ids`` alongside."""
    if config.greedy or len(ids) == 1:
        return int(ids[0])
    scaled = np.asarray(values, dtype=np.float64) / config.temperature
    probabilities = np.where(np.isfinite(scaled), np.exp(scaled - scaled[0]), 0.0)
    total = float(probabilities.sum())
    if not (total > 0.0 and math.isfinite(total)):
        return int(ids[0])
    keep = len(probabilities)
    if config.top_p < 1.0:
        cumulative = 0.0
        for index in range(len(probabilities)):
            cumulative += probabilities[index] / total
            if cumulative >= config.top_p:
                keep = index + 1
                break
    if config.min_p > 0.0:
        floor = config.min_p * probabilities[0]
        kept = 1
        while kept < keep and probabilities[kept] >= floor:
            kept += 1
        keep = kept
    kept_total = 0.0
    for index in range(keep):
        kept_total += probabilities[index]
    threshold = rng.uniform() * kept_total
    cumulative = 0.0
    for index in range(keep):
        cumulative += probabilities[index]
        if threshold <= cumulative:
            return int(ids[index])
    return int(ids[keep - 1])


def host_candidates(logits: np.ndarray, count: int):
    """All (count = 0) or the best ``count`` candidates by (value descending, id ascending),
    NaN last."""
    keyed = np.where(np.isnan(logits), -np.inf, logits)
    order = np.lexsort((np.arange(len(logits)), -keyed))
    if count and count < len(order):
        order = order[:count]
    return logits[order], order


def sample_rows(logits: torch.Tensor, configs: Sequence[SamplingConfig], rngs: Sequence[XorShift64Star]) -> List[int]:
    """One token per row of ``logits`` ([rows, vocab] float32 on the device)."""
    rows, vocab = logits.shape
    tokens: List[Optional[int]] = [None] * rows
    greedy_rows = [i for i, c in enumerate(configs) if c.greedy]
    if greedy_rows:
        ids = ops.argmax_rows(logits if len(greedy_rows) == rows else logits[greedy_rows].contiguous()).cpu().tolist()
        for row, token in zip(greedy_rows, ids):
            tokens[row] = int(token)
    by_k = {}
    for row, config in enumerate(configs):
        if not config.greedy:
            k = config.top_k if 0 < config.top_k <= min(MAX_DEVICE_TOP_K, vocab) else 0
            by_k.setdefault(k, []).append(row)
    for k, group in by_k.items():
        chosen = logits[group].contiguous()
        if k:
            values, ids = ops.topk_rows(chosen, k)
            values, ids = values.cpu().numpy(), ids.cpu().numpy()
            for n, row in enumerate(group):
                tokens[row] = draw_from_candidates(values[n], ids[n], configs[row], rngs[row])
        else:
            host = chosen.cpu().numpy()
            for n, row in enumerate(group):
                count = configs[row].top_k if configs[row].top_k < vocab else 0
                values, ids = host_candidates(host[n], count)
                tokens[row] = draw_from_candidates(values, ids, configs[row], rngs[row])
    return tokens
