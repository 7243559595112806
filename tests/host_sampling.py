"""The sampler's rules once more on the host, candidate list by candidate list, in the order
of the reference (native/src/v2_runtime.cpp:29500-29566, 29686-29743): what the tests draw with
where they want to look at a single cut or count draws, beside the plain implementation's
``sample`` and the C++ reference of the device sampler."""

from __future__ import annotations

import math
from typing import Sequence

import numpy as np

from flyweight_amd.sampling import SamplingConfig, XorShift64Star


def draw_from_candidates(values: Sequence[float], ids: Sequence[int], config: SamplingConfig,
                         rng: XorShift64Star) -> int:
    """``values`` sorted descending (ties by ascending id), ``ids`` alongside. A list of one
    candidate is drawn like any other: the generator moves on, as the reference's does
    (native/src/v2_runtime.cpp:29722-29733)."""
    if config.greedy:
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
