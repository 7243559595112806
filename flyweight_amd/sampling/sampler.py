"""Choosing the next token from a row of logits.

Greedy is an argmax on the device with ties to the lowest id. Otherwise the ``top_k`` best
candidates (value descending, id ascending; 0: all) are considered; probabilities
exp((l - l_max) / T) are formed in float64, ``top_p`` keeps the prefix whose cumulative share
reaches it, ``min_p`` keeps candidates at least that fraction of the best, and the draw walks
the sorted list until the cumulative mass reaches u * kept mass
(native/src/v2_runtime.cpp:29500-29566, 29686-29743). Each request owns an xorshift64*
generator (:29307-29314), so what else is in the batch cannot change its draws.
``sample_rows`` does all of it on the device (``csrc/sampling.hip``).
"""

from __future__ import annotations

import time
from typing import List, Optional, Sequence

import numpy as np
import torch

from ..kernels import ops
from .config import SamplingConfig

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


def pack_settings(configs: Sequence[SamplingConfig], rngs: Sequence[Optional[XorShift64Star]], vocab: int,
                  settings: Optional[np.ndarray] = None, states: Optional[np.ndarray] = None):
    """What the device sampler takes for these rows: float32 [rows, 4] = temperature (0: greedy),
    top_k (0: all), top_p, min_p, and the generators' states, uint64 [rows] (into the given arrays,
    which may be longer, or new ones)."""
    rows = len(configs)
    if vocab > 1 << 24:
        raise ValueError("the device sampler holds top_k in a float32: vocabularies beyond 2^24 are not served")
    if settings is None:
        settings, states = np.zeros((rows, 4), dtype=np.float32), np.zeros(rows, dtype=np.uint64)
    for row, (config, rng) in enumerate(zip(configs, rngs)):
        if config.greedy:
            settings[row] = 0.0
            states[row] = 0
        else:
            settings[row, 0], settings[row, 1] = config.temperature, min(config.top_k, vocab)
            settings[row, 2], settings[row, 3] = config.top_p, config.min_p
            states[row] = rng.state
    return settings, states


def sample_rows(logits: torch.Tensor, configs: Sequence[SamplingConfig], rngs: Sequence[Optional[XorShift64Star]]) -> List[int]:
    """One token per row of ``logits`` ([rows, vocab] float32 on the device), drawn on the device
    (``ops.sample_rows``); the generators of the rows that draw move on."""
    rows, vocab = logits.shape
    if all(config.greedy for config in configs):
        return [int(token) for token in ops.argmax_rows(logits).cpu().tolist()]
    settings, states = pack_settings(configs, rngs, vocab)
    device_settings = torch.from_numpy(settings).to(logits.device)
    device_states = torch.from_numpy(states.view(np.int64)).to(logits.device)
    tokens = ops.sample_rows(logits, device_settings, device_states).cpu().tolist()
    moved_on = device_states.cpu().numpy().view(np.uint64)
    for row, (config, rng) in enumerate(zip(configs, rngs)):
        if not config.greedy:
            rng.state = int(moved_on[row])
    return [int(token) for token in tokens]
