"""In-process helpers of the GPU tests: loading a tiny model and stepping it."""

from __future__ import annotations

from typing import Dict, List, Sequence

import numpy as np

import plain_lfm2 as plain
from helpers import make_model


class Loaded:
    def __init__(self, folder: str, dtype: str):
        from flyweight_amd.engine import load_model
        self.folder = folder
        self.dtype = dtype
        self.config, self.model = load_model(folder, dtype=dtype)
        self.plain_config, self.plain_weights = plain.read_folder(folder)

    def stepper(self, num_pages: int, max_requests: int = 4):
        from flyweight_amd.engine import Stepper
        return Stepper(self.model, num_pages=num_pages, max_requests=max_requests)

    def expected(self, tokens: Sequence[int]) -> np.ndarray:
        return plain.forward(self.plain_config, self.plain_weights, list(tokens))


def feed(stepper, request, tokens: Sequence[int], cuts: Sequence[int]) -> np.ndarray:
    """Feeds ``tokens`` in portions of the given sizes (the last portion takes the rest) and
    returns the logits at every position."""
    from flyweight_amd.engine import StepEntry
    out, at = [], 0
    sizes = list(cuts)
    while at < len(tokens):
        n = min(sizes.pop(0) if sizes else len(tokens) - at, len(tokens) - at)
        out.append(stepper.step([StepEntry(request, list(tokens[at:at + n]), list(range(n)))]).cpu().numpy())
        at += n
    return np.concatenate(out)
