"""Shared by the tests: two tiny LFM2 configurations that differ in every size and option,
model folders with random weights, and a driver for bin/trace_run."""

from __future__ import annotations

import json
import os
import subprocess
import sys
from typing import Dict, List, Sequence

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TRACE_RUN = os.path.join(ROOT, "bin", "trace_run")

# Tiny A: conv/attention alternating via layer_types, 4 heads in 2 groups, head size 16,
# plain feed-forward width, tied head, 3 taps without biases.
TINY_A = dict(
    architectures=["Lfm2ForCausalLM"], model_type="lfm2", vocab_size=256, hidden_size=64, num_hidden_layers=4,
    num_attention_heads=4, num_key_value_heads=2, intermediate_size=160, block_auto_adjust_ff_dim=False,
    norm_eps=1e-5, rope_theta=10000.0, conv_L_cache=3, conv_bias=False, tie_word_embeddings=True,
    max_position_embeddings=384, layer_types=["conv", "full_attention", "conv", "full_attention"])

# Tiny B: attention first, then runs of conv of different length (via full_attn_idxs), 3 heads
# on one kv head, head size 32, width 96 (no power of two), auto-adjusted feed-forward width,
# untied head, 4 taps with biases, another eps and theta.
TINY_B = dict(
    architectures=["Lfm2ForCausalLM"], model_type="lfm2", vocab_size=500, hidden_size=96, num_hidden_layers=6,
    num_attention_heads=3, num_key_value_heads=1, intermediate_size=384, block_auto_adjust_ff_dim=True,
    block_ffn_dim_multiplier=1.5, block_multiple_of=64, norm_eps=1e-6, rope_theta=1000000.0, conv_L_cache=4,
    conv_bias=True, tie_word_embeddings=False, max_position_embeddings=512, full_attn_idxs=[0, 4])

CONFIGS = {"A": TINY_A, "B": TINY_B}

# Largest difference allowed between the engine's logits and the plain float64 model's, as
# a fraction of the largest logit in the comparison (a comparison may be a single row).
# The weights are scaled so that every part of a layer contributes at full size (see
# make_model), which is what lets a fault show, and also what lets rounding through: the
# gated parts multiply up to three rounded numbers. Measured with the straightforward
# kernels over rows of both tiny models: float32 (rounding 6e-8) is off by at most 4e-6 and
# 6e-7 in the root mean square; bfloat16 (rounding 2e-3 at every stored activation, four to
# seven per layer) by 4.5e-2 and 1.1e-2, the same pattern 2^13 times larger. Over every
# comparison of the GPU tests (some six hundred, many of a single row, whose root mean square
# is over one row only) the largest are 1.7e-5 and 1.9e-6 in float32, 5.5e-2 and 1.4e-2 in
# bfloat16. The limits sit a fifth to a quarter above those: a bfloat16 fault of a few per
# cent of the logits does not pass. The float32 run of the same code is what shows the logic
# right; the bfloat16 limits have to tell rounding from a fault, and the tests make faults
# large on purpose.
MAX_TOL = {"float32": 2e-5, "bfloat16": 7e-2}
RMS_TOL = {"float32": 4e-6, "bfloat16": 1.8e-2}


def make_model(folder: str, name: str, seed: int = 0, scale: str = "fan_in") -> str:
    from flyweight_amd.config import config_from_dict
    from flyweight_amd.weights import write_random_model
    return write_random_model(folder, config_from_dict(CONFIGS[name]), seed, scale=scale)


def random_tokens(vocab: int, count: int, seed: int) -> List[int]:
    return np.random.default_rng(seed).integers(0, vocab, size=count).tolist()


def assert_close(found: np.ndarray, expected: np.ndarray, dtype: str, what: str = "") -> None:
    assert found.shape == expected.shape, f"{what}: shape {found.shape} vs {expected.shape}"
    assert np.isfinite(found).all(), f"{what}: non-finite logits"
    scale = max(1.0, float(np.abs(expected).max()))
    error = np.abs(found.astype(np.float64) - expected)
    worst = float(error.max())
    rms = float(np.sqrt(np.mean(error ** 2)))
    where = np.unravel_index(int(error.argmax()), error.shape)
    assert worst <= MAX_TOL[dtype] * scale, (
        f"{what}: largest difference {worst:.3e} at {where} exceeds {MAX_TOL[dtype] * scale:.3e} "
        f"(first row over the limit: {int(np.argmax(error.max(axis=-1) > MAX_TOL[dtype] * scale))})")
    assert rms <= RMS_TOL[dtype] * scale, f"{what}: rms difference {rms:.3e} exceeds {RMS_TOL[dtype] * scale:.3e}"


def run_trace(model_dir: str, dtype: str, out_dir: str, max_tokens: int, steps: Sequence[dict],
              timeout: int = 300) -> Dict[int, np.ndarray]:
    """Feeds ``steps`` to bin/trace_run, waiting for ``done <step>`` after each, and
    returns step -> logits [wanted, vocab]."""
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json")) as handle:
        vocab = json.load(handle)["vocab_size"]
    process = subprocess.Popen(
        [TRACE_RUN, "--model", model_dir, "--dtype", dtype, "--out", out_dir, "--max-tokens", str(max_tokens)],
        stdin=subprocess.PIPE, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    try:
        for step in steps:
            process.stdin.write(json.dumps(step) + "\n")
            process.stdin.flush()
            line = process.stdout.readline()
            if line.strip() != f"done {step['step']}":
                process.stdin.close()
                process.wait(timeout=60)
                raise AssertionError(f"trace_run answered {line!r} to step {step['step']}; stderr: {process.stderr.read()}")
        process.stdin.close()
        code = process.wait(timeout=timeout)
        assert code == 0, f"trace_run exited with {code}: {process.stderr.read()}"
    finally:
        if process.poll() is None:
            process.kill()
    results = {}
    for step in steps:
        wanted = sum(len(e.get("want", [])) for e in step["entries"])
        path = os.path.join(out_dir, f"{step['step']}.f32")
        if wanted:
            data = np.fromfile(path, dtype="<f4")
            assert data.size == wanted * vocab, f"step {step['step']}: {data.size} floats for {wanted} rows of {vocab}"
            results[step["step"]] = data.reshape(wanted, vocab)
        else:
            assert not os.path.exists(path), f"step {step['step']} wanted nothing but wrote a file"
    return results
