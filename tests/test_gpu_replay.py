"""Trace replay through bin/trace_run against the plain implementation: every request
whole; most of it in one step and the last 32 tokens one by one; in portions of changing
size down to two tokens; and mixed, up to four live requests with so few pages that they are
used again. In 32-bit and in bfloat16, for both tiny configurations."""

import os

import numpy as np
import pytest

import plain_lfm2 as plain
from helpers import CONFIGS, assert_close, make_model, random_tokens, run_trace

pytestmark = pytest.mark.gpu

PORTIONS = [7, 2, 16, 3, 2, 64, 5, 2, 33, 2, 2, 65, 9]


def round64(n):
    return (n + 63) // 64 * 64


class TraceBuilder:
    """Collects steps and remembers which (request, position) each written row is."""

    def __init__(self):
        self.steps, self.rows, self.fed, self.live, self.peak = [], {}, {}, set(), 0

    def step(self, entries, end=()):
        number = len(self.steps)
        rows = []
        for request, tokens, want in entries:
            start = self.fed.get(request, 0)
            rows += [(request, start + w) for w in want]
            self.fed[request] = start + len(tokens)
            self.live.add(request)
        self.peak = max(self.peak, sum(round64(self.fed[r]) for r in self.live))
        self.live -= set(end)
        self.steps.append({"step": number, "entries": [{"id": r, "tokens": t, "want": w} for r, t, w in entries],
                           "end": list(end)})
        self.rows[number] = rows


def whole(builder, request, tokens):
    builder.step([(request, tokens, list(range(len(tokens))))], end=[request])


def bulk_and_tail(builder, request, tokens):
    head = len(tokens) - 32
    builder.step([(request, tokens[:head], list(range(head)))])
    for i in range(head, len(tokens)):
        builder.step([(request, [tokens[i]], [0])], end=[request] if i == len(tokens) - 1 else [])


def portions(builder, request, tokens, sizes=PORTIONS):
    at, i = 0, 0
    while at < len(tokens):
        n = min(sizes[i % len(sizes)], len(tokens) - at)
        if len(tokens) - at - n == 1:       # never leave a single token: portions go down to two
            n += 1
        builder.step([(request, tokens[at:at + n], list(range(n)))], end=[request] if at + n == len(tokens) else [])
        at, i = at + n, i + 1


def mixed(builder, prompts, seed):
    """Up to four live requests; each is fed in portions until 12 tokens remain, which are
    then fed one by one (decoding), while others are still in their portions."""
    rng = np.random.default_rng(seed)
    waiting = list(prompts.items())
    live, at = [], {}
    while waiting or live:
        while waiting and len(live) < 4 and (not live or rng.random() < 0.6):
            request, _ = waiting.pop(0)
            live.append(request)
            at[request] = 0
        entries, ended = [], []
        for request in live:
            if len(live) > 1 and rng.random() < 0.2:
                continue                    # a request may be left out of a step
            tokens = prompts[request]
            left = len(tokens) - at[request]
            if left > 12:
                n = int(min(rng.choice([2, 3, 5, 17, 40, 64, 90]), left - 12))
                n = n + 1 if left - 12 - n == 1 else n
                n = max(2, min(n, left - 12)) if left - 12 >= 2 else left - 12
            else:
                n = 1
            entries.append((request, tokens[at[request]:at[request] + n], list(range(n))))
            at[request] += n
            if at[request] == len(tokens):
                ended.append(request)
        if entries:
            builder.step(entries, end=ended)
            live = [r for r in live if r not in ended]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_replay_every_way_of_cutting(tmp_path, name, dtype):
    folder = make_model(str(tmp_path / "model"), name, seed=11)
    config, weights = plain.read_folder(folder)
    vocab, limit = config["vocab_size"], config["max_position_embeddings"]
    lengths = {"w": 200, "t": 190, "p": 230, "m0": 150, "m1": 97, "m2": 200, "m3": 66, "m4": 131, "m5": 35}
    prompts = {r: random_tokens(vocab, min(n, limit), seed=sum(map(ord, r)) + n) for r, n in lengths.items()}
    expected = {r: plain.forward(config, weights, t) for r, t in prompts.items()}

    builder = TraceBuilder()
    whole(builder, "w", prompts["w"])
    bulk_and_tail(builder, "t", prompts["t"])
    portions(builder, "p", prompts["p"])
    mixed(builder, {r: prompts[r] for r in ("m0", "m1", "m2", "m3", "m4", "m5")}, seed=5)
    assert max(len(s["entries"]) for s in builder.steps) == 4
    assert any(len(e["tokens"]) == 1 for s in builder.steps for e in s["entries"] if len(s["entries"]) > 1
               and any(len(o["tokens"]) > 1 for o in s["entries"])), "no step mixes portions with single tokens"
    # the pool is exactly as large as the live requests ever need: pages must be used again
    assert builder.peak < sum(round64(n) for n in lengths.values()) / 2

    results = run_trace(folder, dtype, str(tmp_path / "out"), builder.peak, builder.steps)
    covered = {r: np.zeros(len(t), dtype=bool) for r, t in prompts.items()}
    for number, rows in builder.rows.items():
        if not rows:
            continue
        want = np.stack([expected[r][p] for r, p in rows])
        assert_close(results[number], want, dtype, f"step {number} rows {rows[:3]}...")
        for r, p in rows:
            covered[r][p] = True
    assert all(c.all() for c in covered.values()), "some position was never compared"


def test_trace_run_protocol(tmp_path):
    """`done <step>` after every step, files only where something is wanted, exit 0 at the
    end of the input, and a clear failure for a token outside the vocabulary."""
    folder = make_model(str(tmp_path / "model"), "A", seed=2)
    steps = [{"step": 3, "entries": [{"id": "x", "tokens": [1, 2, 3], "want": []}], "end": []},
             {"step": 9, "entries": [{"id": "x", "tokens": [4, 5], "want": [1]}, {"id": 7, "tokens": [9], "want": [0]}], "end": ["x", 7]},
             {"step": 10, "entries": [], "end": []}]
    results = run_trace(folder, "float32", str(tmp_path / "out"), 128, steps)
    assert set(results) == {9} and results[9].shape == (2, 256)
    assert sorted(os.listdir(tmp_path / "out")) == ["9.f32"]
    config, weights = plain.read_folder(folder)
    assert_close(results[9][0], plain.forward(config, weights, [1, 2, 3, 4, 5])[4], "float32")
    assert_close(results[9][1], plain.forward(config, weights, [9])[0], "float32")
    bad = [{"step": 0, "entries": [{"id": "x", "tokens": [256], "want": [0]}], "end": []}]
    with pytest.raises(AssertionError, match="outside the vocabulary"):
        run_trace(folder, "float32", str(tmp_path / "out2"), 64, bad)
