"""Logits behind a context of more than 32,000 tokens against the plain model: what the serving
workloads run (block tables of more than 512 pages, hundreds of runs of keys per decoded row,
four query heads of a group per workgroup in the prompt kernel, recorded decode steps whose
context bucket grows under a live request), in float32 and in bfloat16.

A narrow model (conv, attention, conv, attention; four heads of 64 channels on one kv head)
keeps the plain model's work to one full attention over the long sequence. The q and k norm
weights are scaled so that the softmax picks a few keys out of the thousands: with random
weights as they come every row would average over all keys, and a page that a kernel missed
or read twice would move the result by less than bfloat16's rounding. (Measured with the
factor below: the engine is off by 7.8e-6 of the largest logit in float32 and 4.2e-2 in
bfloat16; with one of the 512 key pages zeroed, or two of them swapped, by 1.3e-1 to 2.0e-1 in
both. With the weights as drawn a bfloat16 run was off by 9.7e-3 with or without the fault.)

One request: the prompt in portions of 2,048 tokens, the last one ending 40 tokens before
position 32,768, then 64 tokens one by one (position 32,768 = page 512 is crossed on the way).
Four requests of unequal lengths (one of them the same long sequence, the others with tokens of
their own) on the pages the first run gave back: portions of all four in every step, sized so
that all prompts end in the same step, then 64 steps of four decoded tokens."""

import numpy as np
import pytest

import plain_lfm2 as plain
from helpers import assert_close, random_tokens

pytestmark = pytest.mark.gpu

LONG = dict(
    architectures=["Lfm2ForCausalLM"], model_type="lfm2", vocab_size=320, hidden_size=256, num_hidden_layers=4,
    num_attention_heads=4, num_key_value_heads=1, intermediate_size=384, block_auto_adjust_ff_dim=False,
    norm_eps=1e-5, rope_theta=1000000.0, conv_L_cache=3, conv_bias=False, tie_word_embeddings=True,
    max_position_embeddings=33024, layer_types=["conv", "full_attention", "conv", "full_attention"])
PROMPTS = {"long": 32728, "b": 12000, "c": 5000, "d": 700}
DECODED = 64
SHARPER = 2.5           # the factor on the q and k norm weights (scores: its square)


@pytest.fixture(scope="module")
def case(tmp_path_factory):
    """(model folder, {request: tokens}, {request: expected logits of the last 65 positions})."""
    import os
    from flyweight_amd.config import config_from_dict
    from flyweight_amd.weights import SafetensorsFile, write_file, write_random_model
    root = tmp_path_factory.mktemp("long")
    base = write_random_model(str(root / "base"), config_from_dict(LONG), seed=11, scale="fan_in")
    with SafetensorsFile(os.path.join(base, "model.safetensors")) as handle:
        tensors = {n: handle.tensor(n) for n in handle.names()}
    tokens = {name: random_tokens(LONG["vocab_size"], length + DECODED, seed=50 + i) for i, (name, length) in enumerate(PROMPTS.items())}
    folder = str(root / "sharp")
    os.makedirs(folder)
    write_file(os.path.join(folder, "model.safetensors"),
               {n: (t * SHARPER if n.endswith(("q_layernorm.weight", "k_layernorm.weight")) else t) for n, t in tensors.items()})
    config_from_dict(LONG).save(folder)
    config, weights = plain.read_folder(folder)
    return folder, tokens, {name: plain.forward_tail(config, weights, tokens[name], DECODED + 1) for name in tokens}


def portions_of(length: int, steps: int):
    """``length`` tokens cut into ``steps`` portions that differ by at most one token."""
    return [length // steps + (1 if i < length % steps else 0) for i in range(steps)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_logits_behind_a_long_context(case, dtype):
    from flyweight_amd.engine import StepEntry, Stepper, load_model
    folder, tokens, want = case
    _, model = load_model(folder, dtype=dtype)
    pages = sum((len(t) + 63) // 64 for t in tokens.values())
    stepper = Stepper(model, num_pages=pages + 2, max_requests=4)

    # one request
    stepper.admit("long")
    sequence, prompt = tokens["long"], PROMPTS["long"]
    got = []
    for at in range(0, prompt, 2048):
        n = min(2048, prompt - at)
        out = stepper.step([StepEntry("long", sequence[at:at + n], [n - 1] if at + n == prompt else [])])
    got.append(out.cpu().numpy())
    for at in range(prompt, prompt + DECODED):
        got.append(stepper.step([StepEntry("long", sequence[at:at + 1], [0])]).cpu().numpy())
    assert_close(np.concatenate(got), want["long"], dtype, f"{dtype}: one request, 2,048-token portions and {DECODED} decoded tokens")
    stepper.release("long")
    stepper.cache.check_invariants()
    assert stepper.cache.groups[0].pool.in_use == 0

    # four requests of unequal length side by side, on the pages given back
    steps = 16
    plan = {name: portions_of(PROMPTS[name], steps) for name in PROMPTS}
    order = ["c", "long", "d", "b"]
    for name in order:
        stepper.admit(name)
    at = {name: 0 for name in order}
    got = {name: [] for name in order}
    for step in range(steps):
        entries = []
        for name in order:
            n = plan[name][step]
            entries.append(StepEntry(name, tokens[name][at[name]:at[name] + n], [n - 1] if step == steps - 1 else []))
            at[name] += n
        out = stepper.step(entries)
    for row, name in enumerate(order):
        assert at[name] == PROMPTS[name]
        got[name].append(out[row:row + 1].cpu().numpy())
    for _ in range(DECODED):
        out = stepper.step([StepEntry(name, tokens[name][at[name]:at[name] + 1], [0]) for name in order]).cpu().numpy()
        for row, name in enumerate(order):
            got[name].append(out[row:row + 1])
            at[name] += 1
    for name in order:
        assert_close(np.concatenate(got[name]), want[name], dtype, f"{dtype}: request {name} of {PROMPTS[name]} tokens beside three others")
        stepper.release(name)
    stepper.cache.check_invariants()
    assert stepper.cache.groups[0].pool.in_use == 0
    if dtype == "bfloat16":
        assert stepper.graph_replays > 0       # the decoded tokens came from recorded steps
