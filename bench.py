"""Measures the engine on the LFM2-1.2B shape with random weights on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the whole batch. Prints ONE JSON line: decoded tokens a second
at batch 8 over the timed steps (``value``), the same at batch 1 and 64 and over all 512 tokens
that follow the 2,048-token prompts (``points``), the 2,048-token prefill up to its first token
(``prefill``) and the decode step's achieved fraction of the HBM roofline (``roofline``); the
two serving workloads (64 requests behind 32,768-token prompts on the LFM2-350M shape, 128 requests
of mixed lengths on the LFM2-2.6B shape) run at full size and give their tokens a second in
``points`` as well.
Peaks are the MI355X's published ones: HBM 8 TB/s, dense bfloat16 MFMA 2.5 PFLOP/s;
``attainable`` gives the same two fractions against a large copy and a large library product
measured in the same run.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK = 2.5e15

# The LFM2-1.2B shape, the headline configuration
SHAPE = dict(
    architectures=["Lfm2ForCausalLM"], model_type="lfm2", vocab_size=65536, hidden_size=2048, num_hidden_layers=16,
    num_attention_heads=32, num_key_value_heads=8, intermediate_size=12288, block_auto_adjust_ff_dim=True,
    block_ffn_dim_multiplier=1.0, block_multiple_of=256, norm_eps=1e-5, rope_theta=1000000.0, conv_L_cache=3,
    conv_bias=False, tie_word_embeddings=True, max_position_embeddings=4096, full_attn_idxs=[2, 5, 8, 10, 12, 14])
PROMPT = 2048
CONTEXT = 4096

# The two serving workloads beside the headline (the LFM2-350M shape under long contexts, the
# LFM2-2.6B shape under mixed traffic); run with --workload, they print one JSON line of their own.
SHAPE_350M = dict(SHAPE, hidden_size=1024, num_attention_heads=16, intermediate_size=6656, max_position_embeddings=34816)
SHAPE_2P6B = dict(SHAPE, num_hidden_layers=30, intermediate_size=10752, max_position_embeddings=9216,
                  full_attn_idxs=[2, 6, 10, 14, 18, 21, 24, 27])
WORKLOADS = {
    # 64 requests with 32,768-token prompts in portions of 2,048, 256 new tokens each: the cache is the load
    "long-context": dict(shape=SHAPE_350M, name="LFM2-350M shape", requests=64, prompt=(32768, 32768), output=(256, 256)),
    # 128 requests, prompts of 64..8,192 tokens and 128..1,024 new tokens, under continuous batching
    "mixed": dict(shape=SHAPE_2P6B, name="LFM2-2.6B shape", requests=128, prompt=(64, 8192), output=(128, 1024)),
}


def log(text: str) -> None:
    print(f"[bench] {text}", file=sys.stderr, flush=True)


DRAWING = dict(temperature=0.8, top_k=40, top_p=0.95, min_p=0.05)   # the reference's command-line defaults
DECODE_STEPS_PER_TURN = 4      # decode steps the engine runs on the device before the host is asked again


def steps_per_turn(steps: int, warmup: int) -> int:
    """The engine's decode_steps_per_turn for a run (the last turn of the warm-up and of the timed
    steps is cut to the steps that are left, so exactly as many steps run as were asked for)."""
    return max(1, min(DECODE_STEPS_PER_TURN, steps))


def decode_run(torch, model, config, batch: int, steps: int, warmup: int, seed: int = 0, prompt: int = PROMPT,
               context: int = CONTEXT, sampling: dict = None):
    """``batch`` requests with prompts of ``prompt`` tokens (``sampling``: how they draw their tokens; default:
    the most likely one); returns (seconds for ``steps`` decode steps, mean context, bytes the step must read).
    With ``warmup`` 0 the timed steps begin right behind the prompts' first tokens (the graph of a batch size
    that has not run before is recorded inside the timed region then: run the same call once before)."""
    import numpy as np
    from flyweight_amd import Runtime
    from flyweight_amd.engine import accounting
    # requests admitted earlier decode while later prompts are still running (continuous
    # batching), so they are up to one token for every portion of the later prompts ahead when the
    # timed steps begin
    portion = min(prompt, PROMPT)
    new_tokens = warmup + steps + batch * -(-prompt // portion) + 2 + DECODE_STEPS_PER_TURN
    if prompt + new_tokens > context:
        raise ValueError(f"a context of {context} does not hold a prompt of {prompt} and {new_tokens} new tokens")
    pages_each = (prompt + new_tokens + 63) // 64
    turn = steps_per_turn(steps, warmup)
    runtime = Runtime(model, context_limit=context, parallel_sequences=batch, num_pages=pages_each * batch,
                      max_batch_tokens=portion + batch, prefill_rows=portion, decode_steps_per_turn=turn).prepare()
    rng = np.random.default_rng(seed)
    for _ in range(batch):
        runtime.task_submit(rng.integers(0, config.vocab_size, prompt).tolist(), new_tokens, **(sampling or {}))
    # prompts: until every request has produced its first token
    while any(r.computed < len(r.prompt) for r in runtime.scheduler.requests.values()):
        runtime.engine_step()

    def decode(count: int) -> None:
        """Exactly ``count`` decode steps of the whole batch (a turn of the engine may hold several)."""
        tokens = 0
        while tokens < count * batch:
            runtime.decode_steps_per_turn = min(turn, count - tokens // batch)      # never past the steps asked for
            tokens += sum(1 for event in runtime.engine_step() if event[2] == 0)
        assert tokens == count * batch, "a step did not decode the whole batch"

    decode(warmup)
    requests = list(runtime.scheduler.requests.values())
    before = sum(r.computed for r in requests) / batch
    torch.cuda.synchronize()
    began = time.perf_counter()
    decode(steps)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - began
    mean_context = before + 1 + (steps - 1) / 2.0      # keys a row sees, averaged over requests and steps
    cache = runtime.stepper.cache
    step_bytes = accounting.step_weight_bytes(model.model) + batch * (
        mean_context * accounting.cache_bytes_per_token(cache) + accounting.state_bytes_per_request(cache))
    runtime.close()
    return elapsed, mean_context, step_bytes


def prefill_run(torch, model, config, repeats: int = 5, behind: int = 0, context: int = CONTEXT):
    """The median time of one step of 2,048 prompt tokens (logits at the last) behind ``behind`` cached tokens
    of the same request, and the flops of that step."""
    import statistics
    import numpy as np
    from flyweight_amd import Runtime, StepEntry
    from flyweight_amd.engine import accounting
    runtime = Runtime(model, context_limit=context, parallel_sequences=1, num_pages=(behind + PROMPT) // 64 + 1).prepare()
    rng = np.random.default_rng(1)
    times = []
    for i in range(repeats + 1):
        runtime.admit(i)
        for _ in range(behind // PROMPT):
            runtime.step([StepEntry(i, rng.integers(0, config.vocab_size, PROMPT).tolist(), [])])
        tokens = rng.integers(0, config.vocab_size, PROMPT).tolist()
        torch.cuda.synchronize()
        began = time.perf_counter()
        runtime.step([StepEntry(i, tokens, [PROMPT - 1])])
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - began
        runtime.release(i)
        if i > 0:       # the first run loads kernels
            times.append(elapsed)
    lm = model.model
    flops = (accounting.product_flops_per_token(lm) * PROMPT + accounting.head_flops_per_row(lm)
             + accounting.attention_flops(lm, PROMPT, behind))
    runtime.close()
    return statistics.median(times), flops


def first_token_run(torch, model, config, repeats: int = 5):
    """The median time of ``generate(prompt, 1)`` for a 2,048-token prompt: from the call to the first token
    in the caller's hands (the request submitted and planned, the prompt's one step, the most likely token found
    on the device and read back), as the reference times its prompt (src/flyweight/runtime_benchmark.py:129-216)."""
    import statistics
    import numpy as np
    from flyweight_amd import Runtime
    runtime = Runtime(model, context_limit=CONTEXT, parallel_sequences=1, num_pages=PROMPT // 64 + 1,
                      max_batch_tokens=PROMPT, prefill_rows=PROMPT).prepare()
    rng = np.random.default_rng(2)
    times = []
    for i in range(repeats + 1):
        tokens = rng.integers(0, config.vocab_size, PROMPT).tolist()
        torch.cuda.synchronize()
        began = time.perf_counter()
        produced = runtime.generate(tokens, 1)
        elapsed = time.perf_counter() - began
        assert len(produced) == 1
        if i > 0:
            times.append(elapsed)
    runtime.close()
    return statistics.median(times)


def generation_run(torch, model, config, batch: int, new_tokens: int = 512):
    """``batch`` requests with 2,048-token prompts that generate ``new_tokens`` tokens each, to the end: decoded
    tokens a second from the moment every prompt has run until the last request has finished (requests admitted
    earlier have decoded a few tokens beside the later prompts by then; those are not counted), and the mean
    context of that stretch. The same job with eight new tokens runs first on the same runtime, so every decode
    step of the timed stretch is a recorded one."""
    import numpy as np
    from flyweight_amd import Runtime
    pages_each = (PROMPT + new_tokens + 63) // 64
    runtime = Runtime(model, context_limit=CONTEXT, parallel_sequences=batch, num_pages=pages_each * batch,
                      max_batch_tokens=PROMPT + batch, prefill_rows=PROMPT, decode_steps_per_turn=DECODE_STEPS_PER_TURN).prepare()
    rng = np.random.default_rng(3)
    for count in (8, new_tokens):
        for _ in range(batch):
            runtime.task_submit(rng.integers(0, config.vocab_size, PROMPT).tolist(), count)
        while any(r.computed < len(r.prompt) for r in runtime.scheduler.requests.values()):
            runtime.engine_step()
        torch.cuda.synchronize()
        began = time.perf_counter()
        tokens = 0
        while runtime.scheduler.has_work():
            tokens += sum(1 for event in runtime.engine_step() if event[2] == 0)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - began
    runtime.close()
    return tokens / elapsed


def attainable_run(torch):
    """What this GPU gives a plain program: GB/s of a 1 GiB device-to-device copy (bytes read plus
    bytes written) and TFLOP/s of the library's 8192-cubed bfloat16 product of random numbers."""
    def timed(work, repeats: int = 10) -> float:
        for _ in range(3):
            work()
        torch.cuda.synchronize()
        began = time.perf_counter()
        for _ in range(repeats):
            work()
        torch.cuda.synchronize()
        return (time.perf_counter() - began) / repeats
    size = 1 << 30
    source = torch.zeros(size, dtype=torch.uint8, device="cuda")
    target = torch.empty_like(source)
    copy_gbs = 2 * size / timed(lambda: target.copy_(source)) / 1e9
    del source, target
    side = 8192
    a = torch.randn(side, side, device="cuda").to(torch.bfloat16)
    b = torch.randn(side, side, device="cuda").to(torch.bfloat16)
    out = torch.empty(side, side, dtype=torch.bfloat16, device="cuda")
    product_tflops = 2 * side ** 3 / timed(lambda: torch.matmul(a, b.T, out=out)) / 1e12
    return copy_gbs, product_tflops


def serving_run(torch, workload: str, requests: int, seed: int = 0) -> dict:
    """Submits every request of a workload at once and steps the engine until all are done."""
    import numpy as np
    from flyweight_amd import Model, Runtime
    from flyweight_amd.config import config_from_dict
    spec = WORKLOADS[workload]
    config = config_from_dict(spec["shape"])
    log(f"building the {spec['name']} with random bfloat16 weights")
    model = Model.random(config, seed=0, dtype="bfloat16")
    rng = np.random.default_rng(seed)
    prompts = rng.integers(spec["prompt"][0], spec["prompt"][1] + 1, requests).tolist()
    outputs = rng.integers(spec["output"][0], spec["output"][1] + 1, requests).tolist()
    context = max(p + o for p, o in zip(prompts, outputs))
    pages = sum((p + o + 63) // 64 for p, o in zip(prompts, outputs))
    # a step holds 2,048 tokens: the decoded tokens of the running requests first, portions of prompts in the rest
    runtime = Runtime(model, context_limit=context, parallel_sequences=requests, num_pages=pages,
                      max_batch_tokens=PROMPT, prefill_rows=PROMPT, decode_steps_per_turn=DECODE_STEPS_PER_TURN).prepare()
    # a short request first: every kernel and library is loaded before the clock starts
    runtime.generate(rng.integers(0, config.vocab_size, 100).tolist(), 4)
    for prompt, output in zip(prompts, outputs):
        runtime.task_submit(rng.integers(0, config.vocab_size, prompt).tolist(), output)
    log(f"{requests} requests, {sum(prompts)} prompt tokens, {sum(outputs)} tokens to generate")
    generated = finished = steps = 0
    steps_before = runtime.info["steps"]
    torch.cuda.synchronize()
    began = last = time.perf_counter()
    while runtime.scheduler.has_work():
        events = runtime.engine_step()
        steps += 1
        generated += sum(1 for e in events if e[2] == 0)
        finished += sum(1 for e in events if e[2] == 1)
        errors = [e for e in events if e[2] == 2]
        assert not errors, f"a request failed: {runtime.task_error(errors[0][0])}"
        if time.perf_counter() - last > 20.0:
            last = time.perf_counter()
            log(f"step {steps}: {generated} tokens generated, {finished} requests finished")
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - began
    assert finished == requests and generated == sum(outputs), (finished, generated)
    info = runtime.info
    preemptions = info["preemptions"]
    steps = info["steps"] - steps_before       # a turn of the engine may hold several decode steps
    runtime.close()
    return {
        "metric": f"tokens/s, prompt and generated ({workload} workload, {spec['name']})",
        "value": round((sum(prompts) + generated) / elapsed, 1), "unit": "tokens/s", "n_gpus": 1,
        "generated_per_s": round(generated / elapsed, 1), "seconds": round(elapsed, 3), "steps": steps,
        "steps_with_prompt_tokens": {"count": info["prefill_calls"], "seconds": round(info["prefill_ns"] * 1e-9, 3)},
        "decode_only_steps": {"count": steps - info["prefill_calls"], "seconds": round(info["decode_ns"] * 1e-9, 3)},
        "higher_is_better": True, "dtype": "bf16", "data": "synthetic: seeded uniform token ids and lengths, random-init weights",
        "config": config_record(config, spec["name"], requests=requests, prompt_tokens=sum(prompts),
                                generated_tokens=generated, longest_context=context, portion=PROMPT, cache_pages=pages,
                                preemptions=preemptions, decode_steps_per_turn=DECODE_STEPS_PER_TURN),
    }


def config_record(config, name: str, **more) -> dict:
    """Every size of the run, flat."""
    record = {"model": name, "layers": config.num_hidden_layers, "layers_of_named_config": config.num_hidden_layers,
              "hidden": config.hidden_size, "heads": config.num_attention_heads, "kv_heads": config.num_key_value_heads,
              "head_dim": config.head_dim, "ff_dim": config.ff_dim, "vocab": config.vocab_size,
              "attention_layers": len(config.full_attn_idxs), "conv_L_cache": config.conv_L_cache}
    record.update(more)
    return record


def further_points(torch, args, points: dict) -> None:
    """Decode and prefill at further sizes: more requests, a model that allows 128,000 positions run at a
    4,096-token context, and the LFM2-350M shape behind 32,768-token contexts. Tokens a second, and for each
    the fraction of the published peak that bounds it (``*_frac``)."""
    from flyweight_amd import Model
    from flyweight_amd.config import config_from_dict
    config = config_from_dict(dict(SHAPE, max_position_embeddings=128000))
    model = Model.random(config, seed=0, dtype="bfloat16")
    # (at least 64 and 32 steps: a run of a few turns right behind a model's creation times that as well)
    for batch, steps in ((8, max(args.steps, 64)), (64, max(args.steps, 32)), (128, max(args.steps, 32)), (256, max(args.steps, 32))):
        name = f"decode_b{batch}" + ("_maxpos128k" if batch <= 64 else "")
        log(f"decode at batch {batch}, max_position_embeddings 128,000, context {CONTEXT}")
        seconds, _, step_bytes = decode_run(torch, model, config, batch, steps, min(args.warmup, 8))
        points[name] = round(batch * steps / seconds, 1)
        points[name + "_frac"] = round(step_bytes / (seconds / steps) / 1e9 / HBM_PEAK_GBS, 4)
    # requests that draw their tokens with the reference's command-line defaults, each from its own generator
    drawing = DRAWING
    for batch, steps in ((8, min(args.steps, 64)), (64, min(args.steps, 32))):
        log(f"decode at batch {batch}, tokens drawn (temperature 0.8, top_k 40, top_p 0.95, min_p 0.05)")
        seconds, _, _ = decode_run(torch, model, config, batch, steps, min(args.warmup, 8), sampling=drawing)
        points[f"decode_b{batch}_drawn"] = round(batch * steps / seconds, 1)
    del model
    torch.cuda.empty_cache()
    long_context = 32768
    config = config_from_dict(SHAPE_350M)
    model = Model.random(config, seed=0, dtype="bfloat16")
    log("LFM2-350M shape: a 2,048-token portion behind 30,720 cached tokens")
    seconds, flops = prefill_run(torch, model, config, repeats=3, behind=long_context - PROMPT, context=long_context + 2048)
    points["prefill_2048_behind_30720_350m"] = round(PROMPT / seconds, 1)
    points["prefill_2048_behind_30720_350m_frac"] = round(flops / seconds / MFMA_BF16_PEAK, 4)
    log("LFM2-350M shape: decode at batch 64 behind 32,768-token prompts")
    steps = min(args.steps, 32)
    seconds, _, step_bytes = decode_run(torch, model, config, 64, steps, min(args.warmup, 4), prompt=long_context,
                                        context=long_context + 2048)
    points["decode_b64_ctx32k_350m"] = round(64 * steps / seconds, 1)
    points["decode_b64_ctx32k_350m_frac"] = round(step_bytes / (seconds / steps) / 1e9 / HBM_PEAK_GBS, 4)
    del model
    torch.cuda.empty_cache()
    # the two serving workloads at full size: whole jobs through the scheduler, tokens (prompt and generated) a
    # second; `--workload` runs one of them alone and prints a line of its own with the run's other figures
    for workload in ("long-context", "mixed"):
        requests = WORKLOADS[workload]["requests"]
        record = serving_run(torch, workload, requests)
        points[f"serving_{workload.replace('-', '_')}_{requests}req"] = record["value"]
        points[f"serving_{workload.replace('-', '_')}_{requests}req_generated_per_s"] = record["generated_per_s"]


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=256)
    parser.add_argument("--warmup", type=int, default=16)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--skip-points", action="store_true", help="only the headline batch")
    parser.add_argument("--skip-further", action="store_true", help="without the points at further sizes")
    parser.add_argument("--only", choices=("decode", "prefill"), help="run one phase and print no JSON (for profiling)")
    parser.add_argument("--drawn", action="store_true", help="with --only decode: the requests draw their tokens "
                        "(temperature 0.8, top_k 40, top_p 0.95, min_p 0.05) instead of taking the most likely one")
    parser.add_argument("--workload", choices=("headline",) + tuple(WORKLOADS), default="headline",
                        help="headline: the LFM2-1.2B decode and prefill figures; the others: a whole serving run")
    parser.add_argument("--requests", type=int, help="requests of a serving workload (default: as the workload names)")
    args = parser.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print(f"bench.py measures one GPU: this engine has no multi-GPU path (asked for {args.gpus})", flush=True)
        return 2
    if PROMPT + args.warmup + args.steps + 256 + 2 + DECODE_STEPS_PER_TURN > CONTEXT:
        print("bench.py: warmup + steps must leave the 4,096-token context room", flush=True)
        return 2

    import torch
    from flyweight_amd import Model
    from flyweight_amd.config import config_from_dict

    if args.workload != "headline":
        print(json.dumps(serving_run(torch, args.workload, args.requests or WORKLOADS[args.workload]["requests"])), flush=True)
        return 0
    config = config_from_dict(SHAPE)
    log("building the LFM2-1.2B shape with random bfloat16 weights")
    model = Model.random(config, seed=0, dtype="bfloat16")

    if args.only == "decode":
        elapsed, _, _ = decode_run(torch, model, config, args.batch, args.steps, args.warmup, sampling=DRAWING if args.drawn else None)
        log(f"{args.batch * args.steps / elapsed:.1f} tokens/s")
        return 0
    log("prefill of 2,048 tokens")
    step_s, prefill_flops = prefill_run(torch, model, config)
    if args.only == "prefill":
        log(f"{PROMPT / step_s:.1f} tokens/s")
        return 0
    prefill_s = first_token_run(torch, model, config)
    log(f"the prompt's step alone {step_s * 1e3:.3f} ms, generate(prompt, 1) {prefill_s * 1e3:.3f} ms")

    log(f"decode at batch {args.batch}: {args.warmup} warm-up and {args.steps} timed steps")
    elapsed, mean_context, step_bytes = decode_run(torch, model, config, args.batch, args.steps, args.warmup)
    value = args.batch * args.steps / elapsed
    achieved = step_bytes / (elapsed / args.steps) / 1e9

    points = {}
    if not args.skip_points:
        for batch, steps in ((1, min(args.steps, 128)), (64, min(args.steps, 64))):
            log(f"decode at batch {batch}")
            seconds, _, point_bytes = decode_run(torch, model, config, batch, steps, min(args.warmup, 8))
            points[f"decode_b{batch}"] = round(batch * steps / seconds, 1)
            points[f"decode_b{batch}_frac"] = round(point_bytes / (seconds / steps) / 1e9 / HBM_PEAK_GBS, 4)
        # the whole stretch the headline configuration names: 512 generated tokens behind 2,048-token prompts
        for batch in (1, 8, 64):
            log(f"decode at batch {batch}: all 512 generated tokens")
            points[f"decode_b{batch}_512tok"] = round(generation_run(torch, model, config, batch), 1)

    log("a large copy and a large library product, for what the GPU gives a plain program")
    copy_gbs, product_tflops = attainable_run(torch)
    if not args.skip_points and not args.skip_further:
        del model
        torch.cuda.empty_cache()
        further_points(torch, args, points)

    print(json.dumps({
        "metric": "decode tok/s @ batch 8 (LFM2-1.2B shape, 2,048-token prompts, context 4,096)",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(elapsed / args.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic: seeded uniform token ids, random-init weights",
        "config": config_record(config, "LFM2-1.2B shape", global_batch=args.batch, prompt_len=PROMPT, seq_len=CONTEXT,
                                decode_steps_per_turn=steps_per_turn(args.steps, args.warmup), parallelism="single GPU"),
        # generate(prompt, 1): to the first token in the caller's hands; step_ms: the prompt's one step alone
        "prefill": {"value": round(PROMPT / prefill_s, 1), "tokens": PROMPT, "ms": round(prefill_s * 1e3, 3),
                    "frac": round(prefill_flops / prefill_s / MFMA_BF16_PEAK, 4), "step_ms": round(step_s * 1e3, 3),
                    "step_frac": round(prefill_flops / step_s / MFMA_BF16_PEAK, 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": points,
        # the same two fractions against what was measured on this GPU instead of the published peaks
        "attainable": {"copy_gbs": round(copy_gbs, 1), "product_tflops": round(product_tflops, 1),
                       "roofline_frac": round(achieved / copy_gbs, 4),
                       "prefill_frac": round(prefill_flops / step_s / (product_tflops * 1e12), 4)},
    }), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
