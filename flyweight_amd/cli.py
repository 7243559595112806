"""Command line, after the reference's ``flyweight`` (src/flyweight/cli.py:1030-1184): the
same subcommand names and the same names, meanings and defaults of options where the
reference has them. The engine works on token ids: where the reference takes ``--prompt
TEXT`` and a chat template, this takes ``--tokens IDS`` (the form the reference's own
``benchmark --tokens`` has, src/flyweight/cli.py:1134-1137).

  flyweight-amd generate MODEL --tokens 1,2,3 [--max-tokens 64] [--temperature 0.8] ...
  flyweight-amd benchmark MODEL [--tokens IDS] [--warmup 3] [--iterations 128] [--context 2048]
  flyweight-amd inspect MODEL
  flyweight-amd random-weights --config CONFIG.json --seed S --out DIR
  flyweight-amd replay --model DIR --dtype bfloat16 --out DIR --max-tokens N   (steps on stdin)
"""

from __future__ import annotations

import argparse
import json
import statistics
import sys
import time
from typing import List, Optional


def _token_list(text: str) -> List[int]:
    try:
        return [int(part) for part in text.replace(",", " ").split()]
    except ValueError:
        raise argparse.ArgumentTypeError(f"token ids are integers separated by commas or spaces, got {text!r}") from None


def _add_model(parser: argparse.ArgumentParser) -> None:
    parser.add_argument("model", metavar="MODEL", help="model folder (config.json and model.safetensors)")
    parser.add_argument("--dtype", default="bfloat16", choices=("bfloat16", "float32"),
                        help="bfloat16 (serving kernels) or float32 (everything in true 32-bit)")


def _add_runtime(parser: argparse.ArgumentParser, context_default: int) -> None:
    group = parser.add_argument_group("runtime")
    group.add_argument("--context", "--context-window", dest="context_window", type=int, default=context_default,
                       metavar="N", help=f"maximum prompt + output tokens (default {context_default})")
    group.add_argument("--parallel", type=int, default=1, metavar="N", help="requests that may be live at once")
    group.add_argument("--num-pages", type=int, metavar="N",
                       help="cache pages of 64 tokens in every page group (default: every live request at the full context)")
    group.add_argument("--prefill-rows", type=int, default=512, metavar="N", help="most tokens of one prompt portion")
    group.add_argument("--max-batch-tokens", type=int, default=2048, metavar="N", help="most tokens of one step")
    group.add_argument("--decode-steps-per-turn", type=int, default=1, metavar="N",
                       help="decode steps that may run back to back on the device before the host reads their tokens "
                            "(greedy requests without stop tokens; tokens then arrive in bursts)")


def build_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(prog="flyweight-amd", description="LFM2 inference on the AMD Instinct MI355X")
    commands = parser.add_subparsers(dest="command", required=True)

    generate = commands.add_parser("generate", help="generate the tokens that follow a prompt, print them, exit")
    _add_model(generate)
    request = generate.add_argument_group("request")
    request.add_argument("--tokens", "--prompt", dest="tokens", type=_token_list, metavar="IDS",
                         help="the prompt as token ids, e.g. 1,2,3")
    request.add_argument("--tokens-file", metavar="FILE", help="a file of token ids instead of --tokens")
    request.add_argument("--max-tokens", "--max-new-tokens", dest="max_new_tokens", type=int, default=64, metavar="N",
                         help="stop after this many new tokens")
    request.add_argument("--stop-token", dest="stop_tokens", type=int, action="append", default=[], metavar="ID",
                         help="a token id that ends the output when it is produced; repeat the option for several (without it: the eos id of the model's configuration)")
    request.add_argument("--ignore-eos", action="store_true",
                         help="do not end at the model's eos id either: only --stop-token ids and --max-tokens end the output")
    sampling = generate.add_argument_group("sampling")
    sampling.add_argument("--temperature", type=float, default=0.8, metavar="X", help="divides the logits before the draw; 0 always takes the most likely token")
    sampling.add_argument("--top-k", type=int, default=40, metavar="N", help="draw among the N most likely tokens only (0: among all)")
    sampling.add_argument("--top-p", type=float, default=0.95, metavar="X",
                          help="keep the most likely tokens until their probabilities add up to X, a number in (0, 1]")
    sampling.add_argument("--min-p", type=float, default=0.05, metavar="X",
                          help="leave out tokens less probable than X times the most probable one; X in [0, 1], 0 keeps all")
    sampling.add_argument("--seed", type=int, metavar="N", help="start the request's random stream here, so that a run can be repeated")
    _add_runtime(generate, 32768)

    benchmark = commands.add_parser("benchmark", help="time the prompt with its first token, then decode steps, and print the figures as JSON")
    _add_model(benchmark)
    benchmark.add_argument("--tokens", type=_token_list, default=[0], metavar="IDS", help="token ids of the prompt, comma-separated")
    benchmark.add_argument("--warmup", type=int, default=3, metavar="N", help="decode steps before the clock starts")
    benchmark.add_argument("--iterations", type=int, default=128, metavar="N", help="decode steps under the clock")
    benchmark.add_argument("--temperature", type=float, default=0.0)
    benchmark.add_argument("--top-k", type=int, default=0)
    benchmark.add_argument("--top-p", type=float, default=0.0)
    benchmark.add_argument("--kernel-profile", action="store_true",
                           help="bracket every kernel call with events and add GPU time per kernel to the report "
                                "(steps then run launch by launch, not from recorded graphs; also FLYWEIGHT_KERNEL_PROFILE=1)")
    _add_runtime(benchmark, 2048)

    inspect = commands.add_parser("inspect", help="print the configuration, derived sizes and tensor table as JSON")
    inspect.add_argument("model", metavar="MODEL")

    random_weights = commands.add_parser("random-weights", help="write a model folder with random weights")
    random_weights.add_argument("--config", required=True, metavar="FILE", help="a config.json of a registered architecture")
    random_weights.add_argument("--seed", type=int, default=0)
    random_weights.add_argument("--out", required=True, metavar="DIR")
    random_weights.add_argument("--dtype", default="bfloat16", choices=("bfloat16", "float32"),
                                help="storage precision of the matrices")

    replay = commands.add_parser("replay", help="replay a trace of steps from standard input and write logits")
    replay.add_argument("--model", required=True, metavar="DIR")
    replay.add_argument("--dtype", required=True, choices=("bfloat16", "float32"))
    replay.add_argument("--out", required=True, metavar="DIR")
    replay.add_argument("--max-tokens", required=True, type=int, metavar="N")
    return parser


def _runtime(args, context: Optional[int] = None):
    from .engine import Model, Runtime
    model = Model(args.model, dtype=args.dtype)
    limit = min(context or args.context_window, model.spec.max_positions)
    return model, Runtime(model, context_limit=limit, parallel_sequences=args.parallel, num_pages=args.num_pages,
                          prefill_rows=args.prefill_rows, max_batch_tokens=args.max_batch_tokens,
                          decode_steps_per_turn=args.decode_steps_per_turn).prepare()


def _generate(args) -> int:
    tokens = args.tokens
    if args.tokens_file:
        with open(args.tokens_file, "r", encoding="utf-8") as handle:
            tokens = _token_list(handle.read())
    if not tokens:
        print("generate: give the prompt with --tokens IDS or --tokens-file FILE", file=sys.stderr)
        return 2
    model, runtime = _runtime(args)
    stops = list(args.stop_tokens)
    if not stops and not args.ignore_eos and model.spec.eos_token_id is not None:
        stops = [model.spec.eos_token_id]
    produced = runtime.generate(tokens, args.max_new_tokens, stop_tokens=stops, temperature=args.temperature,
                                top_k=args.top_k, top_p=args.top_p, min_p=args.min_p, seed=args.seed)
    print(" ".join(str(t) for t in produced))
    return 0


def _benchmark(args) -> int:
    """The reference's protocol (src/flyweight/runtime_benchmark.py:129-216, cli.py:1749-1794):
    prompt + first token as one latency, then warm-up decodes, then timed decodes."""
    import torch
    from .kernels import ops
    if args.kernel_profile:
        ops.kernel_profile(True)
    began = time.perf_counter()
    model, runtime = _runtime(args)
    torch.cuda.synchronize()
    prepare_seconds = time.perf_counter() - began
    total = args.warmup + args.iterations
    arrivals: List[float] = []

    def on_token(_token: int):
        torch.cuda.synchronize()
        arrivals.append(time.perf_counter())

    began = time.perf_counter()
    top_p = args.top_p if args.top_p > 0 else 1.0
    runtime.generate(args.tokens, total + 1, callback=on_token, temperature=args.temperature, top_k=args.top_k,
                     top_p=top_p, min_p=0.0)
    first = arrivals[0] - began
    gaps = [b - a for a, b in zip(arrivals, arrivals[1:])][args.warmup:]
    measured = sum(gaps)
    ordered = sorted(gaps)
    pick = lambda q: ordered[min(len(ordered) - 1, int(q * len(ordered)))] if ordered else 0.0   # noqa: E731
    # a short stretch can overstate the sustained rate: the first and the last window side by side show a decay
    window = min(32, max(1, len(gaps) // 2))
    rate = lambda part: len(part) / sum(part) if sum(part) > 0 else 0.0     # noqa: E731
    report = {
        "prepare_seconds": prepare_seconds,
        "prompt_tokens": len(args.tokens),
        "prompt_and_first_token_seconds": first,
        "iterations": len(gaps),
        "decode_tokens_per_second": len(gaps) / measured if measured > 0 else 0.0,
        "median_seconds": statistics.median(gaps) if gaps else 0.0,
        "p90_seconds": pick(0.90),
        "p99_seconds": pick(0.99),
        "decode_first_window_tokens_per_second": rate(gaps[:window]),
        "decode_last_window_tokens_per_second": rate(gaps[-window:]),
        "request_seconds": (arrivals[-1] - began) if arrivals else 0.0,
        "generated_tokens": len(arrivals),
    }
    if ops.kernel_profile_active():
        report["kernels"] = ops.kernel_profile_report()
    print(json.dumps(report))
    return 0


def _inspect(args) -> int:
    from .config import load_config
    from .engine.model import declared_tensors
    config = load_config(args.model)
    spec = config.model_spec()
    tensors = declared_tensors(spec)
    parameters = sum(int(__import__("math").prod(d.shape)) for d in tensors.values())
    print(json.dumps({
        "architecture": spec.architecture,
        "config": config.to_dict(),
        "derived": {"head_dim": getattr(config, "head_dim", None), "ff_dim": getattr(config, "ff_dim", None),
                    "layers": len(spec.layers), "parameters": parameters},
        "tensors": {name: {"shape": list(decl.shape), "role": decl.role} for name, decl in tensors.items()},
    }, indent=2))
    return 0


def _random_weights(args) -> int:
    import torch
    from .config import config_from_dict
    from .weights import write_random_model
    with open(args.config, "r", encoding="utf-8") as handle:
        config = config_from_dict(json.load(handle))
    dtype = torch.bfloat16 if args.dtype == "bfloat16" else torch.float32
    print(write_random_model(args.out, config, args.seed, dtype))
    return 0


def main(argv: Optional[List[str]] = None) -> int:
    args = build_parser().parse_args(argv)
    try:
        if args.command == "generate":
            return _generate(args)
        if args.command == "benchmark":
            return _benchmark(args)
        if args.command == "inspect":
            return _inspect(args)
        if args.command == "random-weights":
            return _random_weights(args)
        if args.command == "replay":
            from .engine.trace import replay
            return replay(args.model, args.dtype, args.out, args.max_tokens, sys.stdin, sys.stdout)
    except (ValueError, RuntimeError, OSError) as error:
        print(f"flyweight-amd: {error}", file=sys.stderr)
        return 1
    return 2


if __name__ == "__main__":
    sys.exit(main())
