"""Trace replay: feeds given token ids through the model step by step and writes logits.

It samples nothing and has no forward pass, cache or loader of its own: it drives the
same model, step function, cache manager and kernels that generation uses. Steps arrive as
JSON lines; see ``bin/trace_run``.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
from typing import IO, List, Optional

PAGE_SIZE = 64
MAX_LIVE_SLOTS = 64     # state slots are memory per request: bounded even when the pool is large


def build_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(
        prog="trace_run",
        description="Replay a trace of steps (JSON lines on standard input) through the engine and write the "
                    "logits at the wanted places to OUT/<step>.f32 (little-endian float32, [wanted, vocab]).")
    parser.add_argument("--model", required=True, metavar="DIR", help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", required=True, choices=("bfloat16", "float32"),
                        help="bfloat16: the kernels and precisions that serving uses; float32: everything in true 32-bit")
    parser.add_argument("--out", required=True, metavar="DIR", help="where the logits files go")
    parser.add_argument("--max-tokens", required=True, type=int, metavar="N",
                        help="the most tokens live requests hold at any time, each request rounded up to a multiple "
                             f"of {PAGE_SIZE}; the cache pool is made for this many. As many requests may be live "
                             f"as the pool has pages (a request holds at least one), at most {MAX_LIVE_SLOTS}")
    parser.add_argument("--device", default="cuda:0", help=argparse.SUPPRESS)
    return parser


def replay(model_dir: str, dtype: str, out_dir: str, max_tokens: int, lines: IO[str], done: IO[str],
           device: str = "cuda:0") -> int:
    import numpy as np
    import torch

    from .model import load_model
    from .step import StepEntry, Stepper

    if max_tokens <= 0:
        raise ValueError("--max-tokens must be positive")
    os.makedirs(out_dir, exist_ok=True)
    _, model = load_model(model_dir, dtype=dtype, device=device)
    num_pages = (max_tokens + PAGE_SIZE - 1) // PAGE_SIZE
    stepper = Stepper(model, num_pages=num_pages, max_requests=min(num_pages, MAX_LIVE_SLOTS), page_size=PAGE_SIZE)
    for number, line in enumerate(lines):
        line = line.strip()
        if not line:
            continue
        try:
            record = json.loads(line)
        except json.JSONDecodeError as error:
            raise ValueError(f"input line {number + 1} is not JSON: {error}") from None
        step = record["step"]
        entries: List[StepEntry] = []
        for item in record.get("entries", []):
            request = item["id"]
            if not stepper.is_live(request):
                stepper.admit(request)
            entries.append(StepEntry(request, [int(t) for t in item["tokens"]], [int(p) for p in item.get("want", [])]))
        if entries:
            logits = stepper.step(entries)
            if logits is not None:
                host = logits.to(torch.float32).cpu().numpy().astype("<f4", copy=False)
                host.tofile(os.path.join(out_dir, f"{step}.f32"))
        for request in record.get("end", []):
            if stepper.is_live(request):
                stepper.release(request)
        done.write(f"done {step}\n")
        done.flush()
    return 0


def main(argv: Optional[List[str]] = None) -> int:
    args = build_parser().parse_args(argv)
    try:
        return replay(args.model, args.dtype, args.out, args.max_tokens, sys.stdin, sys.stdout, device=args.device)
    except Exception as error:      # one line on stderr, non-zero exit: the caller sees which step failed
        print(f"trace_run: {type(error).__name__}: {error}", file=sys.stderr, flush=True)
        return 1


if __name__ == "__main__":
    sys.exit(main())
