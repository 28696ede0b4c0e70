"""Trace replay: feeds given token ids through a model step by step and writes logits.

It samples nothing and schedules nothing; it drives the engine's own model, step function,
cache and kernels.  The reference's nearest tool is ``generate-token-ids``
(`src/app/cli/inspect.zig:246-312`), which feeds given ids one by one through the forward
function.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Standard input holds one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step in which something is wanted, ``OUT/<step>.f32`` receives the logits at the
wanted places as little-endian float32 [wanted, vocab]; after every step a line
``done <step>`` is printed.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
from typing import List, Optional

import numpy as np
import torch

from ..errors import ZinferError
from .batch import StepEntry
from .engine import Engine

PAGE_SIZE = 16
MAX_LIVE_REQUESTS = 16


def make_engine(model_dir: str, dtype: str, max_tokens: int, device: str = "cuda:0",
                page_size: int = PAGE_SIZE, poison_freed: bool = False) -> Engine:
    from ..models.build import load_model
    _, model = load_model(model_dir, dtype, device)
    # max_tokens counts every live request rounded up to 64 tokens; with pages that do not
    # divide 64 a request of 64 tokens still needs ceil(64 / page_size) of them
    units = (max_tokens + 63) // 64
    num_pages = max((max_tokens + page_size - 1) // page_size,
                    units * ((64 + page_size - 1) // page_size) if 64 % page_size else 0)
    return Engine(model, page_size=page_size, num_pages=num_pages,
                  max_requests=MAX_LIVE_REQUESTS, poison_freed=poison_freed)


def run_trace(engine: Engine, lines, out_dir: str, report=None) -> int:
    """Runs every step of ``lines`` (an iterable of JSON texts); returns the number of steps."""
    os.makedirs(out_dir, exist_ok=True)
    n = 0
    for line in lines:
        line = line.strip()
        if not line:
            continue
        obj = json.loads(line)
        step = obj["step"]
        entries = [StepEntry(e["id"], [int(t) for t in e["tokens"]],
                             [int(w) for w in e.get("want", [])])
                   for e in obj.get("entries", [])]
        logits = engine.step(entries, end=obj.get("end", []))
        if logits.shape[0] > 0:
            arr = logits.detach().to("cpu", torch.float32).numpy().astype("<f4", copy=False)
            arr.tofile(os.path.join(out_dir, f"{step}.f32"))
        n += 1
        if report is not None:
            report(step)
    return n


def main(argv: Optional[List[str]] = None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder that receives <step>.f32")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64)")
    ap.add_argument("--device", default="cuda:0")
    args = ap.parse_args(argv)
    try:
        engine = make_engine(args.model, args.dtype, args.max_tokens, args.device)

        def report(step):
            sys.stdout.write(f"done {step}\n")
            sys.stdout.flush()

        run_trace(engine, sys.stdin, args.out, report)
    except ZinferError as e:
        print(f"trace_run: {type(e).__name__}: {e}", file=sys.stderr)
        return 1
    return 0


if __name__ == "__main__":
    sys.exit(main())
