"""Trace replay: feeds given token ids through a model step by step and writes logits.

It samples nothing and schedules nothing; it drives the engine's own model, step function,
cache and kernels.  The reference's nearest tool is ``generate-token-ids``
(`src/app/cli/inspect.zig:246-312`), which feeds given ids one by one through the forward
function.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N
              [--page-size P] [--num-pages N] [--max-requests R]

Standard input holds one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

An entry may also say where its tokens begin, ``"start": 12``: the number of tokens the
request must hold already.  A trace that leaves tokens out or brings them twice is then an
error that names the request and the gap, instead of logits at positions nobody meant.

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

from ..errors import StepError, ZinferError
from .batch import StepEntry
from .engine import Engine

PAGE_SIZE = 16
MAX_LIVE_REQUESTS = 16


def pages_for(max_tokens: int, page_size: int) -> int:
    """Pages that hold ``max_tokens`` tokens of live requests, each request's count rounded up
    to 64: with pages that do not divide 64 a request of 64 tokens still needs
    ceil(64 / page_size) of them."""
    units = (max_tokens + 63) // 64
    return max((max_tokens + page_size - 1) // page_size,
               units * ((64 + page_size - 1) // page_size) if 64 % page_size else 0)


def make_engine(model_dir: str, dtype: str, max_tokens: int, device: str = "cuda:0",
                page_size: int = PAGE_SIZE, poison_freed: bool = False,
                num_pages: Optional[int] = None,
                max_requests: int = MAX_LIVE_REQUESTS) -> Engine:
    """The engine a replay drives.  ``num_pages`` overrides the pool size that ``max_tokens``
    gives; ``max_requests`` is the number of request slots."""
    from ..models.build import load_model
    if page_size < 1 or max_requests < 1 or (num_pages is not None and num_pages < 1):
        raise StepError("page size, number of pages and request slots must be at least 1")
    _, model = load_model(model_dir, dtype, device)
    if num_pages is None:
        num_pages = pages_for(max_tokens, page_size)
    return Engine(model, page_size=page_size, num_pages=num_pages,
                  max_requests=max_requests, poison_freed=poison_freed)


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
        entries = []
        for e in obj.get("entries", []):
            if e.get("start") is not None:
                held = engine.length(e["id"]) if engine.has_request(e["id"]) else 0
                start = int(e["start"])
                if start != held:
                    what = f"tokens {held}..{start - 1} were never given" if start > held \
                        else f"tokens {start}..{held - 1} are held already"
                    raise StepError(f"PositionGap: step {step}, request {e['id']!r} starts at "
                                    f"{start} but holds {held} tokens ({what})")
            entries.append(StepEntry(e["id"], [int(t) for t in e["tokens"]],
                                     [int(w) for w in e.get("want", [])]))
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
    ap.add_argument("--page-size", type=int, default=PAGE_SIZE,
                    help=f"tokens a page of the cache holds (default {PAGE_SIZE})")
    ap.add_argument("--num-pages", type=int, default=None,
                    help="pages of the cache pool (default: what --max-tokens needs)")
    ap.add_argument("--max-requests", type=int, default=MAX_LIVE_REQUESTS,
                    help=f"request slots (default {MAX_LIVE_REQUESTS})")
    ap.add_argument("--device", default="cuda:0")
    args = ap.parse_args(argv)
    try:
        engine = make_engine(args.model, args.dtype, args.max_tokens, args.device,
                             page_size=args.page_size, num_pages=args.num_pages,
                             max_requests=args.max_requests)

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
