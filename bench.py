#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on the Qwen3-8B shape with random bfloat16
weights (one MI355X).

    python bench.py --gpus 1 --steps K --warmup W

A "step" is one decode step of the batch.  The default run has the layer sizes of the
Qwen3-8B configuration (36 layers, hidden 4096, 32 query heads on 8 kv heads of 128,
intermediate 12288, vocabulary 151936), a batch of 8 requests with 2048-token prompts of
random ids, pages of 16 tokens; ``value`` is decoded tokens a second over exactly K timed
steps after W warm-up steps, through the engine's own scheduler, step function, cache and
kernels.  The same line reports a 2048-token prefill, the decode step's HBM roofline and
decode at batch 1 and 64.  The reference publishes no numbers, so ``vs_baseline`` is null.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0                      # MI355X HBM3E, published
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

QWEN3_8B = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=36,
                hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
                intermediate_size=12288, vocab_size=151936, rope_theta=1000000.0,
                rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=40960,
                torch_dtype="bfloat16")


def random_model(raw: dict, dtype: str, seed: int, device: str, store: str = None):
    """Model of the given shape with weights drawn on the device: matrices and the embedding
    N(0, 0.02), norm gains 1 + U(-0.1, 0.1).  ``store`` is the dtype the drawn values are
    rounded to (default: the compute dtype)."""
    import torch
    from zinfer_amd.config import Qwen3Config
    from zinfer_amd.models.build import build_model, declare_tensors
    cfg = Qwen3Config.from_dict(raw)
    spec = cfg.model_spec()
    store = torch.bfloat16 if (store or dtype) == "bfloat16" else torch.float32
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    tensors = {}
    for name, decl in declare_tensors(spec).items():
        if decl.optional and spec.tie_word_embeddings:
            continue
        if decl.init == "gain":
            t = 1.0 + (torch.rand(decl.shape, generator=gen, device=device) * 0.2 - 0.1)
        else:
            t = torch.randn(decl.shape, generator=gen, device=device, dtype=torch.float32) * 0.02
        tensors[name] = t.to(store)
        del t
    model = build_model(spec, tensors, dtype, device)
    del tensors
    torch.cuda.empty_cache()
    return cfg, model


def weight_bytes_per_step(cfg, elem: int) -> int:
    """Bytes of weights a decode step has to read: every matrix once (layers and head) and
    the norm gains (32-bit); the embedding rows of the batch are negligible and left out."""
    H, I, hd = cfg.hidden_size, cfg.intermediate_size, cfg.head_dim
    qkv = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * hd * H
    per_layer = qkv + H * cfg.num_attention_heads * hd + 2 * I * H + H * I
    gains = cfg.num_hidden_layers * (2 * H + 2 * hd) + H
    return (cfg.num_hidden_layers * per_layer + cfg.vocab_size * H) * elem + gains * 4


def kv_bytes_per_token(cfg, elem: int) -> int:
    return 2 * cfg.num_hidden_layers * cfg.num_key_value_heads * cfg.head_dim * elem


def prefill_flops(cfg, T: int) -> float:
    """2 flops per multiply-add: the layers' matrices for T tokens, causal attention
    (QK^T and PV over T (T + 1) / 2 pairs), the head for one row."""
    H, I, hd, nH = cfg.hidden_size, cfg.intermediate_size, cfg.head_dim, cfg.num_attention_heads
    qkv = (nH + 2 * cfg.num_key_value_heads) * hd * H
    per_layer = qkv + H * nH * hd + 3 * I * H
    linear = 2.0 * T * per_layer * cfg.num_hidden_layers
    attn = 2.0 * 2.0 * (T * (T + 1) / 2) * hd * nH * cfg.num_hidden_layers
    return linear + attn + 2.0 * cfg.vocab_size * H


def run_prefill(llm, cfg, T: int, seed: int):
    import torch
    from zinfer_amd.engine import StepEntry
    g = torch.Generator().manual_seed(seed)
    eng = llm.engine
    times = []
    for i in range(3):                       # the first pass warms caches and work buffers
        toks = torch.randint(0, cfg.vocab_size, (T,), generator=g).tolist()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = eng.step([StepEntry(f"prefill{i}", toks, [T - 1])], end=[f"prefill{i}"])
        eng.argmax(logits)
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
    return min(times[1:])


def run_decode(llm, cfg, batch: int, prompt_len: int, steps: int, warmup: int, seed: int):
    """Prefills ``batch`` requests through the scheduler, runs ``warmup`` untimed decode
    steps, then times exactly ``steps`` steps.  Returns (seconds, mean context length)."""
    import torch
    from zinfer_amd.sampling import SamplingParams
    g = torch.Generator().manual_seed(seed)
    sched = llm.new_scheduler()
    sched.max_step_tokens = max(sched.max_step_tokens, prompt_len)
    sched.chunk_size = sched.max_step_tokens
    # requests admitted early decode while later prompts are still being run, so they may be
    # up to ``batch`` tokens ahead; none may finish before the timed steps are over
    params = SamplingParams(temperature=0.0, max_new_tokens=warmup + steps + batch + 8,
                            ignore_eos=True)
    for _ in range(batch):
        sched.add_request(torch.randint(0, cfg.vocab_size, (prompt_len,), generator=g).tolist(),
                          params)
    while sched.waiting or any(r.pending > 1 or not r.generated for r in sched.running):
        sched.step()                         # prompts, one or more per step
    assert len(sched.running) == batch
    most = sched.multi_step

    def run_exactly(n):
        """``n`` decode steps of the whole batch; the scheduler may run several in a row on
        the device per call, never more than are still to do."""
        done = 0
        while done < n:
            sched.multi_step = min(most, n - done)
            sched.step()
            assert sched.last_steps >= 1
            done += sched.last_steps
        assert done == n

    run_exactly(warmup)
    torch.cuda.synchronize()
    ctx0 = sum(r.n_computed for r in sched.running) / batch
    t0 = time.perf_counter()
    run_exactly(steps)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ctx1 = sum(r.n_computed for r in sched.running) / batch
    assert len(sched.running) == batch and sched.n_preemptions == 0
    for r in list(sched.running):
        sched._finish(r, "bench")
    return dt, (ctx0 + ctx1) / 2 + 0.5


def check_fp32(llm, cfg, raw, args) -> dict:
    """The same random weights (bfloat16 values widened) through the 32-bit path: FMA
    products, wave attention, 32-bit cache.  Reports the largest difference of the last
    position's logits relative to their largest magnitude, and whether the arg-max agrees."""
    import torch
    from zinfer_amd.engine import Engine, StepEntry
    T = args.check_fp32
    g = torch.Generator().manual_seed(args.seed + 99)
    toks = torch.randint(0, cfg.vocab_size, (T,), generator=g).tolist()
    want = [T - 1]
    lb = llm.engine.step([StepEntry("chk", toks, want)], end=["chk"]).float().clone()
    # same seed, same draws, rounded to bfloat16 as the serving model's, then widened
    _, model32 = random_model(raw, "float32", args.seed, "cuda:0", store="bfloat16")
    eng32 = Engine(model32, page_size=16, num_pages=(T + 15) // 16 + 1, max_requests=2)
    t0 = time.perf_counter()
    lf = eng32.step([StepEntry("chk", toks, want)], end=["chk"]).float()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    err = float((lb - lf).abs().max() / lf.abs().max())
    return {"tokens": T, "rel_max_diff": round(err, 5), "fp32_ms": round(dt * 1e3, 1),
            "argmax_equal": bool(int(lb.argmax()) == int(lf.argmax()))}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--multi-step", type=int, default=8,
                    help="most decode steps in a row on the device without the host between")
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=2048)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the 36 of the "
                    "configuration (both numbers are reported)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip decode at batch 1 and 64")
    ap.add_argument("--check-fp32", type=int, default=0, metavar="TOKENS",
                    help="also run a prompt of TOKENS tokens through a true 32-bit engine with "
                         "the same weights and report how far the logits are apart")
    ap.add_argument("--seed", type=int, default=0)
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py runs on one GPU only (asked for {args.gpus}): this engine has no "
              "multi-GPU path")
        return 2
    import torch
    from zinfer_amd.entrypoints import LLM

    raw = dict(QWEN3_8B)
    if args.layers is not None:
        raw["num_hidden_layers"] = args.layers
    device = "cuda:0"
    t_build = time.perf_counter()
    cfg, model = random_model(raw, args.dtype, args.seed, device)
    elem = 2 if args.dtype == "bfloat16" else 4
    max_batch = args.batch if args.no_points else max(args.batch, 64)
    ctx_cap = args.prompt_len + args.warmup + args.steps + max_batch + 64
    llm = LLM.__new__(LLM)
    from zinfer_amd.engine import Engine
    llm.config, llm.model = cfg, model
    page = 16
    tokens = max(max_batch * ctx_cap, args.prefill_tokens + 64)
    llm.engine = Engine(model, page_size=page, num_pages=(tokens + page - 1) // page + 8,
                        max_requests=max_batch)
    llm.scheduler_options = dict(max_step_tokens=max(2048, args.prompt_len), chunk_size=None,
                                 max_seqs=max_batch, eos_token_ids=(),
                                 multi_step=args.multi_step)
    build_s = time.perf_counter() - t_build

    pre_s = run_prefill(llm, cfg, args.prefill_tokens, args.seed + 1)
    dt, mean_ctx = run_decode(llm, cfg, args.batch, args.prompt_len, args.steps, args.warmup,
                              args.seed + 2)
    value = args.batch * args.steps / dt
    step_bytes = weight_bytes_per_step(cfg, elem) + args.batch * mean_ctx * kv_bytes_per_token(cfg, elem)
    achieved = step_bytes / (dt / args.steps) / 1e9
    points = {}
    if not args.no_points:
        for b in (1, 64):
            k = max(16, args.steps // 4)
            d, _ = run_decode(llm, cfg, b, args.prompt_len, k, min(args.warmup, 4), args.seed + 3 + b)
            points[f"decode_b{b}"] = round(b * k / d, 1)
    peak = PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]
    flops = prefill_flops(cfg, args.prefill_tokens)
    line = {
        "metric": "decode tok/s, Qwen3-8B shape, batch %d, %d-token prompts" % (args.batch, args.prompt_len),
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(dt / args.steps * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {"model": "Qwen3-8B shape, random weights", "layers": cfg.num_hidden_layers,
                   "layers_of_config": QWEN3_8B["num_hidden_layers"],
                   "hidden_size": cfg.hidden_size, "num_attention_heads": cfg.num_attention_heads,
                   "num_key_value_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                   "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
                   "global_batch": args.batch, "prompt_len": args.prompt_len,
                   "seq_len": int(round(mean_ctx)), "page_size": page,
                   "parallelism": "single GPU", "sampling": "greedy",
                   "steps_in_a_row": llm.scheduler_options["multi_step"]},
        "prefill": {"value": round(args.prefill_tokens / pre_s, 1), "tokens": args.prefill_tokens,
                    "ms": round(pre_s * 1e3, 3), "frac": round(flops / pre_s / peak, 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": points,
        "build_s": round(build_s, 1),
    }
    if args.check_fp32:
        line["fp32_check"] = check_fp32(llm, cfg, raw, args)
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
