#!/usr/bin/env python3
"""Throughput of the engine with random bfloat16 weights on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

The default run (``--workload decode``) has the layer sizes of the Qwen3-8B configuration (36
layers, hidden 4096, 32 query heads on 8 kv heads of 128, intermediate 12288, vocabulary
151936), a batch of 8 requests with 2048-token prompts of random ids and pages of 16 tokens.
A "step" is one decode step of the batch; ``value`` is decoded tokens a second over exactly K
timed steps after W warm-up steps, through the engine's own scheduler, step function, cache
and kernels.  The same line reports a 2048-token prefill, the decode step's HBM roofline,
decode at batch 1 and 64, prefills of 512 and 8192 tokens and, unless ``--no-points``, the two
other workloads below in short form.

``--workload continuous``: the Qwen3-14B shape (40 layers, hidden 5120, 40 / 8 heads of 128,
intermediate 17408): 32 requests arrive together, prompt lengths uniform in [128, 4096], 256
greedy tokens each, prompts cut into 512-token portions that run beside the other requests'
decode tokens, through the product's scheduler.  ``value`` is all tokens (prompt and
generated) a second.

``--workload long-context``: the Qwen3-32B shape (64 layers, hidden 5120, 64 / 8 heads of 128,
intermediate 25600; 65.5 GB of weights): a 2048-token prefill, then decode at batch 1, 8 and
64 with every request's context just below 8192 tokens; the cache pool is sized for
64 x 8192 tokens (137 GB).

The reference publishes no numbers, so ``vs_baseline`` is null.
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
PAGE = 16


def _shape(layers, hidden, heads, inter, tied=False):
    return dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=layers,
                hidden_size=hidden, num_attention_heads=heads, num_key_value_heads=8,
                head_dim=128, intermediate_size=inter, vocab_size=151936, rope_theta=1000000.0,
                rms_norm_eps=1e-6, tie_word_embeddings=tied, max_position_embeddings=40960,
                torch_dtype="bfloat16")


# (the three smaller shapes tie the head to the embedding)
SHAPES = {"0.6b": _shape(28, 1024, 16, 3072, True), "1.7b": _shape(28, 2048, 16, 6144, True),
          "4b": _shape(36, 2560, 32, 9728, True), "8b": _shape(36, 4096, 32, 12288),
          "14b": _shape(40, 5120, 40, 17408), "32b": _shape(64, 5120, 64, 25600)}
SHAPE_NAMES = {"0.6b": "Qwen3-0.6B", "1.7b": "Qwen3-1.7B", "4b": "Qwen3-4B", "8b": "Qwen3-8B",
               "14b": "Qwen3-14B", "32b": "Qwen3-32B"}


def build_llm(raw: dict, dtype: str, seed: int, pool_tokens: int, max_seqs: int, **sched):
    """The engine over the product's random-weights mode (matrices and the embedding
    N(0, 0.02), norm gains 1 + U(-0.1, 0.1), drawn on the device) with a pool for
    ``pool_tokens`` tokens."""
    from zinfer_amd.entrypoints import LLM
    return LLM(config=raw, random_seed=seed, dtype=dtype, device="cuda:0", page_size=PAGE,
               num_pages=(pool_tokens + PAGE - 1) // PAGE + 8, max_seqs=max_seqs, **sched)


def drop(llm) -> None:
    """Gives the model's and the pool's memory back before the next shape is built."""
    import gc
    import torch
    import zinfer_amd.ops as ops
    llm.engine._graphs.clear()
    llm.engine = llm.model = None
    ops._workspaces.clear()
    gc.collect()
    torch.cuda.empty_cache()


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


def linear_flops_per_token(cfg) -> float:
    H, I, hd, nH = cfg.hidden_size, cfg.intermediate_size, cfg.head_dim, cfg.num_attention_heads
    qkv = (nH + 2 * cfg.num_key_value_heads) * hd * H
    return 2.0 * (qkv + H * nH * hd + 3 * I * H) * cfg.num_hidden_layers


def prefill_flops(cfg, T: int) -> float:
    """2 flops per multiply-add: the layers' matrices for T tokens, causal attention
    (QK^T and PV over T (T + 1) / 2 pairs), the head for one row."""
    attn = 2.0 * 2.0 * (T * (T + 1) / 2) * cfg.head_dim * cfg.num_attention_heads \
        * cfg.num_hidden_layers
    return linear_flops_per_token(cfg) * T + attn + 2.0 * cfg.vocab_size * cfg.hidden_size


def prefill_record(cfg, T: int, seconds: float, peak: float, mfma_rate=None) -> dict:
    """``frac``: of the published peak; ``frac_of_mfma_loop``: of what a loop of MFMAs alone
    reaches on random operands on this card (``ops.measure_mfma_rate``)."""
    flops = prefill_flops(cfg, T)
    out = {"value": round(T / seconds, 1), "tokens": T, "ms": round(seconds * 1e3, 3),
           "frac": round(flops / seconds / peak, 4)}
    if mfma_rate:
        out["mfma_loop_tflops"] = round(mfma_rate / 1e12, 1)
        out["frac_of_mfma_loop"] = round(flops / seconds / mfma_rate, 4)
    return out


def run_prefill(llm, cfg, T: int, seed: int) -> float:
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


def decode_lead(batch: int, prompt_len: int, step_tokens: int) -> int:
    """How many tokens the first request of ``batch`` may have decoded by the time the last
    one's prompt is through: a step's token budget is shared between one prompt's portion and
    the decode tokens of the requests already running."""
    room = max(1, step_tokens - batch)
    return batch * ((prompt_len + room - 1) // room)


def run_decode(llm, cfg, batch: int, prompt_len: int, steps: int, warmup: int, seed: int,
               classes: bool = False):
    """Prefills ``batch`` requests through the scheduler, runs ``warmup`` untimed decode
    steps, then times exactly ``steps`` steps.  Returns (seconds, mean context length), and
    with ``classes`` a third value: where a step's time goes (see ``step_classes``)."""
    import torch
    from zinfer_amd.sampling import SamplingParams
    g = torch.Generator().manual_seed(seed)
    sched = llm.new_scheduler()
    sched.max_step_tokens = max(sched.max_step_tokens, min(prompt_len, 8192))
    sched.chunk_size = sched.max_step_tokens
    # requests admitted early decode while later prompts are still being run, so they may be
    # many tokens ahead; none may finish before the timed steps are over
    ahead = decode_lead(batch, prompt_len, sched.chunk_size)
    params = SamplingParams(temperature=0.0, max_new_tokens=warmup + steps + ahead + 8,
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
    if classes:
        llm.engine.step_trace = []
    t0 = time.perf_counter()
    run_exactly(steps)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ctx1 = sum(r.n_computed for r in sched.running) / batch
    assert len(sched.running) == batch and sched.n_preemptions == 0
    where = None
    if classes:
        trace, llm.engine.step_trace = llm.engine.step_trace, None
        where = step_classes(llm.engine, sched, trace, steps, dt)
    for r in list(sched.running):
        sched._finish(r, "bench")
    return (dt, (ctx0 + ctx1) / 2 + 0.5) + ((where,) if classes else ())


def step_classes(eng, sched, trace, steps: int, seconds: float) -> dict:
    """Where a decode step's time goes, in milliseconds a step.  ``host``: the host's work for
    the timed steps (packing metadata, launching), which runs beside the device's;
    ``device``: between the events around the timed steps' kernels; the classes: a graph of
    the same step with only that class's kernels, replayed (``Engine.class_times``: products =
    the layers' matrix products with what is fused into them (norms, SwiGLU, residual sums),
    attention = attention over the cache, in steps of up to 32 sequences with the per-head
    norm, rotation and cache write; norm_rope_write = those as kernels of their own;
    head_sampling = final norm, head, arg-max)."""
    from zinfer_amd.engine import StepEntry
    host = sum(r[2] + r[3] for r in trace) / steps
    device = sum(r[4].elapsed_time(r[5]) for r in trace) / 1e3 / steps
    entries = [StepEntry(r.id, [r.generated[-1]], [0]) for r in sched.running]
    t = eng.class_times(entries)
    out = {k + "_ms": round(v * 1e3, 4) for k, v in t.items() if k != "step"}
    out["classes_sum_ms"] = round(sum(v for k, v in t.items() if k != "step") * 1e3, 4)
    out["graph_step_ms"] = round(t["step"] * 1e3, 4)
    out["device_ms"] = round(device * 1e3, 4)
    out["host_ms"] = round(host * 1e3, 4)
    out["wall_ms"] = round(seconds / steps * 1e3, 4)
    return out


def decode_roofline(cfg, elem: int, batch: int, mean_ctx: float, seconds_per_step: float,
                    measured_gbs: float = None) -> dict:
    """``measured``: what a kernel that only reads (16-byte non-temporal loads, 8 in flight a
    lane, a workgroup 64 KB in a row, 2 GiB from HBM, the best pass between two events over 256
    to 4096 workgroups) reaches on this card."""
    step_bytes = weight_bytes_per_step(cfg, elem) + batch * mean_ctx * kv_bytes_per_token(cfg, elem)
    achieved = step_bytes / seconds_per_step / 1e9
    out = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
           "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4)}
    if measured_gbs:
        out["measured_read"] = round(measured_gbs, 1)
        out["frac_of_measured"] = round(achieved / measured_gbs, 4)
    return out


def config_of(cfg, shape: str, **more) -> dict:
    out = {"model": f"{SHAPE_NAMES[shape]} shape, random weights",
           "layers": cfg.num_hidden_layers,
           "layers_of_config": SHAPES[shape]["num_hidden_layers"],
           "hidden_size": cfg.hidden_size, "num_attention_heads": cfg.num_attention_heads,
           "num_key_value_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
           "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
           "page_size": PAGE, "parallelism": "single GPU", "sampling": "greedy"}
    out.update(more)
    return out


# --------------------------------------------------------------------------- continuous batching
def run_continuous(llm, cfg, elem: int, n_requests: int, lo: int, hi: int, new_tokens: int,
                   seed: int) -> dict:
    """All requests arrive together; the scheduler admits them, cuts their prompts into
    portions beside the decode tokens of the others, decodes, finishes and frees.  The
    workload runs three times with the same requests; the third pass is timed (the first
    settles work buffers and captures the decode graph of every batch shape that occurs, the
    second records the runs of decode steps whose shape came a second time: a server that has
    been up for a while)."""
    import torch
    from zinfer_amd.sampling import SamplingParams
    eng = llm.engine
    out = {}
    for timed in (False, False, True):
        g = torch.Generator().manual_seed(seed)
        lens = torch.randint(lo, hi + 1, (n_requests,), generator=g).tolist()
        sched = llm.new_scheduler()
        params = SamplingParams(temperature=0.0, max_new_tokens=new_tokens, ignore_eos=True)
        for n in lens:
            sched.add_request(torch.randint(0, cfg.vocab_size, (n,), generator=g).tolist(), params)
        eng.step_trace = []
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        first_done = None
        prompts_done = None
        while sched.has_work():
            done = sched.step()
            if prompts_done is None and not sched.waiting and \
                    all(r.generated for r in sched.running):
                torch.cuda.synchronize()
                prompts_done = time.perf_counter() - t0
            if done and first_done is None:
                first_done = time.perf_counter() - t0
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        trace, eng.step_trace = eng.step_trace, None
        if not timed:
            continue
        generated = sum(len(r.generated) for r in sched.finished.values())
        assert generated == n_requests * new_tokens
        prompt_tokens = sum(lens)
        mixed = [r for r in trace if r[6]]                  # steps with a prompt portion

        def summary(rows):
            if not rows:
                return None
            dev = sum(r[4].elapsed_time(r[5]) for r in rows) / 1e3
            return {"steps": len(rows), "tokens": sum(r[0] for r in rows),
                    "host_pack_ms": round(sum(r[2] for r in rows) / len(rows) * 1e3, 3),
                    "host_launch_ms": round(sum(r[3] for r in rows) / len(rows) * 1e3, 3),
                    "device_ms": round(dev / len(rows) * 1e3, 3), "device_s": round(dev, 3)}

        mixed_s = summary(mixed)
        # roofline of the mean step with a prompt portion: its matrices' flops and the bytes
        # it must read (every weight once, the cache of the live requests about once)
        if mixed_s:
            t_step = mixed_s["device_ms"] / 1e3
            toks = mixed_s["tokens"] / mixed_s["steps"]
            flops = linear_flops_per_token(cfg) * toks
            mixed_s["tokens_per_step"] = round(toks, 1)
            mixed_s["frac_mfma"] = round(flops / t_step / PEAK_FLOPS["bf16"], 4)
            mixed_s["frac_hbm_weights"] = round(
                weight_bytes_per_step(cfg, elem) / t_step / 1e9 / HBM_PEAK_GBS, 4)
        out = {"seconds": round(dt, 3), "total_tok_s": round((prompt_tokens + generated) / dt, 1),
               "decode_tok_s": round(generated / dt, 1), "prompt_tokens": prompt_tokens,
               "generated_tokens": generated, "engine_steps": sched.n_steps,
               "scheduler_calls": len(trace), "preemptions": sched.n_preemptions,
               "prompts_done_s": round(prompts_done or 0.0, 3),
               "first_finished_s": round(first_done or 0.0, 3),
               "device_busy_frac": round(sum(r[4].elapsed_time(r[5]) for r in trace) / 1e3 / dt, 4),
               "mixed_steps": mixed_s, "decode_calls": summary([r for r in trace if not r[6]])}
    return out


def main_continuous(args) -> int:
    raw = dict(SHAPES[args.shape or "14b"])
    if args.layers is not None:
        raw["num_hidden_layers"] = args.layers
    n, lo, hi, new = args.requests, args.prompt_min, args.prompt_max, args.new_tokens
    t_build = time.perf_counter()
    step_tokens = args.step_tokens or args.chunk
    llm = build_llm(raw, args.dtype, args.seed, n * (hi + new + PAGE), n,
                    max_step_tokens=step_tokens, chunk_size=args.chunk,
                    multi_step=args.multi_step)
    cfg = llm.config
    build_s = time.perf_counter() - t_build
    llm.engine.capture_runs = not args.no_run_graphs
    elem = 2 if args.dtype == "bfloat16" else 4
    res = run_continuous(llm, cfg, elem, n, lo, hi, new, args.seed + 7)
    line = {"metric": f"continuous batching tok/s (prompt + generated), "
                      f"{SHAPE_NAMES[args.shape or '14b']} shape, {n} requests",
            "value": res["total_tok_s"], "unit": "tokens/s", "n_gpus": 1,
            "steps": res["engine_steps"], "warmup": res["engine_steps"],
            "ms_per_step": round(res["seconds"] / max(res["engine_steps"], 1) * 1e3, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
            "config": config_of(cfg, args.shape or "14b", requests=n, prompt_min=lo,
                                prompt_max=hi, new_tokens=new, chunk_size=args.chunk,
                                max_step_tokens=step_tokens,
                                steps_in_a_row=args.multi_step),
            "continuous": res, "build_s": round(build_s, 1)}
    print(json.dumps(line))
    return 0


# --------------------------------------------------------------------------- long context
def run_long_context(llm, cfg, elem: int, context: int, batches, steps: int, seed: int) -> dict:
    """Decode with every request's context just below ``context``: prompts of
    ``context - steps - warm-up`` tokens are run through the scheduler, then the timed steps
    end at ``context``."""
    out = {}
    for b in batches:
        warm = 16
        prompt_len = context - steps - warm - b * ((context + 8191) // 8192) - 8
        dt, mean_ctx = run_decode(llm, cfg, b, prompt_len, steps, warm, seed + b)
        out[f"decode_b{b}"] = round(b * steps / dt, 1)
        out[f"decode_b{b}_ms"] = round(dt / steps * 1e3, 3)
        out[f"decode_b{b}_ctx"] = int(round(mean_ctx))
        out[f"decode_b{b}_hbm_frac"] = decode_roofline(cfg, elem, b, mean_ctx, dt / steps)["frac"]
    return out


def main_long_context(args) -> int:
    import torch
    shape = args.shape or "32b"
    raw = dict(SHAPES[shape])
    if args.layers is not None:
        raw["num_hidden_layers"] = args.layers
    context = args.context
    batches = tuple(int(b) for b in args.batches.split(","))
    t_build = time.perf_counter()
    llm = build_llm(raw, args.dtype, args.seed, max(batches) * (context + PAGE), max(batches),
                    max_step_tokens=8192, multi_step=args.multi_step)
    cfg = llm.config
    build_s = time.perf_counter() - t_build
    elem = 2 if args.dtype == "bfloat16" else 4
    free, total = torch.cuda.mem_get_info()
    pre_s = run_prefill(llm, cfg, args.prefill_tokens, args.seed + 1)
    steps = max(16, min(args.steps, 64))
    res = run_long_context(llm, cfg, elem, context, batches, steps, args.seed + 2)
    peak = PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]
    hb = 8 if 8 in batches else max(batches)      # the batch of the headline
    line = {"metric": f"decode tok/s at context {context}, {SHAPE_NAMES[shape]} shape, batch {hb}",
            "value": res[f"decode_b{hb}"], "unit": "tokens/s", "n_gpus": 1, "steps": steps,
            "warmup": 16, "ms_per_step": res[f"decode_b{hb}_ms"], "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
            "config": config_of(cfg, shape, global_batch=hb, seq_len=context,
                                pool_tokens=max(batches) * (context + PAGE),
                                steps_in_a_row=args.multi_step),
            "prefill": prefill_record(cfg, args.prefill_tokens, pre_s, peak),
            "roofline": {"bound": "hbm", "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": res[f"decode_b{hb}_hbm_frac"],
                         "achieved": round(res[f"decode_b{hb}_hbm_frac"] * HBM_PEAK_GBS, 1)},
            "points": res, "weights_gb": round(weight_bytes_per_step(cfg, elem) / 1e9, 1),
            "pool_gb": round(llm.engine.cache.kv_bytes() / 1e9, 1),
            "free_gb_after_build": round(free / 1e9, 1), "build_s": round(build_s, 1)}
    print(json.dumps(line))
    return 0


# --------------------------------------------------------------------------- the default line
def check_fp32(llm, cfg, raw, seed: int, T: int) -> dict:
    """What bfloat16 costs at this shape: the same random weights (bfloat16 values widened)
    through the true 32-bit path (FMA products, 32-bit attention, 32-bit cache) beside the
    serving engine, on one prompt of ``T`` tokens: its first 512 tokens as one step, the rest
    as a second, then one decode token (the 32-bit arg-max) at context ``T``.  For each of the
    three places: the largest difference of the logits relative to their largest magnitude,
    the root-mean-square difference relative to their root-mean-square, and whether the
    arg-max agrees."""
    import torch
    from zinfer_amd.engine import Engine, StepEntry
    from zinfer_amd.models.build import random_model
    g = torch.Generator().manual_seed(seed + 99)
    toks = torch.randint(0, cfg.vocab_size, (T,), generator=g).tolist()
    head = min(512, T)
    # same seed, same draws, rounded to bfloat16 as the serving model's, then widened
    _, model32 = random_model(raw, seed, "float32", "cuda:0", store_dtype="bfloat16")
    eng32 = Engine(model32, page_size=PAGE, num_pages=(T + 1 + PAGE - 1) // PAGE + 1,
                   max_requests=2)
    out = {"tokens": T}
    t0 = time.perf_counter()
    cuts = [("prefill_%d" % head, toks[:head])]
    if T > head:
        cuts.append(("prefill_%d" % T, toks[head:]))
    nxt = None
    for name, part in cuts + [("decode_ctx%d" % T, None)]:
        part = [nxt] if part is None else part
        entry = [StepEntry("chk", part, [len(part) - 1])]
        lb = llm.engine.step(entry).float().clone()
        lf = eng32.step(entry).float()
        nxt = int(lf.argmax())
        out[name] = {
            "rel_max_diff": round(float((lb - lf).abs().max() / lf.abs().max()), 5),
            "rel_rms_diff": round(float((lb - lf).pow(2).mean().sqrt() / lf.pow(2).mean().sqrt()), 5),
            "argmax_equal": bool(int(lb.argmax()) == nxt)}
    torch.cuda.synchronize()
    out["seconds"] = round(time.perf_counter() - t0, 2)
    llm.engine.release("chk")
    eng32.release("chk")
    del eng32, model32
    import gc
    gc.collect()
    torch.cuda.empty_cache()
    return out


def main_decode(args) -> int:
    shape = args.shape or "8b"
    raw = dict(SHAPES[shape])
    if args.layers is not None:
        raw["num_hidden_layers"] = args.layers
    max_batch = args.batch if args.no_points else max(args.batch, 64)
    step_tokens = max(2048, args.prompt_len)
    ctx_cap = args.prompt_len + args.warmup + args.steps + 64 \
        + decode_lead(max_batch, args.prompt_len, min(step_tokens, 8192))
    longest_prefill = args.prefill_tokens if args.no_points else max(args.prefill_tokens, 8192)
    tokens = max(max_batch * ctx_cap, longest_prefill + 64)
    t_build = time.perf_counter()
    llm = build_llm(raw, args.dtype, args.seed, tokens, max_batch,
                    max_step_tokens=step_tokens, multi_step=args.multi_step)
    cfg = llm.config
    build_s = time.perf_counter() - t_build
    llm.engine.capture_runs = not args.no_run_graphs
    elem = 2 if args.dtype == "bfloat16" else 4
    peak = PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]

    import zinfer_amd.ops as ops
    measured_gbs = ops.measure_read_bandwidth("cuda:0") / 1e9
    pre_s = run_prefill(llm, cfg, args.prefill_tokens, args.seed + 1)
    # what the matrix cores sustain on random operands with nothing else to do (the chip's
    # power limit sets it, far under the 2.4 GHz figure): bfloat16 only
    mfma_rate = ops.measure_mfma_rate("cuda:0") if args.dtype == "bfloat16" else None
    dt, mean_ctx, where = run_decode(llm, cfg, args.batch, args.prompt_len, args.steps,
                                     args.warmup, args.seed + 2, classes=True)
    value = args.batch * args.steps / dt
    points = {}
    if not args.no_points:
        for b in (1, 64):
            k = max(16, args.steps // 4)
            d, ctx = run_decode(llm, cfg, b, args.prompt_len, k, args.warmup, args.seed + 3 + b)
            points[f"decode_b{b}"] = round(b * k / d, 1)
            points[f"decode_b{b}_hbm_frac"] = decode_roofline(cfg, elem, b, ctx, d / k)["frac"]
        for T in (512, 1024, 8192):
            s = run_prefill(llm, cfg, T, args.seed + 5)
            points[f"prefill_{T}"] = round(T / s, 1)
            points[f"prefill_{T}_frac"] = round(prefill_flops(cfg, T) / s / peak, 4)
    line = {
        "metric": "decode tok/s, %s shape, batch %d, %d-token prompts"
                  % (SHAPE_NAMES[shape], args.batch, args.prompt_len),
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(dt / args.steps * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": config_of(cfg, shape, global_batch=args.batch, prompt_len=args.prompt_len,
                            seq_len=int(round(mean_ctx)), steps_in_a_row=args.multi_step),
        "prefill": prefill_record(cfg, args.prefill_tokens, pre_s, peak, mfma_rate),
        "roofline": decode_roofline(cfg, elem, args.batch, mean_ctx, dt / args.steps,
                                    measured_gbs),
        "classes": where,
        "points": points,
        "build_s": round(build_s, 1),
    }
    check_tokens = args.check_fp32 if args.check_fp32 is not None else \
        (0 if args.no_points or args.dtype != "bfloat16" else 2048)
    if check_tokens:
        line["fp32_check"] = check_fp32(llm, cfg, raw, args.seed, check_tokens)
    if not args.no_points and args.layers is None and args.dtype == "bfloat16":
        # the other two workloads in short form (their own modes report them in full)
        drop(llm)
        n = 32
        llm = build_llm(SHAPES["14b"], args.dtype, args.seed, n * (4096 + 256 + PAGE), n,
                        max_step_tokens=512, chunk_size=512, multi_step=args.multi_step)
        res = run_continuous(llm, llm.config, elem, n, 128, 4096, 256, args.seed + 7)
        points["continuous_14b_total"] = res["total_tok_s"]
        points["continuous_14b_decode"] = res["decode_tok_s"]
        points["continuous_14b_seconds"] = res["seconds"]
        points["continuous_14b_preemptions"] = res["preemptions"]
        drop(llm)
        if args.long_context_points:
            llm = build_llm(SHAPES["32b"], args.dtype, args.seed, 64 * (8192 + PAGE), 64,
                            max_step_tokens=8192, multi_step=args.multi_step)
            pre32 = run_prefill(llm, llm.config, 2048, args.seed + 1)
            points["prefill_2048_32b"] = round(2048 / pre32, 1)
            points["prefill_2048_32b_frac"] = round(prefill_flops(llm.config, 2048) / pre32 / peak, 4)
            res = run_long_context(llm, llm.config, elem, 8192, (1, 8, 64), 16, args.seed + 2)
            for k, v in res.items():
                if not k.endswith("_ctx"):
                    points[k.replace("decode_", "decode_32b_ctx8192_")] = v
            drop(llm)
    print(json.dumps(line))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--workload", default="decode", choices=["decode", "continuous", "long-context"])
    ap.add_argument("--shape", default=None, choices=sorted(SHAPES),
                    help="layer sizes (default: 8b for decode, 14b for continuous, 32b for "
                         "long-context)")
    ap.add_argument("--multi-step", type=int, default=8,
                    help="most decode steps in a row on the device without the host between")
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=2048)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the "
                    "configuration has (both numbers are reported)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true",
                    help="only the headline: no other batches, prompt lengths or workloads")
    ap.add_argument("--no-long-context-points", dest="long_context_points", action="store_false",
                    help="leave the 32B-shape points out of the default line")
    ap.add_argument("--check-fp32", type=int, default=None, metavar="TOKENS",
                    help="also run a prompt of TOKENS tokens and one decode token through a true "
                         "32-bit engine with the same weights and report how far the logits "
                         "are apart (default: 2048, with --no-points 0 = not at all)")
    ap.add_argument("--requests", type=int, default=32, help="continuous: requests")
    ap.add_argument("--prompt-min", type=int, default=128)
    ap.add_argument("--prompt-max", type=int, default=4096)
    ap.add_argument("--new-tokens", type=int, default=256)
    ap.add_argument("--chunk", type=int, default=512, help="continuous: tokens of a prompt per step")
    ap.add_argument("--step-tokens", type=int, default=None,
                    help="continuous: token budget of a step (default: the chunk, so that a "
                         "prompt's portion and the decode tokens beside it fill whole tiles)")
    ap.add_argument("--context", type=int, default=8192, help="long-context: context decoded at")
    ap.add_argument("--batches", default="1,8,64",
                    help="long-context: the batch sizes decoded at (the pool holds the largest)")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-run-graphs", action="store_true",
                    help="decode steps in a row replay one graph per step instead of one for the run")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py runs on one GPU only (asked for {args.gpus}): this engine has no "
              "multi-GPU path")
        return 2
    return {"decode": main_decode, "continuous": main_continuous,
            "long-context": main_long_context}[args.workload](args)


if __name__ == "__main__":
    sys.exit(main())
