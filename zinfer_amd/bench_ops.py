"""Per-kernel benchmark at a model's sizes, the counterpart of the reference's ``bench-ops``
(`src/app/cli/tools/bench/ops.zig:12-49`: every kernel alone, warm-up iterations first, then
``ns/iter`` and a throughput figure, `:516-543`).  Operands are random; weights are rotated
through several copies so that reads come from HBM, not from the 256 MB cache.

    python -m zinfer_amd.bench_ops [model_dir | --shape 8b] [--tokens 1,8,64,2048] [--iters N]
        [--only gemm|attention|elementwise]
"""
from __future__ import annotations

import argparse
import math
import sys
from typing import List

import torch

SHAPES = {"8b": dict(hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
                     intermediate_size=12288, vocab_size=151936),
          "14b": dict(hidden_size=5120, num_attention_heads=40, num_key_value_heads=8, head_dim=128,
                      intermediate_size=17408, vocab_size=151936),
          "32b": dict(hidden_size=5120, num_attention_heads=64, num_key_value_heads=8, head_dim=128,
                      intermediate_size=25600, vocab_size=151936)}


def _time(fn, iters: int, warmup: int = 3) -> float:
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / iters * 1e-3      # seconds


def bench_gemms(cfg: dict, tokens: List[int], iters: int, dev: str) -> None:
    from . import ops
    H, I, hd = cfg["hidden_size"], cfg["intermediate_size"], cfg["head_dim"]
    qkv_n = (cfg["num_attention_heads"] + 2 * cfg["num_key_value_heads"]) * hd
    shapes = [("qkv_proj", qkv_n, H, "store"), ("o_proj", H, cfg["num_attention_heads"] * hd, "acc"),
              ("gate_up+swiglu", 2 * I, H, "swiglu"), ("down_proj", H, I, "acc"),
              ("lm_head", cfg["vocab_size"], H, "f32")]
    for name, N, K, kind in shapes:
        copies = max(2, min(12, int(1.2e9 // (N * K * 2))))
        ws = []
        for _ in range(copies):
            w = (torch.randn(N, K, device=dev) * 0.02).to(torch.bfloat16)
            ws.append(ops.pretile_weight(w) if ops.can_pretile(w) else w)
            del w
        tiled = ops.can_pretile(ws[0])
        for M in tokens:
            if name == "lm_head" and M > 64:
                continue
            a = torch.randn(M, K, device=dev).to(torch.bfloat16)
            if kind == "swiglu":
                out = torch.empty(M, N // 2, device=dev, dtype=torch.bfloat16)
            elif kind == "store":
                out = torch.empty(M, N, device=dev, dtype=torch.bfloat16)
            else:
                out = torch.zeros(M, N, device=dev, dtype=torch.float32)
            i = [0]

            def run():
                w = ws[i[0] % copies]
                i[0] += 1
                if kind == "swiglu":
                    ops.gemm_swiglu(a, w, out, w_tiled=tiled)
                else:
                    ops.gemm(a, w, out, accumulate=(kind == "acc"), w_tiled=tiled)
            t = _time(run, iters)
            print(f"gemm {name:15s} M={M:5d} N={N:6d} K={K:6d}: {t * 1e6:9.1f} us/iter  "
                  f"{N * K * 2 / t / 1e12:6.2f} TB/s weights  {2.0 * M * N * K / t / 1e12:8.1f} TFLOP/s",
                  flush=True)
        del ws


def bench_attention(cfg: dict, tokens: List[int], iters: int, dev: str, ctx: int) -> None:
    from . import ops
    nH, nKV, hd, ps = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], 16
    for M in tokens:
        decode = M <= 64
        n_seqs, q_len = (M, 1) if decode else (1, M)
        c = ctx if decode else max(ctx, M)
        pages_per = (c + ps - 1) // ps
        n_pages = n_seqs * pages_per
        q = torch.randn(n_seqs * q_len, nH * hd, device=dev).to(torch.bfloat16)
        kp = torch.randn(n_pages, nKV * ps * hd, device=dev).to(torch.bfloat16)
        vp = torch.randn(n_pages, nKV * ps * hd, device=dev).to(torch.bfloat16)
        bt = torch.randperm(n_pages, device=dev).int().view(n_seqs, pages_per)
        q_start = (torch.arange(n_seqs + 1, device=dev) * q_len).int()
        ctx_len = torch.full((n_seqs,), c, device=dev, dtype=torch.int32)
        seq_index = torch.repeat_interleave(torch.arange(n_seqs, device=dev), q_len).int()
        out = torch.empty_like(q)
        run = lambda: ops.paged_attention(q, kp, vp, bt, q_start, ctx_len, seq_index, out,
                                          1.0 / math.sqrt(hd), 0, nH, nKV, hd, ps, q_len, c,
                                          n_single=n_seqs if decode else 0)
        t = _time(run, iters)
        if decode:
            kv_bytes = n_seqs * c * nKV * hd * 2 * 2
            print(f"attention decode  seqs={n_seqs:3d} ctx={c:6d}: {t * 1e6:9.1f} us/iter  "
                  f"{kv_bytes / t / 1e12:6.2f} TB/s keys+values", flush=True)
        else:
            pairs = q_len * (c - q_len) + q_len * (q_len + 1) / 2
            print(f"attention prefill q={q_len:5d} ctx={c:6d}: {t * 1e6:9.1f} us/iter  "
                  f"{4.0 * pairs * hd * nH / t / 1e12:8.1f} TFLOP/s", flush=True)


def bench_elementwise(cfg: dict, tokens: List[int], iters: int, dev: str) -> None:
    from . import ops
    from .parts.position import rotary_tables
    H, I, hd = cfg["hidden_size"], cfg["intermediate_size"], cfg["head_dim"]
    nH, nKV = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    cos, sin = (t.to(dev) for t in rotary_tables(hd, 1e6, 8192))
    for M in tokens:
        x = torch.randn(M, H, device=dev)
        gain = torch.ones(H, device=dev)
        out = torch.empty(M, H, device=dev, dtype=torch.bfloat16)
        t = _time(lambda: ops.rmsnorm(x, gain, 1e-6, out), iters)
        print(f"rmsnorm            M={M:5d} W={H}: {t * 1e6:9.1f} us/iter  "
              f"{M * H * 6 / t / 1e9:8.1f} GB/s", flush=True)
        gu = torch.randn(M, 2 * I, device=dev).to(torch.bfloat16)
        act = torch.empty(M, I, device=dev, dtype=torch.bfloat16)
        t = _time(lambda: ops.swiglu(gu, act), iters)
        print(f"swiglu             M={M:5d} I={I}: {t * 1e6:9.1f} us/iter  "
              f"{M * I * 6 / t / 1e9:8.1f} GB/s", flush=True)
        qkv = torch.randn(M, (nH + 2 * nKV) * hd, device=dev).to(torch.bfloat16)
        qo = torch.empty(M, nH * hd, device=dev, dtype=torch.bfloat16)
        pages = (M + 15) // 16 + 1
        kp = torch.zeros(pages, nKV * 16 * hd, device=dev, dtype=torch.bfloat16)
        vp = torch.zeros_like(kp)
        pos = torch.arange(M, device=dev, dtype=torch.int32) % 8192
        slots = torch.arange(M, device=dev, dtype=torch.int32)
        g = torch.ones(hd, device=dev)
        t = _time(lambda: ops.qk_norm_rope_kv_write(qkv, g, g, 1e-6, cos, sin, pos, slots, kp, vp,
                                                    qo, nH, nKV, hd, 16), iters)
        print(f"qk_norm_rope_kv    M={M:5d}: {t * 1e6:9.1f} us/iter", flush=True)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="bench-ops", description=__doc__.split("\n\n")[0])
    ap.add_argument("model_dir", nargs="?", default=None)
    ap.add_argument("--shape", default="8b", choices=sorted(SHAPES))
    ap.add_argument("--tokens", default="1,8,64,2048")
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--ctx", type=int, default=2048)
    ap.add_argument("--only", default=None, choices=["gemm", "attention", "elementwise"])
    ap.add_argument("--device", default="cuda:0")
    args = ap.parse_args(argv)
    if args.model_dir:
        from .config import load_config
        c = load_config(args.model_dir)
        cfg = {k: getattr(c, k) for k in SHAPES["8b"]}
    else:
        cfg = SHAPES[args.shape]
    tokens = [int(t) for t in args.tokens.split(",")]
    print("Zinfer op benchmark")
    print(f"kernel_isa: gfx950  iterations: {args.iters}  sizes: {cfg}")
    if args.only in (None, "gemm"):
        bench_gemms(cfg, tokens, args.iters, args.device)
    if args.only in (None, "attention"):
        bench_attention(cfg, tokens, args.iters, args.device, args.ctx)
    if args.only in (None, "elementwise"):
        bench_elementwise(cfg, tokens, args.iters, args.device)
    return 0


if __name__ == "__main__":
    sys.exit(main())
