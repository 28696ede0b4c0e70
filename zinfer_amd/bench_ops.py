"""Per-kernel benchmark at a model's sizes, the counterpart of the reference's ``bench-ops``
(`src/app/cli/tools/bench/ops.zig:12-49`: every kernel alone, warm-up iterations first, then
``ns/iter`` and a throughput figure, `:516-543`).  Operands are random; weights are rotated
through several copies so that reads come from HBM, not from the 256 MB cache.

    python -m zinfer_amd.bench_ops [model_dir | --shape 8b] [--tokens 1,8,64,2048] [--iters N]
        [--only gemm|attention|elementwise]
    python -m zinfer_amd.bench_ops model_dir --tune [--plans-out FILE]

``--tune`` measures, for the four projection widths of the model, every plan the kernels for
17 to 64 tokens take (weight streaming with its row groups and split, the 17-to-128-token
kernel with its split), and for 1 to 16 tokens the residual sums' split along K, each in a
replayed graph over rotating weights, and writes the fastest into ``kernel_plans.json`` of the
model folder, which ``load_model`` reads.  It also prints what the rules for widths without an
entry would have chosen and how much slower that is.
"""
from __future__ import annotations

import argparse
import math
import sys
from typing import List

import torch

SHAPES = {"0.6b": dict(hidden_size=1024, num_attention_heads=16, num_key_value_heads=8, head_dim=128,
                       intermediate_size=3072, vocab_size=151936),
          "1.7b": dict(hidden_size=2048, num_attention_heads=16, num_key_value_heads=8, head_dim=128,
                       intermediate_size=6144, vocab_size=151936),
          "4b": dict(hidden_size=2560, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
                     intermediate_size=9728, vocab_size=151936),
          "8b": dict(hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
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


def _graph_time(fn, copies: int, replays: int = 6) -> float:
    """Seconds per call of ``fn(i)`` (i = 0 .. copies - 1, one weight copy each) in a captured
    graph of ``copies`` calls, the best of ``replays`` replays."""
    for i in range(copies):
        fn(i)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for i in range(copies):
            fn(i)
    graph.replay()
    best = float("inf")
    for _ in range(replays):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        graph.replay()
        b.record()
        b.synchronize()
        best = min(best, a.elapsed_time(b) * 1e-3 / copies)
    return best


def candidate_plans(M: int, N: int, K: int, swiglu: bool):
    """Every plan of the kernels for 17 to 64 tokens that ``ops.check_plans`` accepts."""
    from . import ops
    out = []
    for ks in (1,) if swiglu else (1, 2, 4, 8, 16):
        out.append(["mid", ks])
    for rg in (2, 4) if swiglu else (1, 2, 4):
        for ks in (1,) if swiglu else (1, 2, 4, 8):
            out.append(["skinny", rg, ks])
    good = []
    for plan in out:
        try:
            ops.check_plans({"plans": {f"{N}x{K}" + (":swiglu" if swiglu else ""):
                                       {str(ops.plan_bucket(M)): plan}}})
        except Exception:
            continue
        if plan[0] == "mid" and (K // plan[1]) < 512:
            continue
        good.append(plan)
    return good


def tune(cfg: dict, dev: str, log=print) -> dict:
    """The fastest plan per width and bucket, as a table ``ops.load_plans`` takes."""
    from . import ops
    H, I, hd = cfg["hidden_size"], cfg["intermediate_size"], cfg["head_dim"]
    qkv_n = (cfg["num_attention_heads"] + 2 * cfg["num_key_value_heads"]) * hd
    shapes = [("qkv_proj", qkv_n, H, "store"), ("o_proj", H, cfg["num_attention_heads"] * hd, "acc"),
              ("gate_up+swiglu", 2 * I, H, "swiglu"), ("down_proj", H, I, "acc")]
    table = ops._measured_plans()
    result = {"_": "measured by bench-ops --tune on this model's own widths",
              "plans": {}, "decode_acc": {}}
    losses = []
    for name, N, K, kind in shapes:
        if not (N % 64 == 0 and K % 64 == 0):
            log(f"{name}: {N} x {K} does not pre-tile, no plans apply")
            continue
        # more copies in turn than the 256 MB last-level cache holds: the weights come from HBM
        copies = max(3, min(96, -(-600_000_000 // (N * K * 2))))
        ws = [ops.pretile_weight((torch.randn(N, K, device=dev) * 0.02).to(torch.bfloat16))
              for _ in range(copies)]
        key = f"{N}x{K}" + (":swiglu" if kind == "swiglu" else "")
        saved = table["plans"].pop(key, None)
        entry = {}
        for M in ops.PLAN_BUCKETS:
            a = torch.randn(M, K, device=dev).to(torch.bfloat16)
            if kind == "swiglu":
                out = torch.empty(M, N // 2, device=dev, dtype=torch.bfloat16)
                call = lambda i: ops.gemm_swiglu(a, ws[i], out, w_tiled=True)
            elif kind == "store":
                out = torch.empty(M, N, device=dev, dtype=torch.bfloat16)
                call = lambda i: ops.gemm(a, ws[i], out, w_tiled=True)
            else:
                out = torch.zeros(M, N, device=dev, dtype=torch.float32)
                call = lambda i: ops.gemm(a, ws[i], out, accumulate=True, w_tiled=True)
            rule = list(ops._small_plan(M, N, K, True, swiglu=(kind == "swiglu")) or ())
            times = {}
            for plan in candidate_plans(M, N, K, kind == "swiglu"):
                table["plans"][key] = {str(M): plan}
                try:
                    times[tuple(plan)] = _graph_time(call, copies)
                except Exception as e:            # a configuration a launcher refuses
                    log(f"  {name} M={M} {plan}: refused ({e})")
                table["plans"].pop(key, None)
            best = min(times, key=times.get)
            entry[str(M)] = list(best)
            t_rule = times.get(tuple(rule))
            loss = (t_rule / times[best] - 1.0) if t_rule else float("nan")
            losses.append(loss)
            log(f"tune {name:15s} {N:6d} x {K:6d} M={M:2d}: best {list(best)} "
                f"{times[best] * 1e6:7.1f} us ({N * K * 2 / times[best] / 1e12:.2f} TB/s); "
                f"rule {rule} {'%.1f us, +%.0f %%' % (t_rule * 1e6, loss * 100) if t_rule else 'not measured'}")
        result["plans"][key] = entry
        if saved is not None:
            table["plans"][key] = saved
        if kind == "acc" and N <= 8192:
            # 1 to 16 tokens: the one-launch epilogue that leaves the next norm's inputs, or a
            # split along K whose reduce adds the residual and norms
            M = 8
            a = torch.randn(M, K, device=dev).to(torch.bfloat16)
            res = torch.zeros(M, N, device=dev, dtype=torch.float32)
            gain = torch.ones(N, device=dev)
            xg = torch.empty(M, N, device=dev, dtype=torch.bfloat16)
            sq = torch.empty(N // 16, 16, device=dev, dtype=torch.float32)
            akey = f"{N}x{K}"
            saved = table["decode_acc"].pop(akey, None)
            times = {}
            if ops.norm_emit_plan(M, N, K, ws[0], True) is not None:
                times[None] = _graph_time(lambda i: ops.gemm_emit(a, ws[i], res, gain, xg, sq), copies)
            else:
                times[None] = _graph_time(lambda i: ops.gemm(a, ws[i], res, True, w_tiled=True), copies)
            for rg in (1, 2, 4):
                for ks in (2, 3, 4, 6, 8):
                    plan = ["skinny", rg, ks]
                    try:
                        ops.check_plans({"decode_acc": {akey: plan}})
                    except Exception:
                        continue
                    if (K // 64) % ks != 0 and K // (64 * ks) < 8:
                        continue
                    table["decode_acc"][akey] = plan
                    try:
                        times[tuple(plan)] = _graph_time(
                            lambda i: ops.gemm_sum_norm(a, ws[i], res, gain, 1e-6, xg), copies)
                    except Exception as e:
                        log(f"  {name} decode {plan}: refused ({e})")
                    table["decode_acc"].pop(akey, None)
            best = min(times, key=lambda k: times[k])
            # the split has to win clearly: its norm is done, but so is the other's nearly
            if best is not None and times[best] < 0.97 * times[None]:
                result["decode_acc"][akey] = list(best)
            log(f"tune {name:15s} {N:6d} x {K:6d} M= 8 residual sum: one launch "
                f"{times[None] * 1e6:.1f} us; best split {best} {times[best] * 1e6:.1f} us")
            if saved is not None:
                table["decode_acc"][akey] = saved
        del ws
    ok = [l for l in losses if l == l]
    if ok:
        log(f"tune: the rules' choice is on average {sum(ok) / len(ok) * 100:.1f} % slower than the "
            f"best plan (worst {max(ok) * 100:.0f} %) over {len(ok)} products")
    ops.check_plans(result)
    return result


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="bench-ops", description=__doc__.split("\n\n")[0])
    ap.add_argument("model_dir", nargs="?", default=None)
    ap.add_argument("--shape", default="8b", choices=sorted(SHAPES))
    ap.add_argument("--tokens", default="1,8,64,2048")
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--ctx", type=int, default=2048)
    ap.add_argument("--only", default=None, choices=["gemm", "attention", "elementwise"])
    ap.add_argument("--device", default="cuda:0")
    ap.add_argument("--tune", action="store_true",
                    help="measure the plans for this model's widths and write kernel_plans.json")
    ap.add_argument("--plans-out", default=None,
                    help="with --tune: where to write the plans (default: the model folder)")
    args = ap.parse_args(argv)
    if args.model_dir:
        from .config import load_config
        c = load_config(args.model_dir)
        cfg = {k: getattr(c, k) for k in SHAPES["8b"]}
    else:
        cfg = SHAPES[args.shape]
    if args.tune:
        import json
        import os
        from . import ops
        out = args.plans_out or (os.path.join(args.model_dir, ops.PLAN_FILE) if args.model_dir
                                 else None)
        if out is None:
            print("bench-ops --tune needs a model folder or --plans-out", file=sys.stderr)
            return 2
        plans = tune(cfg, args.device)
        with open(out, "w", encoding="utf-8") as f:
            json.dump(plans, f, indent=1)
        print(f"wrote {out}: {len(plans['plans'])} widths, {len(plans['decode_acc'])} residual sums")
        return 0
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
