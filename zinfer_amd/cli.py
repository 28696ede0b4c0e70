"""The command line, in the manner of the reference's ``zinfer`` binary
(`src/app/cli.zig:11-289` dispatch, `src/app/cli/usage.zig:6-65` usage,
`src/app/cli/args.zig:91-148,352-501` positional forms, presets and flags): sub-commands by
name, ``[model_dir]`` first and optional, then the prompt, ``max_new_tokens``,
``think|no-think``, then ``--flag value`` pairs with the reference's names and meanings.
Prompts are token ids (``1,2,3``); text is out of this engine's scope.  Options the reference
has for things this engine does not build (quantised backends and caches, CPU threads) are
parsed and refused or ignored with a message.
"""
from __future__ import annotations

import sys
import time
from typing import List, Optional, Tuple

DEFAULT_MODEL_DIR = "models/Qwen3-0.6B"          # `src/app/cli/args.zig:7`

USAGE = """Usage:
  zinfer inspect-config [model_dir]
  zinfer inspect-weights [model_dir]
  zinfer inspect-tensor [model_dir] <tensor_name> [count]
  zinfer generate-token-ids [model_dir] <seed_ids_csv> <steps>
  zinfer generate [model_dir] <ids_csv> [max_new_tokens] [think|no-think] [flags...]
  zinfer bench [model_dir] <ids_csv> [max_new_tokens]
  zinfer bench-batch [model_dir] <ids_csv> <batch_size> [max_new_tokens]
  zinfer bench-continuous [model_dir] <ids_csv> <batch_size> <total_requests> [max_new_tokens]
  zinfer bench-ops [model_dir] [--shape 8b|14b|32b] [--tokens 1,8,64,2048] [--iters N]
  zinfer random-model <config.json> <out_dir> [--seed <u64>] [--dtype bfloat16|float32]

Defaults:
  model_dir = models/Qwen3-0.6B
  generate max_new_tokens = 64, bench max_new_tokens = 16

Flags:
  --seed <u64>                 --temperature <f32>        --top-p <f32>
  --top-k <usize>              --min-p <f32>              --presence-penalty <f32>
  --frequency-penalty <f32>    --repetition-penalty <f32> --stream
  --backend <auto|bf16>        --kv-cache <auto|bf16|fp32>
  --threads <usize>            (accepted, unused: the GPU grid replaces the thread pool)
  --dtype <bfloat16|float32>   --page-size <n>            --max-tokens <n>
  --max-step-tokens <n>        --chunk <n>                --max-seqs <n>
  --ignore-eos                 --device <cuda:0>          --multi-step <n>
"""


class CliError(Exception):
    """InvalidCommand, MissingFlagValue, UnknownFlag, ... (`src/app/cli/args.zig`)."""


def parse_token_ids(csv: str) -> List[int]:
    """`src/app/cli/token_ids.zig:3-18`: comma separated, blanks trimmed, empty parts skipped."""
    out = []
    for part in csv.split(","):
        part = part.strip(" ")
        if part:
            if not part.isdigit():
                raise CliError(f"InvalidCommand: {part!r} is not a token id")
            out.append(int(part))
    return out


def _is_flag(a: str) -> bool:
    return a.startswith("--")


def _split_flags(args: List[str]) -> Tuple[List[str], List[str]]:
    for i, a in enumerate(args):
        if _is_flag(a):
            return args[:i], args[i:]
    return args, []


class Options:
    def __init__(self, max_new_tokens: int, think: bool = False):
        from .sampling import thinking_defaults
        self.max_new_tokens = max_new_tokens
        self.think = think
        self.sampling = thinking_defaults(think)        # `args.zig:352-373`
        self.stream = False
        self.kv_cache = "auto"
        self.dtype = "bfloat16"
        self.page_size = 16
        self.max_tokens: Optional[int] = None
        self.max_step_tokens = 2048
        self.chunk: Optional[int] = None
        self.max_seqs = 64
        self.multi_step = 8
        self.ignore_eos = False
        self.device = "cuda:0"
        self.seed = 0


_FLOAT_FLAGS = {"--temperature": "temperature", "--top-p": "top_p", "--min-p": "min_p",
                "--presence-penalty": "presence_penalty",
                "--frequency-penalty": "frequency_penalty",
                "--repetition-penalty": "repetition_penalty"}


def parse_flags(flags: List[str], opt: Options) -> None:
    """`src/app/cli/args.zig:395-501`."""
    i = 0

    def value() -> str:
        nonlocal i
        i += 1
        if i >= len(flags):
            raise CliError(f"MissingFlagValue: {flags[i - 1]}")
        return flags[i]

    while i < len(flags):
        a = flags[i]
        if not _is_flag(a):
            raise CliError(f"InvalidCommand: unexpected {a!r}")
        if a in _FLOAT_FLAGS:
            setattr(opt.sampling, _FLOAT_FLAGS[a], float(value()))
        elif a == "--top-k":
            opt.sampling.top_k = int(value())
        elif a == "--seed":
            opt.seed = int(value())
            opt.sampling.seed = opt.seed
        elif a == "--stream":
            opt.stream = True
        elif a == "--backend":
            v = value()
            if v in ("q8", "q6", "q4"):
                raise CliError(f"InvalidBackendScheme: {v} (quantised weights are not built)")
            if v not in ("auto", "bf16"):
                raise CliError(f"InvalidBackendScheme: {v}")
        elif a == "--kv-cache":
            v = value()
            if v == "q8":
                raise CliError("InvalidKvCacheScheme: q8 (a quantised cache is not built)")
            if v not in ("auto", "bf16", "fp32"):
                raise CliError(f"InvalidKvCacheScheme: {v}")
            opt.kv_cache = v
        elif a == "--threads":
            value()
        elif a in ("--system", "--stop", "--q8-layout"):
            raise CliError(f"UnknownFlag: {a} belongs to the text front end or the quantised "
                           "cache, which this engine does not build")
        elif a == "--dtype":
            opt.dtype = value()
        elif a == "--page-size":
            opt.page_size = int(value())
        elif a == "--max-tokens":
            opt.max_tokens = int(value())
        elif a == "--max-step-tokens":
            opt.max_step_tokens = int(value())
        elif a == "--chunk":
            opt.chunk = int(value())
        elif a == "--max-seqs":
            opt.max_seqs = int(value())
        elif a == "--multi-step":
            opt.multi_step = int(value())
        elif a == "--ignore-eos":
            opt.ignore_eos = True
        elif a == "--device":
            opt.device = value()
        else:
            raise CliError(f"UnknownFlag: {a}")
        i += 1


def parse_generate(args: List[str], default_new: int) -> Tuple[str, List[int], Options]:
    """``[model_dir] <ids> [max_new_tokens] [think|no-think] [flags]``: the model folder is
    there when the third positional is a number (`args.zig:100-131`)."""
    pos, flags = _split_flags(args)
    if not pos:
        raise CliError("InvalidCommand: a prompt is needed")
    model_dir = DEFAULT_MODEL_DIR
    if len(pos) >= 3 and pos[2].isdigit():
        model_dir, pos = pos[0], pos[1:]
    elif len(pos) >= 2 and not pos[1].isdigit() and pos[1] not in ("think", "no-think"):
        model_dir, pos = pos[0], pos[1:]
    ids = parse_token_ids(pos[0])
    rest = pos[1:]
    max_new = default_new
    if rest and rest[0].isdigit():
        max_new = int(rest[0])
        rest = rest[1:]
    think = False
    if rest:
        if rest[0] not in ("think", "no-think"):
            raise CliError(f"InvalidThinkingMode: {rest[0]}")
        think = rest[0] == "think"
        rest = rest[1:]
    if rest:
        raise CliError(f"InvalidCommand: unexpected {rest[0]!r}")
    opt = Options(max_new, think)
    parse_flags(flags, opt)
    opt.sampling.max_new_tokens = opt.max_new_tokens
    opt.sampling.ignore_eos = opt.ignore_eos
    return model_dir, ids, opt


def _llm(model_dir: str, opt: Options, max_tokens: Optional[int] = None):
    from .entrypoints import LLM
    kv = None if opt.kv_cache == "auto" else ("bfloat16" if opt.kv_cache == "bf16" else "float32")
    return LLM(model_dir, dtype=opt.dtype, device=opt.device, page_size=opt.page_size,
               max_tokens=opt.max_tokens or max_tokens, max_step_tokens=opt.max_step_tokens,
               chunk_size=opt.chunk, max_seqs=opt.max_seqs, kv_dtype=kv,
               multi_step=opt.multi_step)


# ------------------------------------------------------------------------- commands
def cmd_inspect_config(args: List[str]) -> int:
    """`src/app/cli/inspect.zig:8-34`."""
    from .config import entry_for, load_config, read_config_json
    model_dir = args[0] if args else DEFAULT_MODEL_DIR
    cfg = load_config(model_dir)
    print("Zinfer model inspection")
    print(f"model_dir: {model_dir}")
    print(f"model_type: {cfg.model_type}")
    print(f"architecture: {entry_for(read_config_json(model_dir)).name}")
    for key in ("hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
                "num_key_value_heads", "head_dim", "vocab_size", "max_position_embeddings"):
        print(f"{key}: {getattr(cfg, key)}")
    print(f"rope_theta: {int(cfg.rope_theta)}")
    print(f"rms_norm_eps: {cfg.rms_norm_eps:e}")
    print(f"torch_dtype: {cfg.torch_dtype}")
    print(f"tie_word_embeddings: {str(cfg.tie_word_embeddings).lower()}")
    return 0


def cmd_inspect_weights(args: List[str]) -> int:
    """`src/app/cli/inspect.zig:36-72`."""
    import os
    from .weights import SafetensorsFile
    model_dir = args[0] if args else DEFAULT_MODEL_DIR
    path = os.path.join(model_dir, "model.safetensors")
    with SafetensorsFile(path) as f:
        print("Zinfer weights inspection")
        print(f"weights_path: {path}")
        print(f"file_size: {os.path.getsize(path)}")
        print(f"tensor_count: {len(f.infos)}")
        for k, v in f.metadata.items():
            print(f"metadata.{k}: {v}")
        for name in ("model.embed_tokens.weight", "model.layers.0.self_attn.q_proj.weight",
                     "model.layers.0.self_attn.k_proj.weight",
                     "model.layers.0.mlp.gate_proj.weight", "model.norm.weight",
                     "lm_head.weight"):
            if name in f.infos:
                i = f.infos[name]
                print(f"tensor {name}: dtype={i.dtype} shape={list(i.shape)} "
                      f"offsets=[{i.begin}, {i.end}]")
    return 0


def cmd_inspect_tensor(args: List[str]) -> int:
    """`src/app/cli/inspect.zig:74-107`: ``[model_dir] <tensor_name> [count]``."""
    import os
    from .weights import SafetensorsFile
    if not args:
        raise CliError("InvalidCommand: a tensor name is needed")
    model_dir, name, count = DEFAULT_MODEL_DIR, args[0], 8
    if len(args) >= 2 and not args[1].isdigit():
        model_dir, name = args[0], args[1]
        if len(args) >= 3:
            count = int(args[2])
    elif len(args) >= 2:
        count = int(args[1])
    with SafetensorsFile(os.path.join(model_dir, "model.safetensors")) as f:
        if name not in f.infos:
            raise CliError(f"TensorNotFound: {name}")
        i = f.infos[name]
        vals = f.tensor(name).float().reshape(-1)[:count].tolist()
        print(f"tensor {name}: dtype={i.dtype} shape={list(i.shape)}")
        print("values: " + ", ".join(f"{v:.6f}" for v in vals))
    return 0


def cmd_generate_token_ids(args: List[str]) -> int:
    """`src/app/cli/inspect.zig:246-312`: greedy from raw ids, no end-of-sequence check;
    prints prompt and generated ids in one list as the reference does."""
    from .sampling import SamplingParams
    pos, flags = _split_flags(args)
    if len(pos) == 3:
        model_dir, csv, steps = pos[0], pos[1], int(pos[2])
    elif len(pos) == 2:
        model_dir, csv, steps = DEFAULT_MODEL_DIR, pos[0], int(pos[1])
    else:
        raise CliError("InvalidCommand: generate-token-ids [model_dir] <seed_ids_csv> <steps>")
    ids = parse_token_ids(csv)
    if not ids:
        raise CliError("EmptySeed")
    opt = Options(steps)
    parse_flags(flags, opt)
    llm = _llm(model_dir, opt, max_tokens=(len(ids) + steps + 63) // 64 * 64)
    out = llm.generate([ids], SamplingParams(temperature=0.0, max_new_tokens=steps,
                                             ignore_eos=True))[0] if steps > 0 else []
    print("Zinfer generated token ids")
    print(f"seed: {csv}")
    print(f"steps: {steps}")
    print("tokens: [" + ", ".join(str(t) for t in ids + out) + "]")
    return 0


def cmd_generate(args: List[str]) -> int:
    """`src/app/cli/generate.zig:7-37` with token ids in place of text."""
    model_dir, ids, opt = parse_generate(args, 64)
    if not ids:
        raise CliError("EmptyPrompt")
    llm = _llm(model_dir, opt, max_tokens=(len(ids) + opt.max_new_tokens + 63) // 64 * 64)
    if not opt.stream:
        out = llm.generate([ids], opt.sampling)[0]
        print(",".join(str(t) for t in out))
        return 0
    sched = llm.new_scheduler()
    rid = sched.add_request(ids, opt.sampling)
    shown = 0
    while sched.has_work():
        sched.step()
        req = sched.finished.get(rid) or next(r for r in sched.running + list(sched.waiting)
                                              if r.id == rid)
        for t in req.generated[shown:]:
            sys.stdout.write(("," if shown else "") + str(t))
            sys.stdout.flush()
            shown += 1
    sys.stdout.write("\n")
    return 0


def _bench_common(args: List[str], n_extra: int):
    pos, flags = _split_flags(args)
    need = 1 + n_extra
    model_dir = DEFAULT_MODEL_DIR
    if len(pos) >= need + 1 and not pos[0].replace(",", "").replace(" ", "").isdigit():
        model_dir, pos = pos[0], pos[1:]
    if len(pos) < need:
        raise CliError("InvalidCommand")
    ids = parse_token_ids(pos[0])
    extra = [int(v) for v in pos[1:1 + n_extra]]
    max_new = int(pos[need]) if len(pos) > need else 16          # `args.zig:237`
    opt = Options(max_new)
    parse_flags(flags, opt)
    return model_dir, ids, extra, opt


def _weights_bytes(llm) -> int:
    seen, total = set(), 0
    stack = [llm.model]
    import torch
    while stack:
        o = stack.pop()
        if isinstance(o, torch.Tensor):
            if o.data_ptr() not in seen and o.device.type != "meta":
                seen.add(o.data_ptr())
                total += o.numel() * o.element_size()
        elif isinstance(o, (list, tuple)):
            stack.extend(o)
        elif hasattr(o, "__dict__") and o.__class__.__module__.startswith("zinfer_amd"):
            stack.extend(v for k, v in vars(o).items() if k not in ("ctx", "spec", "cos", "sin"))
    return total


def cmd_bench(args: List[str], mode: str) -> int:
    """`src/app/cli/tools/bench/runtime.zig:12-99` (bench), `:135-224` (bench-batch),
    `:226-310` (bench-continuous): timers around prefill and decode, greedy, the same keys."""
    import torch
    from .engine import StepEntry
    from .sampling import SamplingParams
    n_extra = {"bench": 0, "bench-batch": 1, "bench-continuous": 2}[mode]
    model_dir, ids, extra, opt = _bench_common(args, n_extra)
    batch = extra[0] if extra else 1
    total = extra[1] if len(extra) > 1 else batch
    per_req = (len(ids) + opt.max_new_tokens + 63) // 64 * 64
    opt.max_seqs = max(batch, 1)
    llm = _llm(model_dir, opt, max_tokens=per_req * batch)
    params = SamplingParams(temperature=0.0, max_new_tokens=opt.max_new_tokens,
                            ignore_eos=opt.ignore_eos)
    print({"bench": "Zinfer benchmark", "bench-batch": "Zinfer batch benchmark",
           "bench-continuous": "Zinfer continuous batch benchmark"}[mode])
    print(f"model_dir: {model_dir}")
    print(f"backend: {opt.dtype}")
    print(f"kv_cache: {llm.engine.cache.groups[0].k.dtype if llm.engine.cache.groups else '-'}")
    print("kernel_isa: gfx950")
    if mode == "bench-continuous":
        sched = llm.new_scheduler()
        for _ in range(total):
            sched.add_request(ids, params)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        done = sched.run()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        decoded = sum(len(r.generated) for r in done.values())
        print(f"batch_size: {batch}")
        print(f"total_requests: {total}")
        print(f"prompt_tokens: {len(ids)}")
        print(f"decode_tokens: {decoded}")
        print(f"service_ms: {dt * 1e3:.3f}")
        print(f"service_tok_s: {(decoded + total * len(ids)) / dt:.3f}")
        print(f"decode_tok_s: {decoded / dt:.3f}")
    else:
        eng = llm.engine
        names = [f"b{i}" for i in range(batch)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        toks = []
        for n in names:                       # prompts one after the other, as the reference
            logits = eng.step([StepEntry(n, ids, [len(ids) - 1])])
            toks.append(eng.argmax(logits)[0])
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        eos = () if opt.ignore_eos else llm.model.spec.eos_token_ids
        live = {n: t for n, t in zip(names, toks) if t not in eos}
        decoded = 0
        for _ in range(opt.max_new_tokens):
            if not live:
                break
            order = list(live)
            logits = eng.step([StepEntry(n, [live[n]], [0]) for n in order])
            decoded += len(order)
            for n, t in zip(order, eng.argmax(logits)):
                if t in eos:
                    del live[n]
                else:
                    live[n] = t
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        if batch > 1:
            print(f"batch_size: {batch}")
        print(f"prompt_tokens: {len(ids)}")
        print(f"decode_tokens: {decoded}")
        print(f"prefill_ms: {(t1 - t0) * 1e3:.3f}")
        print(f"decode_ms: {(t2 - t1) * 1e3:.3f}")
        print(f"prefill_tok_s: {len(ids) * batch / (t1 - t0):.3f}")
        print(f"decode_tok_s: {decoded / max(t2 - t1, 1e-12):.3f}")
    wb = _weights_bytes(llm)
    kb = llm.engine.cache.kv_bytes()
    print(f"weights_bytes: {wb}")
    print(f"weights_mib: {wb / 1048576:.3f}")
    print(f"kv_cache_bytes: {kb}")
    print(f"kv_cache_mib: {kb / 1048576:.3f}")
    return 0


def cmd_random_model(args: List[str]) -> int:
    """Random-weights mode: a model folder (config.json, model.safetensors) from a
    configuration file and a seed."""
    import json
    import torch
    from .config import entry_for
    from .weights import write_model_dir
    pos, flags = _split_flags(args)
    if len(pos) != 2:
        raise CliError("InvalidCommand: random-model <config.json> <out_dir>")
    opt = Options(0)
    parse_flags(flags, opt)
    with open(pos[0]) as f:
        raw = json.load(f)
    cfg = entry_for(raw).config_type.from_dict(raw)
    dtype = torch.bfloat16 if opt.dtype in ("bfloat16", "bf16") else torch.float32
    write_model_dir(pos[1], cfg, opt.seed, dtype)
    print(f"wrote {pos[1]} (seed {opt.seed}, {opt.dtype})")
    return 0


def main(argv: Optional[List[str]] = None) -> int:
    from .errors import ZinferError
    argv = list(sys.argv[1:] if argv is None else argv)
    if not argv or argv[0] in ("-h", "--help", "help"):
        sys.stdout.write(USAGE)
        return 0
    cmd, args = argv[0], argv[1:]
    try:
        if cmd == "inspect-config":
            return cmd_inspect_config(args)
        if cmd == "inspect-weights":
            return cmd_inspect_weights(args)
        if cmd == "inspect-tensor":
            return cmd_inspect_tensor(args)
        if cmd == "generate-token-ids":
            return cmd_generate_token_ids(args)
        if cmd == "generate":
            return cmd_generate(args)
        if cmd in ("bench", "bench-batch", "bench-continuous"):
            return cmd_bench(args, cmd)
        if cmd == "random-model":
            return cmd_random_model(args)
        if cmd == "bench-ops":
            from .bench_ops import main as bench_ops_main
            return bench_ops_main(args)
        if cmd in ("quantize", "tokenize", "decode-ids", "generate-chat", "chat", "probe-linear",
                   "probe-block", "probe-model", "bench-suite"):
            print(f"zinfer: {cmd!r} belongs to what this engine does not build (text front "
                  "end, quantisation, CPU probes)", file=sys.stderr)
            return 2
        print(f"zinfer: unknown command {cmd!r}\n", file=sys.stderr)     # `cli.zig:286`
        sys.stderr.write(USAGE)
        return 2
    except (CliError, ZinferError, FileNotFoundError, ValueError) as e:
        print(f"zinfer: {type(e).__name__}: {e}", file=sys.stderr)
        return 1


if __name__ == "__main__":
    sys.exit(main())
