"""The command line, in the manner of the reference's ``zinfer`` binary
(`src/app/cli.zig:11-289` dispatch, `src/app/cli/usage.zig:6-65` usage,
`src/app/cli/args.zig:91-148,352-501` positional forms, presets and flags): sub-commands by
name, ``[model_dir]`` first and optional, then the prompt, ``max_new_tokens``,
``think|no-think``, then ``--flag value`` pairs with the reference's names and meanings.
Prompts are token ids (``1,2,3``), or text when the model folder brings a tokenizer
(``tokenizer.json``, or ``vocab.json`` + ``merges.txt`` + ``tokenizer_config.json``).  Options
the reference has for things this engine does not build (quantised backends and caches, CPU
threads) are parsed and refused or ignored with a message.
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
  zinfer probe-linear [model_dir] <tensor_name> [input_index] [rows_to_print]
  zinfer probe-block [model_dir] [layer_index] [input_index] [count]
  zinfer probe-model [model_dir] [token_id] [top_k]
  zinfer generate-token-ids [model_dir] <seed_ids_csv> <steps>
  zinfer generate [model_dir] <text|ids_csv> [max_new_tokens] [think|no-think] [flags...]
  zinfer generate-chat [model_dir] <messages_json_path> [max_new_tokens] [think|no-think] [flags...]
  zinfer chat [model_dir] [max_new_tokens] [think|no-think] [flags...]
  zinfer tokenize [model_dir] <text>
  zinfer decode-ids [model_dir] <ids_csv>
  zinfer serve-batch [model_dir] --requests <file.jsonl> [--out <file.jsonl>] [flags...]
  zinfer replay --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N   (steps on stdin)
  zinfer bench [model_dir] <ids_csv> [max_new_tokens]
  zinfer bench-batch [model_dir] <ids_csv> <batch_size> [max_new_tokens]
  zinfer bench-continuous [model_dir] <ids_csv> <batch_size> <total_requests> [max_new_tokens]
  zinfer bench-suite [model_dir]
  zinfer bench-ops [model_dir] [--shape 0.6b|1.7b|4b|8b|14b|32b] [--tokens 1,8,64,2048] [--iters N]
                   [--tune [--plans-out kernel_plans.json]]
  zinfer random-model <config.json> <out_dir> [--seed <u64>] [--dtype bfloat16|float32]

Defaults:
  model_dir = models/Qwen3-0.6B
  generate max_new_tokens = 64, generate-chat/chat max_new_tokens = 128, bench max_new_tokens = 16

Flags:
  --seed <u64>                 --temperature <f32>        --top-p <f32>
  --top-k <usize>              --min-p <f32>              --presence-penalty <f32>
  --frequency-penalty <f32>    --repetition-penalty <f32> --stream
  --system <text>              --stop <text> (repeatable; text prompts only)
  --load <path>  --save <path> (chat only: a session to start from, and to write at the end)
  --backend <auto|bf16>        --kv-cache <auto|bf16|fp32>
  --threads <usize>            (accepted, unused: the GPU grid replaces the thread pool)
  --dtype <bfloat16|float32>   --page-size <n>            --max-tokens <n>
  --max-step-tokens <n>        --chunk <n>                --max-seqs <n>
  --ignore-eos                 --device <cuda:0>          --multi-step <n>
  --config <config.json> --random-weights <seed>   (weights drawn from the seed; no folder read)
  --debug-tables               (every step's block tables and slots checked on the device first)
  --classes                    (bench, bench-batch: a decode step's time per class of kernels)
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
        self.stop: List[str] = []                       # `args.zig:433-436`
        self.system: Optional[str] = None
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
        self.debug_tables = False       # check every step's block tables on the device
        self.classes = False            # bench: a decode step's time per class of kernels
        self.load_path: Optional[str] = None            # chat only (`args.zig:437-446`)
        self.save_path: Optional[str] = None
        self.config_path: Optional[str] = None          # with --random-weights: no model folder
        self.random_weights: Optional[int] = None


_FLOAT_FLAGS = {"--temperature": "temperature", "--top-p": "top_p", "--min-p": "min_p",
                "--presence-penalty": "presence_penalty",
                "--frequency-penalty": "frequency_penalty",
                "--repetition-penalty": "repetition_penalty"}


def parse_flags(flags: List[str], opt: Options, chat: bool = False) -> None:
    """`src/app/cli/args.zig:395-501`.  ``chat``: the flags that only the chat loop has."""
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
        elif a == "--stop":
            opt.stop.append(value())
        elif a == "--system":
            opt.system = value()
        elif a in ("--load", "--save") and chat:
            setattr(opt, a[2:] + "_path", value())
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
        elif a == "--q8-layout":
            raise CliError("UnknownFlag: --q8-layout belongs to the quantised cache, which "
                           "this engine does not build")
        elif a == "--config":
            opt.config_path = value()
        elif a == "--random-weights":
            opt.random_weights = int(value())
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
        elif a == "--debug-tables":
            opt.debug_tables = True
        elif a == "--classes":
            opt.classes = True
        elif a == "--device":
            opt.device = value()
        else:
            raise CliError(f"UnknownFlag: {a}")
        i += 1


def _looks_like_ids(text: str) -> bool:
    return bool(text) and all(c.isdigit() or c in ", " for c in text) and any(c.isdigit() for c in text)


def parse_generate_text(args: List[str], default_new: int) -> Tuple[str, str, Options]:
    """``[model_dir] <prompt> [max_new_tokens] [think|no-think] [flags]``: the model folder is
    there when the third positional is a number (`args.zig:100-131`).  The prompt stays a
    string: token ids or text."""
    pos, flags = _split_flags(args)
    if not pos:
        raise CliError("InvalidCommand: a prompt is needed")
    model_dir = DEFAULT_MODEL_DIR
    if len(pos) >= 3 and pos[2].isdigit():
        model_dir, pos = pos[0], pos[1:]
    elif len(pos) >= 2 and not pos[1].isdigit() and pos[1] not in ("think", "no-think"):
        model_dir, pos = pos[0], pos[1:]
    prompt = pos[0]
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
    return model_dir, prompt, opt


def parse_generate(args: List[str], default_new: int) -> Tuple[str, List[int], Options]:
    """The same with a prompt of token ids."""
    model_dir, prompt, opt = parse_generate_text(args, default_new)
    return model_dir, parse_token_ids(prompt), opt


def _llm(model_dir: str, opt: Options, max_tokens: Optional[int] = None):
    from .entrypoints import LLM
    kv = None if opt.kv_cache == "auto" else ("bfloat16" if opt.kv_cache == "bf16" else "float32")
    if (opt.config_path is None) != (opt.random_weights is None):
        raise CliError("MissingFlagValue: --config <config.json> and --random-weights <seed> "
                       "go together")
    if opt.config_path is not None:
        # weights drawn from the seed instead of read from a folder; the positional model
        # folder, if one was given, is not opened
        model_dir = None
    return LLM(model_dir, config=opt.config_path, random_seed=opt.random_weights, dtype=opt.dtype, device=opt.device, page_size=opt.page_size,
               max_tokens=opt.max_tokens or max_tokens, max_step_tokens=opt.max_step_tokens,
               chunk_size=opt.chunk, max_seqs=opt.max_seqs, kv_dtype=kv,
               multi_step=opt.multi_step, debug_tables=opt.debug_tables)


def _text_hooks(model_dir: str):
    """The tokenizer and templates of the architecture that ``model_dir``'s config.json names
    (`src/model/runtime/decoder_registry.zig:16-19`): the command line knows no family's."""
    from .config import entry_for, read_config_json
    entry = entry_for(read_config_json(model_dir))
    if entry.text is None:
        raise CliError(f"NoTextFrontEnd: the architecture {entry.name} brings no tokenizer and "
                       "no prompt template; give token ids")
    return entry.text


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
    # every key of the typed configuration, whatever the architecture; numbers as the
    # reference prints them (theta as an integer, eps in scientific notation)
    for key, value in cfg.to_dict().items():
        if key in ("model_type", "architectures"):
            continue
        if isinstance(value, bool):
            value = str(value).lower()
        elif isinstance(value, float):
            value = int(value) if value >= 1.0 and value == int(value) else f"{value:e}"
        print(f"{key}: {value}")
    return 0


def cmd_inspect_weights(args: List[str]) -> int:
    """`src/app/cli/inspect.zig:36-72`."""
    import os
    from .config import load_config
    from .models.build import declare_tensors
    from .weights import SafetensorsFile
    model_dir = args[0] if args else DEFAULT_MODEL_DIR
    path = os.path.join(model_dir, "model.safetensors")
    # what is shown: the tensors outside the layers and those of the first layer, by the
    # names the architecture of config.json declares
    spec = load_config(model_dir).model_spec()
    first_layer, any_layer = spec.layer_prefix.format(0), spec.layer_prefix.split("{")[0]
    shown = [n for n in declare_tensors(spec)
             if n.startswith(first_layer) or not n.startswith(any_layer)]
    with SafetensorsFile(path) as f:
        print("Zinfer weights inspection")
        print(f"weights_path: {path}")
        print(f"file_size: {os.path.getsize(path)}")
        print(f"tensor_count: {len(f.infos)}")
        for k, v in f.metadata.items():
            print(f"metadata.{k}: {v}")
        for name in shown:
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


def _probe_args(args: List[str], n_numbers: int, defaults, name_first: bool = False):
    """``[model_dir] [name] [numbers...]`` of the probe commands (`src/app/cli.zig:47-135`):
    the model folder is the first positional when it is no number (and, for a command that
    takes a name, when two words come before the numbers); numbers left out take their
    defaults.  Returns (model_dir, name or None, numbers, options)."""
    pos, flags = _split_flags(args)
    words = 0
    while words < len(pos) and not pos[words].isdigit():
        words += 1
    want = 1 if name_first else 0
    if words not in (want, want + 1) or len(pos) - words > n_numbers:
        raise CliError("InvalidCommand")
    model_dir = pos[0] if words == want + 1 else DEFAULT_MODEL_DIR
    name = pos[words - 1] if name_first else None
    numbers = [int(v) for v in pos[words:]]
    numbers += list(defaults[len(numbers):])
    opt = Options(0)
    parse_flags(flags, opt)
    return model_dir, name, numbers, opt


def _numbers(values) -> str:
    return "[" + ", ".join(f"{float(v):.6f}" for v in values) + "]"


def cmd_probe_linear(args: List[str]) -> int:
    """`src/app/cli/inspect.zig:109-151`: a vector that is 1 at ``input_index`` and 0 elsewhere
    through the matrix ``tensor_name``, by the engine's own product; the first outputs."""
    import os
    import torch
    from .models.build import parse_dtype
    from .parts import BuildContext
    from .parts.linear import Linear, place_matrix
    from .weights import SafetensorsFile
    model_dir, name, (index, rows_to_print), opt = _probe_args(args, 2, (0, 8), name_first=True)
    path = os.path.join(model_dir, "model.safetensors")
    with SafetensorsFile(path) as f:
        if name not in f.infos:
            raise CliError(f"TensorNotFound: {name}")
        if len(f.infos[name].shape) != 2:
            raise CliError(f"InvalidTensorRank: {name} has shape {list(f.infos[name].shape)}")
        rows, cols = f.infos[name].shape
        if index >= cols:
            raise CliError(f"InputIndexOutOfBounds: {index}, the matrix has {cols} columns")
        ctx = BuildContext(parse_dtype(opt.dtype), torch.device(opt.device))
        linear = Linear(place_matrix(f.tensor(name), ctx))
    x = torch.zeros((1, cols), dtype=ctx.act_dtype, device=ctx.device)
    x[0, index] = 1.0
    out = torch.empty((1, rows), dtype=torch.float32, device=ctx.device)
    linear.forward(x, out)
    print("Zinfer linear probe")
    print(f"tensor: {name}")
    print(f"weights_path: {path}")
    print(f"shape: [{rows}, {cols}]")
    print(f"input_index: {index}")
    print("first_outputs: " + _numbers(out[0, :rows_to_print].tolist()))
    return 0


def cmd_probe_block(args: List[str]) -> int:
    """`src/app/cli/inspect.zig:153-204`: a hidden vector that is 1 at ``input_index`` through
    block ``layer_index`` alone, as a new request's first token; the first outputs."""
    import torch
    model_dir, _, (layer, index, count), opt = _probe_args(args, 3, (0, 0, 8))
    llm = _llm(model_dir, opt, max_tokens=64)
    spec = llm.model.spec
    if index >= spec.hidden_size:
        raise CliError(f"InputIndexOutOfBounds: {index}, hidden_size is {spec.hidden_size}")
    if layer >= len(llm.model.blocks):
        raise CliError(f"LayerIndexOutOfBounds: {layer}, the model has {len(llm.model.blocks)}")
    hidden = torch.zeros((1, spec.hidden_size), dtype=torch.float32, device=opt.device)
    hidden[0, index] = 1.0
    out, cache_len = llm.engine.probe_block(layer, hidden)
    print("Zinfer block probe")
    print(f"layer_index: {layer}")
    print(f"input_index: {index}")
    print(f"cache_len: {cache_len}")
    print("first_outputs: " + _numbers(out[0, :count].tolist()))
    return 0


def cmd_probe_model(args: List[str]) -> int:
    """`src/app/cli/inspect.zig:206-244`: one token through the whole model as a new request;
    the largest logits."""
    from .engine import StepEntry
    model_dir, _, (token, top_k), opt = _probe_args(args, 2, (0, 8))
    llm = _llm(model_dir, opt, max_tokens=64)
    logits = llm.engine.step([StepEntry("probe", [token], [0])], end=["probe"])[0]
    top = logits.topk(min(top_k, logits.numel()))
    print("Zinfer model probe")
    print(f"token_id: {token}")
    for value, at in zip(top.values.tolist(), top.indices.tolist()):
        print(f"top_logit token={at} value={value:.6f}")
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
    """`src/app/cli/generate.zig:7-37`: a text prompt goes through the family's chat template
    and the tokenizer and the answer is printed as text; a prompt of token ids is run as it is
    and the answer is printed as ids."""
    model_dir, prompt, opt = parse_generate_text(args, 64)
    if not _looks_like_ids(prompt):
        hooks = _text_hooks(model_dir)
        print("Zinfer generate")
        print(f"mode: {'think' if opt.think else 'no-think'}")
        print(f"prompt: {prompt}")
        return _generate_text(model_dir, hooks.render_single_user(prompt, opt.think, opt.system),
                              opt)
    ids = parse_token_ids(prompt)
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
        req = sched.request(rid)
        for t in req.generated[shown:]:
            sys.stdout.write(("," if shown else "") + str(t))
            sys.stdout.flush()
            shown += 1
    sys.stdout.write("\n")
    return 0


def _respond(llm, tok, ids: List[int], opt: Options, stops: List[str]) -> str:
    """Generates from ``ids`` until an end-of-sequence id, the token limit or a stop sequence
    and returns the answer; with ``--stream`` it is printed piece by piece on the way, except
    for a tail that may still grow into a stop sequence
    (`src/app/cli/runtime/generator.zig:60-140`, `runtime/streaming.zig:41-65`)."""
    from .text import analyze_generated_text
    sched = llm.new_scheduler()
    rid = sched.add_request(ids, opt.sampling)
    printed, response, seen = 0, None, 0
    while sched.has_work() and response is None:
        sched.step()
        generated = sched.request(rid).generated
        # token by token, as the reference looks at its text: a step may bring several
        for k in range(seen + 1, len(generated) + 1):
            text = tok.decode(generated[:k])
            printable, hit, response_len = analyze_generated_text(text, stops)
            if opt.stream and printable > printed:
                sys.stdout.write(text[printed:printable])
                sys.stdout.flush()
                printed = printable
            if hit:
                response = text[:response_len]
                sched.abort(rid, "stop")
                break
        seen = len(generated)
    if response is None:
        response = tok.decode(sched.request(rid).generated)
    if opt.stream:
        sys.stdout.write(response[printed:])
        sys.stdout.flush()
    return response


def _generate_text(model_dir: str, prompt_text: str, opt: Options) -> int:
    """Encodes the rendered prompt, generates and prints the answer."""
    from .text import effective_stop_sequences
    tok = _text_hooks(model_dir).load_tokenizer(model_dir)
    ids = tok.encode(prompt_text)
    if not ids:
        raise CliError("EmptyPrompt")
    llm = _llm(model_dir, opt, max_tokens=(len(ids) + opt.max_new_tokens + 63) // 64 * 64)
    stops = effective_stop_sequences(llm.model.spec.default_stop_sequences, opt.stop)
    sys.stdout.write("response: ")
    response = _respond(llm, tok, ids, opt, stops)
    if not opt.stream:
        sys.stdout.write(response)
    sys.stdout.write("\n")
    return 0


def cmd_generate_chat(args: List[str]) -> int:
    """`src/app/cli/generate.zig:39-75`: the prompt is a JSON file of messages."""
    model_dir, path, opt = parse_generate_text(args, 128)
    from .text.chat import load_messages, with_system
    hooks = _text_hooks(model_dir)
    messages = with_system(load_messages(path), opt.system)
    print("Zinfer generate-chat")
    print(f"mode: {'think' if opt.think else 'no-think'}")
    print(f"messages_path: {path}")
    return _generate_text(model_dir, hooks.render_messages(messages, opt.think), opt)


def parse_chat(args: List[str]) -> Tuple[str, Options]:
    """``[model_dir] [max_new_tokens] [think|no-think] [flags]`` (`args.zig:189-226`): a first
    positional that is no number is the model folder."""
    pos, flags = _split_flags(args)
    model_dir, max_new = DEFAULT_MODEL_DIR, 128
    if pos and not pos[0].isdigit() and pos[0] not in ("think", "no-think"):
        model_dir, pos = pos[0], pos[1:]
    if pos and pos[0].isdigit():
        max_new, pos = int(pos[0]), pos[1:]
    think = False
    if pos:
        if pos[0] not in ("think", "no-think"):
            raise CliError(f"InvalidThinkingMode: {pos[0]}")
        think, pos = pos[0] == "think", pos[1:]
    if pos:
        raise CliError(f"InvalidCommand: unexpected {pos[0]!r}")
    opt = Options(max_new, think)
    opt.max_seqs = 1                    # one conversation: the pool holds one full context
    parse_flags(flags, opt, chat=True)
    opt.sampling.max_new_tokens = opt.max_new_tokens
    opt.sampling.ignore_eos = opt.ignore_eos
    return model_dir, opt


def _session_options(opt: Options) -> dict:
    """What a saved session says about how it was made (`chat.zig:120-183`)."""
    s = opt.sampling
    return {"thinking_mode": "think" if opt.think else "no-think",
            "max_new_tokens": opt.max_new_tokens, "seed": opt.seed, "backend": opt.dtype,
            "kv_cache": opt.kv_cache, "stream_output": opt.stream, "system_prompt": opt.system,
            "sampling": {"temperature": s.temperature, "top_p": s.top_p, "top_k": s.top_k,
                         "min_p": s.min_p, "presence_penalty": s.presence_penalty,
                         "frequency_penalty": s.frequency_penalty,
                         "repetition_penalty": s.repetition_penalty},
            "stop_sequences": list(opt.stop)}


def cmd_chat(args: List[str], lines=None) -> int:
    """`src/app/cli/chat.zig:226-312`: a conversation line by line on standard input.  Every
    turn renders the whole history and runs it as a new request; ``/exit`` ``/quit`` end it,
    ``/clear`` empties the history, ``/save <path>`` and ``/load <path>`` write and read a
    session; ``--load`` and ``--save`` do the same at the start and at the end."""
    from .text import Message, effective_stop_sequences
    from .text.chat import load_messages, with_system
    from .text.session import save_session
    model_dir, opt = parse_chat(args)
    hooks = _text_hooks(model_dir)
    tok = hooks.load_tokenizer(model_dir)
    llm = _llm(model_dir, opt)
    stops = effective_stop_sequences(llm.model.spec.default_stop_sequences, opt.stop)
    print("Zinfer chat")
    print(f"model_dir: {model_dir}")
    print(f"mode: {'think' if opt.think else 'no-think'}")
    print("commands: /exit /quit /clear /save <path> /load <path>")
    history = with_system(load_messages(opt.load_path) if opt.load_path else [], opt.system)
    for raw in (sys.stdin if lines is None else lines):
        sys.stdout.write("user> ")
        sys.stdout.flush()
        line = raw.rstrip("\r\n")
        if not line:
            continue
        if line in ("/exit", "/quit"):
            break
        if line == "/clear":
            history = with_system([], opt.system)
            print("history cleared")
            continue
        if line.startswith("/save ") or line.startswith("/load "):
            path = line[6:].strip(" ")
            if not path:
                raise CliError(f"MissingFlagValue: {line[:5]}")
            if line.startswith("/save "):
                save_session(path, history, model_dir, _session_options(opt))
                print(f"saved: {path}")
            else:
                history = with_system(load_messages(path), opt.system)
                print(f"loaded: {path}")
            continue
        history.append(Message("user", line))
        ids = tok.encode(hooks.render_messages(history, opt.think))
        sys.stdout.write("assistant> ")
        response = _respond(llm, tok, ids, opt, stops)
        if not opt.stream:
            sys.stdout.write(response)
        sys.stdout.write("\n")
        sys.stdout.flush()
        history.append(Message("assistant", hooks.assistant_history_content(response)))
    if opt.save_path:
        save_session(opt.save_path, history, model_dir, _session_options(opt))
    return 0


def _dir_and_one(args: List[str], what: str) -> Tuple[str, str]:
    pos, flags = _split_flags(args)
    if flags or len(pos) not in (1, 2):
        raise CliError(f"InvalidCommand: [model_dir] <{what}>")
    return (pos[0], pos[1]) if len(pos) == 2 else (DEFAULT_MODEL_DIR, pos[0])


def cmd_tokenize(args: List[str]) -> int:
    """`src/app/cli/tools/text.zig:5-36`."""
    model_dir, text = _dir_and_one(args, "text")
    ids = _text_hooks(model_dir).load_tokenizer(model_dir).encode(text)
    print("Zinfer tokenize")
    print(f"text: {text}")
    print("ids: [" + ", ".join(str(i) for i in ids) + "]")
    return 0


def cmd_decode_ids(args: List[str]) -> int:
    """`src/app/cli/tools/text.zig:38-75`."""
    model_dir, csv = _dir_and_one(args, "ids_csv")
    ids = parse_token_ids(csv)
    print("Zinfer decode-ids")
    print("ids: [" + ", ".join(str(i) for i in ids) + "]")
    print(f"text: {_text_hooks(model_dir).load_tokenizer(model_dir).decode(ids)}")
    return 0


def cmd_serve_batch(args: List[str]) -> int:
    """Runs the scheduler over a file of requests, one JSON object a line:
    ``{"id": ..., "prompt": [ids] | "text": "...", "max_new_tokens": n, "temperature": ...,
    "top_k": ..., "top_p": ..., "min_p": ..., "seed": ..., "ignore_eos": bool}``; unknown keys
    are an error, missing ones take the command's flags.  Writes one line per request,
    in the order they finish: ``{"id", "tokens", "finish_reason"[, "text"]}``.  The nearest
    thing in the reference is its continuous-batch benchmark (`src/app/cli/tools/bench/
    runtime.zig:226-310`), which admits the same prompt again and again."""
    import json
    from dataclasses import replace
    pos, flags = _split_flags(args)
    requests_path, out_path, rest = None, None, []
    i = 0
    while i < len(flags):
        if flags[i] in ("--requests", "--out"):
            if i + 1 >= len(flags):
                raise CliError(f"MissingFlagValue: {flags[i]}")
            if flags[i] == "--requests":
                requests_path = flags[i + 1]
            else:
                out_path = flags[i + 1]
            i += 2
        else:
            rest.append(flags[i])
            i += 1
    if requests_path is None or len(pos) > 1:
        raise CliError("InvalidCommand: serve-batch [model_dir] --requests <file.jsonl>")
    model_dir = pos[0] if pos else DEFAULT_MODEL_DIR
    opt = Options(64)
    opt.sampling = replace(opt.sampling, temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0)
    parse_flags(rest, opt)
    opt.sampling.max_new_tokens = opt.max_new_tokens
    opt.sampling.ignore_eos = opt.ignore_eos
    allowed = {"id", "prompt", "text", "max_new_tokens", "temperature", "top_k", "top_p", "min_p",
               "presence_penalty", "frequency_penalty", "repetition_penalty", "seed", "ignore_eos"}
    tok = None
    todo = []
    with open(requests_path, "r", encoding="utf-8") as f:
        for n, line in enumerate(f):
            if not line.strip():
                continue
            raw = json.loads(line)
            extra = set(raw) - allowed
            if extra or ("prompt" in raw) == ("text" in raw):
                raise CliError(f"InvalidRequest: line {n + 1}: one of prompt/text, no other keys "
                               f"than {sorted(allowed)} (found {sorted(extra)})")
            if "text" in raw:
                if tok is None:
                    tok = _text_hooks(model_dir).load_tokenizer(model_dir)
                ids = tok.encode(raw["text"])
            else:
                ids = [int(t) for t in raw["prompt"]]
            sp = replace(opt.sampling, **{k: raw[k] for k in raw if k not in ("id", "prompt", "text")})
            todo.append((raw.get("id", n), ids, sp))
    if not todo:
        raise CliError("InvalidRequest: no requests")
    llm = _llm(model_dir, opt)
    sched = llm.new_scheduler()
    for rid, ids, sp in todo:
        sched.add_request(ids, sp, request_id=rid)
    out = open(out_path, "w", encoding="utf-8") if out_path else sys.stdout
    t0 = time.perf_counter()
    n_tokens = 0
    try:
        while sched.has_work():
            for req in sched.step():
                rec = {"id": req.id, "tokens": req.generated, "finish_reason": req.finish_reason}
                if tok is not None:
                    rec["text"] = tok.decode(req.generated)
                n_tokens += len(req.generated)
                out.write(json.dumps(rec, ensure_ascii=False) + "\n")
                out.flush()
                sched.pop_finished(req.id)      # written out: the scheduler keeps nothing of it
    finally:
        if out_path:
            out.close()
    dt = time.perf_counter() - t0
    print(f"serve-batch: {len(todo)} requests, {n_tokens} generated tokens, {dt:.3f} s, "
          f"{n_tokens / dt:.1f} tok/s, {sched.n_steps} steps, {sched.n_preemptions} preemptions",
          file=sys.stderr)
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


def cmd_bench(args: List[str], mode: str, llm=None) -> int:
    """`src/app/cli/tools/bench/runtime.zig:12-99` (bench), `:135-224` (bench-batch),
    `:226-310` (bench-continuous): timers around prefill and decode, greedy, the same keys.
    ``llm``: an engine that is already loaded (its pool must hold the run)."""
    import torch
    from .engine import StepEntry
    from .sampling import SamplingParams
    n_extra = {"bench": 0, "bench-batch": 1, "bench-continuous": 2}[mode]
    model_dir, ids, extra, opt = _bench_common(args, n_extra)
    batch = extra[0] if extra else 1
    total = extra[1] if len(extra) > 1 else batch
    per_req = (len(ids) + opt.max_new_tokens + 63) // 64 * 64
    opt.max_seqs = max(batch, 1)
    if llm is None:
        llm = _llm(model_dir, opt, max_tokens=per_req * batch)
    params = SamplingParams(temperature=0.0, max_new_tokens=opt.max_new_tokens,
                            ignore_eos=opt.ignore_eos)
    print({"bench": "Zinfer benchmark", "bench-batch": "Zinfer batch benchmark",
           "bench-continuous": "Zinfer continuous batch benchmark"}[mode])
    print(f"model_dir: {model_dir}")
    print(f"backend: {opt.dtype}")
    print(f"kv_cache: {llm.engine.cache.groups[0].k.dtype if llm.engine.cache.groups else '-'}")
    print("q8_layout: none")                    # (the reference's quantised cache: not built)
    print("kernel_isa: gfx950")
    print("threads: 0")                         # (no host thread pool: the device's grid)
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
        classes = None
        if opt.classes and live and eng.use_graphs:
            # where a decode step's time goes: the step once per class of kernels
            classes = eng.class_times([StepEntry(n, [live[n]], [0]) for n in live])
        for n in names:                       # what the requests hold goes back
            eng.release(n)
        eng.cache.check()
        if batch > 1:
            print(f"batch_size: {batch}")
        print(f"prompt_tokens: {len(ids)}")
        print(f"decode_tokens: {decoded}")
        print("tokenize_ms: 0.000")             # (the prompt comes as token ids)
        print(f"prefill_ms: {(t1 - t0) * 1e3:.3f}")
        print(f"decode_ms: {(t2 - t1) * 1e3:.3f}")
        print(f"prefill_tok_s: {len(ids) * batch / (t1 - t0):.3f}")
        print(f"decode_tok_s: {decoded / max(t2 - t1, 1e-12):.3f}")
        if classes is not None:
            for name, t in classes.items():
                print(f"decode_step_{name}_ms: {t * 1e3:.4f}")
    wb = _weights_bytes(llm)
    kb = llm.engine.cache.kv_bytes()
    print(f"weights_bytes: {wb}")
    print(f"weights_mib: {wb / 1048576:.3f}")
    print(f"kv_cache_bytes: {kb}")
    print(f"kv_cache_mib: {kb / 1048576:.3f}")
    return 0


SUITE_PROFILES = (("short", 16), ("medium", 32), ("long", 64))
SUITE_DECODE_TOKENS = 2


def cmd_bench_suite(args: List[str]) -> int:
    """`src/app/cli/tools/bench/runtime.zig:101-133`: the single-request benchmark over a
    short, a medium and a long prompt with two decoded tokens each, on one loaded engine.
    The reference's profiles are texts through its tokenizer and run once per quantised
    backend; here they are prompt lengths in tokens (ids made up), since a folder may bring
    no tokenizer, and there is the one backend."""
    pos, flags = _split_flags(args)
    if len(pos) > 1:
        raise CliError("InvalidCommand: bench-suite [model_dir]")
    model_dir = pos[0] if pos else DEFAULT_MODEL_DIR
    opt = Options(SUITE_DECODE_TOKENS)
    parse_flags(flags, opt)
    opt.max_seqs = 1
    longest = max(n for _, n in SUITE_PROFILES)
    llm = _llm(model_dir, opt, max_tokens=(longest + SUITE_DECODE_TOKENS + 63) // 64 * 64)
    vocab = llm.model.spec.vocab_size
    print("Zinfer perf-gate suite")
    print(f"model_dir: {model_dir}")
    print("threads: 0")
    print(f"kv_cache: {opt.kv_cache}")
    print("q8_layout: none")
    print("kernel_isa: gfx950")
    for name, n in SUITE_PROFILES:
        print(f"\n[suite] profile={name} backend={opt.dtype} decode_tokens={SUITE_DECODE_TOKENS}")
        csv = ",".join(str((7 + 13 * i) % vocab) for i in range(n))
        cmd_bench([model_dir, csv, str(SUITE_DECODE_TOKENS)] + flags + ["--ignore-eos"], "bench",
                  llm=llm)
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
    device = "cuda:0" if torch.cuda.is_available() else None   # the same values either way
    write_model_dir(pos[1], cfg, opt.seed, dtype, device=device)
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
        if cmd == "probe-linear":
            return cmd_probe_linear(args)
        if cmd == "probe-block":
            return cmd_probe_block(args)
        if cmd == "probe-model":
            return cmd_probe_model(args)
        if cmd == "generate-token-ids":
            return cmd_generate_token_ids(args)
        if cmd == "generate":
            return cmd_generate(args)
        if cmd == "generate-chat":
            return cmd_generate_chat(args)
        if cmd == "chat":
            return cmd_chat(args)
        if cmd == "tokenize":
            return cmd_tokenize(args)
        if cmd == "decode-ids":
            return cmd_decode_ids(args)
        if cmd == "serve-batch":
            return cmd_serve_batch(args)
        if cmd == "replay":
            from .engine.replay import main as replay_main
            return replay_main(args)
        if cmd in ("bench", "bench-batch", "bench-continuous"):
            return cmd_bench(args, cmd)
        if cmd == "bench-suite":
            return cmd_bench_suite(args)
        if cmd == "random-model":
            return cmd_random_model(args)
        if cmd == "bench-ops":
            from .bench_ops import main as bench_ops_main
            return bench_ops_main(args)
        if cmd == "quantize":
            print("zinfer: 'quantize' belongs to what this engine does not build (quantised "
                  "weights)", file=sys.stderr)
            return 2
        print(f"zinfer: unknown command {cmd!r}\n", file=sys.stderr)     # `cli.zig:286`
        sys.stderr.write(USAGE)
        return 2
    except (CliError, ZinferError, FileNotFoundError, ValueError) as e:
        print(f"zinfer: {type(e).__name__}: {e}", file=sys.stderr)
        return 1


if __name__ == "__main__":
    sys.exit(main())
