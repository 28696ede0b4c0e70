"""The scheduler over the real engine on the GPU: the stated tiny workload with seeded sampling,
preemption and recomputation under a pool that is too small, a model folder in several files,
and a tied head that the kernels read from a copy in their own order."""
import json
import os

import numpy as np
import pytest
import torch

import plain
import tiny
from gpu_util import DEV

pytestmark = pytest.mark.gpu

GOLDEN, M64 = 0x9E3779B97F4A7C15, (1 << 64) - 1


def _plain_sampled(cfg, w, prompt, params: dict, seed: int, index: int, n: int):
    """What the plain model and the plain sampler generate for the request that was added as
    number ``index``: the scheduler gives it the stream seeded with seed ^ (index * golden)."""
    rng = plain.PlainRng((seed ^ (index * GOLDEN)) & M64)
    toks = list(prompt)
    for _ in range(n):
        logits = plain.model_forward_batched(cfg, w, toks)[-1].float().numpy()
        toks.append(plain.sample_token(logits, toks, params, rng))
    return toks[len(prompt):]


def test_the_stated_tiny_workload_with_seeded_sampling(tmp_path):
    """Tiny B in 32-bit, pages of 8: five requests with prompts of 1, 9, 33, 64 and 130 tokens,
    prompts in portions of 24 beside the decode tokens of the others, 20 tokens each at
    temperature 0.8 / top-k 50 from a seeded stream: the tokens of the plain model under the
    plain sampler."""
    from zinfer_amd.entrypoints import LLM
    from zinfer_amd.sampling import SamplingParams
    path = tiny.model_dir_of("B", str(tmp_path), torch.float32)
    cfg, w = tiny.CONFIGS["B"], tiny.weights_of("B", torch.float32)
    prompts = [tiny.random_tokens(n, cfg["vocab_size"], 300 + n) for n in (1, 9, 33, 64, 130)]
    llm = LLM(path, dtype="float32", device=DEV, page_size=8, max_tokens=512,
              max_step_tokens=32, chunk_size=24)
    sp = SamplingParams(temperature=0.8, top_k=50, seed=17, max_new_tokens=20, ignore_eos=True)
    sched = llm.new_scheduler()
    ids = [sched.add_request(p, sp) for p in prompts]
    mixed_steps = 0
    engine_step = llm.engine.step

    def watched(entries, end=()):
        nonlocal mixed_steps
        sizes = [len(e.tokens) for e in entries]
        assert sum(sizes) <= 32 and max(sizes) <= 24
        if max(sizes) > 1 and any(n == 1 and llm.engine.has_request(e.request_id)
                                  for n, e in zip(sizes, entries)):
            mixed_steps += 1
        return engine_step(entries, end)
    llm.engine.step = watched
    sched.run()
    assert mixed_steps >= 3, "portions of prompts must have run beside decode tokens"
    assert not llm.engine.cache.requests
    llm.engine.cache.check()
    params = dict(temperature=0.8, top_k=50)
    for i, (rid, prompt) in enumerate(zip(ids, prompts)):
        got = sched.finished[rid].generated
        assert got == _plain_sampled(cfg, w, prompt, params, 17, i, 20), f"request {i}"


@pytest.mark.parametrize("sampling", ["greedy", "seeded"])
def test_preemption_recomputes_to_the_same_tokens(sampling, tmp_path):
    """A pool too small for all requests: at least one running request is preempted (its pages
    freed, its tokens and random stream kept) and later recomputed from its prompt and what it
    had generated.  Every request still gets the tokens of the plain implementation."""
    from zinfer_amd.entrypoints import LLM
    from zinfer_amd.sampling import SamplingParams
    path = tiny.model_dir_of("B", str(tmp_path), torch.float32)
    cfg, w = tiny.CONFIGS["B"], tiny.weights_of("B", torch.float32)
    prompts = [tiny.random_tokens(n, cfg["vocab_size"], 400 + n) for n in (33, 64, 40, 17)]
    # 20 new tokens each: 53 + 84 + 60 + 37 tokens = 7 + 11 + 8 + 5 = 31 pages of 8; 22 are there
    llm = LLM(path, dtype="float32", device=DEV, page_size=8, num_pages=22,
              max_step_tokens=48, chunk_size=24, multi_step=4)
    if sampling == "greedy":
        sp = SamplingParams(temperature=0.0, max_new_tokens=20, ignore_eos=True)
    else:
        sp = SamplingParams(temperature=0.9, top_k=40, top_p=0.95, seed=5, max_new_tokens=20,
                            ignore_eos=True)
    sched = llm.new_scheduler()
    ids = [sched.add_request(p, sp) for p in prompts]
    while sched.has_work():
        sched.step()
        llm.engine.cache.check()
    assert sched.n_preemptions >= 1
    assert sum(r.preemptions for r in sched.finished.values()) == sched.n_preemptions
    assert not llm.engine.cache.requests and llm.engine.cache.num_free_pages() == [22]
    for i, (rid, prompt) in enumerate(zip(ids, prompts)):
        got = sched.finished[rid].generated
        assert sched.finished[rid].finish_reason == "length"
        if sampling == "greedy":
            assert got == plain.greedy_generate(cfg, w, prompt, 20), f"request {i}"
        else:
            want = _plain_sampled(cfg, w, prompt, dict(temperature=0.9, top_k=40, top_p=0.95),
                                  5, i, 20)
            assert got == want, f"request {i}"


def test_a_folder_in_several_files_gives_the_same_logits(tmp_path):
    from test_weights import _write_sharded
    from zinfer_amd.engine import StepEntry
    from zinfer_amd.engine.replay import make_engine
    from zinfer_amd.weights import SafetensorsFile
    single = tiny.model_dir_of("B", str(tmp_path), torch.bfloat16)
    with SafetensorsFile(os.path.join(single, "model.safetensors")) as f:
        tensors = {n: f.tensor(n) for n in f.names()}
    sharded = _write_sharded(str(tmp_path / "sharded"), tiny.TINY_B, tensors, 3)
    toks = tiny.random_tokens(40, tiny.TINY_B["vocab_size"], 8)
    outs = []
    for path in (single, sharded):
        eng = make_engine(path, "bfloat16", 64, DEV, page_size=8)
        outs.append(eng.step([StepEntry("r", toks, [0, 20, 39])], end=["r"]).clone())
    assert torch.equal(outs[0], outs[1])


def test_a_tied_head_reads_a_copy_in_the_kernels_order(tmp_path):
    """Tied embeddings with a vocabulary that pre-tiles (a multiple of 64): the embedding stays
    in rows for the gather and the head's product reads a second, pre-tiled copy; prompt
    portions and decode steps give the plain model's logits."""
    from zinfer_amd.config import Qwen3Config
    from zinfer_amd.engine import StepEntry
    from zinfer_amd.engine.replay import make_engine
    from zinfer_amd.models.build import declare_tensors
    from zinfer_amd.weights import draw_tensors, write_model_dir
    raw = dict(tiny.TINY_D, vocab_size=1216)
    cfg = Qwen3Config.from_dict(raw)
    path = write_model_dir(str(tmp_path / "tied"), cfg, 77, torch.bfloat16)
    w = draw_tensors(declare_tensors(cfg.model_spec()), 77, torch.bfloat16, tied=True)
    eng = make_engine(path, "bfloat16", 256, DEV)
    head = eng.model.head
    assert head.tiled and head.weight.data_ptr() != eng.model.embedding.data_ptr()
    toks = tiny.random_tokens(90, raw["vocab_size"], 12)
    ref = plain.model_forward_batched(raw, w, toks).numpy()
    got = [eng.step([StepEntry("r", toks[:70], list(range(70)))]).cpu().numpy()]
    for t in range(70, 90):
        got.append(eng.step([StepEntry("r", toks[t:t + 1], [0])]).cpu().numpy())
    got = np.concatenate(got)
    err = np.abs(got - ref).max(axis=1) / np.abs(ref).max()
    assert err.max() <= 2e-2, f"first wrong position {int(np.argmax(err > 2e-2))}: {err.max():.3g}"


@pytest.mark.parametrize("dtype,tolerance", [("float32", 2e-5), ("bfloat16", 2e-2)])
def test_thirty_six_layers_against_the_plain_model(dtype, tolerance, tmp_path):
    """The depth of the served models at tiny widths: a whole prompt, then decode steps, with
    the tolerances of the shallow configurations (rounding must not pile up layer by layer)."""
    from zinfer_amd.config import Qwen3Config
    from zinfer_amd.engine import StepEntry
    from zinfer_amd.engine.replay import make_engine
    from zinfer_amd.models.build import declare_tensors
    from zinfer_amd.weights import draw_tensors, write_model_dir
    raw = dict(tiny.TINY_D, num_hidden_layers=36, hidden_size=256, num_attention_heads=4,
               num_key_value_heads=2, head_dim=64, intermediate_size=768, vocab_size=1024,
               tie_word_embeddings=False)
    cfg = Qwen3Config.from_dict(raw)
    store = torch.float32 if dtype == "float32" else torch.bfloat16
    path = write_model_dir(str(tmp_path / "deep"), cfg, 5, store, device=DEV)
    w = {k: v.cpu() for k, v in draw_tensors(declare_tensors(cfg.model_spec()), 5, store,
                                             device=DEV).items()}
    toks = tiny.random_tokens(96, raw["vocab_size"], 3)
    ref = plain.model_forward_batched(raw, w, toks).numpy()
    eng = make_engine(path, dtype, 128, DEV)
    got = [eng.step([StepEntry("r", toks[:80], list(range(80)))]).cpu().numpy()]
    for t in range(80, 96):
        got.append(eng.step([StepEntry("r", toks[t:t + 1], [0])]).cpu().numpy())
    got = np.concatenate(got)
    err = np.abs(got - ref).max(axis=1) / np.abs(ref).max()
    assert err.max() <= tolerance, f"position {int(err.argmax())}: {err.max():.3g}"


def test_bench_commands_print_the_reference_keys_and_class_times(tmp_path, capsys):
    """`zinfer bench` and `bench-batch` over a tiny model: the reference's report keys
    (`src/app/cli/tools/bench/runtime.zig:81-98`), with --classes a decode step's time per
    class of kernels, and nothing held afterwards (the command checks its cache itself)."""
    from zinfer_amd import cli
    path = tiny.model_dir_of("D", str(tmp_path), torch.bfloat16)
    for cmd, extra, batch in (("bench", [], 1), ("bench-batch", ["3"], 3)):
        rc = cli.main([cmd, path, "5,6,7,8,9"] + extra + ["6", "--ignore-eos", "--classes",
                                                          "--max-tokens", "512"])
        out = capsys.readouterr().out
        assert rc == 0, out
        keys = {line.split(":")[0] for line in out.splitlines() if ":" in line}
        for key in ("model_dir", "backend", "kv_cache", "q8_layout", "kernel_isa", "threads",
                    "prompt_tokens", "decode_tokens", "tokenize_ms", "prefill_ms", "decode_ms",
                    "prefill_tok_s", "decode_tok_s", "weights_bytes", "weights_mib",
                    "kv_cache_bytes", "kv_cache_mib"):
            assert key in keys, (cmd, key)
        assert f"decode_tokens: {6 * batch}" in out
        times = {k: float(line.split(":")[1]) for line in out.splitlines()
                 for k in [line.split(":")[0]] if k.startswith("decode_step_")}
        assert set(times) == {f"decode_step_{c}_ms" for c in
                              ("products", "attention", "norm_rope_write", "head_sampling",
                               "other", "step")}
        assert times["decode_step_products_ms"] > 0 and times["decode_step_attention_ms"] > 0
        # (each class is a graph replay of its own: on a model this small the replays' own cost
        # can outweigh the kernels, so the classes' sum is only bounded from below)
        parts = sum(v for k, v in times.items() if k != "decode_step_step_ms")
        assert parts >= 0.5 * times["decode_step_step_ms"]
    # the suite: the same report for three prompt lengths on one loaded engine
    # (`src/app/cli/tools/bench/runtime.zig:101-133`)
    assert cli.main(["bench-suite", path]) == 0
    out = capsys.readouterr().out
    assert out.startswith(f"Zinfer perf-gate suite\nmodel_dir: {path}\n")
    assert [l.split()[1] for l in out.splitlines() if l.startswith("[suite] ")] == \
        ["profile=short", "profile=medium", "profile=long"]
    assert out.count("decode_tokens: 2\n") == 3
    assert [int(l.split(":")[1]) for l in out.splitlines() if l.startswith("prompt_tokens:")] == \
        [n for _, n in cli.SUITE_PROFILES]
