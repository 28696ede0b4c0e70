"""Each part alone on the GPU against the plain functions, the entry point's greedy
generation, and (c)'s generality: parts defined here, in the test, are registered, built
from a model folder and stepped without a change to the framework's files: a mixer with
state of its own, and a model whose layers differ (full and windowed attention), run in an
order that names layers twice and lets a run read another run's cache."""
import json
import os
from dataclasses import dataclass
from typing import Optional

import numpy as np
import pytest
import torch

import plain
import tiny
import traces
from gpu_util import DEV, rel_err

pytestmark = pytest.mark.gpu
F64 = torch.float64


# ----------------------------------------------------------------------------- harness
class _StubModel:
    """Just enough of a model for an Engine to hand out pages and build step contexts."""

    def __init__(self, needs, dtype):
        from zinfer_amd.config.specs import ModelSpec, ScheduleEntry
        from zinfer_amd.parts import BuildContext
        self.ctx = BuildContext(dtype, torch.device(DEV))
        self._needs = needs
        self.spec = ModelSpec(vocab_size=100, hidden_size=8, max_positions=4096, layers=(),
                              schedule=tuple(ScheduleEntry(0) for _ in needs), final_norm=None,
                              tie_word_embeddings=True)

    def cache_needs(self):
        return self._needs

    parts = ()      # the parts under test: they are asked for hints and shown their caches

    def hint_providers(self):
        return [q for p in self.parts for q in p.hint_providers()]

    def accept_caches(self, caches):
        for p, c in zip(self.parts, caches):
            if hasattr(p, "accept_cache"):
                p.accept_cache(c)


class _context:
    """Step context for {request: n_tokens}: pages are reserved on entry, lengths are
    committed (and pages a window has passed given back) on exit, as Engine.step does."""

    def __init__(self, eng, cuts):
        self.eng, self.cuts = eng, cuts

    def __enter__(self):
        from zinfer_amd.engine import StepEntry
        entries = []
        for rid, n in self.cuts.items():
            if not self.eng.cache.has_request(rid):
                self.eng.cache.add_request(rid)
            self.eng.cache.reserve(rid, self.eng.cache.length(rid) + n)
            entries.append(StepEntry(rid, [0] * n, []))
        return self.eng._build_context(entries)

    def __exit__(self, *exc):
        for rid, n in self.cuts.items():
            self.eng.cache.commit(rid, self.eng.cache.length(rid) + n)


def _rand(shape, seed, scale=1.0, dtype=torch.float32):
    return (torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale).to(dtype)


# ----------------------------------------------------------------------------- parts alone
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rms_norm_part(dtype):
    from zinfer_amd.config.specs import RmsNormSpec
    from zinfer_amd.parts import BuildContext, build_part
    part = build_part("norm", RmsNormSpec(80, 3e-6), BuildContext(dtype, torch.device(DEV)), "n.")
    assert list(part.declare()) == ["n.weight"] and part.declare()["n.weight"].shape == (80,)
    g = 1 + 0.1 * _rand((80,), 1)
    part.bind({"n.weight": g.to(dtype)})
    x = _rand((7, 80), 2, 3.0)
    out = torch.empty((7, 80), dtype=dtype, device=DEV)
    part.forward(x.to(DEV), out)
    want = plain.rms_norm(x, g.to(dtype), 3e-6)
    assert rel_err(out, want) <= (2e-5 if dtype == torch.float32 else 2 ** -8)


def test_rotary_tables_follow_the_plain_angles():
    from zinfer_amd.parts.position import rotary_tables
    for hd, theta in ((16, 1e4), (128, 1e6), (48, 5e4)):
        cos, sin = rotary_tables(hd, theta, 300)
        for p in (0, 1, 2, 77, 299):
            c, s = plain.rope_cos_sin(p, hd, theta)
            assert torch.allclose(cos[p].double(), c, atol=1e-7)
            assert torch.allclose(sin[p].double(), s, atol=1e-7)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu_part(dtype):
    from zinfer_amd.config.specs import SwiGluSpec
    from zinfer_amd.engine import Engine
    from zinfer_amd.parts import build_part
    stub = _StubModel([], dtype)
    eng = Engine(stub, num_pages=4, max_requests=2)
    part = build_part("feed_forward", SwiGluSpec(96, 200), stub.ctx, "mlp.")
    w = {"mlp.gate_proj.weight": _rand((200, 96), 3, 0.1, dtype),
         "mlp.up_proj.weight": _rand((200, 96), 4, 0.1, dtype),
         "mlp.down_proj.weight": _rand((96, 200), 5, 0.1, dtype)}
    part.bind(w)
    h = _rand((5, 96), 6, 1.0, dtype)
    residual = _rand((5, 96), 7)
    res = residual.clone().to(DEV)
    with _context(eng, {"a": 5}) as ctx:
        part.forward(h.to(DEV), res, ctx)
    want = residual.double() + plain.linear(
        plain.swiglu(plain.linear(h, w["mlp.gate_proj.weight"]),
                     plain.linear(h, w["mlp.up_proj.weight"])), w["mlp.down_proj.weight"])
    assert rel_err(res, want) <= (2e-5 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("qk_norm,window,rope", [(True, None, True), (False, 9, True),
                                                 (True, None, False)])
def test_attention_part(dtype, qk_norm, window, rope):
    """The attention mixer alone over two steps (a portion, then single tokens) against the
    plain single-query attention with the same projections."""
    from zinfer_amd.config.specs import GqaAttentionSpec, NoPositionSpec, RotaryHalfSplitSpec
    from zinfer_amd.engine import Engine
    from zinfer_amd.parts import build_part
    H, nH, nKV, hd, eps, theta = 96, 6, 2, 32, 1e-5, 1e4
    pos_spec = RotaryHalfSplitSpec(hd, theta, 256) if rope else NoPositionSpec()
    spec = GqaAttentionSpec(H, nH, nKV, hd, eps if qk_norm else None, pos_spec, window)
    stub = _StubModel([None], dtype)
    part = build_part("mixer", spec, stub.ctx, "a.")
    stub._needs = [part.cache_need()]
    stub.parts = (part,)
    eng = Engine(stub, page_size=16, num_pages=8, max_requests=2, poison_freed=True)
    w = {"a.q_proj.weight": _rand((nH * hd, H), 1, 0.1, dtype),
         "a.k_proj.weight": _rand((nKV * hd, H), 2, 0.1, dtype),
         "a.v_proj.weight": _rand((nKV * hd, H), 3, 0.1, dtype),
         "a.o_proj.weight": _rand((H, nH * hd), 4, 0.1, dtype)}
    if qk_norm:
        w["a.q_norm.weight"] = (1 + 0.1 * _rand((hd,), 5)).to(dtype)
        w["a.k_norm.weight"] = (1 + 0.1 * _rand((hd,), 6)).to(dtype)
    assert set(part.declare()) == set(w)
    part.bind(w)
    T = 40
    h = _rand((T, H), 7, 1.0, dtype)
    # plain: token after token
    ks, vs, want = [], [], []
    for p in range(T):
        q = plain.linear(h[p], w["a.q_proj.weight"])
        k = plain.linear(h[p], w["a.k_proj.weight"])
        v = plain.linear(h[p], w["a.v_proj.weight"])
        if qk_norm:
            q = plain.per_head_rms_norm(q, nH, hd, w["a.q_norm.weight"], eps)
            k = plain.per_head_rms_norm(k, nKV, hd, w["a.k_norm.weight"], eps)
        if rope:
            q, k = plain.rope_heads(q, nH, hd, p, theta), plain.rope_heads(k, nKV, hd, p, theta)
        ks.append(k.reshape(nKV, hd)); vs.append(v.reshape(nKV, hd))
        o = plain.attention_single_query(q, torch.stack(ks), torch.stack(vs), nH, nKV, hd, window)
        want.append(plain.linear(o, w["a.o_proj.weight"]))
    want = torch.stack(want)
    got = torch.zeros((T, H), device=DEV)
    done = 0
    for n in (23, 1, 1, 13, 2):
        with _context(eng, {"r": n}) as ctx:
            part.forward(h[done:done + n].to(DEV).contiguous(), got[done:done + n], ctx,
                         eng.views[0])
        done += n
    assert rel_err(got, want) <= (2e-5 if dtype == torch.float32 else 1.5e-2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(dtype, tmp_path):
    from zinfer_amd.entrypoints import LLM
    from zinfer_amd.sampling import SamplingParams
    name = "D" if dtype == "bfloat16" else "B"
    store = torch.float32 if dtype == "float32" else torch.bfloat16
    path = tiny.model_dir_of(name, str(tmp_path), store)
    cfg, w = tiny.CONFIGS[name], tiny.weights_of(name, store)
    prompts = [tiny.random_tokens(n, cfg["vocab_size"], 40 + n) for n in (1, 9, 33, 64, 130)]
    llm = LLM(path, dtype=dtype, device=DEV, page_size=tiny.PAGE_SIZE[name], max_tokens=448,
              max_step_tokens=48, chunk_size=24)
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=12,
                                                ignore_eos=True))
    assert not llm.engine.cache.requests
    for p, got in zip(prompts, outs):
        if dtype == "float32":
            assert got == plain.greedy_generate(cfg, w, p, 12)
        else:       # a near-tie may flip in bfloat16: every token must be a near-best one
            toks = list(p)
            for g in got:
                logits = plain.model_forward_batched(cfg, w, toks)[-1]
                assert logits[g] >= logits.max() - 0.04 * logits.abs().max()
                toks.append(g)
    # seeded sampling: the same seed gives the same tokens, alone or in a batch
    sp = SamplingParams(temperature=0.8, top_k=50, seed=3, max_new_tokens=10, ignore_eos=True)
    alone = llm.generate([prompts[2]], sp)[0]
    again = llm.generate([prompts[2]], sp)[0]
    assert alone == again and len(alone) == 10
    # the device sampler (top_k 50) and the host sampler (whole vocabulary: top_k 0 with the
    # same cut made by top_k) see the same stream: with penalties and top-p as well
    sp2 = SamplingParams(temperature=0.7, top_k=20, top_p=0.8, repetition_penalty=1.1, seed=11,
                         max_new_tokens=8, ignore_eos=True)
    batch = llm.generate([prompts[1], prompts[3]], sp2)
    assert [len(b) for b in batch] == [8, 8]
    if dtype == "float32":
        from zinfer_amd.sampling import Xoshiro256pp, sample_token
        toks, rng = list(prompts[1]), Xoshiro256pp(11)      # request index 0: seed ^ 0
        for g in batch[0]:
            logits = plain.model_forward_batched(cfg, w, toks)[-1].float().numpy()
            assert g == sample_token(logits, toks, sp2, rng)
            toks.append(g)
    # without penalties several decode steps run in a row on the device: the same tokens as
    # with the host between all steps, also when a request stops in the middle of a run
    sp3 = SamplingParams(temperature=0.9, top_k=30, top_p=0.9, seed=21, max_new_tokens=21,
                         ignore_eos=True)
    before = llm.engine.steps_run
    runs = llm.generate(prompts[1:4], sp3)
    assert [len(r) for r in runs] == [21, 21, 21]
    single = LLM(path, dtype=dtype, device=DEV, page_size=tiny.PAGE_SIZE[name], max_tokens=448,
                 max_step_tokens=48, chunk_size=24, multi_step=1)
    assert single.generate(prompts[1:4], sp3) == runs
    assert llm.engine.steps_run - before == single.engine.steps_run
    stop = runs[0][12]
    first = runs[0].index(stop)
    for params in (SamplingParams(temperature=0.9, top_k=30, top_p=0.9, seed=21,
                                  max_new_tokens=21, stop_token_ids=(stop,)),
                   SamplingParams(temperature=0.0, max_new_tokens=19, stop_token_ids=(stop,))):
        a, b = llm.generate(prompts[1:4], params), single.generate(prompts[1:4], params)
        assert a == b
        assert not llm.engine.cache.requests and not single.engine.cache.requests
    assert llm.generate(prompts[1:4], SamplingParams(
        temperature=0.9, top_k=30, top_p=0.9, seed=21, max_new_tokens=21,
        stop_token_ids=(stop,)))[0] == runs[0][:first]
    if dtype == "float32":
        toks, rng = list(prompts[1]), Xoshiro256pp(21)
        for g in runs[0]:
            logits = plain.model_forward_batched(cfg, w, toks)[-1].float().numpy()
            assert g == sample_token(logits, toks, sp3, rng)
            toks.append(g)


# ----------------------------------------------------------------------------- toy parts
@dataclass(frozen=True)
class ToyStateSpec:
    """A mixer with state of its own: s <- decay * s + W_in h_t ; out_t = W_out s."""
    hidden_size: int
    state_size: int
    decay: float


def _register_toy_state():
    from zinfer_amd.parts import Mixer, StateNeed, TensorDecl, register_part

    class ToyStateMixer(Mixer):
        def declare(self):
            s = self.spec
            return {self.prefix + "in.weight": TensorDecl((s.state_size, s.hidden_size)),
                    self.prefix + "out.weight": TensorDecl((s.hidden_size, s.state_size))}

        def bind(self, tensors):
            self.w_in = tensors[self.prefix + "in.weight"].float().to(self.ctx.device)
            self.w_out = tensors[self.prefix + "out.weight"].float().to(self.ctx.device)

        def cache_need(self):
            return StateNeed((self.spec.state_size,), torch.float32)

        def forward(self, h, residual, step, cache):
            u = h.float() @ self.w_in.T                      # [T, S]
            start = 0
            for n, slot in zip(step.q_lens, step.slots):     # each request's tokens in order
                s = cache.state[slot]
                for t in range(start, start + n):
                    s = self.spec.decay * s + u[t]
                    residual[t] += s @ self.w_out.T
                cache.state[slot] = s
                start += n

    register_part("mixer", ToyStateSpec, ToyStateMixer)


@dataclass(frozen=True)
class ToyConfig:
    hidden_size: int
    state_size: int
    decay: float
    window: int
    vocab_size: int
    kind: str                  # "state" or "mixed"
    model_type: str = "toy"

    @classmethod
    def from_dict(cls, raw):
        return cls(**{k: raw[k] for k in ("hidden_size", "state_size", "decay", "window",
                                          "vocab_size", "kind")})

    def to_dict(self):
        return dict(architectures=["ToyForCausalLM"], model_type="toy",
                    hidden_size=self.hidden_size, state_size=self.state_size, decay=self.decay,
                    window=self.window, vocab_size=self.vocab_size, kind=self.kind)

    def model_spec(self):
        from zinfer_amd.config.specs import (GqaAttentionSpec, ModelSpec, PreNormBlockSpec,
                                             RmsNormSpec, RotaryHalfSplitSpec, ScheduleEntry,
                                             SwiGluSpec)
        H = self.hidden_size
        norm = RmsNormSpec(H, 1e-5)
        ff = SwiGluSpec(H, 2 * H)
        rope = RotaryHalfSplitSpec(32, 1e4, 512)
        full = GqaAttentionSpec(H, 4, 2, 32, 1e-5, rope, None)
        win = GqaAttentionSpec(H, 4, 2, 32, None, rope, self.window)
        state = ToyStateSpec(H, self.state_size, self.decay)
        blk = lambda m: PreNormBlockSpec(mixer=m, feed_forward=ff, mixer_norm=norm, ff_norm=norm)
        if self.kind == "state":
            layers = (blk(state), blk(full), blk(state))
            schedule = (ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(2))
        else:   # layers differ; 0 and 1 run twice; the last run reads the cache of run 1
            layers = (blk(full), blk(win))
            schedule = (ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0),
                        ScheduleEntry(1, cache_of=1))
        # the "state" kind also scales its embedding rows and scales and caps its logits
        extra = dict(embedding_multiplier=3.0, logit_scale=40.0, logit_softcap=2.5) \
            if self.kind == "state" else {}
        return ModelSpec(vocab_size=self.vocab_size, hidden_size=H, max_positions=512,
                         layers=layers, schedule=schedule, final_norm=norm,
                         tie_word_embeddings=True, **extra)


class ToyTokenizer:
    """One id per byte; the text front end of the toy architecture."""

    def encode(self, text):
        return list(text.encode("utf-8"))

    def decode(self, ids):
        return bytes(int(i) % 256 for i in ids).decode("latin-1")


def _toy_text_hooks():
    from zinfer_amd.config import TextHooks
    return TextHooks(
        load_tokenizer=lambda model_dir: ToyTokenizer(),
        render_messages=lambda messages, thinking: "".join(f"[{m.role}:{m.content}]" for m in messages),
        render_single_user=lambda text, thinking, system=None:
            (f"[system:{system}]" if system else "") + f"[user:{text}]" + ("?" if thinking else "!"),
        assistant_history_content=lambda content: content)


def _toy_plain(cfg: ToyConfig, w, toks):
    """Whole sequence, token after token, from the plain part functions."""
    spec = cfg.model_spec()
    H = cfg.hidden_size
    caches = [([], []) for _ in spec.schedule]
    states = [torch.zeros(cfg.state_size, dtype=F64) for _ in spec.schedule]
    rows = []
    for p, tok in enumerate(toks):
        x = w["model.embed_tokens.weight"][tok].to(F64) * spec.embedding_multiplier
        for pos, e in enumerate(spec.schedule):
            pre = f"model.layers.{e.layer}."
            blk = spec.layers[e.layer]
            n = plain.rms_norm(x, w[pre + "input_layernorm.weight"], 1e-5)
            m = blk.mixer
            if isinstance(m, ToyStateSpec):
                states[pos] = m.decay * states[pos] + plain.linear(n, w[pre + "self_attn.in.weight"])
                x = x + plain.linear(states[pos], w[pre + "self_attn.out.weight"])
            else:
                q = plain.linear(n, w[pre + "self_attn.q_proj.weight"])
                k = plain.linear(n, w[pre + "self_attn.k_proj.weight"])
                v = plain.linear(n, w[pre + "self_attn.v_proj.weight"])
                if m.qk_norm_eps is not None:
                    q = plain.per_head_rms_norm(q, 4, 32, w[pre + "self_attn.q_norm.weight"], 1e-5)
                    k = plain.per_head_rms_norm(k, 2, 32, w[pre + "self_attn.k_norm.weight"], 1e-5)
                q, k = plain.rope_heads(q, 4, 32, p, 1e4), plain.rope_heads(k, 2, 32, p, 1e4)
                src = pos if e.cache_of is None else e.cache_of
                if e.cache_of is None:
                    caches[pos][0].append(k.reshape(2, 32)); caches[pos][1].append(v.reshape(2, 32))
                o = plain.attention_single_query(q, torch.stack(caches[src][0]),
                                                 torch.stack(caches[src][1]), 4, 2, 32, m.window)
                x = x + plain.linear(o, w[pre + "self_attn.o_proj.weight"])
            mm = plain.rms_norm(x, w[pre + "post_attention_layernorm.weight"], 1e-5)
            x = x + plain.linear(plain.swiglu(plain.linear(mm, w[pre + "mlp.gate_proj.weight"]),
                                              plain.linear(mm, w[pre + "mlp.up_proj.weight"])),
                                 w[pre + "mlp.down_proj.weight"])
        logits = plain.linear(plain.rms_norm(x, w["model.norm.weight"], 1e-5),
                              w["model.embed_tokens.weight"]) * spec.logit_scale
        if spec.logit_softcap is not None:
            logits = spec.logit_softcap * torch.tanh(logits / spec.logit_softcap)
        rows.append(logits)
    return torch.stack(rows).numpy()


def _toy_text_through_the_command_line(path, cfg):
    """Text in and out with the toy architecture's own tokenizer and template, which the
    command line takes from the registry entry of the folder's config.json."""
    import contextlib
    import io
    from zinfer_amd import cli
    from zinfer_amd.entrypoints import LLM, SamplingParams
    prompt = "[system:be brief][user:hi]!"
    ids = list(prompt.encode())
    llm = LLM(path, dtype="float32", device=DEV, page_size=16, max_tokens=128)
    want = llm.generate([ids], SamplingParams(temperature=0.0, max_new_tokens=5, ignore_eos=True))[0]
    out = io.StringIO()
    with contextlib.redirect_stdout(out):
        rc = cli.main(["generate", path, "hi", "5", "no-think", "--system", "be brief",
                       "--dtype", "float32", "--temperature", "0", "--repetition-penalty", "1",
                       "--ignore-eos"])
    assert rc == 0, out.getvalue()
    assert "response: " + ToyTokenizer().decode(want) in out.getvalue()
    out = io.StringIO()
    with contextlib.redirect_stdout(out):
        assert cli.main(["tokenize", path, "hi"]) == 0
    assert "ids: [104, 105]" in out.getvalue()


@pytest.mark.parametrize("kind", ["state", "mixed"])
def test_toy_architecture_registered_built_and_stepped(kind, tmp_path):
    """A model folder of an architecture that exists only in this test: config.json names
    it, the registry finds it, the loader binds its tensors, the cache manager gives it
    state slots / windowed pages, the engine steps it under every cutting."""
    from zinfer_amd.config import register_architecture, unregister_architecture
    from zinfer_amd.engine import StepEntry
    from zinfer_amd.engine.replay import make_engine
    from zinfer_amd.parts import unregister_part
    from zinfer_amd.weights import SafetensorsFile, write_model_dir
    _register_toy_state()
    register_architecture("ToyForCausalLM", ToyConfig, model_type="toy", text=_toy_text_hooks())
    try:
        cfg = ToyConfig(hidden_size=64, state_size=24, decay=0.9, window=19, vocab_size=300,
                        kind=kind)
        path = write_model_dir(str(tmp_path / "toy"), cfg, seed=5, dtype=torch.float32)
        if kind == "state":
            _toy_text_through_the_command_line(path, cfg)
        with SafetensorsFile(os.path.join(path, "model.safetensors")) as f:
            w = {n: f.tensor(n) for n in f.names()}
        requests = {f"q{i}": tiny.random_tokens(n, 300, 70 + i) for i, n in enumerate((50, 7, 90, 33))}
        ref = {rid: _toy_plain(cfg, w, t) for rid, t in requests.items()}
        outs = {}
        for mode in ("whole", "portions", "mixed", "prefill_then_32"):
            steps = {"whole": traces.whole, "portions": traces.changing_portions,
                     "mixed": traces.mixed, "prefill_then_32": traces.prefill_then_single}[mode](requests)
            eng = make_engine(path, "float32", traces.peak_tokens(steps, 64), DEV, poison_freed=True)
            if kind == "state":
                assert len(eng.cache.state_pools) == 2 and len(eng.cache.groups) == 1
            else:
                assert len(eng.cache.groups) == 2      # full and windowed pages apart
                assert eng.views[3].k_pool.data_ptr() == eng.views[1].k_pool.data_ptr()
                assert not eng.views[3].writes
            got_steps = {}
            for st in steps:
                lg = eng.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in st["entries"]],
                              end=st["end"])
                if lg.shape[0]:
                    got_steps[st["step"]] = lg.cpu().numpy()
            eng.cache.check()
            outs[mode] = traces.collect(steps, got_steps, 300)
            for rid in requests:
                err = np.abs(outs[mode][rid] - ref[rid]).max() / np.abs(ref[rid]).max()
                assert err <= 2e-5, f"{kind} {mode} {rid}: {err:.3g}"
        if kind == "mixed":
            # the windowed group gave pages back while requests were still running
            steps = traces.changing_portions({"w": requests["q2"]})
            eng = make_engine(path, "float32", 128, DEV)
            for st in steps:
                eng.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in st["entries"]])
            held = [g.pages.num_held for g in eng.cache.groups]
            assert held[0] == 6 and held[1] <= 3       # 90 tokens: 6 pages; window 19: <= 3
            # several decode steps in a row on the device, over page edges of both groups
            one = make_engine(path, "float32", 512, DEV)
            many = make_engine(path, "float32", 512, DEV)
            heads = {r: t[:n] for (r, t), n in zip(requests.items(), (50, 7, 61, 33))}
            for eng in (one, many):
                lg = eng.step([StepEntry(r, t, [len(t) - 1]) for r, t in heads.items()])
                first = eng.argmax(lg)
            drawn = many.decode_steps([StepEntry(r, [t], [0]) for r, t in zip(heads, first)], 21)
            cur = first
            for s in range(21):
                lg = one.step([StepEntry(r, [t], [0]) for r, t in zip(heads, cur)])
                cur = one.argmax(lg)
                assert cur == drawn[s], f"step {s}"
            for eng in (one, many):
                eng.cache.check()
            assert [g.pages.num_held for g in one.cache.groups] == \
                [g.pages.num_held for g in many.cache.groups]
    finally:
        unregister_architecture("ToyForCausalLM")
        unregister_part("mixer", ToyStateSpec)


# ----------------------------------------------------------------------------- more toy parts
# Another norm, another position encoding and a feed-forward with routing, defined here and
# registered from the test: nothing in the framework's files knows of them.
@dataclass(frozen=True)
class ToyLayerNormSpec:
    """(x - mean) / sqrt(var + eps) * w, without a bias."""
    width: int
    eps: float


@dataclass(frozen=True)
class ToyLearnedPositionSpec:
    """A learned vector per position, added to every query and key head."""
    head_dim: int
    max_positions: int


@dataclass(frozen=True)
class ToyRoutedSpec:
    """Top-1 of ``n_experts`` small ReLU networks, weighted by the router's probability."""
    hidden_size: int
    inner_size: int
    n_experts: int


def _register_toy_parts():
    from zinfer_amd.parts import FeedForward, Norm, PositionEncoding, TensorDecl, register_part

    class ToyLayerNorm(Norm):
        def declare(self):
            return {self.prefix + "weight": TensorDecl((self.spec.width,), init="gain")}

        def bind(self, tensors):
            self.w = tensors[self.prefix + "weight"].float().to(self.ctx.device)

        def forward(self, x, out):
            mu = x.mean(-1, keepdim=True)
            var = ((x - mu) ** 2).mean(-1, keepdim=True)
            out.copy_(((x - mu) / torch.sqrt(var + self.spec.eps) * self.w).to(out.dtype))
            return out

    class ToyLearnedPosition(PositionEncoding):
        custom_apply = True

        def declare(self):
            s = self.spec
            return {self.prefix + "pos_table": TensorDecl((s.max_positions, s.head_dim))}

        def bind(self, tensors):
            self.table = tensors[self.prefix + "pos_table"].float().to(self.ctx.device)

        def apply(self, q, k, positions):
            add = self.table[positions.long()][:, None, :]
            q.add_(add.to(q.dtype))
            k.add_(add.to(k.dtype))

    class ToyRouted(FeedForward):
        def declare(self):
            s, p = self.spec, self.prefix
            return {p + "router.weight": TensorDecl((s.n_experts, s.hidden_size)),
                    p + "w_in": TensorDecl((s.n_experts, s.inner_size, s.hidden_size)),
                    p + "w_out": TensorDecl((s.n_experts, s.hidden_size, s.inner_size))}

        def bind(self, tensors):
            dev = self.ctx.device
            self.router = tensors[self.prefix + "router.weight"].float().to(dev)
            self.w_in = tensors[self.prefix + "w_in"].float().to(dev)
            self.w_out = tensors[self.prefix + "w_out"].float().to(dev)

        def forward(self, h, residual, step):
            h = h.float()
            prob = torch.softmax(h @ self.router.T, dim=-1)          # 32-bit router
            weight, expert = prob.max(dim=-1)
            for e in range(self.spec.n_experts):
                y = torch.relu(h @ self.w_in[e].T) @ self.w_out[e].T
                residual += ((expert == e) * weight)[:, None] * y

    register_part("norm", ToyLayerNormSpec, ToyLayerNorm)
    register_part("position", ToyLearnedPositionSpec, ToyLearnedPosition)
    register_part("feed_forward", ToyRoutedSpec, ToyRouted)


@dataclass(frozen=True)
class ToyRoutedConfig:
    hidden_size: int
    inner_size: int
    n_experts: int
    n_layers: int
    vocab_size: int
    model_type: str = "toy_routed"
    HEADS, KV_HEADS, HEAD_DIM, MAX_POS, EPS = 3, 1, 16, 256, 1e-4

    @classmethod
    def from_dict(cls, raw):
        return cls(**{k: raw[k] for k in ("hidden_size", "inner_size", "n_experts", "n_layers",
                                          "vocab_size")})

    def to_dict(self):
        return dict(architectures=["ToyRoutedForCausalLM"], model_type="toy_routed",
                    hidden_size=self.hidden_size, inner_size=self.inner_size,
                    n_experts=self.n_experts, n_layers=self.n_layers, vocab_size=self.vocab_size)

    def model_spec(self):
        from zinfer_amd.config.specs import (GqaAttentionSpec, ModelSpec, PreNormBlockSpec,
                                             ScheduleEntry)
        H = self.hidden_size
        norm = ToyLayerNormSpec(H, self.EPS)
        attn = GqaAttentionSpec(H, self.HEADS, self.KV_HEADS, self.HEAD_DIM, None,
                                ToyLearnedPositionSpec(self.HEAD_DIM, self.MAX_POS), None)
        ff = ToyRoutedSpec(H, self.inner_size, self.n_experts)
        blk = PreNormBlockSpec(mixer=attn, feed_forward=ff, mixer_norm=norm, ff_norm=norm)
        return ModelSpec(vocab_size=self.vocab_size, hidden_size=H, max_positions=self.MAX_POS,
                         layers=(blk,) * self.n_layers,
                         schedule=tuple(ScheduleEntry(i) for i in range(self.n_layers)),
                         final_norm=norm, tie_word_embeddings=False)


def _toy_routed_plain(cfg: ToyRoutedConfig, w, toks):
    """Whole sequence in 64-bit, token after token; returns the logits and, per token and
    layer, the margin between the two best router probabilities."""
    nH, nKV, hd, eps = cfg.HEADS, cfg.KV_HEADS, cfg.HEAD_DIM, cfg.EPS
    W = {k: v.to(F64) for k, v in w.items()}

    def layer_norm(x, g):
        mu = x.mean()
        return (x - mu) / torch.sqrt(((x - mu) ** 2).mean() + eps) * g

    caches = [([], []) for _ in range(cfg.n_layers)]
    rows, margins = [], []
    for p, tok in enumerate(toks):
        x = W["model.embed_tokens.weight"][tok]
        for i in range(cfg.n_layers):
            pre = f"model.layers.{i}."
            n = layer_norm(x, W[pre + "input_layernorm.weight"])
            q = plain.linear(n, W[pre + "self_attn.q_proj.weight"]).reshape(nH, hd)
            k = plain.linear(n, W[pre + "self_attn.k_proj.weight"]).reshape(nKV, hd)
            v = plain.linear(n, W[pre + "self_attn.v_proj.weight"]).reshape(nKV, hd)
            q = q + W[pre + "self_attn.pos_table"][p]
            k = k + W[pre + "self_attn.pos_table"][p]
            caches[i][0].append(k); caches[i][1].append(v)
            o = plain.attention_single_query(q.reshape(-1), torch.stack(caches[i][0]),
                                             torch.stack(caches[i][1]), nH, nKV, hd, None)
            x = x + plain.linear(o, W[pre + "self_attn.o_proj.weight"])
            m = layer_norm(x, W[pre + "post_attention_layernorm.weight"])
            prob = plain.softmax(plain.linear(m, W[pre + "mlp.router.weight"]))
            e = int(prob.argmax())
            top2 = prob.topk(2).values
            margins.append(float(top2[0] - top2[1]))
            y = plain.linear(torch.relu(plain.linear(m, W[pre + "mlp.w_in"][e])),
                             W[pre + "mlp.w_out"][e])
            x = x + prob[e] * y
        rows.append(plain.linear(layer_norm(x, W["model.norm.weight"]), W["lm_head.weight"]))
    return torch.stack(rows).numpy(), min(margins)


def test_toy_norm_position_and_routed_feed_forward(tmp_path):
    """A layer norm, a learned position encoding applied by the part itself and a routed
    feed-forward, all defined in this file, make a model that the engine builds from its
    folder and steps under every cutting; compared with the same formulas in 64-bit."""
    from zinfer_amd.config import register_architecture, unregister_architecture
    from zinfer_amd.engine import StepEntry
    from zinfer_amd.engine.replay import make_engine
    from zinfer_amd.parts import unregister_part
    from zinfer_amd.weights import SafetensorsFile, write_model_dir
    _register_toy_parts()
    register_architecture("ToyRoutedForCausalLM", ToyRoutedConfig, model_type="toy_routed")
    try:
        cfg = ToyRoutedConfig(hidden_size=48, inner_size=40, n_experts=3, n_layers=2,
                              vocab_size=211)
        path = write_model_dir(str(tmp_path / "toy_routed"), cfg, seed=9, dtype=torch.float32)
        with SafetensorsFile(os.path.join(path, "model.safetensors")) as f:
            w = {n: f.tensor(n) for n in f.names()}
        assert all(any(key in n for n in w) for key in ("router", "pos_table", "w_in", "w_out"))
        requests = {f"t{i}": tiny.random_tokens(n, 211, 90 + i) for i, n in enumerate((41, 5, 70, 18))}
        ref, margin = {}, 1.0
        for rid, t in requests.items():
            ref[rid], mg = _toy_routed_plain(cfg, w, t)
            margin = min(margin, mg)
        assert margin > 1e-5, "two experts nearly tie: the 32-bit router might pick the other"
        for mode in ("whole", "portions", "mixed"):
            steps = {"whole": traces.whole, "portions": traces.changing_portions,
                     "mixed": traces.mixed}[mode](requests)
            eng = make_engine(path, "float32", traces.peak_tokens(steps, 64), DEV, poison_freed=True)
            assert not eng.use_graphs          # the toy parts do not claim to be graph-safe
            got_steps = {}
            for st in steps:
                lg = eng.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in st["entries"]],
                              end=st["end"])
                if lg.shape[0]:
                    got_steps[st["step"]] = lg.cpu().numpy()
            eng.cache.check()
            out = traces.collect(steps, got_steps, 211)
            for rid in requests:
                err = np.abs(out[rid] - ref[rid]).max() / np.abs(ref[rid]).max()
                assert err <= 2e-5, f"{mode} {rid}: {err:.3g}"
    finally:
        unregister_architecture("ToyRoutedForCausalLM")
        unregister_part("norm", ToyLayerNormSpec)
        unregister_part("position", ToyLearnedPositionSpec)
        unregister_part("feed_forward", ToyRoutedSpec)


# ----------------------------------------------------------------------------- a mixer with a cache and hints of its own
# One shared key row and one value row per token, of different widths, kept in 64-bit whatever
# the engine's cache dtype is; and a way of its own to cut a step (tiles of 5 queries), which
# it asks the engine to pack with the step's metadata.  Nothing in the framework knows of it.
@dataclass(frozen=True)
class ToyLatentSpec:
    hidden_size: int
    key_dim: int
    value_dim: int
    tile: int


def _register_toy_latent(seen):
    from zinfer_amd.parts import KVNeed, Mixer, StepHints, TensorDecl, register_part

    class ToyLatentMixer(Mixer):
        def __init__(self, spec, ctx, prefix):
            super().__init__(spec, ctx, prefix)
            self.hint_key = ("toy_latent", spec.tile)

        def declare(self):
            s, p = self.spec, self.prefix
            return {p + "q.weight": TensorDecl((s.key_dim, s.hidden_size)),
                    p + "k.weight": TensorDecl((s.key_dim, s.hidden_size)),
                    p + "v.weight": TensorDecl((s.value_dim, s.hidden_size)),
                    p + "o.weight": TensorDecl((s.hidden_size, s.value_dim))}

        def bind(self, tensors):
            self.w = {n: tensors[self.prefix + n + ".weight"].double().to(self.ctx.device)
                      for n in "qkvo"}

        def cache_need(self):
            s = self.spec
            return KVNeed(1, s.key_dim, None, value_dim=s.value_dim, dtype=torch.float64)

        def accept_cache(self, cache):
            seen["accepted"] = (cache.k_pool.dtype, cache.k_pool.shape[1], cache.v_pool.shape[1])

        def step_hints(self, shape):
            t = self.spec.tile
            tiles = [(i, j) for i, n in enumerate(shape.q_lens) for j in range((n + t - 1) // t)]
            seen["asked"] = seen.get("asked", 0) + 1
            return StepHints({"tiles": np.asarray(tiles, dtype=np.int32).reshape(-1, 2)},
                             {"n_tiles": len(tiles), "longest": max(shape.ctx_lens)})

        def forward(self, h, residual, step, cache):
            s, ps = self.spec, cache.page_size
            hints = step.hints[self.hint_key]
            tiles = hints.arrays["tiles"]
            assert tiles.device.type == torch.device(DEV).type and tiles.dtype == torch.int32
            assert tiles.shape == (hints.numbers["n_tiles"], 2)
            assert hints.numbers["longest"] == max(step.ctx_lens)
            kv = step.kv_tables(cache.group)
            q, k, v = (h.double() @ self.w[n].T for n in "qkv")
            slots = kv.slot_mapping.long()
            cache.k_pool.view(-1, s.key_dim)[slots] = k
            cache.v_pool.view(-1, s.value_dim)[slots] = v
            first = [0]
            for n in step.q_lens:
                first.append(first[-1] + n)
            done = 0
            for i, j in tiles.cpu().tolist():        # the step, tile by tile as the hints cut it
                n, c = step.q_lens[i], step.ctx_lens[i]
                pages = kv.block_table[i, :(c + ps - 1) // ps].long()
                K = cache.k_pool[pages].view(-1, s.key_dim)
                V = cache.v_pool[pages].view(-1, s.value_dim)
                for t in range(j * s.tile, min((j + 1) * s.tile, n)):
                    pos = c - n + t
                    a = torch.softmax(K[:pos + 1] @ q[first[i] + t] / s.key_dim ** 0.5, dim=0)
                    residual[first[i] + t] += ((a @ V[:pos + 1]) @ self.w["o"].T).float()
                    done += 1
            assert done == step.n_tokens

    register_part("mixer", ToyLatentSpec, ToyLatentMixer)


@dataclass(frozen=True)
class ToyLatentConfig:
    hidden_size: int
    key_dim: int
    value_dim: int
    vocab_size: int
    model_type: str = "toy_latent"

    @classmethod
    def from_dict(cls, raw):
        return cls(**{k: raw[k] for k in ("hidden_size", "key_dim", "value_dim", "vocab_size")})

    def to_dict(self):
        return dict(architectures=["ToyLatentForCausalLM"], model_type="toy_latent",
                    hidden_size=self.hidden_size, key_dim=self.key_dim, value_dim=self.value_dim,
                    vocab_size=self.vocab_size)

    def model_spec(self):
        from zinfer_amd.config.specs import (GqaAttentionSpec, ModelSpec, PreNormBlockSpec,
                                             RmsNormSpec, RotaryHalfSplitSpec, ScheduleEntry,
                                             SwiGluSpec)
        H = self.hidden_size
        norm = RmsNormSpec(H, 1e-5)
        ff = SwiGluSpec(H, 2 * H)
        full = GqaAttentionSpec(H, 4, 2, 16, 1e-5, RotaryHalfSplitSpec(16, 1e4, 256), None)
        latent = ToyLatentSpec(H, self.key_dim, self.value_dim, 5)
        blk = lambda m: PreNormBlockSpec(mixer=m, feed_forward=ff, mixer_norm=norm, ff_norm=norm)
        return ModelSpec(vocab_size=self.vocab_size, hidden_size=H, max_positions=256,
                         layers=(blk(latent), blk(full), blk(latent)),
                         schedule=tuple(ScheduleEntry(i) for i in range(3)), final_norm=norm,
                         tie_word_embeddings=True)


def _toy_latent_plain(cfg: ToyLatentConfig, w, toks):
    caches = [([], []) for _ in range(3)]
    rows = []
    for p, tok in enumerate(toks):
        x = w["model.embed_tokens.weight"][tok].to(F64)
        for layer in range(3):
            pre = f"model.layers.{layer}."
            n = plain.rms_norm(x, w[pre + "input_layernorm.weight"], 1e-5)
            if layer == 1:
                q = plain.per_head_rms_norm(plain.linear(n, w[pre + "self_attn.q_proj.weight"]),
                                            4, 16, w[pre + "self_attn.q_norm.weight"], 1e-5)
                k = plain.per_head_rms_norm(plain.linear(n, w[pre + "self_attn.k_proj.weight"]),
                                            2, 16, w[pre + "self_attn.k_norm.weight"], 1e-5)
                v = plain.linear(n, w[pre + "self_attn.v_proj.weight"])
                q, k = plain.rope_heads(q, 4, 16, p, 1e4), plain.rope_heads(k, 2, 16, p, 1e4)
                caches[layer][0].append(k.reshape(2, 16)); caches[layer][1].append(v.reshape(2, 16))
                o = plain.attention_single_query(q, torch.stack(caches[layer][0]),
                                                 torch.stack(caches[layer][1]), 4, 2, 16, None)
                x = x + plain.linear(o, w[pre + "self_attn.o_proj.weight"])
            else:
                q, k, v = (plain.linear(n, w[pre + f"self_attn.{m}.weight"]) for m in "qkv")
                caches[layer][0].append(k); caches[layer][1].append(v)
                a = plain.softmax(torch.stack(caches[layer][0]) @ q / cfg.key_dim ** 0.5)
                x = x + plain.linear(a @ torch.stack(caches[layer][1]), w[pre + "self_attn.o.weight"])
            mm = plain.rms_norm(x, w[pre + "post_attention_layernorm.weight"], 1e-5)
            x = x + plain.linear(plain.swiglu(plain.linear(mm, w[pre + "mlp.gate_proj.weight"]),
                                              plain.linear(mm, w[pre + "mlp.up_proj.weight"])),
                                 w[pre + "mlp.down_proj.weight"])
        rows.append(plain.linear(plain.rms_norm(x, w["model.norm.weight"], 1e-5),
                                 w["model.embed_tokens.weight"]))
    return torch.stack(rows).numpy()


def test_toy_mixer_with_cache_widths_dtype_and_step_hints_of_its_own(tmp_path):
    """A mixer defined here keeps keys 24 wide and values 40 wide in 64-bit pools under a
    32-bit engine, beside an ordinary attention layer with pools of its own, and has the
    engine pack its own way of cutting a step (tiles of 5 queries) into the step's upload:
    built from a folder and stepped under every cutting without a change to the framework."""
    from zinfer_amd.config import register_architecture, unregister_architecture
    from zinfer_amd.engine import StepEntry
    from zinfer_amd.engine.replay import make_engine
    from zinfer_amd.parts import unregister_part
    from zinfer_amd.weights import SafetensorsFile, write_model_dir
    seen = {}
    _register_toy_latent(seen)
    register_architecture("ToyLatentForCausalLM", ToyLatentConfig, model_type="toy_latent")
    try:
        cfg = ToyLatentConfig(hidden_size=64, key_dim=24, value_dim=40, vocab_size=190)
        path = write_model_dir(str(tmp_path / "toy_latent"), cfg, seed=13, dtype=torch.float32)
        with SafetensorsFile(os.path.join(path, "model.safetensors")) as f:
            w = {n: f.tensor(n) for n in f.names()}
        requests = {f"l{i}": tiny.random_tokens(n, 190, 60 + i) for i, n in enumerate((37, 4, 66, 21))}
        ref = {rid: _toy_latent_plain(cfg, w, t) for rid, t in requests.items()}
        for mode in ("whole", "portions", "mixed", "prefill_then_32"):
            steps = {"whole": traces.whole, "portions": traces.changing_portions,
                     "mixed": traces.mixed, "prefill_then_32": traces.prefill_then_single}[mode](requests)
            eng = make_engine(path, "float32", traces.peak_tokens(steps, 16), DEV)
            # the two latent layers share a group (64-bit, 24 and 40 wide), the attention
            # layer has its own (32-bit, 2 heads of 16 both ways)
            assert len(eng.cache.groups) == 2 and not eng.use_graphs
            lat, att = eng.cache.groups
            assert lat.k.dtype == torch.float64 and att.k.dtype == torch.float32
            assert lat.k.shape[2] == 16 * 24 and lat.v.shape[2] == 16 * 40 and lat.k.shape[0] == 2
            assert att.k.shape[2] == att.v.shape[2] == 2 * 16 * 16
            assert seen["accepted"] == (torch.float64, 16 * 24, 16 * 40)
            asked = seen.get("asked", 0)
            got_steps = {}
            for st in steps:
                lg = eng.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in st["entries"]],
                              end=st["end"])
                if lg.shape[0]:
                    got_steps[st["step"]] = lg.cpu().numpy().copy()
            assert seen["asked"] == asked + len(steps), "one call a step for both latent layers"
            eng.cache.check()
            out = traces.collect(steps, got_steps, 190)
            for rid in requests:
                err = np.abs(out[rid] - ref[rid]).max() / np.abs(ref[rid]).max()
                assert err <= 2e-5, f"{mode} {rid}: {err:.3g}"
    finally:
        unregister_architecture("ToyLatentForCausalLM")
        unregister_part("mixer", ToyLatentSpec)
