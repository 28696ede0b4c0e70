"""The scheduler above the step function: admits requests, cuts prompts into portions under
a token budget, decodes, finishes and frees.

What the reference has of this (`src/model/runtime/optimized_decoder/batch.zig`): a fixed
number of slots (`:31-73`), first-come admission into a freed slot (`:194-199`), one token
per active request per round (`:116-136`), finish on an end-of-sequence id, which is checked
before it is forwarded and neither stored nor counted (`:120-125`), or after
``max_new_tokens`` (`:131-135`).  Its prefill is the whole prompt at once and its cache can
never run out; portions, the budget and what happens when pages run out are this engine's:

* a waiting request is admitted only when its next portion fits into free pages;
* when a running request cannot get the page it needs, the most recently admitted running
  request is preempted: its pages are freed, it keeps its generated tokens and its random
  stream, goes to the front of the waiting queue and later recomputes prompt + generated;
* a request that can never run (a token id beyond the vocabulary, a prompt longer than the
  position table or than the whole pool, an empty prompt) is rejected when it is added: it
  finishes at once with ``finish_reason`` "rejected" and the reason in ``error``, and the
  next ``step()`` hands it back among the finished; the other requests never see it;
* a request that is alone and still outgrows the pool while it decodes finishes with
  ``finish_reason`` "cache" and keeps its tokens.

When every running request decodes and nobody waits, up to ``multi_step`` decode steps run in
a row on the device without the host between them; tokens that a request drew after its
end-of-sequence id are thrown away, which costs at most ``multi_step - 1`` steps of that row.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..errors import CacheFull, StepError
from ..sampling import SamplingParams, Xoshiro256pp, sample_token
from .batch import StepEntry


@dataclass
class Request:
    id: object
    prompt: List[int]
    params: SamplingParams
    generated: List[int] = field(default_factory=list)
    n_computed: int = 0                # tokens whose keys and values are in the cache
    rng: Xoshiro256pp = None
    finished: bool = False
    finish_reason: Optional[str] = None
    preemptions: int = 0
    error: Optional[str] = None        # why the request was rejected
    counts: Optional[Dict[int, int]] = None    # occurrences of each token so far (penalties)

    @property
    def tokens(self) -> List[int]:
        return self.prompt + self.generated

    @property
    def pending(self) -> int:
        return len(self.prompt) + len(self.generated) - self.n_computed


@dataclass
class PlannedEntry:
    request: Request
    n_tokens: int
    samples: bool                      # the portion reaches the end of the known tokens


class Scheduler:
    def __init__(self, engine, *, max_step_tokens: int = 2048, chunk_size: Optional[int] = None,
                 max_seqs: int = 64, eos_token_ids: Sequence[int] = (), multi_step: int = 8):
        if max_step_tokens < 1 or max_seqs < 1:
            raise ValueError("max_step_tokens and max_seqs must be at least 1")
        self.engine = engine
        self.cache = engine.cache
        self.max_step_tokens = max_step_tokens
        self.chunk_size = chunk_size or max_step_tokens
        self.max_seqs = min(max_seqs, self.cache.max_requests)
        self.eos_token_ids = tuple(eos_token_ids)
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []           # in admission order
        self.finished: Dict[object, Request] = {}
        self._next_id = 0
        self.multi_step = multi_step        # most decode steps in a row without the host
        self.n_steps = 0                    # engine steps so far
        self.last_steps = 0                 # engine steps the last call of step() ran
        self.n_preemptions = 0
        self._rejected: List[Request] = []   # finished when added; handed back by step()

    # ------------------------------------------------------------------ requests
    def add_request(self, prompt: Sequence[int], params: Optional[SamplingParams] = None,
                    request_id=None) -> object:
        """Queues a request and returns its id.  An id that a live request (waiting, running
        or holding pages) has is the caller's mistake and raises; the id of a request that has
        finished may be used again, and its old record then goes.  A request that can never
        run is rejected (see the module's text)."""
        prompt = [int(t) for t in prompt]
        params = params or SamplingParams()
        rid = request_id if request_id is not None else self._next_id
        if self.cache.has_request(rid) or any(r.id == rid for r in self._rejected) or \
                any(r.id == rid for r in self.running) or any(r.id == rid for r in self.waiting):
            raise StepError(f"request id {rid!r} is already in use")
        self.finished.pop(rid, None)
        index = self._next_id
        self._next_id += 1
        # every request has a stream of its own, so its output does not depend on the batch
        rng = Xoshiro256pp((params.seed ^ (index * 0x9E3779B97F4A7C15)) & ((1 << 64) - 1))
        req = Request(rid, prompt, params, rng=rng)
        why = self._why_it_can_never_run(req)
        if why is not None:
            req.finished, req.finish_reason, req.error = True, "rejected", why
            self.finished[rid] = req
            self._rejected.append(req)
        else:
            self.waiting.append(req)
        return rid

    def _why_it_can_never_run(self, req: Request) -> Optional[str]:
        spec = self.engine.model.spec
        if not req.prompt:
            return "EmptyPrompt: a prompt must hold at least one token"
        bad = next((t for t in req.prompt if not (0 <= t < spec.vocab_size)), None)
        if bad is not None:
            return f"TokenIdOutOfBounds: token {bad}, vocabulary {spec.vocab_size}"
        if len(req.prompt) > spec.max_positions:
            return (f"PositionOutOfBounds: a prompt of {len(req.prompt)} tokens, "
                    f"max_position_embeddings is {spec.max_positions}")
        # the prompt and the first generated token must fit into the pool when it is alone
        need = self.cache.pages_at_most(len(req.prompt) + 1, self.chunk_size)
        if any(n > total for n, total in zip(need, self.cache.num_pages())):
            return (f"CacheFull: a prompt of {len(req.prompt)} tokens needs {need} pages, the "
                    f"pool has {self.cache.num_pages()}")
        return None

    def pop_finished(self, rid=None):
        """Takes finished requests out of the scheduler: the one with this id (KeyError if it
        has not finished), or, without an id, all of them as {id: request}.  ``finished``
        otherwise keeps every request's prompt and tokens: a loop that serves for long calls
        this once it has handed a result on."""
        if rid is not None:
            return self.finished.pop(rid)
        done, self.finished = self.finished, {}
        return done

    def has_work(self) -> bool:
        return bool(self.waiting or self.running or self._rejected)

    def request(self, rid) -> Request:
        """The request with this id, wherever it is."""
        if rid in self.finished:
            return self.finished[rid]
        for req in list(self.running) + list(self.waiting):
            if req.id == rid:
                return req
        raise KeyError(rid)

    def abort(self, rid, reason: str = "aborted") -> Request:
        """Ends a request from outside (a stop sequence in its text, a client that left): what
        it holds is given back; the tokens it has generated stay."""
        req = self.request(rid)
        if req.finished:
            return req
        if req in self.running:
            self._finish(req, reason)
        else:
            self.waiting.remove(req)
            if self.cache.has_request(req.id):
                self.cache.release(req.id)
            req.finished, req.finish_reason = True, reason
            self.finished[req.id] = req
        return req

    # ------------------------------------------------------------------ planning
    def plan(self) -> List[PlannedEntry]:
        """Decides what the next step runs.  May preempt; admits from the waiting queue."""
        self._ended_by_plan: List[Request] = []
        while True:
            planned: List[PlannedEntry] = []
            budget = self.max_step_tokens
            # pages and request slots the entries planned so far will take
            taken = [0] * len(self.cache.groups)
            free = self.cache.num_free_pages()
            new_slots = [0]

            def try_add(req: Request, n: int) -> bool:
                need = self.cache.pages_missing(req.id, req.n_computed + n)
                slot = 0 if self.cache.has_request(req.id) else 1
                if new_slots[0] + slot > self.cache.num_free_slots() or \
                        any(t + m > f for t, m, f in zip(taken, need, free)):
                    return False
                for g, m in enumerate(need):
                    taken[g] += m
                new_slots[0] += slot
                planned.append(PlannedEntry(req, n, n == req.pending))
                return True

            starved: Optional[Request] = None
            # 1. requests that decode: one token each
            for req in self.running:
                if req.pending == 1 and req.generated and budget > 0:
                    if try_add(req, 1):
                        budget -= 1
                    elif starved is None:
                        starved = req
            # 2. running requests still in their prompt (or recomputing)
            in_plan = {id(p.request) for p in planned}
            for req in self.running:
                if id(req) in in_plan or req is starved:
                    continue
                if req.pending == 1 and req.generated:
                    continue
                n = min(req.pending, self.chunk_size, budget)
                if n <= 0:
                    continue
                if try_add(req, n):
                    budget -= n
                elif starved is None:
                    starved = req
            # 3. admission, first come first served, only if the next portion fits
            while self.waiting and budget > 0 and len(self.running) < self.max_seqs \
                    and starved is None:
                req = self.waiting[0]
                n = min(req.pending, self.chunk_size, budget)
                if not try_add(req, n):
                    break
                budget -= n
                self.waiting.popleft()
                self.running.append(req)
            if starved is not None and len(self.running) > 1:
                # a running request cannot get its pages: the newest running request yields
                self._preempt(self.running[-1])
                continue
            if starved is not None and len(self.running) == 1 and starved.generated:
                # alone, and its next token still does not fit: it ends here with what it has
                self._finish(starved, "cache")
                self._ended_by_plan.append(starved)
                continue
            if not planned:
                blocked = starved or (self.waiting[0] if self.waiting else None)
                if blocked is not None and not self.running or \
                        (starved is not None and len(self.running) == 1):
                    raise CacheFull(
                        f"CacheFull: request {blocked.id!r} needs "
                        f"{blocked.n_computed + min(blocked.pending, self.chunk_size)} tokens of "
                        "cache but does not fit even alone")
            return planned

    def _preempt(self, req: Request) -> None:
        self.running.remove(req)
        if self.cache.has_request(req.id):
            self.cache.release(req.id)
        req.n_computed = 0
        req.preemptions += 1
        self.n_preemptions += 1
        self.waiting.appendleft(req)

    # ------------------------------------------------------------------ one iteration
    def step(self) -> List[Request]:
        """Plans, runs one step, samples, finishes.  Returns the requests finished by it."""
        rejected, self._rejected = self._rejected, []
        k = self._multi_step_count()
        if k >= 2:
            return rejected + self._decode_multi(k)
        planned = self.plan()
        self.last_steps = 1 if planned else 0
        if not planned:
            return rejected + self._ended_by_plan
        entries = []
        for p in planned:
            toks = p.request.tokens[p.request.n_computed:p.request.n_computed + p.n_tokens]
            entries.append(StepEntry(p.request.id, toks, [p.n_tokens - 1] if p.samples else []))
        logits = self.engine.step(entries)
        self.n_steps += 1
        sampling = [p for p in planned if p.samples]
        next_tokens = self._sample(logits, sampling)
        done: List[Request] = rejected + self._ended_by_plan
        for p in planned:
            p.request.n_computed += p.n_tokens
        for p, tok in zip(sampling, next_tokens):
            if self._accept(p.request, tok):
                done.append(p.request)
        return done

    def _accept(self, req: Request, tok: int) -> bool:
        """Takes a drawn token into the request; True if the request has finished by it."""
        reason = None
        if not req.params.ignore_eos and (tok in self.eos_token_ids
                                          or tok in req.params.stop_token_ids):
            reason = "eos"                    # not stored, not counted
        else:
            req.generated.append(tok)
            if len(req.generated) >= req.params.max_new_tokens:
                reason = "length"
            elif len(req.prompt) + len(req.generated) > self.engine.model.spec.max_positions:
                reason = "context"
        if reason is not None:
            self._finish(req, reason)
        return reason is not None

    def _multi_step_count(self) -> int:
        """How many decode steps may run in a row on the device: every running request must
        decode, be sampled on the device without penalties and have room for that many tokens
        (in its length limits and in free pages), and nobody may wait for admission."""
        if self.multi_step < 2 or self.waiting or not self.running \
                or not getattr(self.engine, "use_graphs", False) \
                or len(self.running) > self.max_step_tokens:
            return 0
        k = self.multi_step
        max_pos = self.engine.model.spec.max_positions
        for req in self.running:
            sp = req.params
            if req.pending != 1 or not req.generated or sp.has_penalties \
                    or not (sp.greedy or 1 <= sp.top_k <= 1024):
                return 0
            k = min(k, sp.max_new_tokens - len(req.generated),
                    max_pos - (len(req.prompt) + len(req.generated)) + 1)
        while k >= 2 and not self.cache.can_reserve(
                [(req.id, req.n_computed + k) for req in self.running]):
            k //= 2
        return k if k >= 2 else 0

    def _decode_multi(self, k: int) -> List[Request]:
        from ..ops import SAMPLE_ROW_DTYPE
        reqs = list(self.running)
        entries = [StepEntry(r.id, [r.generated[-1]], [0]) for r in reqs]
        records = None
        if not all(r.params.greedy for r in reqs):
            records = np.zeros((k, len(reqs)), dtype=SAMPLE_ROW_DTYPE)
            for i, r in enumerate(reqs):
                sp = r.params
                for s in range(k):
                    records[s, i] = (1.0, 1.0, 0.0, 1, 0.0) if sp.greedy else \
                        (sp.temperature, sp.top_p, sp.min_p, sp.top_k, r.rng.float64())
        tokens = self.engine.decode_steps(entries, k, records)
        self.n_steps += k
        self.last_steps = k
        done: List[Request] = []
        for i, r in enumerate(reqs):
            r.n_computed += k
            for s in range(k):
                if self._accept(r, tokens[s][i]):
                    done.append(r)
                    break
        return done

    def _finish(self, req: Request, reason: str) -> None:
        req.finished = True
        req.finish_reason = reason
        self.running.remove(req)
        self.cache.release(req.id)
        self.finished[req.id] = req

    def _sample(self, logits: torch.Tensor, sampling: List[PlannedEntry]) -> List[int]:
        """Greedy rows without penalties: the device arg-max.  Rows whose top_k is 1..1024:
        the device sampler (penalties applied on the device too), with the uniform number
        taken from the request's own stream.  Anything else (the whole vocabulary as
        candidates): the host sampler on a copy of the row."""
        if not sampling:
            return []
        params = [p.request.params for p in sampling]
        if all(sp.greedy and not sp.has_penalties for sp in params):
            return self.engine.argmax(logits)
        if hasattr(self.engine, "sample") and all(
                sp.greedy or 1 <= sp.top_k <= 1024 for sp in params):
            return self._sample_on_device(logits, sampling)
        rows = logits.detach().to("cpu", torch.float32).numpy()
        out = []
        for i, p in enumerate(sampling):
            req = p.request
            out.append(sample_token(rows[i], req.tokens, req.params, req.rng))
        return out

    def _sample_on_device(self, logits: torch.Tensor, sampling: List[PlannedEntry]) -> List[int]:
        from ..ops import SAMPLE_ROW_DTYPE
        V = logits.shape[1]
        rec = np.zeros((len(sampling),), dtype=SAMPLE_ROW_DTYPE)
        pen_rows, pen_tok, pen_cnt = [], [], []
        pen_params = np.zeros((len(sampling), 3), dtype=np.float32)
        pen_params[:, 0] = 1.0
        for i, p in enumerate(sampling):
            req, sp = p.request, p.request.params
            if sp.greedy:          # the arg-max is the draw among the single best candidate
                rec[i] = (1.0, 1.0, 0.0, 1, 0.0)
            else:
                rec[i] = (sp.temperature, sp.top_p, sp.min_p, sp.top_k, req.rng.float64())
            if sp.has_penalties:
                if req.counts is None:
                    req.counts = {}
                    req._counted = 0
                toks = req.tokens
                for t in toks[req._counted:]:
                    if t < V:
                        req.counts[t] = req.counts.get(t, 0) + 1
                req._counted = len(toks)
                pen_rows.extend([i] * len(req.counts))
                pen_tok.extend(req.counts.keys())
                pen_cnt.extend(req.counts.values())
                pen_params[i] = (sp.repetition_penalty, sp.presence_penalty, sp.frequency_penalty)
        pen = None
        if pen_rows:
            pen = (np.asarray(pen_rows, np.int32), np.asarray(pen_tok, np.int32),
                   np.asarray(pen_cnt, np.int32), pen_params)
        return self.engine.sample(logits, rec, pen)

    def run(self) -> Dict[object, Request]:
        """Steps until every request has finished."""
        while self.has_work():
            self.step()
        return self.finished
