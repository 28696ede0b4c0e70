"""The step function: a batch of (request, its next tokens) run as one batch from the cache.

The reference's counterpart runs one token of one request (`src/model/runtime/
optimized_decoder/runtime.zig:103-148`) and loops it for a prompt (`:150-163`); its limits
are kept as errors raised before anything is launched: a token id beyond the vocabulary
(`:109`), a position beyond the table (`src/kernel/attention/rope.zig:135`), a full cache
(`src/model/runtime/optimized_kv_cache/cache.zig:96`).
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ..cache import CacheManager
from ..errors import (CacheFull, ConfigError, PositionOutOfBounds, StepError,
                      TokenIdOutOfBounds)
from ..models.decoder import DecoderModel
from ..parts.base import StepHints, StepShape
from .batch import KVStepTables, Scratch, StepContext, StepEntry


def _pad4(n: int) -> int:
    return (n + 3) // 4 * 4


class Engine:
    """Owns a model, its cache and work buffers; ``step`` is the only way tokens run."""

    GRAPH_PAGE_BUCKET = 64      # decode graphs are captured for block tables this many pages wide
    STEP_TRACE_MAX = 65536      # most records ``step_trace`` keeps
    MAX_GRAPHS = 256            # the least recently replayed graph goes when there are more

    def __init__(self, model: DecoderModel, *, page_size: int = 16, num_pages: int = 256,
                 max_requests: int = 64, kv_dtype: Optional[torch.dtype] = None,
                 poison_freed: bool = False, use_graphs: bool = True,
                 debug_tables: bool = False):
        self.model = model
        self.device = model.ctx.device
        if self.device.type == "cuda":
            # what this model needs is built now, side by side, if it is not built yet
            from ..ops import build
            build.prepare(getattr(model, "kernel_modules", ()))
        spec = model.spec
        needs = model.cache_needs()
        reads = [e.cache_of for e in spec.schedule]
        self.cache = CacheManager(needs, reads, page_size, num_pages, max_requests,
                                  kv_dtype or model.ctx.compute_dtype, self.device,
                                  poison_freed=poison_freed)
        self.views = [self.cache.view(pos) for pos in range(len(spec.schedule))]
        # a mixer whose kernels cannot serve the cache it was given says so now
        model.accept_caches(self.views)
        # the parts that want to know about a step's shape, one per kind
        self._hint_providers = model.hint_providers()
        self.page_size = page_size
        # debugging: every step's block tables and slots are checked on the device against the
        # pool before its kernels run (one small kernel and a wait for its report a step)
        self.debug_tables = debug_tables and self.device.type == "cuda"
        self._scratch = Scratch(self.device)
        self._meta_host = None          # two pinned buffers that take turns
        self._meta_dev: Optional[torch.Tensor] = None
        self._meta_generation = 0
        self.steps_run = 0
        # decode-only steps (one token per request) are launch-bound: they are captured once
        # per batch shape into a HIP graph and replayed
        self.use_graphs = use_graphs and self.device.type == "cuda" \
            and getattr(model, "graph_safe", False)
        self._graphs: Dict[tuple, tuple] = {}
        self.graph_replays = 0
        # several decode steps in a row (``decode_steps``) are also recorded as one graph, from
        # the second time a shape of run comes
        self.capture_runs = True
        self._run_shapes: Dict[tuple, int] = {}
        # measurement: when a list, every step appends (tokens, sequences, seconds of host
        # packing, seconds of host launching, event before, event after the step's kernels,
        # whether a request brought more than one token).  Every record holds two events:
        # whoever switches tracing on empties the list as it reads it (``drain_step_trace``);
        # beyond STEP_TRACE_MAX records the oldest go.
        self.step_trace: Optional[list] = None

    # ------------------------------------------------------------------ requests
    def has_request(self, rid) -> bool:
        return self.cache.has_request(rid)

    def length(self, rid) -> int:
        return self.cache.length(rid)

    def release(self, rid) -> None:
        self.cache.release(rid)

    # ------------------------------------------------------------------ the step
    def step(self, entries: Sequence[StepEntry], end: Sequence[object] = ()) -> torch.Tensor:
        """Runs the tokens of ``entries`` as one batch and returns float32 logits
        [number of wanted places, vocab] in the order of the entries and of their ``want``.
        Requests in ``end`` give back what they hold after the step.  On an error the cache
        is as before: what can be refused is refused before anything runs, and a failure
        inside the run gives back what the step had reserved."""
        seen, wanted_len = self._check_entries(entries)
        for rid in end:
            if rid not in seen and not self.cache.has_request(rid):
                raise StepError(f"request {rid!r} cannot end: it is not live")
        if not self.cache.can_reserve(wanted_len):
            raise CacheFull(f"CacheFull: the step needs more pages or request slots than are "
                            f"free (free pages per group: {self.cache.num_free_pages()})")
        if entries:
            added = self._reserve(wanted_len)
            try:
                decode_only = self.use_graphs and all(len(e.tokens) == 1 for e in entries)
                traced = self.step_trace is not None and self.device.type == "cuda"
                if traced:
                    import time
                    t0 = time.perf_counter()
                ctx = self._build_context(entries, bucket_pages=decode_only)
                if self.debug_tables:
                    self._check_tables(ctx)
                if traced:
                    t1 = time.perf_counter()
                    before = torch.cuda.Event(enable_timing=True)
                    after = torch.cuda.Event(enable_timing=True)
                    before.record()
                logits = self._forward_graphed(ctx) if decode_only \
                    else self.model.forward(ctx, self.views)
                if traced:
                    after.record()
                    self._trace((ctx.n_tokens, ctx.n_seqs, t1 - t0, time.perf_counter() - t1,
                                 before, after, ctx.max_q_len > 1))
            except BaseException:
                self._roll_back(wanted_len, added)
                raise
            for rid, new_len in wanted_len:
                self.cache.commit(rid, new_len)
            self.steps_run += 1
        else:
            logits = torch.empty((0, self.model.spec.vocab_size), dtype=torch.float32,
                                 device=self.device)
        for rid in end:
            self.cache.release(rid)
        return logits

    def probe_block(self, layer: int, hidden: torch.Tensor):
        """Block ``layer`` alone (`src/app/cli/inspect.zig:153-204`): ``hidden`` [T, hidden
        size] is the residual stream at the first T positions of a request made for this
        call; the block runs once over it, with pages of its own from the pool.  Returns the
        stream after the block (float32) and the length the request's cache had then.  What
        the request held goes back before the call returns."""
        spec = self.model.spec
        runs = [pos for pos, e in enumerate(spec.schedule)
                if e.layer == layer and e.cache_of is None]
        if not runs:
            raise StepError(f"no run of the schedule has layer {layer} with a cache of its own")
        T, width = hidden.shape
        if width != spec.hidden_size or T < 1:
            raise StepError(f"hidden is {tuple(hidden.shape)}, the stream is [T, {spec.hidden_size}]")
        rid = object()
        entry = StepEntry(rid, [0] * T, [])
        self._check_entries([entry])
        if not self.cache.can_reserve([(rid, T)]):
            raise CacheFull("CacheFull: no pages or request slot for the probe")
        self._reserve([(rid, T)])
        try:
            ctx = self._build_context([entry])
            x = ctx.scratch("residual", (T, spec.hidden_size), torch.float32)
            x.copy_(hidden)
            ctx.norm_ready = ctx.norm_after_block = None
            self.model.blocks[layer].forward(x, ctx, self.views[runs[0]])
            self.cache.commit(rid, T)
            return x.clone(), self.cache.length(rid)
        finally:
            self.cache.release(rid)

    def _trace(self, record) -> None:
        self.step_trace.append(record)
        if len(self.step_trace) > self.STEP_TRACE_MAX:
            del self.step_trace[:len(self.step_trace) - self.STEP_TRACE_MAX]

    def drain_step_trace(self) -> list:
        """The records gathered so far (the list is emptied; tracing stays on)."""
        done, self.step_trace = self.step_trace or [], [] if self.step_trace is not None else None
        return done

    def _check_tables(self, ctx: StepContext) -> None:
        """The device's own look at what the step's kernels will index with (debugging)."""
        from .. import ops
        report = self._scratch.get("table_report", (4,), torch.int32)
        for g, tables in enumerate(ctx.kv):
            report.zero_()
            ops.check_tables(tables.block_table, ctx.ctx_len, tables.slot_mapping, self.page_size,
                             self.cache.groups[g].pages.num_pages, report)
            kind, a, b, value = report.tolist()
            if kind == 1:
                raise StepError(f"BlockTableOutOfBounds: group {g}, sequence {a}, page index {b}: "
                                f"{value} is no page of a pool of "
                                f"{self.cache.groups[g].pages.num_pages} (or a context beyond "
                                "the table)")
            if kind == 2:
                raise StepError(f"SlotOutOfBounds: group {g}, token {a}: slot {value} is no row "
                                "of the pool")

    def _reserve(self, wanted_len) -> List[object]:
        """Adds the requests that are new and reserves every request's pages; returns the
        ids that were added."""
        added = []
        try:
            for rid, new_len in wanted_len:
                if not self.cache.has_request(rid):
                    self.cache.add_request(rid)
                    added.append(rid)
                self.cache.reserve(rid, new_len)
        except BaseException:
            self._roll_back(wanted_len, added)
            raise
        return added

    def _roll_back(self, wanted_len, added) -> None:
        """A step failed after it had reserved: the requests it added go, the pages it
        reserved beyond what the others hold go back.  (Keys and values that kernels may
        already have written lie beyond the requests' lengths and are never read.)"""
        for rid, _ in wanted_len:
            if rid in added:
                if self.cache.has_request(rid):
                    self.cache.release(rid)
            elif self.cache.has_request(rid):
                self.cache.trim(rid)

    def _check_entries(self, entries: Sequence[StepEntry], extra: int = 0):
        """What can be refused before anything runs.  Returns the ids of the entries and
        (id, length after the step plus ``extra`` further tokens) for each."""
        spec = self.model.spec
        seen = set()
        wanted_len = []
        for e in entries:
            if e.request_id in seen:
                raise StepError(f"request {e.request_id!r} appears twice in one step")
            seen.add(e.request_id)
            n = len(e.tokens)
            if n == 0:
                raise StepError(f"request {e.request_id!r}: a portion must hold a token")
            for t in e.tokens:
                if not (0 <= int(t) < spec.vocab_size):
                    raise TokenIdOutOfBounds(f"TokenIdOutOfBounds: token {t} of request "
                                             f"{e.request_id!r}, vocabulary {spec.vocab_size}")
            for w in e.want:
                if not (0 <= int(w) < n):
                    raise StepError(f"request {e.request_id!r}: want {w} outside its {n} tokens")
            start = self.cache.length(e.request_id) if self.cache.has_request(e.request_id) else 0
            if start + n + extra > spec.max_positions:
                raise PositionOutOfBounds(
                    f"PositionOutOfBounds: request {e.request_id!r} would reach position "
                    f"{start + n + extra - 1}, max_position_embeddings is {spec.max_positions}")
            wanted_len.append((e.request_id, start + n + extra))
        return seen, wanted_len

    def decode_steps(self, entries: Sequence[StepEntry], n_steps: int,
                     records: Optional[np.ndarray] = None) -> List[List[int]]:
        """``n_steps`` decode steps in a row without the host between them: every entry brings
        one token; after each step a token is drawn for every request on the device (the
        arg-max, or with ``records`` [n_steps, requests] of ``ops.SAMPLE_ROW_DTYPE`` the
        device sampler) and becomes the request's input of the next step.  Returns the drawn
        tokens [n_steps][requests]; the requests then hold ``n_steps`` more tokens.  Only for
        models whose steps replay as a graph: nothing on the host sees the steps between."""
        from .. import ops
        if not self.use_graphs:
            raise StepError("decode_steps needs a model whose decode steps replay as a graph")
        n = len(entries)
        if n_steps < 1 or n == 0:
            raise StepError("decode_steps: at least one step and one request")
        if any(len(e.tokens) != 1 or list(e.want) != [0] for e in entries):
            raise StepError("decode_steps: every entry brings one token and wants its logits")
        if records is not None and records.shape != (n_steps, n):
            raise StepError(f"decode_steps: records must be [{n_steps}, {n}]")
        extra = n_steps - 1
        _, wanted_len = self._check_entries(entries, extra)
        if not self.cache.can_reserve(wanted_len):
            raise CacheFull(f"CacheFull: {n_steps} steps need more pages or request slots than "
                            f"are free (free pages per group: {self.cache.num_free_pages()})")
        added = self._reserve(wanted_len)
        try:
            traced = self.step_trace is not None and self.device.type == "cuda"
            if traced:
                import time
                t0 = time.perf_counter()
            ctx = self._build_context(entries, bucket_pages=True, extra_tokens=extra)
            if traced:
                t1 = time.perf_counter()
                before = torch.cuda.Event(enable_timing=True)
                after = torch.cuda.Event(enable_timing=True)
                before.record()
            out = self._scratch.get("decoded", (n_steps, n), torch.int32)
            rec = None
            if records is not None:
                # at a fixed address, so that a captured run of steps can be replayed
                rec = self._scratch.get("sample_records", (n_steps, n * 24), torch.uint8)
                rec.copy_(torch.from_numpy(records.view(np.uint8).reshape(n_steps, -1).copy()),
                          non_blocking=False)

            def run_steps():
                for s in range(n_steps):
                    if s:
                        for g, tables in enumerate(ctx.kv):
                            ops.advance_decode(ctx.token_ids, ctx.positions, ctx.ctx_len,
                                               out[s - 1], tables.slot_mapping,
                                               tables.block_table, self.page_size,
                                               advance=(g == 0))
                    logits = self.model.forward(ctx, self.views) if capturing[0] \
                        else self._forward_graphed(ctx)
                    if rec is None:
                        ops.argmax(logits, out[s])
                    else:
                        ops.sample_topk(logits, rec[s], out[s])

            # The whole run of steps as one graph.  A call with a new shape runs step by step
            # (each step's own graph, the kernels between them launched one by one), which
            # settles every work buffer.  The second call with that shape does the same and
            # then records the run once more without running it (some tens of milliseconds,
            # which a shape that comes only once is not worth); later calls replay that
            # record, so that nothing is launched between the steps.
            capturing = [False]
            key = ("run", n, n_steps, rec is not None, tuple(t.max_pages for t in ctx.kv),
                   ctx.meta_offset)
            held = self._graphs.get(key)
            if n_steps > 1 and held is not None and held[2] == self._generations():
                self._graphs[key] = self._graphs.pop(key)
                held[0].replay()
                self.graph_replays += n_steps
            else:
                run_steps()
                seen = self._run_shapes.get(key, 0)
                if len(self._run_shapes) > 4 * self.MAX_GRAPHS:
                    self._run_shapes.clear()
                self._run_shapes[key] = seen + 1
                if n_steps > 1 and self.capture_runs and seen >= 1:
                    torch.cuda.current_stream(self.device).synchronize()
                    graph = torch.cuda.CUDAGraph()
                    capturing[0] = True
                    try:
                        with torch.cuda.graph(graph):
                            run_steps()
                    finally:
                        capturing[0] = False
                    self._graphs = {k: g for k, g in self._graphs.items()
                                    if g[2] == self._generations() and k != key}
                    while len(self._graphs) >= self.MAX_GRAPHS:
                        self._graphs.pop(next(iter(self._graphs)))
                    self._graphs[key] = (graph, None, self._generations())
            if traced:
                after.record()
                self._trace((n * n_steps, n, t1 - t0, time.perf_counter() - t1, before, after,
                             False))
            tokens = out.tolist()
        except BaseException:
            self._roll_back(wanted_len, added)
            raise
        for rid, new_len in wanted_len:
            self.cache.commit(rid, new_len)
        self.steps_run += n_steps
        return tokens

    def class_times(self, entries: Sequence[StepEntry], repeats: int = 20) -> Dict[str, float]:
        """Seconds a decode step of ``entries`` (one token each) spends in each class of kernels
        (``ops.KERNEL_CLASSES``), and in all of them together under "step": for each class a
        graph of the step with only that class's kernels launched is captured and replayed
        ``repeats`` times between two events.  What the runs compute means nothing (the kernels
        of the other classes did not run) and nothing of it is kept: the requests hold what
        they held before.  The reference's per-op timing harness is
        `src/app/cli/tools/bench/ops.zig:516-543`."""
        from .. import ops
        if not self.use_graphs:
            raise StepError("class_times needs a model whose decode steps replay as a graph")
        if not entries or any(len(e.tokens) != 1 for e in entries):
            raise StepError("class_times: every entry brings one token")
        _, wanted_len = self._check_entries(entries)
        if not self.cache.can_reserve(wanted_len):
            raise CacheFull("CacheFull: the step needs more pages or request slots than are free")
        added = self._reserve(wanted_len)
        out: Dict[str, float] = {}
        try:
            ctx = self._build_context(entries, bucket_pages=True)
            self.model.forward(ctx, self.views)           # settles every work buffer's size
            stream = torch.cuda.current_stream(self.device)
            for cls in ops.KERNEL_CLASSES + ("step",):
                only = ops.KERNEL_CLASSES if cls == "step" else (cls,)
                n0 = ops.launch_count()
                with ops.only_classes(only):
                    self.model.forward(ctx, self.views)
                if ops.launch_count() == n0:              # the step has no kernel of this class
                    out[cls] = 0.0
                    continue
                stream.synchronize()
                graph = torch.cuda.CUDAGraph()
                with ops.only_classes(only):
                    with torch.cuda.graph(graph):
                        self.model.forward(ctx, self.views)
                graph.replay()
                before = torch.cuda.Event(enable_timing=True)
                after = torch.cuda.Event(enable_timing=True)
                before.record()
                for _ in range(repeats):
                    graph.replay()
                after.record()
                after.synchronize()
                out[cls] = before.elapsed_time(after) * 1e-3 / repeats
                del graph
        finally:
            self._roll_back(wanted_len, added)
        return out

    def _generations(self) -> tuple:
        from .. import ops
        return (self._scratch.generation, ops.workspace_generation(), self._meta_generation)

    def _forward_graphed(self, ctx: StepContext) -> torch.Tensor:
        """A decode-only step through a captured graph.  The graph holds the addresses of the
        metadata views, work buffers and pools: it is keyed by everything that fixes them
        (sequences, wanted rows and whether they are simply all rows, which decides the kernels
        of the head, width of the block tables) and dropped when a buffer moves."""
        key = (ctx.n_seqs, ctx.n_want, ctx.wants_all_rows, tuple(t.max_pages for t in ctx.kv),
               ctx.meta_offset)
        held = self._graphs.get(key)
        if held is not None and held[2] == self._generations():
            self._graphs[key] = self._graphs.pop(key)      # most recently used last
            held[0].replay()
            self.graph_replays += 1
            return held[1]
        # first time: an eager run settles the sizes of every work buffer (it writes the same
        # keys and values the replay will write again), then capture and replay
        logits = self.model.forward(ctx, self.views)
        if held is not None or any(g[2] != self._generations() for g in self._graphs.values()):
            # a work buffer has moved: every graph that holds its old address is dead
            self._graphs = {k: g for k, g in self._graphs.items()
                            if g[2] == self._generations() and k != key}
        while len(self._graphs) >= self.MAX_GRAPHS:
            self._graphs.pop(next(iter(self._graphs)))
        torch.cuda.current_stream(self.device).synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            logits = self.model.forward(ctx, self.views)
        self._graphs[key] = (graph, logits, self._generations())
        graph.replay()
        return logits

    def argmax(self, logits: torch.Tensor) -> List[int]:
        """First-maximum arg-max of every row, on the device; only the ids come back."""
        from .. import ops
        n = logits.shape[0]
        if n == 0:
            return []
        out = self._scratch.get("argmax", (n,), torch.int32)
        ops.argmax(logits, out)
        return out.tolist()

    def sample(self, logits: torch.Tensor, records, penalties=None) -> List[int]:
        """Draws one token per row on the device.  ``records`` is a numpy array of
        ``ops.SAMPLE_ROW_DTYPE`` (temperature, top_p, min_p, top_k in 1..1024, u);
        ``penalties`` = (rows, tokens, counts, params[n, 3]) numpy arrays or None."""
        from .. import ops
        n = logits.shape[0]
        if n == 0:
            return []
        dev = self.device
        if penalties is not None and len(penalties[0]):
            rows, tokens, counts, params = penalties
            ops.apply_penalties(logits, torch.from_numpy(rows).to(dev),
                                torch.from_numpy(tokens).to(dev), torch.from_numpy(counts).to(dev),
                                torch.from_numpy(params).to(dev))
        rec = torch.from_numpy(records.view(np.uint8).reshape(-1).copy()).to(dev)
        out = self._scratch.get("sampled", (n,), torch.int32)
        ops.sample_topk(logits, rec, out)
        return out.tolist()

    # ------------------------------------------------------------------ metadata
    def _build_context(self, entries: Sequence[StepEntry], bucket_pages: bool = False,
                       extra_tokens: int = 0) -> StepContext:
        """Packs the step's metadata and copies it to the device.  ``extra_tokens``: the block
        tables (and the bound on the context) also cover this many tokens after the step."""
        ps = self.page_size
        n_seqs = len(entries)
        q_lens = [len(e.tokens) for e in entries]
        T = sum(q_lens)
        starts = [self.cache.length(e.request_id) for e in entries]
        ctx_lens = [s + n for s, n in zip(starts, q_lens)]
        slots = [self.cache.state_slot(e.request_id) for e in entries]
        want_rows: List[int] = []
        q_start = [0]
        for e, n in zip(entries, q_lens):
            want_rows.extend(q_start[-1] + int(w) for w in e.want)
            q_start.append(q_start[-1] + n)
        n_want = len(want_rows)
        n_groups = len(self.cache.groups)
        max_pages = max((c + extra_tokens + ps - 1) // ps for c in ctx_lens)
        max_ctx = max(ctx_lens) + extra_tokens
        if bucket_pages:      # a fixed table width (and context bound) per captured graph
            # a part whose kernels' grids follow the width may ask for one of its own
            asked = [w for w in (p.graph_table_pages(max_pages, ps) for p in self._hint_providers)
                     if w is not None]
            if asked:
                max_pages = max(max_pages, *asked)
            else:
                b = self.GRAPH_PAGE_BUCKET
                max_pages = (max_pages + b - 1) // b * b
            max_ctx = max_pages * ps

        # what the parts want to know about the step's shape: their arrays ride in the upload
        shape = StepShape(q_lens, starts, ctx_lens, ps, fixed_shapes=bucket_pages)
        hinted = [(p.hint_key, p.step_hints(shape)) for p in self._hint_providers]
        hinted = [(k, h) for k, h in hinted if h is not None]

        # one packed int32 buffer, one copy to the device
        sizes = [("token_ids", T), ("positions", T), ("seq_index", T), ("q_start", n_seqs + 1),
                 ("ctx_len", n_seqs), ("state_slots", n_seqs), ("want_rows", max(n_want, 1))]
        for i, (_, h) in enumerate(hinted):
            for name, arr in h.arrays.items():
                if arr.dtype != np.int32:
                    raise StepError(f"step hint {name!r} must be an int32 array, is {arr.dtype}")
                sizes.append((f"hint{i}.{name}", arr.size))
        for g in range(n_groups):
            sizes += [(f"slot_mapping{g}", T), (f"block_table{g}", n_seqs * max_pages)]
        offs, total = {}, 0
        for name, n in sizes:
            offs[name] = (total, n)
            total += _pad4(n)
        host = np.zeros((total,), dtype=np.int32)

        def put(name, values):
            o, n = offs[name]
            host[o:o + len(values)] = values

        single = max(q_lens) == 1
        if single:
            put("token_ids", np.fromiter((e.tokens[0] for e in entries), np.int32, n_seqs))
            put("positions", np.asarray(starts, dtype=np.int32))
            put("seq_index", np.arange(n_seqs, dtype=np.int32))
        else:
            put("token_ids", np.concatenate([np.asarray(e.tokens, dtype=np.int32)
                                             for e in entries]))
            put("positions", np.concatenate([np.arange(s, s + n, dtype=np.int32)
                                             for s, n in zip(starts, q_lens)]))
            put("seq_index", np.repeat(np.arange(n_seqs, dtype=np.int32), q_lens))
        put("q_start", np.asarray(q_start, dtype=np.int32))
        put("ctx_len", np.asarray(ctx_lens, dtype=np.int32))
        put("state_slots", np.asarray(slots, dtype=np.int32))
        put("want_rows", np.asarray(want_rows, dtype=np.int32))
        for i, (_, h) in enumerate(hinted):
            for name, arr in h.arrays.items():
                put(f"hint{i}.{name}", arr.reshape(-1))
        rids = [e.request_id for e in entries]
        for g in range(n_groups):
            # the block tables and the slot mapping, written by the cache's native core
            # straight into their places of the buffer
            (bo, bn), (so, sn) = offs[f"block_table{g}"], offs[f"slot_mapping{g}"]
            self.cache.pack_step(g, rids, starts, q_lens, max_pages, host[bo:bo + bn],
                                 host[so:so + sn])

        dev = self._upload(host)

        def view(name):
            o, n = offs[name]
            return dev[o:o + n]

        kv = [KVStepTables(view(f"block_table{g}").view(n_seqs, max_pages),
                           view(f"slot_mapping{g}"), max_pages) for g in range(n_groups)]
        return StepContext(
            n_tokens=T, n_seqs=n_seqs, n_want=n_want, token_ids=view("token_ids"),
            positions=view("positions"), seq_index=view("seq_index"), q_start=view("q_start"),
            ctx_len=view("ctx_len"), state_slots=view("state_slots"),
            want_rows=view("want_rows")[:n_want], kv=kv, max_q_len=max(q_lens),
            max_ctx_len=max_ctx, q_lens=q_lens, ctx_lens=ctx_lens, slots=slots,
            meta_offset=self._meta_dev.data_ptr() if self._meta_dev is not None else 0,
            hints={k: StepHints({name: view(f"hint{i}.{name}").view(arr.shape)
                                 for name, arr in h.arrays.items() if arr.size},
                                dict(h.numbers))
                   for i, (k, h) in enumerate(hinted)},
            wants_all_rows=want_rows == list(range(T)),
            _scratch=self._scratch)

    def _upload(self, host: np.ndarray) -> torch.Tensor:
        """The packed metadata on the device.  Two pinned host buffers take turns, each with an
        event that says when its last copy has left it, so that packing a step never waits
        for the stream: the copy of the step before last is long done.  (The device buffer is
        one: its copy is queued on the stream behind the kernels that read the old contents.)"""
        n = host.shape[0]
        if self.device.type == "cpu":
            return torch.from_numpy(host.copy())
        if self._meta_dev is None or self._meta_dev.numel() < n:
            cap = max(n * 2, 1 << 18)
            self._meta_host = [torch.empty((cap,), dtype=torch.int32, pin_memory=True)
                               for _ in range(2)]
            self._meta_events = [None, None]
            self._meta_turn = 0
            self._meta_dev = torch.empty((cap,), dtype=torch.int32, device=self.device)
            self._meta_generation += 1
        turn = self._meta_turn
        self._meta_turn = 1 - turn
        if self._meta_events[turn] is not None:
            self._meta_events[turn].synchronize()
        pinned = self._meta_host[turn]
        pinned[:n].numpy()[:] = host
        self._meta_dev[:n].copy_(pinned[:n], non_blocking=True)
        event = torch.cuda.Event()
        event.record(torch.cuda.current_stream(self.device))
        self._meta_events[turn] = event
        return self._meta_dev[:n]
