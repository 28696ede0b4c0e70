"""The generic decoder: embedding, a schedule of blocks, final norm, head
(`src/model/layers/decoder_only_stack.zig:48-93`, `src/model/runtime/optimized_decoder/
runtime.zig:103-148`).  Which blocks, with which parts, in which order is data
(``ModelSpec``); nothing here names an architecture."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import ops
from ..config.specs import ModelSpec
from ..errors import ConfigError
from ..parts import BuildContext, TensorDecl, build_part
from ..parts.linear import Linear, place_matrix


class DecoderModel:
    def __init__(self, spec: ModelSpec, ctx: BuildContext):
        self.spec = spec
        self.ctx = ctx
        self.blocks = [build_part("block", b, ctx, spec.layer_prefix.format(i))
                       for i, b in enumerate(spec.layers)]
        self.final_norm = build_part("norm", spec.final_norm, ctx, spec.final_norm_prefix)
        self.graph_safe = self.final_norm.graph_safe and all(b.graph_safe for b in self.blocks)
        # embedding, row gather and head are the model's own launches
        self.kernel_modules = tuple(sorted(
            {"elementwise", "gemm"} | {m for b in self.blocks for m in b.kernel_modules}))
        for pos, e in enumerate(spec.schedule):
            if not (0 <= e.layer < len(self.blocks)):
                raise ConfigError(f"schedule[{pos}] names layer {e.layer} of {len(self.blocks)}")
            if e.cache_of is not None:
                if not (0 <= e.cache_of < pos) or spec.schedule[e.cache_of].cache_of is not None:
                    raise ConfigError(f"schedule[{pos}].cache_of={e.cache_of} must name an "
                                      "earlier run that has a cache of its own")
                if self.blocks[spec.schedule[e.cache_of].layer].cache_need() != \
                        self.blocks[e.layer].cache_need():
                    raise ConfigError(f"schedule[{pos}] cannot read the cache of run "
                                      f"{e.cache_of}: their cache needs differ")

    # ---------------------------------------------------------------- weights
    def declare(self) -> Dict[str, TensorDecl]:
        s = self.spec
        d: Dict[str, TensorDecl] = {s.embed_name: TensorDecl((s.vocab_size, s.hidden_size))}
        for b in self.blocks:
            d.update(b.declare())
        d.update(self.final_norm.declare())
        d[s.head_name] = TensorDecl((s.vocab_size, s.hidden_size),
                                    optional=s.tie_word_embeddings)
        return d

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        s = self.spec
        self.embedding = place_matrix(tensors[s.embed_name], self.ctx)
        for b in self.blocks:
            b.bind(tensors)
        self.final_norm.bind(tensors)
        if s.head_name in tensors:
            self.head = Linear(place_matrix(tensors[s.head_name], self.ctx))
        else:
            # tied: the embedding stands in for the head.  Where the matrix pre-tiles, the
            # head's product reads a second copy in the kernels' own order (the embedding
            # itself stays in rows for the gather); elsewhere both are one tensor.
            self.head = Linear(self.embedding)

    def hint_providers(self):
        """One part per ``hint_key`` among all the blocks' parts: the engine asks each once a
        step for what its kernels want to know about the step's shape."""
        seen = {}
        for b in self.blocks:
            for p in b.hint_providers():
                seen.setdefault(p.hint_key, p)
        return list(seen.values())

    def accept_caches(self, caches) -> None:
        for pos, e in enumerate(self.spec.schedule):
            self.blocks[e.layer].accept_cache(caches[pos])

    # ---------------------------------------------------------------- cache needs
    def cache_needs(self) -> List[Optional[object]]:
        """For each schedule position: the cache need of the run, or None if it has none or
        reads another run's."""
        return [None if e.cache_of is not None else self.blocks[e.layer].cache_need()
                for e in self.spec.schedule]

    # ---------------------------------------------------------------- forward
    def forward(self, step, caches) -> torch.Tensor:
        """Runs the tokens of ``step`` and returns float32 logits [len(step.want_rows), V].
        ``caches[pos]`` is the cache view of schedule position ``pos`` (or None)."""
        s = self.spec
        T = step.n_tokens
        x = step.scratch("residual", (T, s.hidden_size), torch.float32)
        ops.embed(self.embedding, step.token_ids, x, float(s.embedding_multiplier))
        step.norm_ready = None
        for pos, e in enumerate(s.schedule):
            # the norm that reads the stream after this block: the next block's first, or the
            # final norm when every row goes to the head as it lies
            if pos + 1 < len(s.schedule):
                after = getattr(self.blocks[s.schedule[pos + 1].layer], "entry_norm", None)
            else:
                after = self.final_norm if self.final_norm.defers and step.wants_all_rows \
                    else None
            step.norm_after_block = after
            self.blocks[e.layer].forward(x, step, caches[pos])
        left, step.norm_ready, step.norm_after_block = step.norm_ready, None, None
        n_rows = step.n_want
        logits = step.scratch("logits", (n_rows, s.vocab_size), torch.float32)
        if n_rows == 0:
            return logits
        if step.wants_all_rows:
            rows = x
        else:
            left = None
            rows = step.scratch("want_rows", (n_rows, s.hidden_size), torch.float32)
            ops.gather_rows(x, step.want_rows, rows)
        make = lambda: step.scratch("final_normed", (n_rows, s.hidden_size), self.ctx.act_dtype)
        with ops.kernel_class("head_sampling"):      # what a per-class measurement counts these as
            normed = self.final_norm.deferred(rows, make, left)
            if normed is None:
                normed = self.final_norm.forward(rows, make())
            self.head.forward(normed, logits)
            if s.logit_scale != 1.0 or s.logit_softcap is not None:
                ops.scale_cap(logits, float(s.logit_scale), float(s.logit_softcap or 0.0))
        return logits
