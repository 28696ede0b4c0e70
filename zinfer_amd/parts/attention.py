from __future__ import annotations

import math
from typing import Dict

import numpy as np
import torch

from .. import ops
from ..config.specs import GqaAttentionSpec
from ..errors import ConfigError
from .base import KVNeed, Mixer, StepHints, TensorDecl, build_part, register_part
from .linear import Linear, place_gain, place_matrix


class GqaAttention(Mixer):
    """Causal grouped-query attention over a paged cache, in the reference's order
    (`src/model/runtime/optimized_decoder/layer.zig:110-142,188`): q/k/v projections,
    optional per-head RMSNorm of q and k, position encoding of q and k, append (k, v) at the
    token's position, softmax(q K^T / sqrt(hd)) V over the positions up to the token's own
    (query head h reads kv head h // G), output projection added to the residual."""
    graph_safe = True
    accepts_lazy_norm = True       # h is only ever handed to the q/k/v product
    kernel_modules = ("elementwise", "gemm", "attention")


    def __init__(self, spec: GqaAttentionSpec, ctx, prefix):
        super().__init__(spec, ctx, prefix)
        s = spec
        if s.n_heads == 0 or s.n_kv_heads == 0 or s.head_dim == 0:
            raise ConfigError("InvalidDimensions: heads and head_dim must not be 0")
        if s.n_heads % s.n_kv_heads != 0:
            raise ConfigError(f"InvalidGrouping: {s.n_heads} query heads, {s.n_kv_heads} kv heads")
        if s.head_dim % 2 != 0 or s.head_dim > ops.MAX_HEAD_DIM:
            raise ConfigError(f"InvalidHeadDim: head_dim={s.head_dim}: the attention kernels "
                              f"take even head sizes up to {ops.MAX_HEAD_DIM}")
        if s.window is not None and s.window < 1:
            raise ConfigError(f"window={s.window} must be at least 1")
        self.q_width = s.n_heads * s.head_dim
        self.kv_width = s.n_kv_heads * s.head_dim
        self.scale = s.scale if s.scale is not None else 1.0 / math.sqrt(float(s.head_dim))
        self.position = build_part("position", s.position, ctx, prefix)
        self.graph_safe = self.position.graph_safe
        # every layer of this kind cuts a step the same way, whatever its heads: one set of
        # hints a step serves them all
        self.hint_key = ("gqa_attention", ops.PREFILL_QUERY_TILE, ops.DECODE_SPLIT_KEYS)

    def declare(self) -> Dict[str, TensorDecl]:
        s, p = self.spec, self.prefix
        d = {p + "q_proj.weight": TensorDecl((self.q_width, s.hidden_size)),
             p + "k_proj.weight": TensorDecl((self.kv_width, s.hidden_size)),
             p + "v_proj.weight": TensorDecl((self.kv_width, s.hidden_size)),
             p + "o_proj.weight": TensorDecl((s.hidden_size, self.q_width))}
        if s.qk_norm_eps is not None:
            d[p + "q_norm.weight"] = TensorDecl((s.head_dim,), init="gain")
            d[p + "k_norm.weight"] = TensorDecl((s.head_dim,), init="gain")
        d.update(self.position.declare())
        return d

    def bind(self, tensors) -> None:
        p = self.prefix
        q, k, v = (tensors[p + n] for n in ("q_proj.weight", "k_proj.weight", "v_proj.weight"))
        if not (q.dtype == k.dtype == v.dtype):
            q, k, v = q.float(), k.float(), v.float()
        # rows of q, k and v one below the other: each output element keeps its own dot
        # product, so fusing changes no value
        self.qkv = Linear(place_matrix(torch.cat([q, k, v], dim=0), self.ctx))
        self.o = Linear(place_matrix(tensors[p + "o_proj.weight"], self.ctx))
        if self.spec.qk_norm_eps is not None:
            self.q_gain = place_gain(tensors[p + "q_norm.weight"], self.ctx)
            self.k_gain = place_gain(tensors[p + "k_norm.weight"], self.ctx)
        else:
            self.q_gain = self.k_gain = None
        self.position.bind(tensors)

    def cache_need(self):
        return KVNeed(self.spec.n_kv_heads, self.spec.head_dim, self.spec.window)

    def accept_cache(self, cache) -> None:
        # the cache-write and attention kernels keep keys and values in the activations'
        # dtype; there is no converting write
        if cache.k_pool is not None and cache.k_pool.dtype != self.ctx.act_dtype:
            raise ConfigError(f"the cache is kept in the compute dtype ({self.ctx.act_dtype}): "
                              f"a cache of {cache.k_pool.dtype} needs a model built with that "
                              "dtype")

    def step_hints(self, shape) -> StepHints:
        """How the attention kernels cut the step: the tiles of ``ops.PREFILL_QUERY_TILE``
        queries of the sequences that bring more than one token, as (sequence, tile) pairs
        with the tiles that read the most keys first; how many sequences bring exactly one
        token; the longest context among the others."""
        qt = ops.PREFILL_QUERY_TILE
        tiles = [(shape.starts[i] + min(qt * (t + 1), n), i, t)
                 for i, n in enumerate(shape.q_lens) if n > 1 for t in range((n + qt - 1) // qt)]
        tiles.sort(key=lambda x: -x[0])
        arrays = {}
        if tiles:
            arrays["q_tile_map"] = np.asarray([(i, t) for _, i, t in tiles], dtype=np.int32)
        return StepHints(arrays, {
            "n_single": sum(1 for n in shape.q_lens if n == 1),
            "n_query_tiles": len(tiles),
            "prefill_max_ctx": max((c for c, n in zip(shape.ctx_lens, shape.q_lens) if n > 1),
                                   default=None)})

    def graph_table_pages(self, pages: int, page_size: int):
        # contexts within one split of the decode attention get a table width of their own:
        # that kernel then writes the output itself and no merge kernel runs
        short = max(1, ops.DECODE_SPLIT_KEYS // page_size)
        return short if pages <= short else None

    def forward(self, h, residual, step, cache) -> None:
        s = self.spec
        T = h.shape[0]
        act = self.ctx.act_dtype
        tables = self.position.rotation_tables()
        kv = step.kv_tables(cache.group)
        eps = float(s.qk_norm_eps) if s.qk_norm_eps is not None else 0.0
        attn = step.scratch("attn", (T, self.q_width), act)
        window = 0 if s.window is None else int(s.window)
        plain_position = tables is not None or not self.position.custom_apply
        # 17 to 128 tokens: the product runs split along K, and the kernel that norms, rotates
        # and stores takes its partials as they are (one launch less, the same bits)
        partials = self.qkv.forward_partials(h) \
            if plain_position and cache.writes and act == torch.bfloat16 \
            and cache.k_pool.dtype == torch.bfloat16 and s.head_dim % 8 == 0 else None
        if partials is not None:
            qkv = partials
        else:
            qkv = step.scratch("qkv", (T, self.q_width + 2 * self.kv_width), act)
            self.qkv.forward(h, qkv)
        if partials is None and plain_position and step.max_q_len == 1 and cache.writes \
                and step.n_seqs <= ops.FUSED_DECODE_MAX_SEQS and ops.mfma_attention_covers(
                    act, s.n_heads, s.n_kv_heads, s.head_dim, cache.page_size):
            # a decode step: the attention kernel norms and rotates q and k and stores the
            # token's key and value itself (one kernel less, the same bits)
            cos, sin = tables if tables is not None else (None, None)
            ops.decode_attention_fused(
                qkv, self.q_gain, self.k_gain, eps, cos, sin, step.positions, kv.slot_mapping,
                cache.k_pool, cache.v_pool, kv.block_table, step.q_start, step.ctx_len, attn,
                float(self.scale), window, s.n_heads, s.n_kv_heads, s.head_dim, cache.page_size,
                step.max_ctx_len)
            self.o.forward(attn, residual, accumulate=True, step=step)
            return
        q = step.scratch("q", (T, self.q_width), act)
        if plain_position:
            cos, sin = tables if tables is not None else (None, None)
            ops.qk_norm_rope_kv_write(
                qkv, self.q_gain, self.k_gain, eps, cos, sin, step.positions,
                kv.slot_mapping if cache.writes else None, cache.k_pool, cache.v_pool, q,
                s.n_heads, s.n_kv_heads, s.head_dim, cache.page_size)
        else:
            # a position encoding of its own: norm in place, let it change q and k, then store
            ops.qk_norm_rope_kv_write(qkv, self.q_gain, self.k_gain, eps, None, None,
                                      step.positions, None, cache.k_pool, cache.v_pool, None,
                                      s.n_heads, s.n_kv_heads, s.head_dim, cache.page_size)
            self.position.apply(qkv[:, :self.q_width].unflatten(1, (s.n_heads, s.head_dim)),
                                qkv[:, self.q_width:self.q_width + self.kv_width]
                                .unflatten(1, (s.n_kv_heads, s.head_dim)), step.positions)
            ops.qk_norm_rope_kv_write(qkv, None, None, 0.0, None, None, step.positions,
                                      kv.slot_mapping if cache.writes else None,
                                      cache.k_pool, cache.v_pool, q,
                                      s.n_heads, s.n_kv_heads, s.head_dim, cache.page_size)
        hints = step.hints.get(self.hint_key)
        cut = {} if hints is None else dict(
            n_single=hints.numbers["n_single"], n_query_tiles=hints.numbers["n_query_tiles"],
            q_tile_map=hints.arrays.get("q_tile_map"),
            prefill_max_ctx=hints.numbers["prefill_max_ctx"])
        ops.paged_attention(q, cache.k_pool, cache.v_pool, kv.block_table, step.q_start,
                            step.ctx_len, step.seq_index, attn, float(self.scale), window,
                            s.n_heads, s.n_kv_heads, s.head_dim, cache.page_size,
                            step.max_q_len, step.max_ctx_len, **cut)
        self.o.forward(attn, residual, accumulate=True, step=step)


register_part("mixer", GqaAttentionSpec, GqaAttention)
