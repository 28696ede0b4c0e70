"""Specifications of the parts a model is put together from.

A specification is plain data: every size and constant a part needs, nothing about the model
it ends up in.  The reference describes a layer the same way, as a ``Spec`` of sizes plus a
``LayerLayout`` of optional slots (`src/model/layers/rmsnorm_gqa_swiglu_block.zig:10-51`) and
an ``AttentionSpec`` (`src/model/layers/gqa_attention/spec.zig:3-26`); here each slot is a
specification of its own so that layers of one model may differ.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Tuple


@dataclass(frozen=True)
class RmsNormSpec:
    """n = x * w / sqrt(mean(x^2) + eps) over ``width`` elements."""
    width: int
    eps: float


@dataclass(frozen=True)
class RotaryHalfSplitSpec:
    """Rotation of the pairs (i, i + head_dim/2) by position * theta^(-2i/head_dim)."""
    head_dim: int
    theta: float
    max_positions: int


@dataclass(frozen=True)
class NoPositionSpec:
    """No position encoding inside the mixer."""


@dataclass(frozen=True)
class GqaAttentionSpec:
    """Causal grouped-query attention.  ``window`` None = every earlier key; an integer =
    only the last ``window`` positions (the query's own included)."""
    hidden_size: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    qk_norm_eps: Optional[float]          # None: no per-head norm of q and k
    position: object                       # a position-encoding specification
    window: Optional[int] = None
    scale: Optional[float] = None          # None: 1/sqrt(head_dim)


@dataclass(frozen=True)
class SwiGluSpec:
    """down(silu(gate(x)) * up(x))."""
    hidden_size: int
    intermediate_size: int


@dataclass(frozen=True)
class PreNormBlockSpec:
    """x += mixer(norm1(x)); x += ff(norm2(x)).  ``mixer_prefix`` and the other prefixes are
    the tensor-name prefixes below the layer's own prefix."""
    mixer: object
    feed_forward: object
    mixer_norm: object
    ff_norm: object
    mixer_prefix: str = "self_attn."
    ff_prefix: str = "mlp."
    mixer_norm_prefix: str = "input_layernorm."
    ff_norm_prefix: str = "post_attention_layernorm."


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.  ``layer`` indexes ``ModelSpec.layers`` (a layer may be named
    twice); ``cache_of`` None gives this run a cache of its own, an integer makes it read
    the cache that the run at that earlier schedule position writes."""
    layer: int
    cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    """Everything the generic decoder needs: sizes, one block specification per layer, the
    order the layers run in, and tensor names."""
    vocab_size: int
    hidden_size: int
    max_positions: int
    layers: Tuple[object, ...]
    schedule: Tuple[ScheduleEntry, ...]
    final_norm: object
    tie_word_embeddings: bool
    embed_name: str = "model.embed_tokens.weight"
    final_norm_prefix: str = "model.norm."
    head_name: str = "lm_head.weight"
    layer_prefix: str = "model.layers.{}."
    eos_token_ids: Tuple[int, ...] = ()
    default_stop_sequences: Tuple[str, ...] = ()
    embedding_multiplier: float = 1.0       # the embedding row times this enters the stream
    logit_scale: float = 1.0                # logits = head(x) * logit_scale ...
    logit_softcap: Optional[float] = None   # ... then cap * tanh(logits / cap) if given
