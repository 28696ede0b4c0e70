"""Interfaces of the parts a model is put together from, and their registries.

A part is built from its specification (sizes and constants), a build context (compute
dtype, device) and the tensor-name prefix it binds its weights under.  It declares the
tensors it needs, receives them once, and then runs on the tokens of a step.  No part knows
which model it is in: the reference's generic block is parametrised the same way
(`src/model/layers/rmsnorm_gqa_swiglu_block.zig:10-51`), with the family supplying names
(`src/model/families/qwen3/weights.zig:10-35`).

Roles and what each must provide:

* norm            ``forward(x_f32[T, W], out[T, W])``
* position        ``rotation_tables()`` (cos, sin as float32 ``[max_positions, head_dim/2]``) for
                  encodings the fused attention kernel can apply itself, else None and
                  ``apply(q, k, positions)`` which rotates/changes q ``[T, nH, hd]`` and
                  k ``[T, nKV, hd]`` in place
* mixer           ``cache_need()`` -> KVNeed | StateNeed | None;
                  ``forward(h[T, H], residual_f32[T, H], step, cache)`` adds its output to
                  ``residual`` (in 32-bit)
* feed_forward    ``forward(h[T, H], residual_f32[T, H], step)`` adds its output to ``residual``
* block           ``forward(x_f32[T, H], step, cache)`` in place on the residual stream
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, Optional, Tuple

import torch

from ..errors import ConfigError


@dataclass(frozen=True)
class TensorDecl:
    """A tensor a part binds.  ``init`` says how the random-weights mode draws it:
    'normal' = N(0, 0.02), 'gain' = 1 + U(-0.1, 0.1)."""
    shape: Tuple[int, ...]
    init: str = "normal"
    optional: bool = False


@dataclass(frozen=True)
class KVNeed:
    """A cache of keys and values that grows with the context; with ``window`` only the
    last ``window`` positions are ever read, so earlier pages may be given back."""
    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateNeed:
    """Per-request state of fixed size, zero when a request starts."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class BuildContext:
    compute_dtype: torch.dtype      # torch.bfloat16 or torch.float32
    device: torch.device

    @property
    def act_dtype(self) -> torch.dtype:
        """dtype of activations between kernels (the residual stream is always float32)."""
        return self.compute_dtype


class Part:
    """``graph_safe`` says that ``forward`` only launches work on the current stream whose
    arguments depend on the step's device tensors and sizes, never on its host-side lists
    (``q_lens``, ``slots``, ...): only then may a decode step be captured once and replayed."""
    role = ""
    graph_safe = False
    kernel_modules = ()        # names of the HIP kernel libraries the part launches

    def __init__(self, spec, ctx: BuildContext, prefix: str):
        self.spec = spec
        self.ctx = ctx
        self.prefix = prefix

    def declare(self) -> Dict[str, TensorDecl]:
        """Full tensor names -> declaration."""
        return {}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Receives the host tensors it declared (an optional one may be absent)."""


class Norm(Part):
    role = "norm"

    def forward(self, x: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class PositionEncoding(Part):
    """``rotation_tables()`` returns (cos, sin) when the encoding is a half-split rotation
    the attention kernel applies itself.  An encoding of another kind returns None there,
    sets ``custom_apply`` and changes q and k in place in ``apply``; with neither, q and k
    stay as they are."""
    role = "position"
    custom_apply = False

    def rotation_tables(self):
        return None

    def apply(self, q: torch.Tensor, k: torch.Tensor, positions: torch.Tensor) -> None:
        return None


class Mixer(Part):
    role = "mixer"

    def cache_need(self):
        return None

    def forward(self, h, residual, step, cache) -> None:
        raise NotImplementedError


class FeedForward(Part):
    role = "feed_forward"

    def forward(self, h, residual, step) -> None:
        raise NotImplementedError


class Block(Part):
    role = "block"

    def cache_need(self):
        return None

    def forward(self, x, step, cache) -> None:
        raise NotImplementedError


_REGISTRY: Dict[Tuple[str, type], type] = {}
ROLES = ("norm", "position", "mixer", "feed_forward", "block")


def register_part(role: str, spec_type: type, part_type: type) -> None:
    """Makes ``part_type`` the implementation of specifications of ``spec_type`` in ``role``."""
    if role not in ROLES:
        raise ConfigError(f"unknown role {role!r}; roles are {ROLES}")
    _REGISTRY[(role, spec_type)] = part_type


def unregister_part(role: str, spec_type: type) -> None:
    _REGISTRY.pop((role, spec_type), None)


def build_part(role: str, spec, ctx: BuildContext, prefix: str) -> Part:
    try:
        part_type = _REGISTRY[(role, type(spec))]
    except KeyError:
        raise ConfigError(f"no {role} registered for specification {type(spec).__name__}") \
            from None
    return part_type(spec, ctx, prefix)
