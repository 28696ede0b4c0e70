"""Interfaces of the parts a model is put together from, and their registries.

A part is built from its specification (sizes and constants), a build context (compute
dtype, device) and the tensor-name prefix it binds its weights under.  It declares the
tensors it needs, receives them once, and then runs on the tokens of a step.  No part knows
which model it is in: the reference's generic block is parametrised the same way
(`src/model/layers/rmsnorm_gqa_swiglu_block.zig:10-51`), with the family supplying names
(`src/model/families/qwen3/weights.zig:10-35`).

Roles and what each must provide:

* norm            ``forward(x_f32[T, W], out[T, W])``; optionally ``deferred`` and
                  ``residual_sum`` (a norm that lets a neighbouring product do its work)
* position        ``rotation_tables()`` (cos, sin as float32 ``[max_positions, head_dim/2]``) for
                  encodings the fused attention kernel can apply itself, else None and
                  ``apply(q, k, positions)`` which rotates/changes q ``[T, nH, hd]`` and
                  k ``[T, nKV, hd]`` in place
* mixer           ``cache_need()`` -> KVNeed | StateNeed | None;
                  ``forward(h[T, H], residual_f32[T, H], step, cache)`` adds its output to
                  ``residual`` (in 32-bit); optionally ``step_hints`` (what its kernels want
                  to know about a step's shape, packed with the step's metadata),
                  ``graph_table_pages`` and ``accept_cache``
* feed_forward    ``forward(h[T, H], residual_f32[T, H], step)`` adds its output to ``residual``
* block           ``forward(x_f32[T, H], step, cache)`` in place on the residual stream
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Tuple

import numpy as np

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
    last ``window`` positions are ever read, so earlier pages may be given back.  A key row
    is ``head_dim`` wide; a value row ``value_dim`` (None: as wide as a key), so a mixer whose
    values are narrower or wider than its keys (or that keeps one shared latent row:
    ``n_kv_heads`` 1) gets pools of its own widths.  ``dtype``: what the pools hold (None:
    the engine's cache dtype)."""
    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    value_dim: Optional[int] = None
    dtype: Optional[torch.dtype] = None

    @property
    def key_width(self) -> int:
        return self.head_dim

    @property
    def value_width(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim


@dataclass(frozen=True)
class StateNeed:
    """Per-request state of fixed size, zero when a request starts."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class StepShape:
    """The shape of a step as the host knows it before anything is uploaded: per sequence the
    tokens it brings, the tokens it held before and holds after.  ``fixed_shapes``: the step's
    launches may be captured and replayed for other contexts of the same table width, so
    nothing a hint says may depend on the contexts themselves."""
    q_lens: List[int]
    starts: List[int]
    ctx_lens: List[int]
    page_size: int
    fixed_shapes: bool = False


@dataclass
class StepHints:
    """What a part wants to know about a step beyond the common metadata: small int32 arrays
    (the engine packs them into the step's one upload and hands back device views under the
    same names) and host-side numbers."""
    arrays: Dict[str, "np.ndarray"] = field(default_factory=dict)
    numbers: Dict[str, Optional[int]] = field(default_factory=dict)


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

    # Parts whose kernels cut a step's work by its shape (query tiles, splits of a context)
    # say so here: parts with equal ``hint_key`` share one ``step_hints`` call a step, and
    # find its result in ``step.hints[hint_key]``.  None: no hints.
    hint_key = None

    def declare(self) -> Dict[str, TensorDecl]:
        """Full tensor names -> declaration."""
        return {}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Receives the host tensors it declared (an optional one may be absent)."""

    def step_hints(self, shape: "StepShape") -> Optional["StepHints"]:
        """Called once a step (per ``hint_key``) on the host, before the upload."""
        return None

    def graph_table_pages(self, pages: int, page_size: int) -> Optional[int]:
        """The block-table width (>= ``pages``) a captured decode step should be made for, if
        the part's kernels care (their grids follow it); None: the engine's own bucket."""
        return None

    def hint_providers(self) -> List["Part"]:
        """The parts below this one (itself included) that have hints to give."""
        return [self] if self.hint_key is not None else []


class Norm(Part):
    """A norm may let the products next to it do part of its work.  Both ways are optional and
    safe to leave out; the generic block and decoder only ever call these three methods.

    * ``deferred(x, make_out, left)``: a stand-in for the norm's output on the rows ``x`` for a
      consumer that says ``accepts_lazy_norm``: an object with ``shape``, ``materialize()``
      (runs the norm once, returns the activations) and ``fold_into(linear, out, **kw)`` (the
      product of the normed rows with ``linear``'s weight in one kernel, or False).  None:
      the norm simply runs.  ``left``: what ``residual_sum`` left for this norm, or None.
    * ``residual_sum(linear, a, out, step)``: out += a W^T in a kernel that also leaves
      something for this norm, which reads ``out`` next; puts it in ``step.norm_ready`` and
      returns True, or returns False and does nothing."""
    role = "norm"
    defers = False         # whether ``deferred`` can ever give a stand-in

    def forward(self, x: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    def deferred(self, x: torch.Tensor, make_out, left=None):
        return None

    def residual_sum(self, linear, a: torch.Tensor, out: torch.Tensor, step) -> bool:
        return False


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

    def accept_cache(self, cache) -> None:
        """Called once per run of the layer with the cache view the engine made for it; a
        mixer whose kernels cannot serve it (another dtype, another page size) raises
        ``ConfigError`` here, before any request runs."""

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

    def accept_cache(self, cache) -> None:
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
