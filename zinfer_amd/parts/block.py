from __future__ import annotations

from typing import Dict

import torch

from ..config.specs import PreNormBlockSpec
from .base import Block, TensorDecl, build_part, register_part


class PreNormBlock(Block):
    """x += mixer(norm(x)); x += feed_forward(norm(x)): the residual is the un-normed input
    (`src/model/runtime/optimized_decoder/layer.zig:108,188-201`).  The residual stream ``x``
    is float32; both sums happen in 32-bit inside the parts."""

    def __init__(self, spec: PreNormBlockSpec, ctx, prefix):
        super().__init__(spec, ctx, prefix)
        self.mixer_norm = build_part("norm", spec.mixer_norm, ctx, prefix + spec.mixer_norm_prefix)
        self.mixer = build_part("mixer", spec.mixer, ctx, prefix + spec.mixer_prefix)
        self.ff_norm = build_part("norm", spec.ff_norm, ctx, prefix + spec.ff_norm_prefix)
        self.feed_forward = build_part("feed_forward", spec.feed_forward, ctx,
                                       prefix + spec.ff_prefix)
        self.parts = (self.mixer_norm, self.mixer, self.ff_norm, self.feed_forward)
        # the norm that reads the residual stream first, if what a sum leaves for it is of use
        self.entry_norm = self._lazy(self.mixer_norm, self.mixer)
        self.graph_safe = all(p.graph_safe for p in self.parts)
        self.kernel_modules = tuple(sorted({m for p in self.parts for m in p.kernel_modules}))

    def declare(self) -> Dict[str, TensorDecl]:
        d: Dict[str, TensorDecl] = {}
        for part in self.parts:
            d.update(part.declare())
        return d

    def bind(self, tensors) -> None:
        for part in self.parts:
            part.bind(tensors)

    def cache_need(self):
        return self.mixer.cache_need()

    def accept_cache(self, cache) -> None:
        self.mixer.accept_cache(cache)

    def hint_providers(self):
        return [q for p in self.parts for q in p.hint_providers()]

    def _normed(self, norm, consumer, x, step):
        """The consumer's input: the normed activations, or, for a consumer that says it can
        take a norm that has not run, the norm's stand-in (``Norm.deferred``)."""
        make = lambda: step.scratch("normed", x.shape, self.ctx.act_dtype)
        left, step.norm_ready, step.norm_after = step.norm_ready, None, None
        if getattr(consumer, "accepts_lazy_norm", False):
            lazy = norm.deferred(x, make, left)
            if lazy is not None:
                return lazy
        return norm.forward(x, make())

    def _lazy(self, norm, consumer):
        """``norm`` if its reader takes a norm that has not run (and so what a residual sum
        leaves for it), else None."""
        return norm if norm.defers and getattr(consumer, "accepts_lazy_norm", False) else None

    def forward(self, x, step, cache) -> None:
        after_block = step.norm_after_block
        h = self._normed(self.mixer_norm, self.mixer, x, step)
        step.norm_after = self._lazy(self.ff_norm, self.feed_forward)
        self.mixer.forward(h, x, step, cache)
        h = self._normed(self.ff_norm, self.feed_forward, x, step)
        step.norm_after = after_block
        self.feed_forward.forward(h, x, step)
        step.norm_after = None


register_part("block", PreNormBlockSpec, PreNormBlock)
