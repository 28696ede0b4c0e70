from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..config.specs import SwiGluSpec
from .base import FeedForward, TensorDecl, register_part
from .linear import Linear, place_matrix


class SwiGluMlp(FeedForward):
    """d = W_down (silu(W_gate m) * W_up m), added to the residual
    (`src/model/runtime/optimized_decoder/layer.zig:194-201`, `src/kernel/core/cpu.zig:130-147`).
    gate and up rows are stacked into one matrix at load: each output keeps its own dot
    product."""
    graph_safe = True
    accepts_lazy_norm = True
    kernel_modules = ("elementwise", "gemm")


    def declare(self) -> Dict[str, TensorDecl]:
        s, p = self.spec, self.prefix
        return {p + "gate_proj.weight": TensorDecl((s.intermediate_size, s.hidden_size)),
                p + "up_proj.weight": TensorDecl((s.intermediate_size, s.hidden_size)),
                p + "down_proj.weight": TensorDecl((s.hidden_size, s.intermediate_size))}

    def bind(self, tensors) -> None:
        p = self.prefix
        g, u = tensors[p + "gate_proj.weight"], tensors[p + "up_proj.weight"]
        if g.dtype != u.dtype:
            g, u = g.float(), u.float()
        g, u = place_matrix(g, self.ctx), place_matrix(u, self.ctx)
        # bfloat16 on the GPU with sizes the MFMA kernels take: gate and up rows alternate in
        # groups of 16 and the activation runs in the product's epilogue
        self.fused = self.ctx.compute_dtype == torch.bfloat16 and g.shape[0] % 32 == 0 \
            and ops.can_fuse_swiglu(_probe(g))
        stacked = ops.interleave_gate_up(g, u) if self.fused else torch.cat([g, u], dim=0)
        del g, u
        self.gate_up = Linear(stacked)
        self.down = Linear(place_matrix(tensors[p + "down_proj.weight"], self.ctx))

    def forward(self, h, residual, step) -> None:
        T = h.shape[0]
        I = self.spec.intermediate_size
        act = self.ctx.act_dtype
        a = step.scratch("ff_act", (T, I), act)
        if hasattr(h, "materialize"):
            # a norm that has not run: the gate/up product folds it in where it can
            if self.fused and h.fold_into(self.gate_up, a, swiglu=True):
                self.down.forward(a, residual, accumulate=True, step=step)
                return
            h = h.materialize()
        if self.fused and h.dtype == torch.bfloat16:
            ops.gemm_swiglu(h, self.gate_up.weight, a, w_tiled=self.gate_up.tiled)
        else:
            gu = step.scratch("gate_up", (T, 2 * I), act)
            self.gate_up.forward(h, gu)
            ops.swiglu(gu, a)
        self.down.forward(a, residual, accumulate=True, step=step)


class _probe:
    """Shape and placement of the stacked gate/up matrix, without building it."""

    def __init__(self, g: torch.Tensor):
        self.is_cuda, self.dtype, self.shape = g.is_cuda, g.dtype, (2 * g.shape[0], g.shape[1])


register_part("feed_forward", SwiGluSpec, SwiGluMlp)
