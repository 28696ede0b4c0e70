from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..config.specs import RmsNormSpec
from .base import Norm, TensorDecl, register_part
from .linear import place_gain


class RmsNorm(Norm):
    """n = x * w / sqrt(mean(x^2) + eps) (`src/kernel/core/cpu.zig:38-48,73-110`); reads the
    float32 residual stream, writes the activation dtype.

    Under bfloat16 on the GPU the norm can be taken apart by the products around it: the
    weight-streaming product folds it in (``LazyRmsNorm.fold_into``), and the product that
    last adds into the residual can leave the norm's inputs or its whole result
    (``residual_sum``)."""
    graph_safe = True
    defers = True
    kernel_modules = ("elementwise",)


    def declare(self) -> Dict[str, TensorDecl]:
        return {self.prefix + "weight": TensorDecl((self.spec.width,), init="gain")}

    def bind(self, tensors) -> None:
        self.gain = place_gain(tensors[self.prefix + "weight"], self.ctx)

    def forward(self, x: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        ops.rmsnorm(x, self.gain, float(self.spec.eps), out)
        return out

    def deferred(self, x: torch.Tensor, make_out, left=None):
        if not (x.is_cuda and self.ctx.compute_dtype == torch.bfloat16):
            return None
        given = left if left is not None and left.fits(self, x) else None
        return LazyRmsNorm(self, x, make_out, given)

    def residual_sum(self, linear, a: torch.Tensor, out: torch.Tensor, step) -> bool:
        if a.dtype != torch.bfloat16:
            return False
        M, N, K = a.shape[0], linear.out_features, linear.in_features
        if ops.norm_emit_plan(M, N, K, linear.weight, linear.tiled) is not None:
            xg = step.scratch("normed_by_gain", out.shape, torch.bfloat16)
            sq = step.scratch("normed_squares", (N // 16, 16), torch.float32)
            ops.gemm_emit(a, linear.weight, out, self.gain, xg, sq)
            step.norm_ready = GivenRmsNorm(self, out, xg, sq)
            return True
        if ops.sum_norm_plan(M, N, K, linear.weight, linear.tiled) is not None:
            normed = step.scratch("normed_by_sum", out.shape, torch.bfloat16)
            ops.gemm_sum_norm(a, linear.weight, out, self.gain, float(self.spec.eps), normed)
            step.norm_ready = DoneRmsNorm(self, out, normed)
            return True
        return False


class GivenRmsNorm:
    """What the kernel that last added into the residual rows ``x`` left for ``norm``:
    xg = bfloat16(x * gain) and sq [width / 16, 16], the sums of x^2 over each 16 columns per
    token (``ops.gemm_emit``)."""

    def __init__(self, norm: "RmsNorm", x: torch.Tensor, xg: torch.Tensor, sq: torch.Tensor):
        self.norm, self.x, self.xg, self.sq = norm, x, xg, sq

    def fits(self, norm, x: torch.Tensor) -> bool:
        return self.norm is norm and self.x.data_ptr() == x.data_ptr() and self.x.shape == x.shape


class DoneRmsNorm:
    """The norm of the residual rows ``x`` already run by the kernel that last added into them
    (``ops.gemm_sum_norm``): ``normed`` holds the result."""

    def __init__(self, norm: "RmsNorm", x: torch.Tensor, normed: torch.Tensor):
        self.norm, self.x, self.normed = norm, x, normed

    def fits(self, norm, x: torch.Tensor) -> bool:
        return self.norm is norm and self.x.data_ptr() == x.data_ptr() and self.x.shape == x.shape


class LazyRmsNorm:
    """A norm that has not run yet: the residual rows and the norm's parameters.  A consumer
    whose first matrix product can fold the norm in (``Linear.forward``) takes it apart;
    anyone else calls ``materialize()`` and gets the normed activations (computed once).
    ``given``: what the producer of the rows already left of the norm, if anything: its
    inputs (``GivenRmsNorm``) or its whole result (``DoneRmsNorm``)."""

    def __init__(self, norm: "RmsNorm", x: torch.Tensor, make_out, given: GivenRmsNorm = None):
        self.x, self.gain, self.eps = x, norm.gain, float(norm.spec.eps)
        self.shape = x.shape
        self._norm, self._make_out, self._out = norm, make_out, None
        if isinstance(given, DoneRmsNorm):
            given, self._out = None, given.normed
        self.given = given

    @property
    def done(self) -> bool:
        return self._out is not None

    def materialize(self) -> torch.Tensor:
        if self._out is None:
            self._out = self._make_out()
            self._norm.forward(self.x, self._out)
        return self._out

    def fold_into(self, linear, out: torch.Tensor, swiglu: bool = False) -> bool:
        """out = norm(x) W^T (with ``swiglu`` the activation of a stacked gate/up weight) in
        the weight-streaming product, from the residual rows or from what their producer
        left; False (and nothing done) where that kernel does not cover the sizes."""
        M, K = self.shape
        if self.done or not linear.tiled:
            return False
        if swiglu:
            if M > ops.NORM_FOLD_MAX_M:
                return False
        elif ops.norm_gemm_plan(M, linear.out_features, K, linear.weight, True) is None:
            return False
        if self.given is not None:
            ops.gemm_given(self.given.xg, self.given.sq, self.eps, linear.weight, out,
                           swiglu=swiglu)
        else:
            ops.norm_gemm(self.x, self.gain, self.eps, linear.weight, out, swiglu=swiglu)
        return True


register_part("norm", RmsNormSpec, RmsNorm)
