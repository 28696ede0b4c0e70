from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..config.specs import RmsNormSpec
from .base import Norm, TensorDecl, register_part
from .linear import place_gain


class RmsNorm(Norm):
    """n = x * w / sqrt(mean(x^2) + eps) (`src/kernel/core/cpu.zig:38-48,73-110`); reads the
    float32 residual stream, writes the activation dtype."""
    graph_safe = True
    kernel_modules = ("elementwise",)


    def declare(self) -> Dict[str, TensorDecl]:
        return {self.prefix + "weight": TensorDecl((self.spec.width,), init="gain")}

    def bind(self, tensors) -> None:
        self.gain = place_gain(tensors[self.prefix + "weight"], self.ctx)

    def forward(self, x: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        ops.rmsnorm(x, self.gain, float(self.spec.eps), out)
        return out


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


register_part("norm", RmsNormSpec, RmsNorm)
