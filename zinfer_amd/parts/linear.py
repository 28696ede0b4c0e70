"""A weight matrix [out, in] applied as y = x W^T, without bias
(`src/tensor/storage/store.zig:286-319`: y[r] = sum_c W[r, c] x[c])."""
from __future__ import annotations

import torch

from .. import ops


class Linear:
    """``pretile``: a bfloat16 matrix on the GPU whose sizes allow it is re-laid once into the
    MFMA kernels' own order; the copy in rows is not kept here (a caller that also reads the
    matrix by rows, as a tied embedding is read, keeps its own)."""

    def __init__(self, weight: torch.Tensor, pretile: bool = True):
        assert weight.dim() == 2
        self.out_features, self.in_features = weight.shape
        self.tiled = bool(pretile and weight.is_cuda and ops.can_pretile(weight))
        self.weight = ops.pretile_weight(weight) if self.tiled else weight.contiguous()

    def forward(self, x, out: torch.Tensor, accumulate: bool = False, step=None) -> torch.Tensor:
        """out = x W^T, or out += x W^T (``out`` float32) when ``accumulate``.  ``x`` may be a
        norm that has not run yet (what ``Norm.deferred`` gave): it folds itself into the
        product when it can, else it runs first.  With ``accumulate`` and a ``step`` that
        names the norm reading ``out`` next (``step.norm_after``), that norm may have the sum's
        kernel leave something for it (``Norm.residual_sum``, result in ``step.norm_ready``)."""
        if hasattr(x, "materialize"):
            if not accumulate and x.fold_into(self, out):
                return out
            x = x.materialize()
        norm = getattr(step, "norm_after", None) if accumulate else None
        if norm is not None and norm.residual_sum(self, x, out, step):
            return out
        ops.gemm(x, self.weight, out, accumulate, w_tiled=self.tiled)
        return out

    def forward_partials(self, x):
        """The float32 partials [ksplit, T, out] of x W^T where the product is one that runs
        split along K and would need a kernel of its own to add them (17 to 128 tokens), for
        a caller whose next kernel can add them on its way; else None (then ``forward``)."""
        M, K = x.shape
        ks = ops.gemm_partials_plan(M, self.out_features, K, self.weight, self.tiled)
        if ks is None:
            return None
        if hasattr(x, "materialize"):
            x = x.materialize()
        if x.dtype != torch.bfloat16:
            return None
        return ops.gemm_partials(x, self.weight, ks)


def place_matrix(t: torch.Tensor, ctx) -> torch.Tensor:
    """A matrix on the device: bfloat16 stays bfloat16 under a bfloat16 build, a tensor
    stored in 32-bit stays so; a float32 build widens everything (float16 exactly).  A
    matrix stored in float16 or float64 is rounded to bfloat16 under a bfloat16 build: as
    32-bit data it would take twice the bytes and miss the MFMA kernels."""
    if ctx.compute_dtype == torch.float32 and t.dtype == torch.bfloat16 \
            and torch.device(ctx.device).type == "cuda":
        # half the bytes go over the bus; the widening (exact) runs on the device
        from .. import ops
        src = t.to(ctx.device).contiguous()
        out = torch.empty(src.shape, dtype=torch.float32, device=src.device)
        ops.cast(src, out)
        return out
    if ctx.compute_dtype == torch.float32:
        t = t.to(torch.float32)
    elif t.dtype not in (torch.bfloat16, torch.float32):
        t = t.to(torch.bfloat16)
    return t.to(ctx.device).contiguous()


def place_gain(t: torch.Tensor, ctx) -> torch.Tensor:
    """A norm's gain vector, widened to float32 once at load as the reference does
    (`src/model/runtime/optimized_decoder/support.zig:6-19`)."""
    return t.to(torch.float32).to(ctx.device).contiguous()
