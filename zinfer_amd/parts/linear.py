"""A weight matrix [out, in] applied as y = x W^T, without bias
(`src/tensor/storage/store.zig:286-319`: y[r] = sum_c W[r, c] x[c])."""
from __future__ import annotations

import torch

from .. import ops


class Linear:
    def __init__(self, weight: torch.Tensor):
        assert weight.dim() == 2
        self.weight = weight.contiguous()
        self.out_features, self.in_features = weight.shape

    def forward(self, x: torch.Tensor, out: torch.Tensor, accumulate: bool = False) -> torch.Tensor:
        """out = x W^T, or out += x W^T (``out`` float32) when ``accumulate``."""
        ops.gemm(x, self.weight, out, accumulate)
        return out


def place_matrix(t: torch.Tensor, ctx) -> torch.Tensor:
    """A matrix on the device: bfloat16 stays bfloat16 under a bfloat16 build, a tensor
    stored in 32-bit stays so; a float32 build widens everything."""
    if ctx.compute_dtype == torch.float32:
        t = t.to(torch.float32)
    elif t.dtype not in (torch.bfloat16, torch.float32):
        t = t.to(torch.float32)
    return t.to(ctx.device).contiguous()


def place_gain(t: torch.Tensor, ctx) -> torch.Tensor:
    """A norm's gain vector, widened to float32 once at load as the reference does
    (`src/model/runtime/optimized_decoder/support.zig:6-19`)."""
    return t.to(torch.float32).to(ctx.device).contiguous()
