"""Helpers of the GPU tests: tolerances and the comparison with the plain implementation."""
from __future__ import annotations

import torch

DEV = "cuda:0"


def rel_err(got: torch.Tensor, ref: torch.Tensor) -> float:
    """Largest absolute difference, relative to the largest reference magnitude."""
    ref = ref.to(torch.float64).cpu()
    got = got.to(torch.float64).cpu()
    return float((got - ref).abs().max() / ref.abs().max().clamp_min(1e-30))


# float32 kernels accumulate in 32-bit: a few 1e-7 per operation; 2e-5 of the largest
# magnitude leaves room for sums over a few thousand terms and nothing more.
F32_TOL = 2e-5
# bfloat16 storage rounds to 8 bits of mantissa (2^-9 relative per rounding); a kernel's
# output is rounded once, its inputs are exact in the comparison.
BF16_KERNEL_TOL = 2.0 ** -8


def tol(dtype) -> float:
    return F32_TOL if dtype == torch.float32 else BF16_KERNEL_TOL
