"""One flat table of the engine's kernels: name -> (the function that launches it, the csrc
module it lives in, the plain reference it is tested against).  The reference's counterpart is
its table of ops that the per-op benchmark walks (`src/app/cli/tools/bench/ops.zig:12-49`).
References are named, not imported: those under ``tests/`` are no part of the package."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict

from . import (advance_decode, apply_penalties, argmax, argmax_no_alloc, cast,
               decode_attention_fused, embed, gather_rows, gemm, gemm_emit, gemm_given,
               gemm_partials, gemm_sum_norm, gemm_swiglu, norm_gemm, paged_attention, poison_pages,
               qk_norm_rope_kv_write, randinit, rmsnorm, sample_topk, scale_cap, swiglu)


@dataclass(frozen=True)
class KernelEntry:
    launch: Callable
    module: str          # csrc/<module>.hip
    reference: str       # "file:function" of the plain implementation its test compares with


KERNELS: Dict[str, KernelEntry] = {
    "embed": KernelEntry(embed, "elementwise", "tests/kernel_refs.py:embed"),
    "rmsnorm": KernelEntry(rmsnorm, "elementwise", "tests/kernel_refs.py:rmsnorm"),
    "qk_norm_rope_kv_write": KernelEntry(qk_norm_rope_kv_write, "elementwise",
                                         "tests/kernel_refs.py:qk_norm_rope_kv_write"),
    "swiglu": KernelEntry(swiglu, "elementwise", "tests/kernel_refs.py:swiglu"),
    "gather_rows": KernelEntry(gather_rows, "elementwise", "tests/kernel_refs.py:gather_rows"),
    "argmax": KernelEntry(argmax, "elementwise", "tests/kernel_refs.py:argmax"),
    "argmax_no_alloc": KernelEntry(argmax_no_alloc, "elementwise", "tests/kernel_refs.py:argmax"),
    "scale_cap": KernelEntry(scale_cap, "elementwise", "tests/kernel_refs.py:scale_cap"),
    "advance_decode": KernelEntry(advance_decode, "elementwise",
                                  "tests/test_engine_gpu.py:test_decode_steps_in_a_row_equal_single_steps"),
    "cast": KernelEntry(cast, "elementwise", "tests/test_kernels_gpu.py:test_cast_and_poison_pages"),
    "poison_pages": KernelEntry(poison_pages, "elementwise",
                                "tests/test_kernels_gpu.py:test_cast_and_poison_pages"),
    "gemm": KernelEntry(gemm, "gemm", "tests/kernel_refs.py:gemm"),
    "gemm_partials": KernelEntry(gemm_partials, "gemm", "tests/kernel_refs.py:gemm"),
    "gemm_swiglu": KernelEntry(gemm_swiglu, "gemm", "tests/kernel_refs.py:gemm_swiglu"),
    "norm_gemm": KernelEntry(norm_gemm, "gemm", "tests/kernel_refs.py:rmsnorm"),
    "gemm_emit": KernelEntry(gemm_emit, "gemm", "tests/kernel_refs.py:gemm"),
    "gemm_given": KernelEntry(gemm_given, "gemm", "tests/kernel_refs.py:rmsnorm"),
    "gemm_sum_norm": KernelEntry(gemm_sum_norm, "gemm", "tests/kernel_refs.py:rmsnorm"),
    "paged_attention": KernelEntry(paged_attention, "attention",
                                   "tests/kernel_refs.py:paged_attention"),
    "decode_attention_fused": KernelEntry(
        decode_attention_fused, "attention",
        "tests/test_kernels_gpu.py:test_decode_attention_fused_equals_the_two_kernels"),
    "apply_penalties": KernelEntry(apply_penalties, "sampling",
                                   "zinfer_amd/sampling/sampler.py:adjust_logits"),
    "sample_topk": KernelEntry(sample_topk, "sampling",
                               "zinfer_amd/sampling/sampler.py:sample_token"),
    "randinit": KernelEntry(randinit, "randinit", "zinfer_amd/weights/counter_rng.py:draw"),
}
