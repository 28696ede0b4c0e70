"""One flat table of the engine's kernels: name -> (the function that launches it, the csrc
module it lives in, where the reference implementation states the formula it computes).  The
reference's counterpart is its table of ops that the per-op benchmark walks
(`src/app/cli/tools/bench/ops.zig:12-49`).  Kernels without a counterpart there (paging,
batching, fusions of two of the reference's operations) name the operations they are made of,
or say "own"."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict

from . import (advance_decode, apply_penalties, argmax, argmax_no_alloc, cast, check_tables,
               decode_attention_fused, embed, gather_rows, gemm, gemm_emit, gemm_given,
               gemm_partials, gemm_sum_norm, gemm_swiglu, mfma_loop, norm_gemm, paged_attention,
               poison_pages,
               qk_norm_rope_kv_write, randinit, rmsnorm, sample_topk, scale_cap, stream_read,
               swiglu)


@dataclass(frozen=True)
class KernelEntry:
    launch: Callable
    module: str          # csrc/<module>.hip
    formula: str         # file:lines of the reference implementation, or "own: ..."


_LINEAR = "src/kernel/core/cpu.zig:21-36"
_RMSNORM = "src/kernel/core/cpu.zig:38-48,73-110"
_ATTENTION = "src/kernel/attention/basic.zig:5-76"
_QK = "src/kernel/core/cpu.zig:50-71; src/kernel/attention/rope.zig:25-34,67-90"

KERNELS: Dict[str, KernelEntry] = {
    "embed": KernelEntry(embed, "elementwise", "src/model/layers/decoder_only_stack.zig:48-93"),
    "rmsnorm": KernelEntry(rmsnorm, "elementwise", _RMSNORM),
    "qk_norm_rope_kv_write": KernelEntry(
        qk_norm_rope_kv_write, "elementwise",
        _QK + "; src/model/runtime/optimized_kv_cache/cache.zig:21-107"),
    "swiglu": KernelEntry(swiglu, "elementwise", "src/kernel/core/cpu.zig:130-147"),
    "gather_rows": KernelEntry(gather_rows, "elementwise", "own: rows whose logits are wanted"),
    "argmax": KernelEntry(argmax, "elementwise", "src/model/layers/logits.zig:47-59"),
    "argmax_no_alloc": KernelEntry(argmax_no_alloc, "elementwise",
                                   "src/model/layers/logits.zig:47-59"),
    "scale_cap": KernelEntry(scale_cap, "elementwise", "own: logit scale and tanh cap"),
    "advance_decode": KernelEntry(advance_decode, "elementwise",
                                  "own: positions and slots of the next decode step"),
    "cast": KernelEntry(cast, "elementwise", "src/tensor/formats/bfloat16.zig:3-13"),
    "poison_pages": KernelEntry(poison_pages, "elementwise", "own: NaN into pages given back"),
    "gemm": KernelEntry(gemm, "gemm", _LINEAR),
    "gemm_partials": KernelEntry(gemm_partials, "gemm", _LINEAR),
    "gemm_swiglu": KernelEntry(gemm_swiglu, "gemm", _LINEAR + "; src/kernel/core/cpu.zig:130-147"),
    "norm_gemm": KernelEntry(norm_gemm, "gemm", _RMSNORM + "; " + _LINEAR),
    "gemm_emit": KernelEntry(gemm_emit, "gemm", _LINEAR + "; " + _RMSNORM),
    "gemm_given": KernelEntry(gemm_given, "gemm", _RMSNORM + "; " + _LINEAR),
    "gemm_sum_norm": KernelEntry(gemm_sum_norm, "gemm", _LINEAR + "; " + _RMSNORM),
    "paged_attention": KernelEntry(paged_attention, "attention", _ATTENTION),
    "decode_attention_fused": KernelEntry(decode_attention_fused, "attention",
                                          _QK + "; " + _ATTENTION),
    "apply_penalties": KernelEntry(apply_penalties, "sampling",
                                   "src/sampling/sampler.zig:186-201"),
    "sample_topk": KernelEntry(sample_topk, "sampling", "src/sampling/sampler.zig:18-91"),
    "randinit": KernelEntry(randinit, "randinit", "own: counter-based random weights"),
    "check_tables": KernelEntry(check_tables, "elementwise",
                                "own: a step's block tables and slots against the pool"),
    "stream_read": KernelEntry(stream_read, "elementwise",
                               "own: the read stream bandwidths are measured against"),
    "mfma_loop": KernelEntry(mfma_loop, "gemm",
                             "own: MFMAs alone, the rate the tiled products are measured against"),
}
