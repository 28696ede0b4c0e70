"""The engine's operations: thin wrappers that check shapes on the host and launch the
hand-written HIP kernels on torch's current stream.  There is no other implementation: a
tensor that is not on the GPU, or a kernel library that cannot be built or loaded, is an
error.  Kernels take every size a configuration allows or refuse it with a clear message.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from ..errors import KernelUnavailable
from . import build

_DT = {torch.float32: 0, torch.bfloat16: 1}
_vp = ctypes.c_void_p


def _stream() -> ctypes.c_void_p:
    return _vp(torch.cuda.current_stream().cuda_stream)


def _ptr(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return _vp(None) if t is None else _vp(t.data_ptr())


def _need_gpu(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelUnavailable(
                "the HIP kernels run on GPU tensors only; got a tensor on "
                f"{t.device} (there is no CPU path)")
        if t is not None and not t.is_contiguous():
            raise KernelUnavailable(f"kernel operands must be contiguous; got strides {t.stride()}")


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelUnavailable(f"kernels take float32 or bfloat16, not {t.dtype}") from None


def _check(code: int, what: str) -> None:
    if code != 0:
        raise KernelUnavailable(f"{what}: launch failed with code {code}")


def _i32(t: torch.Tensor, what: str) -> None:
    if t.dtype != torch.int32:
        raise KernelUnavailable(f"{what} must be int32, is {t.dtype}")


# ------------------------------------------------------------------------- elementwise
def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor) -> None:
    """out[t, :] = table[ids[t], :] widened to float32 (no scale factor)."""
    _need_gpu(table, ids, out)
    _i32(ids, "ids")
    T, H = out.shape
    if table.shape[1] != H or ids.shape[0] != T or out.dtype != torch.float32:
        raise KernelUnavailable(f"embed: table {tuple(table.shape)}, ids {tuple(ids.shape)}, "
                                f"out {tuple(out.shape)} {out.dtype}")
    lib = build.load("elementwise")
    _check(lib.zf_embed(_ptr(table), _dt(table), _ptr(ids), _ptr(out), T, H, _stream()), "embed")


def rmsnorm(x: torch.Tensor, gain: torch.Tensor, eps: float, out: torch.Tensor) -> None:
    """out = x * gain / sqrt(mean(x^2) + eps) over the last axis; x and gain float32."""
    _need_gpu(x, gain, out)
    T, W = x.shape
    if x.dtype != torch.float32 or gain.dtype != torch.float32 or gain.shape != (W,) \
            or out.shape != x.shape:
        raise KernelUnavailable(f"rmsnorm: x {tuple(x.shape)} {x.dtype}, gain "
                                f"{tuple(gain.shape)} {gain.dtype}, out {tuple(out.shape)}")
    lib = build.load("elementwise")
    _check(lib.zf_rmsnorm(_ptr(x), _ptr(gain), _ptr(out), _dt(out), T, W, ctypes.c_float(eps),
                          _stream()), "rmsnorm")


def qk_norm_rope_kv_write(qkv, q_gain, k_gain, eps, cos, sin, positions, slot_mapping, k_pool,
                          v_pool, q_out, n_heads, n_kv_heads, head_dim, page_size) -> None:
    """Per token and head of ``qkv`` [T, (nH + 2 nKV) hd]: optional RMSNorm of q and k heads
    with the [hd] gains, optional half-split rotation from the [max_pos, hd/2] tables at
    ``positions``; q goes to ``q_out`` [T, nH hd] (in place if None), k and v go into the
    pools at ``slot_mapping`` (k in place if None)."""
    _need_gpu(qkv, q_gain, k_gain, cos, sin, positions, slot_mapping, k_pool, v_pool, q_out)
    T = qkv.shape[0]
    width = (n_heads + 2 * n_kv_heads) * head_dim
    if qkv.shape[1] != width or head_dim % 2 != 0:
        raise KernelUnavailable(f"qk_norm_rope_kv_write: qkv {tuple(qkv.shape)} for "
                                f"{n_heads}+2*{n_kv_heads} heads of {head_dim} (even)")
    if (q_gain is None) != (k_gain is None) or (cos is None) != (sin is None):
        raise KernelUnavailable("qk_norm_rope_kv_write: gains and tables come in pairs")
    for g in (q_gain, k_gain):
        if g is not None and (g.dtype != torch.float32 or g.shape != (head_dim,)):
            raise KernelUnavailable("qk_norm_rope_kv_write: a gain must be float32 [head_dim]")
    if cos is not None and (cos.dtype != torch.float32 or cos.shape[1] != head_dim // 2
                            or cos.shape != sin.shape):
        raise KernelUnavailable("qk_norm_rope_kv_write: tables must be float32 [*, head_dim/2]")
    _i32(positions, "positions")
    if slot_mapping is not None:
        _i32(slot_mapping, "slot_mapping")
        if k_pool.dtype != qkv.dtype or v_pool.dtype != qkv.dtype:
            raise KernelUnavailable("qk_norm_rope_kv_write: pools and qkv differ in dtype")
    if q_out is not None and (q_out.dtype != qkv.dtype
                              or q_out.shape != (T, n_heads * head_dim)):
        raise KernelUnavailable("qk_norm_rope_kv_write: q_out must be [T, nH * hd] of qkv's dtype")
    lib = build.load("elementwise")
    _check(lib.zf_qk_norm_rope_kv_write(
        _ptr(qkv), _dt(qkv), _ptr(q_gain), _ptr(k_gain), ctypes.c_float(eps), _ptr(cos),
        _ptr(sin), _ptr(positions), _ptr(slot_mapping), _ptr(k_pool), _ptr(v_pool), _ptr(q_out),
        T, n_heads, n_kv_heads, head_dim, page_size, _stream()), "qk_norm_rope_kv_write")


def swiglu(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    """out[t, j] = silu(gate_up[t, j]) * gate_up[t, I + j]."""
    _need_gpu(gate_up, out)
    T, I = out.shape
    if gate_up.shape != (T, 2 * I) or gate_up.dtype != out.dtype:
        raise KernelUnavailable(f"swiglu: gate_up {tuple(gate_up.shape)}, out {tuple(out.shape)}")
    lib = build.load("elementwise")
    _check(lib.zf_swiglu(_ptr(gate_up), _ptr(out), _dt(out), T, I, _stream()), "swiglu")


def gather_rows(x: torch.Tensor, idx: torch.Tensor, out: torch.Tensor) -> None:
    _need_gpu(x, idx, out)
    _i32(idx, "idx")
    n, H = out.shape
    if x.shape[1] != H or idx.shape[0] != n or x.dtype != torch.float32 or out.dtype != x.dtype:
        raise KernelUnavailable("gather_rows: float32 [T, H] -> [n, H]")
    lib = build.load("elementwise")
    _check(lib.zf_gather_rows(_ptr(x), _ptr(idx), _ptr(out), n, H, _stream()), "gather_rows")


def argmax(logits: torch.Tensor, out: torch.Tensor) -> None:
    """out[r] = index of the first maximum of logits[r, :]."""
    _need_gpu(logits, out)
    _i32(out, "out")
    n, V = logits.shape
    if logits.dtype != torch.float32 or out.shape != (n,):
        raise KernelUnavailable("argmax: float32 [n, V] -> int32 [n]")
    lib = build.load("elementwise")
    _check(lib.zf_argmax(_ptr(logits), _ptr(out), n, V, _stream()), "argmax")


# ------------------------------------------------------------------------- matrix product
def gemm(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False) -> None:
    """out = a w^T (w is [N, K]); with ``accumulate`` out += a w^T, in 32-bit."""
    _need_gpu(a, w, out)
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K or out.shape != (M, N):
        raise KernelUnavailable(f"gemm: a {tuple(a.shape)}, w {tuple(w.shape)}, "
                                f"out {tuple(out.shape)}")
    if accumulate and out.dtype != torch.float32:
        raise KernelUnavailable("gemm: accumulation needs a float32 output")
    lib = build.load("gemm")
    _check(lib.zf_gemm_fma(_ptr(a), _dt(a), _ptr(w), _dt(w), _ptr(out), _dt(out), M, N, K,
                           1 if accumulate else 0, _stream()), "gemm")


# ------------------------------------------------------------------------- attention
def paged_attention(q, k_pool, v_pool, block_table, q_start, ctx_len, seq_index, out, scale,
                    window, n_heads, n_kv_heads, head_dim, page_size, max_q_len,
                    max_ctx_len) -> None:
    """Causal grouped-query attention of the step's tokens over the paged cache.  Token t of
    sequence s = seq_index[t] has position ctx_len[s] - q_len[s] + (t - q_start[s]) and reads
    the positions up to its own (the last ``window`` of them if window > 0)."""
    _need_gpu(q, k_pool, v_pool, block_table, q_start, ctx_len, seq_index, out)
    T = q.shape[0]
    if q.shape != (T, n_heads * head_dim) or out.shape != q.shape or out.dtype != q.dtype \
            or k_pool.dtype != q.dtype or v_pool.dtype != q.dtype:
        raise KernelUnavailable("paged_attention: q/out must be [T, nH * hd] of the pools' dtype")
    for t, name in ((block_table, "block_table"), (q_start, "q_start"), (ctx_len, "ctx_len"),
                    (seq_index, "seq_index")):
        _i32(t, name)
    if n_heads % n_kv_heads != 0:
        raise KernelUnavailable("paged_attention: InvalidGrouping")
    if head_dim > 512:
        raise KernelUnavailable(f"paged_attention: head_dim {head_dim} > 512 is not covered")
    if max_ctx_len > block_table.shape[1] * page_size:
        raise KernelUnavailable("paged_attention: block table shorter than the context")
    lib = build.load("attention")
    _check(lib.zf_paged_attention_wave(
        _ptr(q), _ptr(k_pool), _ptr(v_pool), _dt(q), _ptr(block_table), _ptr(q_start),
        _ptr(ctx_len), _ptr(seq_index), _ptr(out), ctypes.c_float(scale), int(window), T,
        n_heads, n_kv_heads, head_dim, page_size, block_table.shape[1], _stream()),
        "paged_attention")
