"""The engine's operations: thin wrappers that check shapes on the host and launch the
hand-written HIP kernels on torch's current stream.  There is no other implementation: a
tensor that is not on the GPU, or a kernel library that cannot be built or loaded, is an
error.  Kernels take every size a configuration allows or refuse it with a clear message.
"""
from __future__ import annotations

import ctypes
import functools
from typing import Optional, Tuple

import torch

from ..errors import KernelUnavailable
from . import build

_DT = {torch.float32: 0, torch.bfloat16: 1}
_vp = ctypes.c_void_p


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> ctypes.c_void_p:
    """torch's current HIP stream of the current device (the capture stream inside a graph
    capture); read through torch's raw-handle call where it has one: a launch costs a few
    microseconds of host time, and building a Stream object was half of that."""
    if _raw_stream is not None:
        return _vp(_raw_stream(torch.cuda.current_device()))
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


# ------------------------------------------------------------------------- kernel classes
# Every launcher belongs to a class of a step's work; the per-class benchmark
# (``Engine.class_times``, the reference's per-op harness is `src/app/cli/tools/bench/
# ops.zig:516-543`) runs a step with only one class's kernels launched, the others left out.
# The outputs of such a run mean nothing; only its time does.
KERNEL_CLASSES = ("products", "attention", "norm_rope_write", "head_sampling", "other")
_class_filter = None        # None: everything launches; else the set of classes that do
_class_override = None      # a caller's label for the launches inside it (the head's product)
_launch_count = 0           # launcher calls that went through


def launch_count() -> int:
    return _launch_count


class only_classes:
    """Within this context only kernels of ``classes`` are launched."""

    def __init__(self, classes):
        unknown = set(classes) - set(KERNEL_CLASSES)
        if unknown:
            raise KernelUnavailable(f"unknown kernel classes {sorted(unknown)}")
        self.classes = frozenset(classes)

    def __enter__(self):
        global _class_filter
        self._before, _class_filter = _class_filter, self.classes

    def __exit__(self, *exc):
        global _class_filter
        _class_filter = self._before


class kernel_class:
    """Launches inside this context count as ``name`` whatever their launcher's own class."""

    def __init__(self, name: str):
        self.name = name

    def __enter__(self):
        global _class_override
        self._before, _class_override = _class_override, self.name

    def __exit__(self, *exc):
        global _class_override
        _class_override = self._before


def _left_out(cls: str) -> bool:
    return _class_filter is not None and (_class_override or cls) not in _class_filter


def _launches(cls: str):
    """Marks a launcher with its class; under ``only_classes`` a launcher of another class
    returns without launching."""
    def deco(fn):
        @functools.wraps(fn)
        def launcher(*args, **kwargs):
            global _launch_count
            if _class_filter is not None and (_class_override or cls) not in _class_filter:
                return None
            _launch_count += 1
            return fn(*args, **kwargs)
        launcher.kernel_class = cls
        return launcher
    return deco


# ------------------------------------------------------------------------- elementwise
@_launches("other")
def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> None:
    """out[t, :] = table[ids[t], :] widened to float32, times ``scale``."""
    _need_gpu(table, ids, out)
    _i32(ids, "ids")
    T, H = out.shape
    if table.shape[1] != H or ids.shape[0] != T or out.dtype != torch.float32:
        raise KernelUnavailable(f"embed: table {tuple(table.shape)}, ids {tuple(ids.shape)}, "
                                f"out {tuple(out.shape)} {out.dtype}")
    lib = build.load("elementwise")
    _check(lib.zf_embed(_ptr(table), _dt(table), _ptr(ids), _ptr(out), T, H,
                        ctypes.c_float(scale), _stream()), "embed")


@_launches("head_sampling")
def scale_cap(x: torch.Tensor, scale: float = 1.0, cap: float = 0.0) -> None:
    """In place on float32: x = x * scale, then with cap > 0: x = cap * tanh(x / cap)."""
    _need_gpu(x)
    if x.dtype != torch.float32 or cap < 0.0:
        raise KernelUnavailable("scale_cap: a float32 tensor and a cap that is not negative")
    lib = build.load("elementwise")
    _check(lib.zf_scale_cap(_ptr(x), ctypes.c_longlong(x.numel()), ctypes.c_float(scale),
                            ctypes.c_float(cap), _stream()), "scale_cap")


@_launches("norm_rope_write")
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


@_launches("norm_rope_write")
def qk_norm_rope_kv_write(qkv, q_gain, k_gain, eps, cos, sin, positions, slot_mapping, k_pool,
                          v_pool, q_out, n_heads, n_kv_heads, head_dim, page_size) -> None:
    """Per token and head of ``qkv`` [T, (nH + 2 nKV) hd]: optional RMSNorm of q and k heads
    with the [hd] gains, optional half-split rotation from the [max_pos, hd/2] tables at
    ``positions``; q goes to ``q_out`` [T, nH hd] (in place if None), k and v go into the
    pools at ``slot_mapping`` (k in place if None).  Pools of a shape the MFMA attention
    kernels cover (``mfma_attention_covers``) are written in those kernels' own order.

    ``qkv`` may also be the float32 partials [ksplit, T, (nH + 2 nKV) hd] of a product split
    along K (``gemm_partials``): the kernel adds them in split order and rounds to bfloat16
    on its way, as the kernel that only adds them would have (bfloat16 pools, ``q_out`` and
    ``slot_mapping`` given)."""
    partials = qkv if qkv.dim() == 3 else None
    if partials is not None:
        if partials.dtype != torch.float32 or not partials.is_contiguous() or q_out is None \
                or slot_mapping is None or k_pool.dtype != torch.bfloat16 \
                or head_dim % 8 != 0 or head_dim > 512:
            raise KernelUnavailable("qk_norm_rope_kv_write: partials must be contiguous float32 "
                                    "[ksplit, T, width], with q_out, slot_mapping and bfloat16 "
                                    "pools, head_dim a multiple of 8 up to 512")
        qkv = partials[0]
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
    row_dtype = torch.bfloat16 if partials is not None else qkv.dtype
    if slot_mapping is not None:
        _i32(slot_mapping, "slot_mapping")
        if k_pool.dtype != row_dtype or v_pool.dtype != row_dtype:
            raise KernelUnavailable("qk_norm_rope_kv_write: pools and qkv differ in dtype")
    if q_out is not None and (q_out.dtype != row_dtype
                              or q_out.shape != (T, n_heads * head_dim)):
        raise KernelUnavailable("qk_norm_rope_kv_write: q_out must be [T, nH * hd] of qkv's dtype")
    lib = build.load("elementwise")
    _check(lib.zf_qk_norm_rope_kv_write(
        _ptr(None if partials is not None else qkv), 1 if partials is not None else _dt(qkv),
        _ptr(q_gain), _ptr(k_gain),
        ctypes.c_float(eps), _ptr(cos),
        _ptr(sin), _ptr(positions), _ptr(slot_mapping), _ptr(k_pool), _ptr(v_pool), _ptr(q_out),
        T, n_heads, n_kv_heads, head_dim, page_size,
        1 if mfma_attention_covers(row_dtype, n_heads, n_kv_heads, head_dim, page_size) else 0,
        0 if cos is None else cos.shape[0],
        _ptr(partials), 0 if partials is None else partials.shape[0],
        _stream()), "qk_norm_rope_kv_write")


@_launches("norm_rope_write")
def swiglu(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    """out[t, j] = silu(gate_up[t, j]) * gate_up[t, I + j]."""
    _need_gpu(gate_up, out)
    T, I = out.shape
    if gate_up.shape != (T, 2 * I) or gate_up.dtype != out.dtype:
        raise KernelUnavailable(f"swiglu: gate_up {tuple(gate_up.shape)}, out {tuple(out.shape)}")
    lib = build.load("elementwise")
    _check(lib.zf_swiglu(_ptr(gate_up), _ptr(out), _dt(out), T, I, _stream()), "swiglu")


@_launches("other")
def cast(src: torch.Tensor, out: torch.Tensor) -> None:
    """out = src in the other storage type (bfloat16 <-> float32), element by element."""
    _need_gpu(src, out)
    if src.shape != out.shape or src.dtype == out.dtype:
        raise KernelUnavailable(f"cast: {tuple(src.shape)} {src.dtype} -> {tuple(out.shape)} "
                                f"{out.dtype}")
    lib = build.load("elementwise")
    _check(lib.zf_cast(_ptr(src), _dt(src), _ptr(out), _dt(out), ctypes.c_longlong(src.numel()),
                       _stream()), "cast")


@_launches("other")
def poison_pages(pool: torch.Tensor, pages: torch.Tensor) -> None:
    """pool[:, pages, :] = NaN: ``pool`` [runs, pages, row] float32 or bfloat16, ``pages`` int32."""
    _need_gpu(pool, pages)
    _i32(pages, "pages")
    if pool.dim() != 3 or pages.dim() != 1:
        raise KernelUnavailable("poison_pages: a pool [runs, pages, row] and a list of pages")
    lib = build.load("elementwise")
    _check(lib.zf_poison_pages(_ptr(pool), _dt(pool), _ptr(pages), pages.shape[0], pool.shape[0],
                               ctypes.c_longlong(pool.shape[1]), ctypes.c_longlong(pool.shape[2]),
                               _stream()), "poison_pages")


@_launches("head_sampling")
def gather_rows(x: torch.Tensor, idx: torch.Tensor, out: torch.Tensor) -> None:
    _need_gpu(x, idx, out)
    _i32(idx, "idx")
    n, H = out.shape
    if x.shape[1] != H or idx.shape[0] != n or x.dtype != torch.float32 or out.dtype != x.dtype:
        raise KernelUnavailable("gather_rows: float32 [T, H] -> [n, H]")
    lib = build.load("elementwise")
    _check(lib.zf_gather_rows(_ptr(x), _ptr(idx), _ptr(out), n, H, _stream()), "gather_rows")


@_launches("head_sampling")
def argmax(logits: torch.Tensor, out: torch.Tensor) -> None:
    """out[r] = index of the first maximum of logits[r, :]."""
    _need_gpu(logits, out)
    _i32(out, "out")
    n, V = logits.shape
    if logits.dtype != torch.float32 or out.shape != (n,):
        raise KernelUnavailable("argmax: float32 [n, V] -> int32 [n]")
    lib = build.load("elementwise")
    ws = _workspace("argmax", 2 * n * ((V + 4095) // 4096), torch.float32, logits.device)
    _check(lib.zf_argmax(_ptr(logits), _ptr(out), _ptr(ws), n, V, _stream()), "argmax")


ARGMAX_NO_ALLOC_MAX_PARTIALS = 32768    # ZF_ARGMAX_NO_ALLOC_MAX_PARTIALS in zf_no_alloc.h


@_launches("head_sampling")
def argmax_no_alloc(logits: torch.Tensor, out: torch.Tensor) -> None:
    """``argmax`` for callers that cannot allocate: the partial results live in a fixed device
    array of the library (shared by all calls on a GPU: overlapping calls race), so at most
    n * ceil(V / 4096) = 32768 of them."""
    _need_gpu(logits, out)
    _i32(out, "out")
    n, V = logits.shape
    if logits.dtype != torch.float32 or out.shape != (n,):
        raise KernelUnavailable("argmax_no_alloc: float32 [n, V] -> int32 [n]")
    if n * ((V + 4095) // 4096) > ARGMAX_NO_ALLOC_MAX_PARTIALS:
        raise KernelUnavailable(f"argmax_no_alloc: {n} rows of {V} logits need more than "
                                f"{ARGMAX_NO_ALLOC_MAX_PARTIALS} partial results")
    lib = build.load("elementwise")
    _check(lib.zf_argmax_no_alloc(_ptr(logits), _ptr(out), n, V, _stream()), "argmax_no_alloc")


@_launches("other")
def advance_decode(token_ids: torch.Tensor, positions: torch.Tensor, ctx_len: torch.Tensor,
                   sampled: torch.Tensor, slot_mapping: torch.Tensor, block_table: torch.Tensor,
                   page_size: int, advance: bool) -> None:
    """One decode step on, on the device: with ``advance`` token_ids = sampled, positions and
    ctx_len + 1; always slot_mapping[i] = block_table[i, p // page_size] * page_size +
    p % page_size at the (new) position p.  The caller guarantees that the table holds a page
    there."""
    _need_gpu(token_ids, positions, ctx_len, sampled, slot_mapping, block_table)
    for t, name in ((token_ids, "token_ids"), (positions, "positions"), (ctx_len, "ctx_len"),
                    (sampled, "sampled"), (slot_mapping, "slot_mapping"),
                    (block_table, "block_table")):
        _i32(t, name)
    n = token_ids.shape[0]
    if block_table.dim() != 2 or block_table.shape[0] != n or not block_table.is_contiguous() \
            or any(t.shape != (n,) for t in (positions, ctx_len, sampled, slot_mapping)):
        raise KernelUnavailable("advance_decode: int32 [n] vectors and a contiguous [n, pages] "
                                "block table")
    lib = build.load("elementwise")
    _check(lib.zf_advance_decode(_ptr(token_ids), _ptr(positions), _ptr(ctx_len), _ptr(sampled),
                                 _ptr(slot_mapping), _ptr(block_table), n, block_table.shape[1],
                                 int(page_size), 1 if advance else 0, _stream()),
           "advance_decode")


@_launches("other")
def randinit(out: torch.Tensor, key: int, start: int, kind: str, std: float = 0.02) -> None:
    """out[i] = element ``start + i`` of the random tensor with ``key``
    (`weights/counter_rng.py`: 'normal' = N(0, std), 'gain' = 1 + U(-0.1, 0.1), 'zeros')."""
    from ..weights.counter_rng import KIND
    _need_gpu(out)
    if out.dim() != 1 or kind not in KIND:
        raise KernelUnavailable(f"randinit: a flat tensor and a kind of {sorted(KIND)}")
    lib = build.load("randinit")
    _check(lib.zf_randinit(_ptr(out), _dt(out), ctypes.c_ulonglong(key & ((1 << 64) - 1)),
                           ctypes.c_ulonglong(start), ctypes.c_ulonglong(out.numel()),
                           KIND[kind], ctypes.c_double(std), _stream()), "randinit")


@_launches("other")
def check_tables(block_table: torch.Tensor, ctx_len: torch.Tensor,
                 slot_mapping: Optional[torch.Tensor], page_size: int, num_pages: int,
                 report: torch.Tensor) -> None:
    """Debugging: marks in ``report`` (int32 [4], zeroed by the caller: kind, sequence or token,
    index, value) a block-table entry among those a step's kernels will look up that is no
    page of the pool (kind 1), a context longer than the table's row, or a slot that is no row
    of the pool (kind 2).  The kernels themselves trust their tables; this is the check to
    switch on when they are in doubt (``Engine(debug_tables=True)``)."""
    _need_gpu(block_table, ctx_len, slot_mapping, report)
    for t, name in ((block_table, "block_table"), (ctx_len, "ctx_len"), (report, "report")):
        _i32(t, name)
    if slot_mapping is not None:
        _i32(slot_mapping, "slot_mapping")
    if block_table.dim() != 2 or ctx_len.shape != (block_table.shape[0],) or report.numel() < 4:
        raise KernelUnavailable("check_tables: int32 [n, pages] table, [n] contexts, [4] report")
    lib = build.load("elementwise")
    _check(lib.zf_check_tables(_ptr(block_table), _ptr(ctx_len), _ptr(slot_mapping),
                               block_table.shape[0], block_table.shape[1], int(page_size),
                               int(num_pages), 0 if slot_mapping is None else slot_mapping.shape[0],
                               _ptr(report), _stream()), "check_tables")


@_launches("other")
def stream_read(buf: torch.Tensor, sink: torch.Tensor, workgroups: int = 2048) -> None:
    """Reads ``buf`` once (16-byte non-temporal loads, 8 in flight a lane) and xors it into
    ``sink`` (int32, one word per workgroup): the read stream the weight-streaming kernels are
    measured against (``measure_read_bandwidth``)."""
    _need_gpu(buf, sink)
    _i32(sink, "sink")
    nbytes = buf.numel() * buf.element_size()
    if nbytes % 16 != 0 or sink.numel() < workgroups or not 1 <= workgroups <= 65536:
        raise KernelUnavailable("stream_read: a buffer of a multiple of 16 bytes and a sink of "
                                "one int32 per workgroup (1 to 65536)")
    lib = build.load("elementwise")
    _check(lib.zf_stream_read(_ptr(buf), ctypes.c_longlong(nbytes), _ptr(sink), int(workgroups),
                              _stream()), "stream_read")


def measure_read_bandwidth(device, nbytes: int = 2 << 30, repeats: int = 3) -> float:
    """Bytes a second of the best of ``repeats`` passes of ``stream_read`` over a buffer of
    ``nbytes`` (far more than the last-level cache holds, so it comes from HBM), each pass
    timed by a pair of events; the best of 256 to 4096 workgroups."""
    buf = torch.empty((nbytes // 4,), dtype=torch.int32, device=device)
    buf.zero_()
    sink = torch.zeros((4096,), dtype=torch.int32, device=device)
    best = 0.0
    for wgs in (256, 512, 768, 1024, 2048, 4096):
        stream_read(buf, sink, wgs)                       # warm-up
        for _ in range(repeats):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            stream_read(buf, sink, wgs)
            b.record()
            b.synchronize()
            best = max(best, nbytes / (a.elapsed_time(b) * 1e-3))
    del buf
    return best


@_launches("other")
def mfma_loop(operands: torch.Tensor, out: torch.Tensor, workgroups: int, iters: int) -> None:
    """``iters`` rounds of eight 32x32x16 MFMAs between the operands in ``operands`` (bfloat16
    [6, 64, 8]: four token operands, two weight operands, as the lanes of a wave hold them) in
    every wave of ``workgroups`` workgroups of four; ``out`` float32 [8, 32, 32] takes the first
    wave's accumulators (accumulator n: ``iters`` times tokens n % 4 against weights n / 4).
    Nothing but MFMAs: the rate the matrix cores sustain (``measure_mfma_rate``)."""
    _need_gpu(operands, out)
    if operands.dtype != torch.bfloat16 or tuple(operands.shape) != (6, 64, 8) \
            or not operands.is_contiguous() or out.dtype != torch.float32 \
            or tuple(out.shape) != (8, 32, 32) or not out.is_contiguous():
        raise KernelUnavailable("mfma_loop: operands bfloat16 [6, 64, 8], out float32 [8, 32, 32]")
    lib = build.load("gemm")
    _check(lib.zf_mfma_loop(_ptr(operands), _ptr(out), int(workgroups), int(iters), _stream()),
           "mfma_loop")


MFMA_LOOP_FLOPS = 2.0 * 32 * 32 * 16 * 8 * 4       # a workgroup's flops in one round


def measure_mfma_rate(device, random_operands: bool = True, seconds: float = 0.03) -> float:
    """Flops a second of ``mfma_loop`` on the whole chip, sustained over about ``seconds``
    (launches of a few milliseconds, the first ones untimed: the clock settles under the
    load).  On random operands the chip's power limit sets it, on zeros its clock."""
    g = torch.Generator(device="cpu").manual_seed(5)
    operands = (torch.randn((6, 64, 8), generator=g) if random_operands
                else torch.zeros((6, 64, 8))).to(torch.bfloat16).to(device)
    out = torch.zeros((8, 32, 32), dtype=torch.float32, device=device)
    workgroups, iters = 1024, 8000                  # about 5 ms a launch
    for _ in range(3):
        mfma_loop(operands, out, workgroups, iters)
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    n = 0
    a.record()
    while True:
        mfma_loop(operands, out, workgroups, iters)
        n += 1
        b.record()
        b.synchronize()
        dt = a.elapsed_time(b) * 1e-3
        if dt >= seconds or n >= 64:
            return MFMA_LOOP_FLOPS * workgroups * iters * n / dt


# ------------------------------------------------------------------------- work buffers
_workspaces = {}
_workspace_generation = 0


def workspace_generation() -> int:
    """Goes up whenever a work buffer is (re)allocated: a captured graph that used the old
    buffer must not be replayed."""
    return _workspace_generation


def _workspace(name: str, numel: int, dtype: torch.dtype, device) -> torch.Tensor:
    """A persistent device buffer of at least ``numel`` elements (grown when needed, never
    inside a stream capture once sizes have settled)."""
    global _workspace_generation
    key = (name, str(device), dtype)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < numel:
        buf = torch.empty((max(numel, 1),), dtype=dtype, device=device)
        _workspaces[key] = buf
        _workspace_generation += 1
    return buf


# ------------------------------------------------------------------------- matrix product
_EPI_STORE_BF16, _EPI_STORE_F32, _EPI_ACC_F32, _EPI_SWIGLU = 0, 1, 2, 3
SKINNY_MAX_M = 64
NORM_FOLD_MAX_M = 16


def _skinny_plan(M: int, N: int, K: int, tiled: bool):
    """Row groups of 16 per workgroup and workgroups along K for the weight-streaming kernel:
    enough workgroups to fill 256 CUs, as many rows per workgroup as that allows (the tokens
    are re-read once per workgroup).  Measured on MI355X at the Qwen3-8B sizes."""
    if tiled:
        if M <= 16:
            # one workgroup per CU streams best: the fewest row groups per workgroup that
            # still leave at most 256 workgroups, if that keeps half the CUs busy (384 row
            # groups: 192 workgroups of 2; 320: 160 of 2; 640: 160 of 4); a wide output takes 2
            for rg in (1, 2, 4):
                if N % (16 * rg) == 0 and 128 <= N // (16 * rg) <= 256:
                    return rg, 1
            return (2 if N >= 6144 else 1), 1
        # 17 to 64 tokens.  A wide output fills the chip by its row groups alone.  A narrow one
        # takes about 256 workgroups: the longer K is, the more rows a workgroup keeps (the
        # tokens are read again by every workgroup), and a split along K makes up for the
        # workgroups that costs (4096 x 1024: 256 of one row group; 1024 x 2048: 64 x 4 along
        # K; 2048 x 6144: 64 of two row groups x 4; 4096 x 12288: 64 of four x 4).  Measured on
        # MI355X at the projection widths of the Qwen3 0.6B to 8B shapes.
        if N >= 16384:
            return 4, 1
        if N >= 6144:
            return 2, 1
        rg = 1 if K < 4096 else 2 if K < 8192 else 4
        while rg > 1 and N % (16 * rg) != 0:
            rg //= 2
        wgs, ks = N // (16 * rg), 1
        while 2 * ks * wgs <= 256 and 2 * ks <= 16 and K >= 1024 * ks:
            ks *= 2
        return rg, ks
    if M <= 16:
        rg = 4 if N // 64 >= 256 else 1
        ks = 2 if (rg == 4 and N // 64 < 1024) else 1
    else:
        rg, ks = 4, 1
        while (N // 64) * ks < 192 and ks < 16:
            ks *= 2
    return rg, ks


MID_MAX_M = 128


def _mid_plan(M: int, N: int, K: int, w_tiled: bool, swiglu: bool = False):
    """Workgroups along K if the kernel for 17 to 128 tokens (128 outputs per workgroup, the
    tokens through LDS) covers the product, else None: above 32 tokens, and from 17 on a wide
    output, it beats the weight-streaming kernel, which re-reads the tokens for every few
    rows of the weight, and from 65 to 128 tokens the 128 x 128 tiles, two of whose waves load
    each part of the weight.  Split along K until up to 256 workgroups run, each keeping 1024
    of K.  Measured on MI355X at the Qwen3-8B sizes."""
    if not (w_tiled and 16 < M <= MID_MAX_M and N % 16 == 0
            and K % (256 if M <= 32 else 128) == 0):
        return None
    if M <= 32 and N < 16384:
        return None
    if swiglu:
        return 1
    tiles = (N + 127) // 128
    # up to 64 tokens a workgroup has half the work per k-tile: it may keep as little as 512 of K
    if M <= 64:
        return max(1, min(256 // tiles, K // 512))
    # above, 1024 of K a workgroup, or as little as 512 where that is what it takes to have
    # 128 workgroups (narrow outputs on a short K: 2048 x 2048 at 80 tokens 15.0 -> 12.4 us,
    # 1024 x 3072 15.2 -> 12.7, 2560 x 4096 16.7 -> 15.3)
    return max(1, min(256 // tiles, K // 512, max(K // 1024, (128 + tiles - 1) // tiles)))


_measured = None


def _measured_plans() -> dict:
    global _measured
    if _measured is None:
        import json
        import os
        with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "plans_mi355x.json")) as f:
            _measured = json.load(f)
    return _measured


PLAN_FILE = "kernel_plans.json"     # a model folder may bring plans measured at its own widths
PLAN_BUCKETS = (17, 24, 32, 48, 64)


def plan_bucket(M: int) -> int:
    """The bucket of a number of tokens in 17..64: a plan is kept per bucket, not per M."""
    return 17 if M <= 20 else 24 if M <= 28 else 32 if M <= 32 else 48 if M <= 56 else 64


def check_plans(plans: dict) -> None:
    """Raises ``KernelUnavailable`` unless every entry of a plan table names a configuration
    the launchers accept (what ``load_plans`` takes, and what the tuner writes)."""
    def bad(why):
        raise KernelUnavailable(f"kernel plans: {why}")
    for key, entry in plans.get("plans", {}).items():
        shape, _, kind = key.partition(":")
        try:
            N, K = (int(x) for x in shape.split("x"))
        except ValueError:
            bad(f"{key!r} is not 'NxK' or 'NxK:swiglu'")
        if kind not in ("", "swiglu"):
            bad(f"{key!r}: unknown kind {kind!r}")
        for bucket, plan in entry.items():
            M = int(bucket)
            if M not in PLAN_BUCKETS:
                bad(f"{key}: bucket {bucket} is none of {PLAN_BUCKETS}")
            if plan[0] == "mid" and len(plan) == 2:
                # k-tiles of 256 (up to 32 tokens) or 128, dealt over the workgroups along K
                ks, tk = int(plan[1]), (256 if M <= 32 else 128)
                ok = K % tk == 0 and 1 <= ks <= K // tk and N % 16 == 0
            elif plan[0] == "skinny" and len(plan) == 3:
                rg, ks = int(plan[1]), int(plan[2])
                ok = rg in (1, 2, 4) and N % (16 * rg) == 0 and 1 <= ks <= 16 and K % 64 == 0
            else:
                ok = False
            if ok and kind == "swiglu":
                ok = plan[-1] == 1 and (plan[0] == "mid" or plan[1] >= 2) and N % 32 == 0
            if not ok:
                bad(f"{key} at {bucket} tokens: {plan} is no plan the kernels take")
    for key, plan in plans.get("decode_acc", {}).items():
        if key == "_":
            continue
        N, K = (int(x) for x in key.split("x"))
        if plan is not None and not (
                len(plan) == 3 and plan[0] == "skinny" and plan[1] in (1, 2, 4)
                and N % (16 * plan[1]) == 0 and 2 <= plan[2] <= 16 and N <= 8192 and K % 64 == 0):
            bad(f"decode_acc {key}: {plan} is no plan the kernels take")


def load_plans(path: str) -> int:
    """Merges a plan file (``bench-ops --tune`` writes one) over the built-in table: its
    entries win for their widths.  Returns the number of entries taken."""
    import json
    with open(path, "r", encoding="utf-8") as f:
        plans = json.load(f)
    check_plans(plans)
    table = _measured_plans()
    n = 0
    for key, entry in plans.get("plans", {}).items():
        table["plans"][key] = {str(b): list(p) for b, p in entry.items()}
        n += 1
    for key, plan in plans.get("decode_acc", {}).items():
        if key != "_":
            table["decode_acc"][key] = None if plan is None else list(plan)
            n += 1
    return n


def _small_plan(M: int, N: int, K: int, w_tiled: bool, swiglu: bool = False):
    """Which kernel takes a product of 17 to 128 tokens (None: the tiled kernels):
    ('mid', workgroups along K) or ('skinny', row groups per workgroup, workgroups along K).
    The widths of the served models have measured entries in ``plans_mi355x.json``; other
    widths follow the rules of ``_mid_plan`` and ``_skinny_plan``."""
    if w_tiled and 16 < M <= SKINNY_MAX_M:
        bucket = plan_bucket(M)
        entry = _measured_plans()["plans"].get(f"{N}x{K}" + (":swiglu" if swiglu else ""))
        if entry is not None:
            # a width measured at fewer numbers of tokens: the nearest one on the same side of
            # 32 tokens (the kernels change there)
            same = [int(b) for b in entry if (int(b) <= 32) == (bucket <= 32)]
            if same:
                plan = entry[str(min(same, key=lambda b: abs(b - bucket)))]
                return tuple(plan)
    mid = _mid_plan(M, N, K, w_tiled, swiglu)
    # a short K: what the weight-streaming kernel reads again per workgroup is little, and it
    # stays ahead of the kernel that stages the tokens up to 56 tokens (64 at K <= 1024)
    short_k = w_tiled and 32 < M <= SKINNY_MAX_M and K <= 2048 and (M <= 56 or K <= 1024)
    if mid is not None and not short_k:
        return ("mid", mid)
    if M <= SKINNY_MAX_M:
        if swiglu:
            return ("skinny", 4 if (M > 16 and N >= 12288 and N % 64 == 0) else 2, 1)
        return ("skinny",) + tuple(_skinny_plan(M, N, K, w_tiled))
    return None


def _decode_acc_plan(M: int, N: int, K: int):
    """('skinny', row groups, workgroups along K) if, at 1 to 16 tokens, a residual sum that an
    RMSNorm follows is measured to run faster split along K (the reduce adds the residual and
    norms) than with the one-launch epilogue; else None."""
    if not 0 < M <= NORM_FOLD_MAX_M:
        return None
    plan = _measured_plans()["decode_acc"].get(f"{N}x{K}")
    return tuple(plan) if plan is not None else None


def _tile_variant(M: int, N: int, w_tiled: bool = False, accumulate: bool = False,
                  K: int = 0) -> int:
    """Which tiled kernel: with pre-tiled weights the kernels that take W straight from
    memory (10: 128 x 256 tiles, two workgroups to a CU, when they fill the chip; 12: the same
    tiles with two groups of waves a workgroup where a CU holds one; else 128 x
    128 tiles, 16: with the waves side by side and k-tiles of 128 (weights from HBM, 512
    tokens: qkv of the 8B shape 43 -> 38 us), 6: with 2 x 2 waves, where K is no multiple of
    128); otherwise the kernels that stage both operands through LDS
    (4: 256 x 256 when they still fill the chip, else 0: 128 x 128).  Measured on MI355X at the
    Qwen3-8B and Qwen3-14B sizes."""
    if w_tiled:
        tiles_m = (M + 127) // 128
        tiles = tiles_m * ((N + 255) // 256)
        # from 144 large tiles on they win or draw (140 to 152 tiles: 0.84 to 1.05 of the
        # 128 x 128 tiles' time).  Between one and two 128 x 256 tiles per CU half the CUs hold
        # two workgroups and half one: there the 256-token tiles are measured against the
        # 128 x 128 ones (2048 tokens into 6144 outputs); with few tiles along the tokens (512
        # tokens into 24576 outputs) the large tiles still win (five rows of tiles: 544 tokens
        # into 24576 outputs, 480 large tiles, 143 -> 115 us)
        if tiles >= 144 and not (256 < tiles < 512 and tiles_m > 5):
            # one workgroup to a CU whatever is done: two groups of waves in it, each over
            # half of a long K (o_proj and down at 1280 to 2048 tokens: 3 to 12 % less; at
            # K <= 2048 the blocks handed over at the end cost more than the waves gain)
            if 160 <= tiles <= TILE_PLACES // 2 and K >= 4096 and K % 256 == 0:
                return 12
            return 10
        # (the 128 x 128 tiles of 2 x 2 waves, where two waves load each part of W, only
        # where k-tiles of 128 do not divide K: in 24 products of 136 to 4096 tokens that had
        # them, the waves side by side were level or faster, 12 % in all)
        return 16 if K > 0 and K % 128 == 0 else 6
    tiles = ((M + 255) // 256) * ((N + 255) // 256)
    return 4 if tiles >= 160 else 0


def _tile_ksplit(M: int, N: int, K: int, accumulate: bool = True) -> int:
    """Workgroups per 128 x 128 tile along K: products of a few hundred tokens on a narrow
    output have too few tiles for 256 CUs, or a number that fills them unevenly (160 tiles:
    96 CUs idle; 320: a second round for a quarter of them).  Two workgroups fit a CU, so the
    split is chosen to fill 256 or a multiple of 512 places as evenly as it can, each
    workgroup keeping at least 8 k-tiles of 64.  Every split costs partials of M * N floats,
    written and read again (against the product's own time that is about 400 / K a split),
    and the first one a second launch.  A product that is stored, not added to the residual,
    stays whole once its tiles need a second round anyway (257 and more: 768 tokens of the 8B
    shape's qkv 66 -> 59 us); the residual sum gains from the split up to 383 tiles, since the
    kernel that adds the partials is the norm's as well.  Measured on MI355X at the Qwen3-8B,
    14B and 32B sizes, 256 to 1024 tokens, the weights from HBM."""
    tiles = ((M + 127) // 128) * ((N + 127) // 128)
    if tiles >= 384 or (tiles > 256 and not accumulate):
        return 1
    # one round of 128 x 256 tiles with two groups of waves a workgroup needs no partials: on
    # a short K it beats the split even with the norm's kernel behind it (1280 tokens into
    # 4096 outputs, K = 4096: 64 + 6 against 76 us; 2048 into 2560: 59 + 8 against 75); on a
    # long K the split stays ahead (1024 into 5120, K = 17408: 205 against 237)
    if K < 8192 and _tile_variant(M, N, True, accumulate, K) == 12:
        return 1
    best, best_cost = 1, None
    for ks in range(1, min(8, K // 64 // 8) + 1):
        wgs = tiles * ks
        places = 256 if wgs <= 256 else (wgs + 511) // 512 * 512
        cost = places / wgs + (ks * 400.0 / K + 0.05 if ks > 1 else 0.0)
        if best_cost is None or cost < best_cost - 1e-9:
            best, best_cost = ks, cost
    return best


# Rates per CU (flop/s) of the tiled kernels on pre-tiled weights, from gate/up of the 8B shape
# at 16384 tokens: the 256-token tiles of 256, 192 and 128 outputs (one workgroup to a CU),
# and the 128-token tiles two to a CU ("pair") or one ("alone").
_TILE256_RATE = {20: 5.18e12, 21: 4.52e12, 22: 3.73e12}
_TILE256_WIDTH = {20: 256, 21: 192, 22: 128}
_TILE128_RATE = {10: (5.13e12, 3.85e12), 12: (5.13e12, 4.05e12), 16: (3.8e12, 2.9e12), 6: (3.77e12, 2.7e12)}


@functools.lru_cache(maxsize=None)
def _tile64_covers(M: int, N: int, K: int, accumulate: bool) -> bool:
    """A few hundred tokens on a narrow output, no residual sum: tiles of 64 tokens x 128
    outputs, unsplit.  A CU finishes one such tile in about two thirds of the time of a
    128 x 128 tile, and a second round doubles that, so they are taken where one round holds
    them (up to 288: the last few share CUs), or where the 128-token tiles would need a
    second round themselves while these stay within two.  Measured on MI355X with weights
    that come from HBM (more copies in turn than the last-level cache holds): qkv of the
    8B shape at 272 tokens 36 -> 26 us, o_proj-like 5120 x 8192 at 384 tokens 72 -> 51 us,
    qkv of the 14B shape at 528 to 576 tokens 70 -> 58 us; with 300 to 512 tiles against one
    round of the larger ones they lose (14B qkv at 384 tokens 47 -> 57 us).  A residual sum
    keeps its split along K, whose second kernel is also the norm."""
    if accumulate or not (128 < M <= 640 and K % 128 == 0 and N % 16 == 0 and K <= 8192):
        return False
    cols = (N + 127) // 128
    tiles64, tiles128 = ((M + 63) // 64) * cols, ((M + 127) // 128) * cols
    return tiles64 <= 288 or (tiles128 > 256 and tiles64 <= 512)


def _tile256_time(variant: int, M: int, N: int, K: int) -> float:
    """Estimated seconds of the 256-token tile kernel: rounds of up to 256 tiles, one to a CU."""
    bn = _TILE256_WIDTH[variant]
    tiles = ((M + 255) // 256) * ((N + bn - 1) // bn)
    rounds = (tiles + 255) // 256
    t = rounds * 2.0 * 256 * bn * K / _TILE256_RATE[variant]
    # on a narrow output the 256-token tiles fall behind this estimate once every CU takes
    # more than one (o_proj and down at 8192 tokens and more: by 6 to 20 %)
    return t * (1.08 if (rounds > 1 and N <= 5120) else 1.0) + 4e-6


TILE_PLACES = 512       # workgroups of the 128 x 256 tiles the chip holds at once: two to a CU


def _tile_tail_split(M: int, N: int, K: int):
    """(whole, split) if the 128 x 256 tiles of a product on pre-tiled weights should run with
    their last, short round split along K, else None: ``whole`` tiles fill whole rounds of the
    chip's ``TILE_PLACES`` places, and each of the others goes to ``split`` workgroups.  A
    round of a few tiles takes as long as a full one (512 tokens into the 14B shape's 34816
    gate and up outputs: 544 tiles, 210 us, of which the last 32 take 80); split in four it
    takes a quarter of that, plus what the partials cost: 128 KB a workgroup, written and read
    again, and a second kernel.  The split that the estimate below likes best is taken if it
    saves a fifth of the round or more, which on MI355X (Qwen3-8B and 14B widths, 512 to 4096
    tokens) is where the measured gain begins: 210 -> 165 us above, 768 tokens into 24576
    outputs 156 -> 131, 1024 into 34816 339 -> 307; a last round of more than about 100 tiles
    stays whole (168 tiles in three parts: 210 -> 255 us).  Only splits that leave every part
    an even number of k-tiles, which the kernel's deeper prefetch of W needs."""
    if K % 128 != 0:
        return None
    tiles = ((M + 127) // 128) * ((N + 255) // 256)
    whole = tiles // TILE_PLACES * TILE_PLACES
    tail = tiles - whole
    if whole == 0 or tail == 0 or whole > 2 * TILE_PLACES:
        return None         # (behind three rounds and more the workgroups no longer end together)
    kt = K // 64
    per = 2.0 * 128 * 256 * K
    pair, alone = _TILE128_RATE[10]

    def last_round(workgroups: int, flop: float) -> float:
        return flop / alone if workgroups <= 256 else 2 * flop / pair
    best, best_t = None, 0.8 * last_round(tail, per)
    for split in (2, 4, 8):
        if tail * split > TILE_PLACES or kt % (2 * split) != 0 or kt // split < 8:
            continue
        t = last_round(tail * split, per / split) + 8e-6 + tail * split * 128 * 256 * 4 * 2 / 3e12
        if t < best_t:
            best, best_t = split, t
    return None if best is None else (whole, best)


def _tile128_time(M: int, N: int, K: int, variant: int, ksplit: int) -> float:
    """Estimated seconds of the 128-token tile kernels: rounds of up to 512 tiles, two to a CU
    (a last round of up to 256 tiles runs one to a CU, each faster than two)."""
    bn = 256 if variant in (10, 12) else 128
    tiles = ((M + 127) // 128) * ((N + bn - 1) // bn) * ksplit
    per = 2.0 * 128 * bn * (K / ksplit)
    pair, alone = _TILE128_RATE[variant if ksplit == 1 else 6]
    rem = tiles % 512
    tail = _tile_tail_split(M, N, K) if variant == 10 and ksplit == 1 else None
    if tail is not None:    # the last round split along K, its partials written and read again
        part, wgs = per / tail[1], rem * tail[1]
        last = (part / alone if wgs <= 256 else 2 * part / pair) + 8e-6 \
            + wgs * 128 * 256 * 4 * 2 / 3e12
    else:
        last = 0.0 if rem == 0 else per / alone if rem <= 256 else 2 * per / pair
    t = (tiles // 512) * 2 * per / pair + last
    if ksplit > 1:      # the partials, written and read again, and the second launch
        t += 4e-6 + M * N * 4.0 * ksplit * 2 / 4e12
    return t + 4e-6


@functools.lru_cache(maxsize=None)
def _tile256_variant(M: int, N: int, K: int, accumulate: bool = False):
    """The 256-token tile kernel (20: 256 outputs a tile, 21: 192, 22: 128) if it is expected
    to beat what ``_tile_variant`` and ``_tile_ksplit`` choose by 5 % or more, else None.  One
    workgroup per CU and tile: what counts is how evenly the tiles fill 256 CUs (2048 tokens
    into 6144 outputs are 256 tiles of 256 x 192, where 128 x 128 tiles fill 512 places one
    and a half times: 101 -> 83 us; 14B down at 3072 tokens: 603 -> 441).  Where both kinds
    fill the chip many times over they run equally fast (gate/up at 8192 tokens: 1250 us).
    Times are estimated from rates measured on MI355X; against a sweep of the Qwen3-8B, 14B
    and 32B widths at 512 to 16384 tokens the choice is within 1 % of the best on the whole.
    A residual sum that is split along K keeps its split (the kernel that adds the partials
    also norms)."""
    if M <= 128 or K % 128 != 0 or N % 16 != 0:
        return None
    ks = _tile_ksplit(M, N, K, accumulate)
    if ks > 1 and accumulate:
        return None
    now = _tile128_time(M, N, K, _tile_variant(M, N, True, accumulate, K), ks)
    best = min((20, 21, 22), key=lambda v: _tile256_time(v, M, N, K))
    return best if _tile256_time(best, M, N, K) < 0.95 * now else None


def can_pretile(w: torch.Tensor) -> bool:
    return w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[0] % 64 == 0 \
        and w.shape[1] % 64 == 0


def pretile_weight(w: torch.Tensor) -> torch.Tensor:
    """The bfloat16 kernels' own weight layout, made once at load: [N / 16][K / 64][2][64][8],
    the 16 rows x 64 k of a tile together (2 KB) in the order the lanes of the 16x16x32 MFMA
    pair consume them, so that the weight-streaming kernel reads 1 KB of consecutive memory
    per wave load.  Returned with shape [N, K]; only the kernels know what lies where."""
    N, K = w.shape
    if not can_pretile(w):
        raise KernelUnavailable(f"pretile_weight: bfloat16 [N % 64 == 0, K % 64 == 0], got "
                                f"{tuple(w.shape)} {w.dtype}")
    t = w.view(N // 16, 16, K // 64, 4, 2, 8).permute(0, 2, 4, 3, 1, 5).contiguous()
    return t.view(N, K)


def _gemm_tile_tail(lib, a, w, out, M: int, N: int, K: int, epi: int, tail) -> None:
    whole, split = tail
    tiles = ((M + 127) // 128) * ((N + 255) // 256)
    if not (0 <= whole < tiles and split >= 2):
        raise KernelUnavailable(f"gemm: tail split {tail} of {tiles} tiles")
    ws = _workspace("gemm_tile_tail", (tiles - whole) * split * 128 * 256, torch.float32, a.device)
    _check(lib.zf_gemm_bf16_tile_tail(_ptr(a), _ptr(w), _ptr(out), _ptr(ws), M, N, K, epi, whole,
                                      split, _stream()), "gemm (tiled, last round split along K)")


@_launches("products")
def gemm(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False,
         w_tiled: bool = False, tile_variant: Optional[int] = None,
         tile_tail: Optional[Tuple[int, int]] = None) -> None:
    """out = a w^T (w is [N, K]); with ``accumulate`` out += a w^T, in 32-bit.  ``w_tiled``:
    ``w`` went through ``pretile_weight``.  ``tile_variant`` (tests and measurements): this
    tiled kernel, whatever the number of rows; ``tile_tail`` (whole, split): the 128 x 256
    tiles with the tiles from ``whole`` on split along K (``_tile_tail_split``).

    bfloat16 operands with K a multiple of 8 go to the MFMA kernels (weight streaming for up
    to 16 rows of ``a``, and up to 64 where the kernel for 17 to 128 rows does not cover the
    sizes; LDS-tiled above); everything else, the whole 32-bit path included,
    goes to the FMA kernel, whose results do not depend on how rows are batched."""
    _need_gpu(a, w, out)
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K or out.shape != (M, N):
        raise KernelUnavailable(f"gemm: a {tuple(a.shape)}, w {tuple(w.shape)}, "
                                f"out {tuple(out.shape)}")
    if accumulate and out.dtype != torch.float32:
        raise KernelUnavailable("gemm: accumulation needs a float32 output")
    lib = build.load("gemm")
    if w_tiled and not (a.dtype == torch.bfloat16 and can_pretile(w)):
        raise KernelUnavailable("gemm: a pre-tiled weight needs bfloat16 operands")
    if a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and K % 8 == 0 and M > 0:
        epi = _EPI_ACC_F32 if accumulate else \
            (_EPI_STORE_BF16 if out.dtype == torch.bfloat16 else _EPI_STORE_F32)
        plan = _small_plan(M, N, K, w_tiled) if M > 16 else None
        if tile_tail is not None:
            _gemm_tile_tail(lib, a, w, out, M, N, K, epi, tile_tail)
        elif tile_variant is not None:
            _check(lib.zf_gemm_bf16_tile(_ptr(a), _ptr(w), _ptr(out), M, N, K, epi, tile_variant,
                                         1 if w_tiled else 0, _stream()), "gemm (tiled)")
        elif plan is not None and plan[0] == "mid":
            mid = plan[1]
            ws = _workspace("gemm_splitk", mid * M * N, torch.float32, a.device) if mid > 1 else None
            _check(lib.zf_gemm_bf16_mid(_ptr(a), _ptr(w), _ptr(out), _ptr(ws), M, N, K, epi, mid,
                                        _stream()), "gemm (17 to 128 tokens)")
        elif M <= SKINNY_MAX_M:
            rg, ks = plan[1:] if plan is not None else _skinny_plan(M, N, K, w_tiled)
            ws = _workspace("gemm_splitk", ks * M * N, torch.float32, a.device) if ks > 1 else None
            _check(lib.zf_gemm_bf16_skinny(_ptr(a), _ptr(w), _ptr(out), _ptr(ws), M, N, K, epi,
                                           rg, ks, 1 if w_tiled else 0, _stream()),
                   "gemm (weight streaming)")
        elif w_tiled and _tile64_covers(M, N, K, accumulate):
            _check(lib.zf_gemm_bf16_mid(_ptr(a), _ptr(w), _ptr(out), _ptr(None), M, N, K, epi, 1,
                                        _stream()), "gemm (64-token tiles)")
        else:
            wide = _wide_ksplit(M, N, K) if w_tiled and accumulate else None
            if wide is not None:        # as gemm_sum_norm runs it: the same bits
                ws = _workspace("gemm_splitk", wide * M * N, torch.float32, a.device)
                _check(lib.zf_gemm_bf16_wide_splitk(_ptr(a), _ptr(w), _ptr(out), _ptr(ws), M, N, K,
                                                    epi, wide, _stream()),
                       "gemm (128 x 256 tiles, split along K)")
                return
            big = _tile256_variant(M, N, K, accumulate) if w_tiled else None
            if big is not None:
                _check(lib.zf_gemm_bf16_tile(_ptr(a), _ptr(w), _ptr(out), M, N, K, epi, big, 1,
                                             _stream()), "gemm (256-token tiles)")
                return
            ksplit = _tile_ksplit(M, N, K, accumulate) if w_tiled else 1
            if ksplit > 1:
                ws = _workspace("gemm_splitk", ksplit * M * N, torch.float32, a.device)
                _check(lib.zf_gemm_bf16_tile_splitk(_ptr(a), _ptr(w), _ptr(out), _ptr(ws), M, N,
                                                    K, epi, ksplit, _stream()),
                       "gemm (tiled, split along K)")
                return
            variant = _tile_variant(M, N, w_tiled, accumulate, K)
            tail = _tile_tail_split(M, N, K) if variant == 10 else None
            if tail is not None:
                _gemm_tile_tail(lib, a, w, out, M, N, K, epi, tail)
                return
            _check(lib.zf_gemm_bf16_tile(_ptr(a), _ptr(w), _ptr(out), M, N, K, epi, variant,
                                         1 if w_tiled else 0, _stream()),
                   "gemm (tiled)")
        return
    _check(lib.zf_gemm_fma(_ptr(a), _dt(a), _ptr(w), _dt(w), _ptr(out), _dt(out), M, N, K,
                           1 if accumulate else 0, _stream()), "gemm")


def gemm_partials_plan(M: int, N: int, K: int, w: torch.Tensor, w_tiled: bool):
    """Workgroups along K if ``gemm`` would run a stored product a w^T through the kernel for
    17 to 128 tokens split along K (whose partials a second kernel then adds), else None: the
    partials can instead go to a kernel of the caller's that adds them on its way
    (``gemm_partials``)."""
    if not (w_tiled and w.dtype == torch.bfloat16 and w.is_cuda and 16 < M <= MID_MAX_M):
        return None
    plan = _small_plan(M, N, K, True)
    return plan[1] if plan is not None and plan[0] == "mid" and plan[1] > 1 else None


def gemm_partials(a: torch.Tensor, w: torch.Tensor, ksplit: int) -> torch.Tensor:
    """The float32 partials [ksplit, M, N] of a w^T (``w`` pre-tiled, 17 to 128 rows of
    ``a``) in a work buffer that the next split product overwrites; their sum in split order,
    rounded, is what ``gemm`` stores."""
    _need_gpu(a, w)
    M, K = a.shape
    N = w.shape[0]
    if a.dtype != torch.bfloat16 or w.shape[1] != K or not can_pretile(w) \
            or gemm_partials_plan(M, N, K, w, True) != ksplit:
        raise KernelUnavailable("gemm_partials: not a product that gemm_partials_plan covers")
    ws = _workspace("gemm_splitk", ksplit * M * N, torch.float32, a.device)
    lib = build.load("gemm")
    if not _left_out("products"):
        global _launch_count
        _launch_count += 1
        _check(lib.zf_gemm_bf16_mid_partials(_ptr(a), _ptr(w), _ptr(ws), M, N, K, ksplit,
                                             _stream()), "gemm_partials")
    return ws[:ksplit * M * N].view(ksplit, M, N)


gemm_partials.kernel_class = "products"     # (it hands its work buffer on even when left out)


def norm_gemm_plan(M: int, N: int, K: int, w: torch.Tensor, w_tiled: bool):
    """Row groups per workgroup if ``norm_gemm`` covers the product (the weight-streaming
    kernel without a split over workgroups on a pre-tiled bfloat16 weight), else None."""
    # beyond 16 tokens the lanes' extra work (32-bit rows, gains, conversions for every group
    # of 16 tokens) costs more than the norm kernel it saves (measured)
    if not (w_tiled and 0 < M <= NORM_FOLD_MAX_M and w.dtype == torch.bfloat16):
        return None
    rg, ks = _skinny_plan(M, N, K, True)
    return rg if ks == 1 else None


@_launches("products")
def norm_gemm(x: torch.Tensor, gain: torch.Tensor, eps: float, w: torch.Tensor,
              out: torch.Tensor, swiglu: bool = False) -> None:
    """out = rmsnorm(x, gain, eps) w^T with the norm folded into the weight-streaming product
    (``w`` pre-tiled; with ``swiglu`` the rows of ``w`` alternate gate / up as for
    ``gemm_swiglu`` and out is [M, N / 2]).  x float32 [M <= 64, K]; the sum of squares, the
    scale and the product's sums are 32-bit, the MFMA operands bfloat16(x * gain)."""
    _need_gpu(x, gain, w, out)
    M, K = x.shape
    N = w.shape[0]
    rg = norm_gemm_plan(M, N, K, w, True)
    if swiglu and 0 < M <= SKINNY_MAX_M:
        rg = 4 if (M > 16 and N >= 16384) else 2
    if rg is None or x.dtype != torch.float32 or gain.dtype != torch.float32 \
            or gain.shape != (K,) or w.shape[1] != K or not can_pretile(w) \
            or out.shape != (M, N // 2 if swiglu else N) \
            or (swiglu and out.dtype != torch.bfloat16):
        raise KernelUnavailable(f"norm_gemm: x {tuple(x.shape)} {x.dtype}, w {tuple(w.shape)}, "
                                f"out {tuple(out.shape)} {out.dtype}")
    epi = _EPI_SWIGLU if swiglu else \
        (_EPI_STORE_BF16 if out.dtype == torch.bfloat16 else _EPI_STORE_F32)
    lib = build.load("gemm")
    _check(lib.zf_norm_gemm_bf16_skinny(_ptr(x), _ptr(gain), ctypes.c_float(eps), _ptr(w),
                                        _ptr(out), M, N, K, epi, rg, _stream()), "norm_gemm")


def sum_norm_plan(M: int, N: int, K: int, w: torch.Tensor, w_tiled: bool):
    """The plan if ``gemm_sum_norm`` covers residual += a w^T: a product that is split along K
    anyway (by measurement at 1 to 64 tokens, by rule at 17 to 128, or a few hundred tokens on
    a narrow output), whose partials one kernel can add, sum into the residual and norm; else
    None.  ('mid' | 'tile' | 'wide' | 'skinny', [row groups per workgroup,] workgroups along K)."""
    if not (w_tiled and w.dtype == torch.bfloat16 and w.is_cuda and N % 16 == 0 and N <= 8192):
        return None
    if M <= NORM_FOLD_MAX_M:
        return _decode_acc_plan(M, N, K)
    if M <= MID_MAX_M:
        plan = _small_plan(M, N, K, True)
        return plan if plan is not None and plan[-1] >= 2 else None
    wide = _wide_ksplit(M, N, K)
    if wide is not None:
        return ("wide", wide)
    ks = _tile_ksplit(M, N, K)
    return ("tile", ks) if ks >= 2 else None


def _wide_ksplit(M: int, N: int, K: int):
    """Workgroups along K if a residual sum with the norm behind it should run through 128 x
    256 tiles split along K: 641 to 1280 tokens on a long K, where those tiles alone leave
    half the chip idle (1024 tokens into 4096 outputs: 128 of them) and the 128 x 128 tiles,
    split or not, are slower per flop.  Two to four parts of an even number of k-tiles each,
    as close to 512 workgroups as they get.  Measured on MI355X against what ran before (the
    norm's kernel included): K = 12288 into 4096 at 768 / 1024 / 1280 tokens 113 -> 107, 133
    -> 113, 171 -> 143 us; K = 17408 into 5120 174 -> 149, 222 -> 209, 254 -> 244; K = 25600
    253 -> 205 and 314 -> 289.  With K = 4096 or 5120 the partials cost what the split gains,
    and from 1536 tokens on the tiles fill the chip without it."""
    if not (640 < M <= 1280 and K >= 8192 and K % 128 == 0 and N % 16 == 0):
        return None
    tiles = ((M + 127) // 128) * ((N + 255) // 256)
    fits = [ks for ks in (2, 3, 4) if (K // 64) % (2 * ks) == 0]
    return min(fits, key=lambda ks: abs(tiles * ks - TILE_PLACES)) if fits else None


@_launches("products")
def gemm_sum_norm(a: torch.Tensor, w: torch.Tensor, residual: torch.Tensor, gain: torch.Tensor,
                  eps: float, normed: torch.Tensor) -> None:
    """residual += a w^T in 32-bit (``w`` pre-tiled) and normed = bfloat16(rmsnorm(residual,
    gain, eps)), the norm from the kernel that adds the product's partials."""
    _need_gpu(a, w, residual, gain, normed)
    M, K = a.shape
    N = w.shape[0]
    plan = sum_norm_plan(M, N, K, w, True)
    if plan is None or a.dtype != torch.bfloat16 or w.shape[1] != K or not can_pretile(w) \
            or residual.shape != (M, N) or residual.dtype != torch.float32 \
            or gain.shape != (N,) or gain.dtype != torch.float32 \
            or normed.shape != (M, N) or normed.dtype != torch.bfloat16 \
            or not all(t.is_contiguous() for t in (a, residual, normed)):
        raise KernelUnavailable(f"gemm_sum_norm: a {tuple(a.shape)} {a.dtype}, w "
                                f"{tuple(w.shape)}, residual {tuple(residual.shape)} "
                                f"{residual.dtype}")
    ks = plan[-1]
    ws = _workspace("gemm_splitk", ks * M * N, torch.float32, a.device)
    lib = build.load("gemm")
    if plan[0] == "wide":
        _check(lib.zf_gemm_bf16_wide_splitk_sum_norm(_ptr(a), _ptr(w), _ptr(residual), _ptr(ws),
                                                     _ptr(gain), ctypes.c_float(eps), _ptr(normed),
                                                     M, N, K, ks, _stream()),
               "gemm_sum_norm (128 x 256 tiles)")
    elif plan[0] == "skinny":
        _check(lib.zf_gemm_bf16_skinny_sum_norm(_ptr(a), _ptr(w), _ptr(residual), _ptr(ws),
                                                _ptr(gain), ctypes.c_float(eps), _ptr(normed), M, N,
                                                K, plan[1], ks, _stream()),
               "gemm_sum_norm (weight streaming)")
    else:
        _check(lib.zf_gemm_bf16_splitk_sum_norm(_ptr(a), _ptr(w), _ptr(residual), _ptr(ws),
                                                _ptr(gain), ctypes.c_float(eps), _ptr(normed), M, N,
                                                K, ks, _stream()), "gemm_sum_norm")


def norm_emit_plan(M: int, N: int, K: int, w: torch.Tensor, w_tiled: bool):
    """Row groups per workgroup if ``gemm_emit`` covers out += a w^T (weight-streaming kernel,
    up to 16 tokens, pre-tiled bfloat16 weight, no split over workgroups), else None."""
    if not (w_tiled and 0 < M <= NORM_FOLD_MAX_M and w.dtype == torch.bfloat16 and w.is_cuda):
        return None
    if N <= 8192 and _decode_acc_plan(M, N, K) is not None:
        return None             # measured: the split along K with the norm in its reduce is faster
    rg, ks = _skinny_plan(M, N, K, True)
    return rg if (ks == 1 and rg <= 2) else None


@_launches("products")
def gemm_emit(a: torch.Tensor, w: torch.Tensor, residual: torch.Tensor, gain: torch.Tensor,
              xg: torch.Tensor, sq: torch.Tensor) -> None:
    """residual += a w^T in 32-bit (``w`` pre-tiled) and, for the RMSNorm that reads the sum
    next, from the same epilogue: xg = bfloat16(residual * gain) [M, N] and sq [N / 16, 16] =
    the sums of residual^2 over each 16 columns per token, which ``gemm_given`` takes."""
    _need_gpu(a, w, residual, gain, xg, sq)
    M, K = a.shape
    N = w.shape[0]
    rg = norm_emit_plan(M, N, K, w, True)
    if rg is None or a.dtype != torch.bfloat16 or w.shape[1] != K or not can_pretile(w) \
            or residual.shape != (M, N) or residual.dtype != torch.float32 \
            or gain.shape != (N,) or gain.dtype != torch.float32 \
            or xg.shape != (M, N) or xg.dtype != torch.bfloat16 \
            or sq.shape != (N // 16, 16) or sq.dtype != torch.float32 \
            or not all(t.is_contiguous() for t in (a, residual, xg, sq)):
        raise KernelUnavailable(f"gemm_emit: a {tuple(a.shape)} {a.dtype}, w {tuple(w.shape)}, "
                                f"residual {tuple(residual.shape)} {residual.dtype}")
    lib = build.load("gemm")
    _check(lib.zf_gemm_bf16_skinny_emit(_ptr(a), _ptr(w), _ptr(residual), _ptr(gain), _ptr(xg),
                                        _ptr(sq), M, N, K, rg, _stream()), "gemm_emit")


@_launches("products")
def gemm_given(xg: torch.Tensor, sq: torch.Tensor, eps: float, w: torch.Tensor,
               out: torch.Tensor, swiglu: bool = False) -> None:
    """out = rmsnorm(x) w^T from what ``gemm_emit`` left of x: xg = bfloat16(x * gain) and the
    partial sums of squares sq [groups, 16]; the token's 1 / sqrt(mean(x^2) + eps) scales the
    32-bit sums of the product.  With ``swiglu`` as ``gemm_swiglu``."""
    _need_gpu(xg, sq, w, out)
    M, K = xg.shape
    N = w.shape[0]
    rg = norm_gemm_plan(M, N, K, w, True)
    if swiglu and 0 < M <= NORM_FOLD_MAX_M:
        rg = 2
    if rg is None or xg.dtype != torch.bfloat16 or sq.dtype != torch.float32 \
            or sq.dim() != 2 or sq.shape[1] != 16 or sq.shape[0] * 16 != K \
            or w.shape[1] != K or not can_pretile(w) \
            or out.shape != (M, N // 2 if swiglu else N) \
            or (swiglu and out.dtype != torch.bfloat16) \
            or not all(t.is_contiguous() for t in (xg, sq, out)):
        raise KernelUnavailable(f"gemm_given: xg {tuple(xg.shape)} {xg.dtype}, w {tuple(w.shape)}, "
                                f"out {tuple(out.shape)} {out.dtype}")
    epi = _EPI_SWIGLU if swiglu else \
        (_EPI_STORE_BF16 if out.dtype == torch.bfloat16 else _EPI_STORE_F32)
    lib = build.load("gemm")
    _check(lib.zf_gemm_bf16_skinny_given(_ptr(xg), _ptr(sq), sq.shape[0], ctypes.c_float(eps),
                                         _ptr(w), _ptr(out), M, N, K, epi, rg, _stream()),
           "gemm_given")


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """Rows of the gate and the up projection alternating in groups of 16 (gate 0..15, up
    0..15, gate 16..31, ...): the order ``gemm_swiglu`` wants.  Needs I % 16 == 0."""
    I, K = gate.shape
    return torch.stack([gate.view(I // 16, 16, K), up.view(I // 16, 16, K)], dim=1) \
        .reshape(2 * I, K).contiguous()


def can_fuse_swiglu(w: torch.Tensor) -> bool:
    return w.is_cuda and w.dtype == torch.bfloat16 and w.shape[0] % 64 == 0 and w.shape[1] % 8 == 0


@_launches("products")
def gemm_swiglu(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, w_tiled: bool = False,
                tile_variant: Optional[int] = None,
                tile_tail: Optional[Tuple[int, int]] = None) -> None:
    """out[M, I] = silu(a Wg^T) * (a Wu^T) as bfloat16, with ``w`` [2 I, K] from
    ``interleave_gate_up`` (then possibly ``pretile_weight``): the activation is applied to
    the 32-bit sums in the product's epilogue, nothing of width 2 I is written."""
    _need_gpu(a, w, out)
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K or out.shape != (M, N // 2) or out.dtype != torch.bfloat16 \
            or a.dtype != torch.bfloat16 or not can_fuse_swiglu(w):
        raise KernelUnavailable(f"gemm_swiglu: a {tuple(a.shape)} {a.dtype}, w {tuple(w.shape)} "
                                f"{w.dtype}, out {tuple(out.shape)} {out.dtype}")
    if M == 0:
        return
    lib = build.load("gemm")
    plan = _small_plan(M, N, K, w_tiled, swiglu=True) if M > 16 else None
    if tile_tail is not None:
        _gemm_tile_tail(lib, a, w, out, M, N, K, _EPI_SWIGLU, tile_tail)
    elif tile_variant is not None:
        _check(lib.zf_gemm_bf16_tile(_ptr(a), _ptr(w), _ptr(out), M, N, K, _EPI_SWIGLU,
                                     tile_variant, 1 if w_tiled else 0, _stream()),
               "gemm_swiglu (tiled)")
    elif plan is not None and plan[0] == "mid":
        _check(lib.zf_gemm_bf16_mid(_ptr(a), _ptr(w), _ptr(out), _ptr(None), M, N, K, _EPI_SWIGLU,
                                    1, _stream()), "gemm_swiglu (17 to 128 tokens)")
    elif M <= SKINNY_MAX_M:
        rg = plan[1] if plan is not None else 2
        _check(lib.zf_gemm_bf16_skinny(_ptr(a), _ptr(w), _ptr(out), _ptr(None), M, N, K,
                                       _EPI_SWIGLU, rg, 1, 1 if w_tiled else 0, _stream()),
               "gemm_swiglu (weight streaming)")
    else:
        big = _tile256_variant(M, N, K) if w_tiled else None
        variant = big if big is not None else _tile_variant(M, N, w_tiled, False, K)
        tail = _tile_tail_split(M, N, K) if variant == 10 else None
        if tail is not None:
            _gemm_tile_tail(lib, a, w, out, M, N, K, _EPI_SWIGLU, tail)
            return
        _check(lib.zf_gemm_bf16_tile(_ptr(a), _ptr(w), _ptr(out), M, N, K, _EPI_SWIGLU, variant,
                                     1 if w_tiled else 0, _stream()),
               "gemm_swiglu (tiled)")


# ------------------------------------------------------------------------- attention
MAX_HEAD_DIM = 512          # the wave kernel keeps a head in registers: 8 values a lane
DECODE_SPLIT_KEYS = 256     # keys per split of the decode kernel (DEC_SPLIT in attention.hip)
PREFILL_QUERY_TILE = 32     # queries per tile of the kernels for prompt portions


def mfma_attention_covers(dtype, n_heads, n_kv_heads, head_dim, page_size) -> bool:
    """Whether the bfloat16 MFMA attention kernels serve this shape.  If so, the pools are
    kept in those kernels' own order inside every group of 16 rows (keys ``[hd / 32][16 *
    ((d % 32) / 8) + row][d % 8]``, values ``[hd / 16][16 * (row / 4) + d % 16][row % 4]``);
    otherwise keys are ``[row][hd]`` and values ``[hd][row]`` inside a (page, kv head) block."""
    return dtype == torch.bfloat16 and head_dim in (32, 64, 128, 256) and page_size % 16 == 0 \
        and n_heads // n_kv_heads <= 16


# Up to this many sequences a decode step's attention does the work of qk_norm_rope_kv_write
# itself.  Measured on MI355X (Qwen3-8B shape, context 2100, per layer, against the two kernels
# one after the other): 11.2 -> 8.2 us at batch 1, 15.0 -> 13.1 at 4, 19.1 -> 18.2 at 8,
# 30.2 -> 29.3 at 16, 51.0 -> 50.0 at 32, but 94.6 -> 95.7 at 64, where the chip is busy
# streaming keys and values and a workgroup's longer start costs more than a launch.  At
# context 32768 it gains at batch 1, 8 and 16 alike (245 -> 255, 853 -> 864, 1008 -> 1012
# tokens/s): there one workgroup in 128 also norms and stores a key, at context 2100 one in 9.
FUSED_DECODE_MAX_SEQS = 32


@_launches("attention")
def decode_attention_fused(qkv, q_gain, k_gain, eps, cos, sin, positions, slot_mapping, k_pool,
                           v_pool, block_table, q_start, ctx_len, out, scale, window, n_heads,
                           n_kv_heads, head_dim, page_size, max_ctx_len) -> None:
    """A decode step's attention straight from the q/k/v product: every sequence has exactly
    one token (token s is sequence s's), ``qkv`` [n_seqs, (nH + 2 nKV) hd] is read and not
    changed.  What ``qk_norm_rope_kv_write`` and ``paged_attention`` do one after the other
    (per-head RMSNorm of q and k, rotation at ``positions``, the token's key and value into the
    pools at ``slot_mapping``, attention over the cache) in one kernel less, with the same
    arithmetic and so the same bits.  Only for shapes ``mfma_attention_covers``."""
    _need_gpu(qkv, q_gain, k_gain, cos, sin, positions, slot_mapping, k_pool, v_pool, block_table,
              q_start, ctx_len, out)
    n_seqs = ctx_len.shape[0]
    width = (n_heads + 2 * n_kv_heads) * head_dim
    if not mfma_attention_covers(qkv.dtype, n_heads, n_kv_heads, head_dim, page_size):
        raise KernelUnavailable("decode_attention_fused: bfloat16, head_dim 32/64/128/256, pages "
                                "of a multiple of 16 rows and at most 16 query heads per kv head")
    if qkv.shape != (n_seqs, width) or out.shape != (n_seqs, n_heads * head_dim) \
            or out.dtype != qkv.dtype or k_pool.dtype != qkv.dtype or v_pool.dtype != qkv.dtype:
        raise KernelUnavailable("decode_attention_fused: qkv must be [n_seqs, (nH + 2 nKV) * hd] "
                                "and out [n_seqs, nH * hd], of the pools' dtype")
    if (q_gain is None) != (k_gain is None) or (cos is None) != (sin is None):
        raise KernelUnavailable("decode_attention_fused: gains and tables come in pairs")
    for g in (q_gain, k_gain):
        if g is not None and (g.dtype != torch.float32 or g.shape != (head_dim,)):
            raise KernelUnavailable("decode_attention_fused: a gain must be float32 [head_dim]")
    if cos is not None and (cos.dtype != torch.float32 or cos.shape[1] != head_dim // 2
                            or cos.shape != sin.shape):
        raise KernelUnavailable("decode_attention_fused: tables must be float32 [*, head_dim/2]")
    for t, name in ((block_table, "block_table"), (q_start, "q_start"), (ctx_len, "ctx_len"),
                    (positions, "positions"), (slot_mapping, "slot_mapping")):
        _i32(t, name)
    if q_start.shape[0] != n_seqs + 1 or block_table.shape[0] != n_seqs \
            or positions.shape[0] != n_seqs or slot_mapping.shape[0] != n_seqs:
        raise KernelUnavailable("decode_attention_fused: per-sequence arrays disagree in length")
    if max_ctx_len > block_table.shape[1] * page_size:
        raise KernelUnavailable("decode_attention_fused: block table shorter than the context")
    max_splits = (max_ctx_len + DECODE_SPLIT_KEYS - 1) // DECODE_SPLIT_KEYS
    ws_o = _workspace("attn_o", n_seqs * n_heads * max_splits * head_dim, torch.float32,
                      qkv.device)
    ws_ml = _workspace("attn_ml", n_seqs * n_heads * max_splits * 2, torch.float32, qkv.device)
    lib = build.load("attention")
    _check(lib.zf_attn_decode_fused_bf16(
        _ptr(qkv), _ptr(q_gain), _ptr(k_gain), ctypes.c_float(eps), _ptr(cos), _ptr(sin),
        0 if cos is None else cos.shape[0],
        _ptr(positions), _ptr(slot_mapping), _ptr(k_pool), _ptr(v_pool), _ptr(block_table),
        _ptr(q_start), _ptr(ctx_len), _ptr(out), _ptr(ws_o), _ptr(ws_ml), ctypes.c_float(scale),
        int(window), n_seqs, n_heads, n_kv_heads, head_dim, page_size, block_table.shape[1],
        max_splits, _stream()), "decode_attention_fused")


def _prefill_key_split(n_query_tiles: int, n_kv_heads: int, max_ctx_len: int):
    """(keys per split, splits) if a prompt portion's attention should also split its keys over
    workgroups: few query tiles behind a long context (a 512-token portion at context 4096: 128
    workgroups that walk up to 128 key tiles each) leave half the chip idle and the rest
    waiting on one chain of tiles.  Splits of at least 512 keys, about 512 workgroups; from
    2048 keys on (measured, 481 queries of 40 heads on 8: 4096 keys 223 -> 151 us, 8192 keys
    443 -> 259 us; at 1024 keys the partials cost what the split gains)."""
    wgs = n_query_tiles * n_kv_heads
    if wgs <= 0 or wgs >= 384 or max_ctx_len < 2048:
        return None
    want = (512 + wgs - 1) // wgs
    keys = max(512, ((max_ctx_len + want - 1) // want + 63) // 64 * 64)
    splits = (max_ctx_len + keys - 1) // keys
    return (keys, splits) if splits >= 2 else None


@_launches("attention")
def paged_attention(q, k_pool, v_pool, block_table, q_start, ctx_len, seq_index, out, scale,
                    window, n_heads, n_kv_heads, head_dim, page_size, max_q_len,
                    max_ctx_len, n_single=None, n_query_tiles=None, q_tile_map=None,
                    prefill_max_ctx=None, prefill_variant=0) -> None:
    """Causal grouped-query attention of the step's tokens over the paged cache.  Token t of
    sequence s = seq_index[t] has position ctx_len[s] - q_len[s] + (t - q_start[s]) and reads
    the positions up to its own (the last ``window`` of them if window > 0).  ``n_single`` is
    the number of sequences with exactly one token in this step (None: unknown),
    ``n_query_tiles`` the number of 32-query tiles of the others, ``q_tile_map`` their int32
    (sequence, tile) pairs [n_query_tiles, 2] and ``prefill_max_ctx`` the longest context among
    those sequences (None: unknown): they only decide how the work is cut.
    ``prefill_variant`` picks the kernel for the portions (0: by size; 1: every wave fetches
    its keys and values; 2: they are staged in LDS for a group's heads), for measurements and
    tests.

    bfloat16 with head_dim 32/64/128/256 and a page size that is a multiple of 16 runs the
    MFMA kernels: split-context decode for single tokens, the tiled kernel for portions.
    Everything else runs the 32-bit wave kernel."""
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
    if head_dim > MAX_HEAD_DIM:
        raise KernelUnavailable(f"paged_attention: head_dim {head_dim} > {MAX_HEAD_DIM} is not "
                                "covered")
    if max_ctx_len > block_table.shape[1] * page_size:
        raise KernelUnavailable("paged_attention: block table shorter than the context")
    n_seqs = ctx_len.shape[0]
    if q_start.shape[0] != n_seqs + 1 or block_table.shape[0] != n_seqs or seq_index.shape[0] != T:
        raise KernelUnavailable("paged_attention: per-sequence arrays disagree in length")
    lib = build.load("attention")
    max_pages = block_table.shape[1]
    if mfma_attention_covers(q.dtype, n_heads, n_kv_heads, head_dim, page_size):
        if n_single is None:
            n_single = n_seqs if max_q_len == 1 else -1      # -1: some, not known how many
        if n_single != 0:
            max_splits = (max_ctx_len + DECODE_SPLIT_KEYS - 1) // DECODE_SPLIT_KEYS
            ws_o = _workspace("attn_o", n_seqs * n_heads * max_splits * head_dim, torch.float32,
                              q.device)
            ws_ml = _workspace("attn_ml", n_seqs * n_heads * max_splits * 2, torch.float32,
                               q.device)
            _check(lib.zf_attn_decode_bf16(
                _ptr(q), _ptr(k_pool), _ptr(v_pool), _ptr(block_table), _ptr(q_start),
                _ptr(ctx_len), _ptr(out), _ptr(ws_o), _ptr(ws_ml), ctypes.c_float(scale),
                int(window), n_seqs, n_heads, n_kv_heads, head_dim, page_size, max_pages,
                max_splits, _stream()), "paged_attention (decode)")
        if n_single != n_seqs and max_q_len > 1:
            if q_tile_map is not None:
                _i32(q_tile_map, "q_tile_map")
                if n_query_tiles is None or q_tile_map.shape != (n_query_tiles, 2) \
                        or not q_tile_map.is_cuda or not q_tile_map.is_contiguous():
                    raise KernelUnavailable("paged_attention: q_tile_map must be int32 "
                                            "[n_query_tiles, 2] on the device")
            split = _prefill_key_split(n_query_tiles, n_kv_heads,
                                       prefill_max_ctx if prefill_max_ctx is not None
                                       else max_ctx_len) \
                if n_query_tiles is not None else None
            if split is not None and T * n_heads * split[1] * (head_dim + 2) * 4 > (1 << 28):
                split = None
            ws_o = ws_ml = None
            if split is not None:
                ws_o = _workspace("attn_pre_o", T * n_heads * split[1] * head_dim, torch.float32,
                                  q.device)
                ws_ml = _workspace("attn_pre_ml", T * n_heads * split[1] * 2, torch.float32,
                                   q.device)
            _check(lib.zf_attn_prefill_bf16(
                _ptr(q), _ptr(k_pool), _ptr(v_pool), _ptr(block_table), _ptr(q_start),
                _ptr(ctx_len), _ptr(out), ctypes.c_float(scale), int(window), n_seqs,
                max_q_len, n_heads, n_kv_heads, head_dim, page_size, max_pages,
                1 if n_single != 0 else 0, 1 if max_ctx_len <= 2 * max_q_len else 0,
                _ptr(seq_index), T, _ptr(ws_o), _ptr(ws_ml),
                split[0] if split is not None else 0, split[1] if split is not None else 0,
                _ptr(q_tile_map), n_query_tiles if q_tile_map is not None else 0,
                int(prefill_variant), _stream()), "paged_attention (prefill)")
        return
    _check(lib.zf_paged_attention_wave(
        _ptr(q), _ptr(k_pool), _ptr(v_pool), _dt(q), _ptr(block_table), _ptr(q_start),
        _ptr(ctx_len), _ptr(seq_index), _ptr(out), ctypes.c_float(scale), int(window), T,
        n_heads, n_kv_heads, head_dim, page_size, max_pages, _stream()),
        "paged_attention")


# ------------------------------------------------------------------------- sampling
SAMPLE_MAX_TOP_K = 1024
SAMPLE_ROW_DTYPE = [("temperature", "<f4"), ("top_p", "<f4"), ("min_p", "<f4"), ("top_k", "<i4"),
                    ("u", "<f8")]


@_launches("head_sampling")
def apply_penalties(logits, rows, tokens, counts, params) -> None:
    """In place, for every triple (rows[i], tokens[i], counts[i]): the repetition, presence
    and frequency penalties of ``params[row] = (repetition, presence, frequency)``."""
    _need_gpu(logits, rows, tokens, counts, params)
    for t, name in ((rows, "rows"), (tokens, "tokens"), (counts, "counts")):
        _i32(t, name)
    n, V = rows.shape[0], logits.shape[1]
    if logits.dtype != torch.float32 or params.dtype != torch.float32 \
            or params.shape != (logits.shape[0], 3) or tokens.shape[0] != n or counts.shape[0] != n:
        raise KernelUnavailable("apply_penalties: float32 logits [n, V], params [n, 3], int32 triples")
    lib = build.load("sampling")
    _check(lib.zf_apply_penalties(_ptr(logits), _ptr(rows), _ptr(tokens), _ptr(counts),
                                  _ptr(params), n, V, _stream()), "apply_penalties")


@_launches("head_sampling")
def sample_topk(logits: torch.Tensor, params: torch.Tensor, out: torch.Tensor) -> None:
    """out[r] = a token of row r drawn as the reference's sampler draws it: the top_k
    (1..1024) largest logits, temperature, min-p, top-p, and the uniform number u of the
    row.  ``params`` is a uint8 tensor holding one SAMPLE_ROW_DTYPE record per row."""
    _need_gpu(logits, params, out)
    _i32(out, "out")
    n, V = logits.shape
    if logits.dtype != torch.float32 or params.dtype != torch.uint8 \
            or params.numel() != n * 24 or out.shape != (n,):
        raise KernelUnavailable("sample_topk: float32 logits [n, V], 24-byte records, int32 out [n]")
    lib = build.load("sampling")
    _check(lib.zf_sample_topk(_ptr(logits), _ptr(params), _ptr(out), n, V, _stream()),
           "sample_topk")
