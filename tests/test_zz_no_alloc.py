"""The arg-max entry point that allocates nothing (`zinfer_amd/csrc/zf_no_alloc.h`), called
through ctypes as a caller without torch's wrappers would: against the ordinary arg-max on two
calls in a row, the second with a smaller input that leaves the first call's partial results
in the shared device array; and its refusals."""
import ctypes

import pytest
import torch

from gpu_util import DEV

pytestmark = pytest.mark.gpu

MAX_PARTIALS = 32768
TOO_LARGE, BAD_ARGUMENT = -2, -1


def _lib():
    from zinfer_amd.ops import build
    lib = build.load("elementwise")
    fn = lib.zf_argmax_no_alloc
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    return fn


def _call(fn, logits, out):
    n, V = logits.shape
    stream = torch.cuda.current_stream().cuda_stream
    return fn(logits.data_ptr(), out.data_ptr(), n, V, stream)


def _logits(n, V, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((n, V), generator=g)
    # equal maxima in a row: the first one must win, also across the 4096-wide chunks
    for r in range(n):
        top = float(x[r].max()) + 1.0
        where = torch.randint(0, V, (3,), generator=g)
        x[r, where] = top
    return x.to(DEV)


def test_two_calls_in_a_row_match_the_ordinary_argmax():
    from zinfer_amd import ops
    fn = _lib()
    for (n, V), seed in (((7, 151936), 1), ((3, 5000), 2)):   # the second is smaller
        logits = _logits(n, V, seed)
        want = torch.empty((n,), dtype=torch.int32, device=DEV)
        ops.argmax(logits, want)
        got = torch.full((n,), -1, dtype=torch.int32, device=DEV)
        assert _call(fn, logits, got) == 0
        torch.cuda.synchronize()
        assert got.tolist() == want.tolist()
        # numpy's argmax returns the first of equal maxima
        assert got.tolist() == logits.cpu().numpy().argmax(axis=1).tolist()


def test_it_allocates_nothing():
    fn = _lib()
    logits = _logits(4, 9001, 3)
    out = torch.empty((4,), dtype=torch.int32, device=DEV)
    assert _call(fn, logits, out) == 0           # the first call on the device is set-up
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    stats_before = torch.cuda.memory_stats().get("allocation.all.allocated", 0)
    for _ in range(5):
        assert _call(fn, logits, out) == 0
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats().get("allocation.all.allocated", 0) == stats_before
    assert torch.cuda.mem_get_info()[0] == free_before


def test_sizes_beyond_the_array_are_refused(capfd):
    fn = _lib()
    V = 4096 * 8 + 1                             # 9 chunks a row
    n = MAX_PARTIALS // 9 + 1
    logits = torch.zeros((n, V), device=DEV)
    out = torch.full((n,), -7, dtype=torch.int32, device=DEV)
    assert _call(fn, logits, out) == TOO_LARGE
    assert "partial results" in capfd.readouterr().err
    torch.cuda.synchronize()
    assert out.eq(-7).all()                      # nothing ran
    assert _call(fn, logits[:n - 1], out[:n - 1]) == 0       # the largest size that fits
    torch.cuda.synchronize()
    assert out[:n - 1].eq(0).all()
    assert fn(None, out.data_ptr(), 1, 8, None) == BAD_ARGUMENT
    assert fn(logits.data_ptr(), out.data_ptr(), 1, 0, None) == BAD_ARGUMENT
    assert fn(logits.data_ptr(), out.data_ptr(), 0, 8, None) == 0


def test_the_python_wrapper():
    from zinfer_amd import ops
    from zinfer_amd.errors import KernelUnavailable
    logits = _logits(5, 1210, 4)
    want = torch.empty((5,), dtype=torch.int32, device=DEV)
    got = torch.empty((5,), dtype=torch.int32, device=DEV)
    ops.argmax(logits, want)
    ops.argmax_no_alloc(logits, got)
    assert got.tolist() == want.tolist()
    with pytest.raises(KernelUnavailable, match="partial results"):
        ops.argmax_no_alloc(torch.zeros((ops.ARGMAX_NO_ALLOC_MAX_PARTIALS + 1, 8), device=DEV),
                            torch.zeros((ops.ARGMAX_NO_ALLOC_MAX_PARTIALS + 1,),
                                        dtype=torch.int32, device=DEV))
