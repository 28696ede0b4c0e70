"""Each HIP kernel alone against its plain torch reference (tests/kernel_refs.py), at sizes
other than the engine's tiny configurations: widths and vocabularies that are no power of
two, head sizes in steps of 16, any number of heads and groups."""
import math

import numpy as np
import pytest
import torch

import kernel_refs as ref
from gpu_util import DEV, rel_err, tol

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def _ops():
    import zinfer_amd.ops as ops
    return ops


def _rand(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("V,H,T", [(1000, 96, 7), (777, 80, 33), (50, 4100, 3)])
def test_embed(dtype, V, H, T):
    table = _rand((V, H), dtype, 1)
    ids = torch.randint(0, V, (T,), generator=torch.Generator().manual_seed(2)).int()
    ids[0], ids[-1] = 0, V - 1
    want = torch.empty((T, H))
    ref.embed(table, ids, want)
    got = torch.empty((T, H), device=DEV)
    _ops().embed(table.to(DEV), ids.to(DEV), got)
    assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("T,W,eps", [(5, 80, 1e-6), (3, 4096, 1e-5), (17, 1000, 3e-6), (1, 7, 0.0)])
def test_rmsnorm(out_dtype, T, W, eps):
    x = _rand((T, W), torch.float32, 3, 2.0)
    gain = 1 + 0.1 * _rand((W,), torch.float32, 4)
    want = torch.empty((T, W), dtype=out_dtype)
    ref.rmsnorm(x, gain, eps, want)
    got = torch.empty((T, W), dtype=out_dtype, device=DEV)
    _ops().rmsnorm(x.to(DEV), gain.to(DEV), eps, got)
    assert rel_err(got, want) <= tol(out_dtype)


def test_rmsnorm_reference_vector():
    """[3, 4] with gains [1, 2], eps 0 -> [0.84852814, 2.2627418]
    (the reference's own test, src/kernel/core/cpu.zig:193-204)."""
    x = torch.tensor([[3.0, 4.0]], device=DEV)
    out = torch.empty_like(x)
    _ops().rmsnorm(x, torch.tensor([1.0, 2.0], device=DEV), 0.0, out)
    assert torch.allclose(out.cpu(), torch.tensor([[0.84852814, 2.2627418]]), atol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,I", [(3, 112), (9, 1000), (1, 5)])
def test_swiglu(dtype, T, I):
    gu = _rand((T, 2 * I), dtype, 5, 3.0)
    want = torch.empty((T, I), dtype=dtype)
    ref.swiglu(gu, want)
    got = torch.empty((T, I), dtype=dtype, device=DEV)
    _ops().swiglu(gu.to(DEV), got)
    assert rel_err(got, want) <= tol(dtype)


def test_swiglu_reference_vector():
    """gate [0, 1, -1], up [1, 2, 3] -> [0, 1.4621172, -0.8068243] (cpu.zig:233-245)."""
    gu = torch.tensor([[0.0, 1.0, -1.0, 1.0, 2.0, 3.0]], device=DEV)
    out = torch.empty((1, 3), device=DEV)
    _ops().swiglu(gu, out)
    assert torch.allclose(out.cpu(), torch.tensor([[0.0, 1.4621172, -0.8068243]]), atol=1e-6)


@pytest.mark.parametrize("a_dtype,w_dtype,o_dtype", [
    (torch.float32, torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16, torch.bfloat16),
    (torch.bfloat16, torch.bfloat16, torch.float32), (torch.bfloat16, torch.float32, torch.bfloat16),
    (torch.float32, torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("M,N,K", [(1, 1000, 96), (7, 77, 80), (65, 130, 33), (130, 64, 4100),
                                   (2, 3, 5)])
def test_gemm(a_dtype, w_dtype, o_dtype, M, N, K):
    a = _rand((M, K), a_dtype, 6)
    w = _rand((N, K), w_dtype, 7, 0.05)
    want = torch.empty((M, N), dtype=o_dtype)
    ref.gemm(a, w, want)
    got = torch.full((M, N), float("nan"), dtype=o_dtype, device=DEV)
    _ops().gemm(a.to(DEV), w.to(DEV), got)
    assert rel_err(got, want) <= tol(o_dtype)


@pytest.mark.parametrize("M", [1, 3, 8, 16, 17, 33, 64, 65, 130, 300, 517])
@pytest.mark.parametrize("N,K", [(1000, 136), (96, 64), (777, 320), (4100, 4096), (256, 1032)])
@pytest.mark.parametrize("o_dtype,accumulate", [(torch.bfloat16, False), (torch.float32, False),
                                                (torch.float32, True)])
def test_gemm_bf16_mfma_paths(M, N, K, o_dtype, accumulate):
    """The bfloat16 MFMA kernels (weight streaming up to 64 rows, tiled above) at sizes that
    are no multiples of their tiles, with each epilogue."""
    a = _rand((M, K), torch.bfloat16, 20)
    w = _rand((N, K), torch.bfloat16, 21, 0.05)
    base = _rand((M, N), torch.float32, 22).to(o_dtype)
    want = base.clone()
    ref.gemm(a, w, want, accumulate)
    got = base.clone().to(DEV)
    _ops().gemm(a.to(DEV), w.to(DEV), got, accumulate)
    assert rel_err(got, want) <= (tol(o_dtype) if not accumulate else 2e-5)


@pytest.mark.parametrize("M", [1, 8, 16, 17, 48, 64, 65, 200, 300])
@pytest.mark.parametrize("N,K", [(64, 64), (4160, 1088), (192, 4096), (1024, 320)])
@pytest.mark.parametrize("o_dtype,accumulate", [(torch.bfloat16, False), (torch.float32, True)])
def test_gemm_pretiled_weights(M, N, K, o_dtype, accumulate):
    """The kernels' own weight layout (made once at load) gives the same product."""
    a = _rand((M, K), torch.bfloat16, 30)
    w = _rand((N, K), torch.bfloat16, 31, 0.05)
    base = _rand((M, N), torch.float32, 32).to(o_dtype)
    want = base.clone()
    ref.gemm(a, w, want, accumulate)
    wt = _ops().pretile_weight(w.to(DEV))
    assert wt.shape == w.shape and not torch.equal(wt.cpu(), w)
    got = base.clone().to(DEV)
    _ops().gemm(a.to(DEV), wt, got, accumulate, w_tiled=True)
    assert rel_err(got, want) <= (tol(o_dtype) if not accumulate else 2e-5)
    plain_out = base.clone().to(DEV)
    _ops().gemm(a.to(DEV), w.to(DEV), plain_out, accumulate)
    assert rel_err(got, plain_out) <= (tol(o_dtype) if not accumulate else 2e-5)


@pytest.mark.parametrize("M", [17, 32, 33, 47, 64, 65, 100, 128])
@pytest.mark.parametrize("N,K", [(192, 4096), (4160, 1024), (16448, 512), (320, 384)])
@pytest.mark.parametrize("kind", ["store", "store32", "accumulate", "swiglu"])
def test_gemm_17_to_128_tokens(M, N, K, kind):
    """The kernel for 17 to 128 tokens on pre-tiled weights (the tokens through LDS, 128
    outputs per workgroup, split along K when the tiles are few): outputs that are no
    multiple of its tile, one and several workgroups along K, each epilogue.  The tokens
    differ in scale, so a row that lands in another token's place shows."""
    ops = _ops()
    plan = ops._mid_plan(M, N, K, True, kind == "swiglu")
    if plan is None:
        pytest.skip("the weight-streaming kernel serves this size")
    a = _rand((M, K), torch.bfloat16, 70) * (1 + torch.arange(M)[:, None] % 5).to(torch.bfloat16)
    w = _rand((N, K), torch.bfloat16, 71, 0.05)
    if kind == "swiglu":
        wi = ops.interleave_gate_up(w[:N // 2].to(DEV), w[N // 2:].to(DEV))
        want = torch.empty((M, N // 2), dtype=torch.bfloat16)
        ref.gemm_swiglu(a, wi.cpu(), want)
        got = torch.full((M, N // 2), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.gemm_swiglu(a.to(DEV), ops.pretile_weight(wi), got, w_tiled=True)
        assert rel_err(got, want) <= tol(torch.bfloat16)
        return
    acc = kind == "accumulate"
    o_dtype = torch.bfloat16 if kind == "store" else torch.float32
    base = _rand((M, N), torch.float32, 72).to(o_dtype)
    want = base.clone()
    ref.gemm(a, w, want, acc)
    got = base.clone().to(DEV)
    ops.gemm(a.to(DEV), ops.pretile_weight(w.to(DEV)), got, acc, w_tiled=True)
    assert rel_err(got, want) <= (2e-5 if acc else tol(o_dtype))


@pytest.mark.parametrize("M,N,K", [(m, n, k) for m in (17, 33, 64, 65, 128, 129, 200)
                                   for n, k in ((192, 4096), (4160, 2048), (8192, 1024), (256, 2112))]
                         # widths with measured plans: the weight-streaming kernel split along K
                         # at 1 to 16 tokens and at 17 to 32, the other kernel above
                         + [(1, 5120, 17408), (8, 5120, 17408), (16, 5120, 25600), (17, 5120, 5120),
                            (24, 5120, 17408), (32, 5120, 8192), (40, 5120, 5120), (64, 4096, 12288)]
                         # several hundred tokens on a long K: 128 x 256 tiles split along K
                         + [(700, 512, 8192), (1030, 1344, 8448), (1280, 320, 12288)])
def test_gemm_sum_norm(M, N, K):
    """The residual sum whose split-K partials are added, summed into the residual and normed
    by one kernel, against sum and norm in 64-bit.  Tokens of different scale: another row's
    1 / rms would show."""
    ops = _ops()
    a = _rand((M, K), torch.bfloat16, 80)
    w = _rand((N, K), torch.bfloat16, 81, 0.05)
    base = _rand((M, N), torch.float32, 82, 2.0) * (1 + torch.arange(M).float()[:, None] % 7)
    gain = 1 + 0.1 * _rand((N,), torch.float32, 83)
    eps = 1e-5
    wt = ops.pretile_weight(w.to(DEV))
    plan = ops.sum_norm_plan(M, N, K, wt, True)
    if plan is None:
        pytest.skip("this product is not split along K: the norm runs on its own")
    if (N, K) in ((5120, 17408), (5120, 25600), (5120, 5120), (5120, 8192)) and M <= 32:
        assert plan[0] == "skinny" and plan[-1] >= 2, plan
    if M > 640:
        assert plan[0] == "wide" and (K // 64) % (2 * plan[1]) == 0, plan
    x = base.double() + a.double() @ w.double().T
    want = torch.empty((M, N), dtype=torch.float64)
    ref.rmsnorm(x, gain, eps, want)
    res = base.clone().to(DEV)
    normed = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.gemm_sum_norm(a.to(DEV), wt, res, gain.to(DEV), eps, normed)
    assert rel_err(res, x) <= tol(torch.float32)
    assert rel_err(normed, want) <= tol(torch.bfloat16)
    # the residual has the same bits as from the separate kernels (partials added in the same
    # order); the norm's sum of squares is added over another number of threads
    # (up to 16 tokens the plain product is not split, so its sums come in another order)
    if M > 16:
        res2 = base.clone().to(DEV)
        ops.gemm(a.to(DEV), wt, res2, True, w_tiled=True)
        assert torch.equal(res, res2)


@pytest.mark.parametrize("kind", ["store", "accumulate", "swiglu"])
@pytest.mark.parametrize("K", [192, 256, 64])
@pytest.mark.parametrize("M,N,variant", [(4100, 4160, 10), (2100, 6208, 6)])
def test_gemm_many_large_tiles(kind, K, M, N, variant):
    """Enough 128 x 256 tiles (and, at the second size, 128 x 128 tiles) to fill the chip more
    than once: the kernels that take pre-tiled W straight into their operands and copy the
    tokens straight into LDS, with edges in M and N that are no multiple of the tile; an odd
    and an even number of k-tiles (W one or two k-tiles ahead) and one."""
    ops = _ops()
    assert ops._tile_variant(M, N, True, kind == "accumulate", K) == \
        (16 if variant == 6 and K % 128 == 0 else variant)
    assert variant == 10 or ((M + 127) // 128) * ((N + 127) // 128) >= 384
    _check_tiled(ops, kind, M, N, K, variant)


@pytest.mark.parametrize("kind", ["store", "accumulate", "swiglu"])
@pytest.mark.parametrize("M,N,K", [(2048, 4096, 4096), (1300, 2112, 512), (130, 320, 256),
                                   (257, 576, 768), (1999, 4160, 1024)])
def test_gemm_large_tiles_with_two_groups_of_waves(kind, M, N, K):
    """The 128 x 256 tiles with two groups of four waves in a workgroup, each over half of K,
    which hand each other a column block through LDS at the end: edges in M and N, two to 32
    k-tiles a group, every epilogue, against the plain product; and that the rule takes it
    where one round holds the tiles and K is long."""
    ops = _ops()
    _check_tiled(ops, kind, M, N, K, 12, seed=91)
    assert ops._tile_variant(2048, 4096, True, True, 12288) == 12
    assert ops._tile_variant(2048, 4096, True, True, 2048) == 10


def test_gemm_two_groups_of_waves_need_whole_steps():
    """A K whose k-tiles do not divide over the two groups' pairs of steps is refused."""
    from zinfer_amd.errors import KernelUnavailable
    ops = _ops()
    a = _rand((256, 192), torch.bfloat16, 92).to(DEV)
    wt = ops.pretile_weight(_rand((256, 192), torch.bfloat16, 93).to(DEV))
    out = torch.zeros((256, 256), dtype=torch.float32, device=DEV)
    with pytest.raises(KernelUnavailable):
        ops.gemm(a, wt, out, w_tiled=True, tile_variant=12)


def _check_tiled(ops, kind, M, N, K, variant, seed=35, tile_tail=None):
    """One tiled kernel on pre-tiled W against the plain product."""
    how = dict(tile_variant=variant) if tile_tail is None else dict(tile_tail=tile_tail)
    a = _rand((M, K), torch.bfloat16, seed)
    w = _rand((N, K), torch.bfloat16, seed + 1, 0.05)
    if kind == "swiglu":
        wi = ops.interleave_gate_up(w[:N // 2].to(DEV), w[N // 2:].to(DEV))
        want = torch.empty((M, N // 2), dtype=torch.bfloat16)
        ref.gemm_swiglu(a, wi.cpu(), want)
        got = torch.full((M, N // 2), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.gemm_swiglu(a.to(DEV), ops.pretile_weight(wi), got, w_tiled=True, **how)
        assert rel_err(got, want) <= tol(torch.bfloat16)
        return
    acc = kind == "accumulate"
    base = _rand((M, N), torch.float32, seed + 2).to(torch.float32 if acc else torch.bfloat16)
    want = base.clone()
    ref.gemm(a, w, want, acc)
    got = base.clone().to(DEV)
    ops.gemm(a.to(DEV), ops.pretile_weight(w.to(DEV)), got, acc, w_tiled=True, **how)
    assert rel_err(got, want) <= (2e-5 if acc else tol(torch.bfloat16))


@pytest.mark.parametrize("kind", ["store", "accumulate", "swiglu"])
@pytest.mark.parametrize("M,N,K,whole,split", [
    (300, 2112, 1024, 16, 2), (300, 2112, 1024, 20, 8), (257, 2240, 1536, 0, 3),
    (520, 4160, 640, 80, 5), (4100, 4160, 256, 512, 2), (130, 320, 192, 1, 3),
    (200, 512, 320, 2, 2)])
def test_gemm_large_tiles_with_the_last_round_split_along_k(kind, M, N, K, whole, split):
    """The 128 x 256 tiles with the tiles from ``whole`` on shared by ``split`` workgroups each
    along K and their partials added by a second kernel: edges in M and N that are no multiple
    of the tile, parts of an even and an odd number of k-tiles and parts that are not all
    equal (W one or two k-tiles ahead), every epilogue; against the plain product, and against
    the same tiles unsplit up to the order of the sums."""
    ops = _ops()
    _check_tiled(ops, kind, M, N, K, 10, seed=81, tile_tail=(whole, split))


def test_gemm_last_round_split_is_chosen_and_agrees():
    """Where the rule splits the last round (more than 512 tiles of 128 x 256, a short last
    round, a long K) the product goes through that path, and its result is the unsplit one's
    up to the order in which 32-bit sums are added."""
    ops = _ops()
    M, N, K = 520, 27648 + 256, 4096         # 5 x 109 = 545 tiles: a last round of 33
    tail = ops._tile_tail_split(M, N, K)
    assert tail is not None and tail[0] == 512 and ops._tile_variant(M, N, True, False, K) == 10
    a = _rand((M, K), torch.bfloat16, 83).to(DEV)
    wt = ops.pretile_weight(_rand((N, K), torch.bfloat16, 84, 0.05).to(DEV))
    chosen = torch.empty((M, N), dtype=torch.float32, device=DEV)
    forced = torch.empty_like(chosen)
    whole = torch.empty_like(chosen)
    before = ops.launch_count()
    ops.gemm(a, wt, chosen, w_tiled=True)
    assert ops.launch_count() == before + 1
    ops.gemm(a, wt, forced, w_tiled=True, tile_tail=tail)
    ops.gemm(a, wt, whole, w_tiled=True, tile_variant=10)
    assert torch.equal(chosen, forced)
    assert not torch.equal(chosen, whole) and rel_err(chosen, whole) <= 2e-5
    # the tiles of the whole rounds have the unsplit product's bits
    same = (chosen == whole).float().mean().item()
    assert same > 0.9


@pytest.mark.parametrize("kind", ["store", "accumulate", "swiglu"])
@pytest.mark.parametrize("M,N,K,variant", [
    (256, 256, 128, 20), (700, 640, 384, 20), (513, 448, 640, 20), (2100, 1600, 256, 20),
    (256, 192, 128, 21), (1000, 960, 512, 21), (300, 576, 384, 21), (257, 832, 256, 21),
    (256, 128, 128, 22), (999, 448, 256, 22), (513, 384, 640, 22), (300, 8192 + 64, 128, 22)])
def test_gemm_256_token_tiles(kind, M, N, K, variant):
    """The kernel with one 256-token tile per CU (256, 192 or 128 outputs wide): edges in M and
    N that are no multiple of the tile, one to five rounds of its ring of four k-tiles, more
    tiles than CUs, every epilogue."""
    _check_tiled(_ops(), kind, M, N, K, variant, seed=41)


@pytest.mark.parametrize("M,N,K", [(130, 768, 256), (300, 1088, 384), (520, 1024, 128), (640, 896, 640)])
def test_gemm_64_token_tiles_above_128_tokens(M, N, K):
    """A few hundred tokens on a narrow output go through tiles of 64 tokens x 128 outputs,
    unsplit: edges in M and N, one to five k-tiles of 128, against the plain product and, bit
    for bit, the 128-token tiles."""
    ops = _ops()
    assert ops._tile64_covers(M, N, K, False) and not ops._tile64_covers(M, N, K, True)
    a = _rand((M, K), torch.bfloat16, 61)
    w = _rand((N, K), torch.bfloat16, 62, 0.05)
    wt = ops.pretile_weight(w.to(DEV))
    for dtype in (torch.bfloat16, torch.float32):
        want = torch.empty((M, N), dtype=dtype)
        ref.gemm(a, w, want, False)
        got = torch.full((M, N), float("nan"), dtype=dtype, device=DEV)
        ops.gemm(a.to(DEV), wt, got, w_tiled=True)
        assert rel_err(got, want) <= (2e-5 if dtype == torch.float32 else tol(torch.bfloat16))
        other = torch.empty_like(got)
        ops.gemm(a.to(DEV), wt, other, w_tiled=True, tile_variant=6)
        assert torch.equal(got, other)


def test_gemm_256_token_tiles_are_chosen_and_agree():
    """Where the cost model picks the 256-token tiles the product goes through them, with the
    same bits as through the 128-token tiles: the sums are added in the same order."""
    ops = _ops()
    for M, N, K in [(2048, 6144, 512), (1536, 6144, 256), (3072, 4096, 384)]:
        variant = ops._tile256_variant(M, N, K)
        assert variant in (20, 21, 22), (M, N, K, variant)
        a = _rand((M, K), torch.bfloat16, 51).to(DEV)
        wt = ops.pretile_weight(_rand((N, K), torch.bfloat16, 52, 0.05).to(DEV))
        chosen = torch.empty((M, N), dtype=torch.bfloat16, device=DEV)
        forced = torch.empty_like(chosen)
        small = torch.empty_like(chosen)
        ops.gemm(a, wt, chosen, w_tiled=True)
        ops.gemm(a, wt, forced, w_tiled=True, tile_variant=variant)
        ops.gemm(a, wt, small, w_tiled=True, tile_variant=6)
        assert torch.equal(chosen, forced) and torch.equal(chosen, small)


@pytest.mark.parametrize("variant", [20, 21, 22, 10, 16])
@pytest.mark.parametrize("K", [4096, 12288])
def test_gemm_tiled_kernels_at_a_served_k(variant, K):
    """The tiled kernels at the K the engine runs them with (4096: 128 trips round the
    256-token tiles' ring of four k-tiles of 32; 12288: the down product's), where the offsets
    into both operands are largest: against the plain product and, bit for bit, the 128 x 128
    tiles; 64-token tiles of 128 outputs likewise."""
    ops = _ops()
    M, N = 512, 1024
    a = _rand((M, K), torch.bfloat16, 71)
    w = _rand((N, K), torch.bfloat16, 72, 0.02)
    wt = ops.pretile_weight(w.to(DEV))
    want = torch.empty((M, N), dtype=torch.float32)
    ref.gemm(a, w, want, False)
    got = torch.full((M, N), float("nan"), dtype=torch.float32, device=DEV)
    ops.gemm(a.to(DEV), wt, got, w_tiled=True, tile_variant=variant)
    assert rel_err(got, want) <= 2e-5
    small = torch.empty_like(got)
    ops.gemm(a.to(DEV), wt, small, w_tiled=True, tile_variant=6)
    assert torch.equal(got, small)
    if variant == 20:
        # and the residual sum with its 32-bit accumulate epilogue
        base = _rand((M, N), torch.float32, 73)
        want = base.clone()
        ref.gemm(a, w, want, True)
        got = base.clone().to(DEV)
        ops.gemm(a.to(DEV), wt, got, True, w_tiled=True, tile_variant=variant)
        assert rel_err(got, want) <= 2e-5


@pytest.mark.parametrize("M", [1, 8, 16, 17, 40, 64, 65, 200, 300])
@pytest.mark.parametrize("I,K,tiled", [(32, 64, True), (12288 // 8, 320, True), (96, 136, False),
                                       (352, 4096, True), (8192, 192, True)])
def test_gemm_swiglu(M, I, K, tiled):
    """silu(a Wg^T) * (a Wu^T) in the product's epilogue, against the plain reference, with
    gate and up rows interleaved in groups of 16 (and the result of the separate kernels)."""
    ops = _ops()
    a = _rand((M, K), torch.bfloat16, 40)
    g = _rand((I, K), torch.bfloat16, 41, 0.08)
    u = _rand((I, K), torch.bfloat16, 42, 0.08)
    w = ops.interleave_gate_up(g.to(DEV), u.to(DEV))
    want = torch.empty((M, I), dtype=torch.bfloat16)
    ref.gemm_swiglu(a, w.cpu(), want)
    plain_gu = a.double() @ torch.cat([g, u]).double().T
    assert rel_err(want, (torch.nn.functional.silu(plain_gu[:, :I]) * plain_gu[:, I:])) <= tol(torch.bfloat16)
    if tiled:
        w = ops.pretile_weight(w)
    got = torch.full((M, I), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.gemm_swiglu(a.to(DEV), w, got, w_tiled=tiled)
    assert rel_err(got, want) <= tol(torch.bfloat16)


@pytest.mark.parametrize("M", [1, 8, 16, 17, 33, 64])
@pytest.mark.parametrize("N,K", [(6144, 4096), (4160, 1088), (64, 64), (24576, 320)])
@pytest.mark.parametrize("kind", ["bf16", "f32", "swiglu"])
def test_norm_gemm(M, N, K, kind):
    """The RMSNorm folded into the weight-streaming product against norm-then-product in
    64-bit: 32-bit sum of squares and scale, bfloat16 operands."""
    ops = _ops()
    x = _rand((M, K), torch.float32, 50, 2.0)
    gain = 1 + 0.1 * _rand((K,), torch.float32, 51)
    w = _rand((N, K), torch.bfloat16, 52, 0.05)
    eps = 1e-5
    normed = torch.empty((M, K), dtype=torch.float64)
    ref.rmsnorm(x, gain, eps, normed)
    if ops.norm_gemm_plan(M, N, K, w.to(DEV), True) is None and kind != "swiglu":
        pytest.skip("this size uses a split over workgroups: the norm runs on its own")
    if kind == "swiglu":
        I = N // 2
        wi = ops.interleave_gate_up(w[:I].to(DEV), w[I:].to(DEV))
        want = torch.empty((M, I), dtype=torch.float64)
        ref.gemm_swiglu(normed, wi.cpu(), want)
        got = torch.full((M, I), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.norm_gemm(x.to(DEV), gain.to(DEV), eps, ops.pretile_weight(wi), got, swiglu=True)
    else:
        o_dtype = torch.bfloat16 if kind == "bf16" else torch.float32
        want = normed @ w.double().T
        got = torch.full((M, N), float("nan"), dtype=o_dtype, device=DEV)
        ops.norm_gemm(x.to(DEV), gain.to(DEV), eps, ops.pretile_weight(w.to(DEV)), got)
    # the operands are rounded to bfloat16 once (2^-9 each), the sums are 32-bit
    assert rel_err(got, want) <= 2.0 ** -7


@pytest.mark.parametrize("M", [1, 7, 16])
@pytest.mark.parametrize("H,K1,N2", [(4096, 12288, 6144), (1088, 320, 4160), (64, 64, 128)])
@pytest.mark.parametrize("kind", ["bf16", "f32", "swiglu"])
def test_gemm_emit_then_given(M, H, K1, N2, kind):
    """The residual sum whose epilogue leaves bfloat16(x * gain) and partial sums of x^2 for
    the norm that follows, and the product that takes them, against sum, norm and product
    in 64-bit.  Tokens of different scale: a wrong row's 1 / rms would show."""
    ops = _ops()
    a = _rand((M, K1), torch.bfloat16, 60, 1.0)
    w1 = _rand((H, K1), torch.bfloat16, 61, 0.05)
    base = _rand((M, H), torch.float32, 62, 2.0) * (1 + torch.arange(M).float()[:, None])
    gain = 1 + 0.1 * _rand((H,), torch.float32, 63)
    w2 = _rand((N2, H), torch.bfloat16, 64, 0.05)
    eps = 1e-5
    if ops.norm_emit_plan(M, H, K1, w1.to(DEV), True) is None:
        pytest.skip("this size is not covered: the norm runs on its own")
    x = base.double() + a.double() @ w1.double().T
    res = base.clone().to(DEV)
    xg = torch.full((M, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    sq = torch.full((H // 16, 16), float("nan"), dtype=torch.float32, device=DEV)
    ops.gemm_emit(a.to(DEV), ops.pretile_weight(w1.to(DEV)), res, gain.to(DEV), xg, sq)
    assert rel_err(res, x) <= tol(torch.float32)
    assert rel_err(xg, x * gain.double()) <= tol(torch.bfloat16)
    assert rel_err(sq.sum(0)[:M], (x * x).sum(-1)) <= 1e-5
    assert torch.equal(sq[:, M:], torch.zeros_like(sq[:, M:]))
    normed = torch.empty((M, H), dtype=torch.float64)
    ref.rmsnorm(x, gain, eps, normed)
    if kind == "swiglu":
        I = N2 // 2
        wi = ops.interleave_gate_up(w2[:I].to(DEV), w2[I:].to(DEV))
        want = torch.empty((M, I), dtype=torch.float64)
        ref.gemm_swiglu(normed, wi.cpu(), want)
        got = torch.full((M, I), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.gemm_given(xg, sq, eps, ops.pretile_weight(wi), got, swiglu=True)
    else:
        if ops.norm_gemm_plan(M, N2, H, w2.to(DEV), True) is None:
            pytest.skip("the second product uses a split over workgroups")
        want = normed @ w2.double().T
        got = torch.full((M, N2), float("nan"), dtype=torch.bfloat16 if kind == "bf16"
                         else torch.float32, device=DEV)
        ops.gemm_given(xg, sq, eps, ops.pretile_weight(w2.to(DEV)), got)
    assert rel_err(got, want) <= 2.0 ** -7


@pytest.mark.parametrize("a_dtype", DTYPES)
def test_gemm_accumulate_and_one_hot(a_dtype):
    """out += a w^T in 32-bit; a one-hot row picks a column of W (the reference's
    probe-linear, src/app/cli/inspect.zig:109-151)."""
    M, N, K = 5, 70, 48
    w = _rand((N, K), a_dtype, 8)
    a = torch.zeros((M, K), dtype=a_dtype)
    for m in range(M):
        a[m, (m * 11) % K] = 1.0
    base = _rand((M, N), torch.float32, 9)
    got = base.clone().to(DEV)
    _ops().gemm(a.to(DEV), w.to(DEV), got, accumulate=True)
    want = base + torch.stack([w[:, (m * 11) % K].float() for m in range(M)])
    assert rel_err(got, want) <= 1e-6


def test_gemm_reference_vector():
    """[[1,2,3],[4,5,6]] . [1, .5, -1] = [-1, .5] (src/kernel/core/cpu.zig:177-191)."""
    w = torch.tensor([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]], device=DEV)
    a = torch.tensor([[1.0, 0.5, -1.0]], device=DEV)
    out = torch.empty((1, 2), device=DEV)
    _ops().gemm(a, w, out)
    assert torch.allclose(out.cpu(), torch.tensor([[-1.0, 0.5]]), atol=1e-6)


def test_gemm_row_does_not_depend_on_batch():
    """A row's result is bitwise the same alone and inside a larger batch (float32 path)."""
    a = _rand((70, 200), torch.float32, 10).to(DEV)
    w = _rand((90, 200), torch.float32, 11).to(DEV)
    full = torch.empty((70, 90), device=DEV)
    _ops().gemm(a, w, full)
    for m in (0, 33, 69):
        one = torch.empty((1, 90), device=DEV)
        _ops().gemm(a[m:m + 1].contiguous(), w, one)
        assert torch.equal(one[0], full[m])


def _paged_setup(dtype, nH, nKV, hd, page_size, ctx_lens, q_lens, seed, num_pages=None):
    """Random q and contiguous K/V per sequence, scattered into pages in a shuffled order."""
    g = torch.Generator().manual_seed(seed)
    n = len(ctx_lens)
    pages_per = [(c + page_size - 1) // page_size for c in ctx_lens]
    total = sum(pages_per)
    num_pages = num_pages or total + 3
    perm = torch.randperm(num_pages, generator=g).tolist()
    max_pages = max(pages_per)
    bt = torch.full((n, max_pages), -1, dtype=torch.int32)
    k_pool = torch.full((num_pages, nKV, page_size, hd), float("nan")).to(dtype)
    v_pool = torch.full((num_pages, nKV, hd, page_size), float("nan")).to(dtype)
    Ks, Vs = [], []
    cur = 0
    for s in range(n):
        K = _rand((ctx_lens[s], nKV, hd), dtype, seed * 100 + s)
        V = _rand((ctx_lens[s], nKV, hd), dtype, seed * 100 + 50 + s)
        Ks.append(K); Vs.append(V)
        for i in range(pages_per[s]):
            pg = perm[cur]; cur += 1
            bt[s, i] = pg
            lo, hi = i * page_size, min((i + 1) * page_size, ctx_lens[s])
            k_pool[pg, :, :hi - lo] = K[lo:hi].transpose(0, 1)
            v_pool[pg, :, :, :hi - lo] = V[lo:hi].permute(1, 2, 0)
    T = sum(q_lens)
    q = _rand((T, nH * hd), dtype, seed + 7)
    q_start = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
    seq_index = torch.repeat_interleave(torch.arange(n, dtype=torch.int32),
                                        torch.tensor(q_lens))
    return dict(q=q, k_pool=k_pool.view(num_pages, -1), v_pool=v_pool.view(num_pages, -1),
                block_table=bt, q_start=q_start, ctx_len=torch.tensor(ctx_lens, dtype=torch.int32),
                seq_index=seq_index.int(), Ks=Ks, Vs=Vs)


def _run_attention(s, dtype, nH, nKV, hd, page_size, window, q_lens, ctx_lens, tiles_hint=False,
                   variant=0):
    scale = 1.0 / math.sqrt(hd)
    T = s["q"].shape[0]
    want = torch.empty((T, nH * hd), dtype=dtype)
    ref.paged_attention(s["q"], s["k_pool"], s["v_pool"], s["block_table"], s["q_start"],
                        s["ctx_len"], s["seq_index"], want, scale, window, nH, nKV, hd,
                        page_size, max(q_lens), max(ctx_lens))
    got = torch.full((T, nH * hd), float("nan"), dtype=dtype, device=DEV)
    d = {k: v.to(DEV) for k, v in s.items() if isinstance(v, torch.Tensor)}
    if _ops().mfma_attention_covers(dtype, nH, nKV, hd, page_size):
        # the MFMA kernels read pools in their own order (what qk_norm_rope_kv_write writes)
        d["k_pool"] = ref.tile_k_pool(d["k_pool"], nKV, page_size, hd)
        d["v_pool"] = ref.tile_v_pool(d["v_pool"], nKV, page_size, hd)
    _ops().paged_attention(d["q"], d["k_pool"], d["v_pool"], d["block_table"], d["q_start"],
                           d["ctx_len"], d["seq_index"], got, scale, window, nH, nKV, hd,
                           page_size, max(q_lens), max(ctx_lens),
                           n_single=sum(1 for n in q_lens if n == 1), prefill_variant=variant,
                           **_tile_hints(q_lens, ctx_lens, tiles_hint))
    return got, want


def _tile_hints(q_lens, ctx_lens, on):
    """What the engine passes with a step: the query tiles of the sequences with more than one
    token (heaviest first) and those sequences' longest context."""
    if not on:
        return {}
    tiles = [(c - n + min(32 * (t + 1), n), i, t) for i, (n, c) in enumerate(zip(q_lens, ctx_lens))
             if n > 1 for t in range((n + 31) // 32)]
    tiles.sort(key=lambda x: -x[0])
    tmap = torch.tensor([(i, t) for _, i, t in tiles], dtype=torch.int32, device=DEV).view(-1, 2)
    return dict(n_query_tiles=len(tiles), q_tile_map=tmap if tiles else None,
                prefill_max_ctx=max((c for c, n in zip(ctx_lens, q_lens) if n > 1), default=None))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nH,nKV,hd,page_size,window", [
    (4, 2, 16, 16, 0), (8, 2, 32, 8, 0), (3, 1, 48, 16, 0), (6, 3, 80, 4, 0),
    (8, 8, 64, 16, 0), (5, 5, 128, 32, 0), (4, 1, 112, 16, 0), (4, 2, 32, 16, 19),
    (2, 1, 64, 8, 8), (6, 2, 96, 16, 100)])
def test_paged_attention_mixed_batch(dtype, nH, nKV, hd, page_size, window):
    """Portions of prompts (some starting mid-context) beside single decode tokens."""
    ctx_lens = [37, 150, 1, 64, 129, 16]
    q_lens = [37, 1, 1, 5, 129 - 100, 2]
    s = _paged_setup(dtype, nH, nKV, hd, page_size, ctx_lens, q_lens, seed=3)
    got, want = _run_attention(s, dtype, nH, nKV, hd, page_size, window, q_lens, ctx_lens)
    assert not torch.isnan(got.float()).any(), "a slot outside the context was read"
    assert rel_err(got, want) <= tol(dtype)


@pytest.mark.parametrize("nH,nKV,hd,page_size,window", [
    (8, 2, 32, 16, 0), (32, 8, 128, 16, 0), (6, 6, 64, 32, 0), (16, 1, 64, 16, 0),
    (9, 3, 256, 16, 0), (8, 2, 64, 16, 37), (4, 4, 128, 48, 300), (36, 4, 32, 16, 0),
    (16, 2, 128, 16, 0), (8, 2, 128, 32, 100), (16, 2, 128, 16, 45), (10, 2, 128, 16, 0),
    (6, 2, 64, 48, 20), (4, 2, 128, 64, 0), (24, 2, 64, 16, 0)])
@pytest.mark.parametrize("kind", ["decode", "prefill", "mixed", "whole"])
def test_paged_attention_mfma(nH, nKV, hd, page_size, window, kind):
    """The bfloat16 MFMA kernels: decode tokens over contexts that end at, before and after a
    split's and a page's edge; portions that start mid-context; both in one batch; whole
    prompts (where the waves of a head split its key tiles between them)."""
    dtype = torch.bfloat16
    if kind == "decode":
        ctx_lens = [1, 15, 16, 17, 255, 256, 257, 600, 1025]
        q_lens = [1] * len(ctx_lens)
    elif kind == "whole":
        ctx_lens = [37, 150, 64, 300, 2, 257]
        q_lens = list(ctx_lens)
    elif kind == "prefill":
        ctx_lens = [37, 150, 64, 129, 700, 2]
        q_lens = [37, 50, 33, 129 - 100, 200, 2]
    else:
        ctx_lens = [37, 300, 1, 64, 129, 513, 16]
        q_lens = [37, 1, 1, 5, 29, 1, 2]
    s = _paged_setup(dtype, nH, nKV, hd, page_size, ctx_lens, q_lens, seed=9)
    got, want = _run_attention(s, dtype, nH, nKV, hd, page_size, window, q_lens, ctx_lens)
    assert not torch.isnan(got.float()).any(), "a slot outside the context was read"
    assert rel_err(got, want) <= 2 * tol(dtype)     # probabilities are rounded once more
    # with the engine's hints (the list of query tiles that exist, heaviest first)
    got, want = _run_attention(s, dtype, nH, nKV, hd, page_size, window, q_lens, ctx_lens,
                               tiles_hint=True)
    assert not torch.isnan(got.float()).any(), "a slot outside the context was read"
    assert rel_err(got, want) <= 2 * tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_paged_attention_far_key_stands_out(dtype):
    """One key among hundreds is aligned with the query and scaled up, so that the softmax
    puts all weight on it: the output must be that position's value row.  The position is
    put at a page's first row, a page's last row and the very first token in turn."""
    nH, nKV, hd, ps = 4, 2, 64, 16
    ctx = 700
    for target in (16 * 20, 16 * 31 - 1, 0, ctx - 1):
        s = _paged_setup(dtype, nH, nKV, hd, ps, [ctx], [1], seed=5)
        q = s["q"].view(1, nH, hd).float()
        kp = s["k_pool"].view(-1, nKV, ps, hd)
        page = int(s["block_table"][0, target // ps])
        for kvh in range(nKV):
            direction = q[0, kvh * 2] / q[0, kvh * 2].norm()
            kp[page, kvh, target % ps] = (direction * 400.0).to(dtype)
        got, want = _run_attention(s, dtype, nH, nKV, hd, ps, 0, [1], [ctx])
        for h in (0, 2):   # the heads whose query the key was aligned with
            v_row = s["Vs"][0][target, h // 2].float()
            assert torch.allclose(got.cpu().float()[0, h * hd:(h + 1) * hd], v_row, atol=2e-2), \
                f"target {target}, head {h}"
        assert rel_err(got, want) <= tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_paged_attention_window_edge(dtype):
    """A huge key just outside the window must have no influence; the one just inside takes
    all the weight."""
    nH, nKV, hd, ps, window = 2, 1, 32, 8, 24
    ctx = 100
    pos = ctx - 1
    for target, inside in ((pos - window, False), (pos - window + 1, True)):
        s = _paged_setup(dtype, nH, nKV, hd, ps, [ctx], [1], seed=6)
        q = s["q"].view(1, nH, hd).float()
        kp = s["k_pool"].view(-1, nKV, ps, hd)
        page = int(s["block_table"][0, target // ps])
        kp[page, 0, target % ps] = (q[0, 0] / q[0, 0].norm() * 400.0).to(dtype)
        got, want = _run_attention(s, dtype, nH, nKV, hd, ps, window, [1], [ctx])
        v_row = s["Vs"][0][target, 0].float()
        close = torch.allclose(got.cpu().float()[0, :hd], v_row, atol=2e-2)
        assert close == inside
        assert rel_err(got, want) <= tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nH,nKV,hd,page_size,use_norm,use_rope", [
    (4, 2, 16, 16, True, True), (8, 2, 32, 8, True, True), (3, 1, 48, 16, True, True),
    (5, 5, 128, 4, False, True), (6, 2, 80, 16, True, False), (2, 2, 256, 16, True, True)])
def test_qk_norm_rope_kv_write(dtype, nH, nKV, hd, page_size, use_norm, use_rope):
    from zinfer_amd.parts.position import rotary_tables
    T, num_pages, eps = 11, 9, 1e-5
    width = (nH + 2 * nKV) * hd
    qkv = _rand((T, width), dtype, 12)
    qg = (1 + 0.1 * _rand((hd,), torch.float32, 13)) if use_norm else None
    kg = (1 + 0.1 * _rand((hd,), torch.float32, 14)) if use_norm else None
    cos, sin = rotary_tables(hd, 10000.0, 300) if use_rope else (None, None)
    positions = torch.tensor([0, 1, 2, 299, 150, 7, 8, 9, 63, 64, 65], dtype=torch.int32)
    slots = torch.randperm(num_pages * page_size, generator=torch.Generator().manual_seed(1))[:T].int()
    row = nKV * page_size * hd
    pools = [torch.zeros((num_pages, row), dtype=dtype) for _ in range(4)]
    q_want = torch.empty((T, nH * hd), dtype=dtype)
    ref.qk_norm_rope_kv_write(qkv.clone(), qg, kg, eps, cos, sin, positions, slots, pools[0],
                              pools[1], q_want, nH, nKV, hd, page_size)
    dv = lambda t: None if t is None else t.to(DEV)
    q_got = torch.empty((T, nH * hd), dtype=dtype, device=DEV)
    kp, vp = pools[2].to(DEV), pools[3].to(DEV)
    _ops().qk_norm_rope_kv_write(qkv.to(DEV), dv(qg), dv(kg), eps, dv(cos), dv(sin),
                                 positions.to(DEV), slots.to(DEV), kp, vp, q_got, nH, nKV, hd,
                                 page_size)
    assert rel_err(q_got, q_want) <= tol(dtype)
    if _ops().mfma_attention_covers(dtype, nH, nKV, hd, page_size):
        pools[0] = ref.tile_k_pool(pools[0], nKV, page_size, hd)
        pools[1] = ref.tile_v_pool(pools[1], nKV, page_size, hd)
    assert rel_err(kp, pools[0]) <= tol(dtype)
    assert torch.equal(vp.cpu(), pools[1])
    # in place, nothing stored: q and k come back in the qkv buffer, v is untouched
    want_inplace = qkv.clone()
    ref.qk_norm_rope_kv_write(want_inplace, qg, kg, eps, cos, sin, positions, None, pools[0],
                              pools[1], None, nH, nKV, hd, page_size)
    got_inplace = qkv.to(DEV)
    _ops().qk_norm_rope_kv_write(got_inplace, dv(qg), dv(kg), eps, dv(cos), dv(sin),
                                 positions.to(DEV), None, kp, vp, None, nH, nKV, hd, page_size)
    assert rel_err(got_inplace, want_inplace) <= tol(dtype)


@pytest.mark.parametrize("T", [5, 300])
def test_positions_beyond_the_rotation_tables_read_their_last_row(T):
    """A position that the tables do not hold (the engine refuses such a step before it runs;
    a caller of the kernel alone may not) is taken as the tables' last row, or first: the
    result is that of the clipped positions, and nothing is read out of bounds."""
    from zinfer_amd.parts.position import rotary_tables
    ops = _ops()
    nH, nKV, hd, page_size, rows = 4, 2, 64, 16, 40
    width = (nH + 2 * nKV) * hd
    qkv = _rand((T, width), torch.bfloat16, 21).to(DEV)
    gain = (1 + 0.1 * _rand((hd,), torch.float32, 22)).to(DEV)
    cos, sin = (t.to(DEV) for t in rotary_tables(hd, 10000.0, rows))
    positions = (torch.arange(T, dtype=torch.int32) * 17 - 20)         # -20 .. beyond 40
    assert positions.min() < 0 and positions.max() >= rows
    slots = torch.arange(T, dtype=torch.int32).to(DEV)
    n_pages = (T + page_size - 1) // page_size
    got, want = [], []
    for pos, into in ((positions, got), (positions.clamp(0, rows - 1), want)):
        q = torch.empty((T, nH * hd), dtype=torch.bfloat16, device=DEV)
        kp = torch.zeros((n_pages, nKV * page_size * hd), dtype=torch.bfloat16, device=DEV)
        vp = torch.zeros_like(kp)
        ops.qk_norm_rope_kv_write(qkv, gain, gain, 1e-6, cos, sin, pos.to(DEV), slots, kp, vp, q,
                                  nH, nKV, hd, page_size)
        into += [q, kp, vp]
    for a, b in zip(got, want):
        assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nH,nKV,hd,page_size", [(32, 8, 128, 16), (6, 2, 64, 32), (3, 1, 48, 16),
                                                 (8, 2, 32, 8), (4, 4, 256, 16)])
def test_qk_norm_rope_kv_write_of_hundreds_of_tokens(dtype, nH, nKV, hd, page_size):
    """From 256 tokens on a workgroup takes four tokens in a row and stores the values of four
    consecutive rows at once: portions that start at a page's edge, in the middle of a group of
    four rows and one row before a page's end, single tokens between them, slots in no order
    at all, and a number of tokens that is no multiple of four."""
    from zinfer_amd.parts.position import rotary_tables
    ops, eps = _ops(), 1e-6
    width = (nH + 2 * nKV) * hd
    runs = [(0, 130), (3, 57), (-1, 70), (1, 1), (2, 2), (0, 4), (5, 3)]   # (start row in a fresh page, tokens)
    slots, positions, page = [], [], 0
    for start, n in runs:
        first = page * page_size + (start % page_size)
        slots += list(range(first, first + n))
        positions += list(range(7 + start % page_size, 7 + start % page_size + n))
        page = (first + n + page_size - 1) // page_size + 1
    g = torch.Generator().manual_seed(3)
    extra = (torch.randperm(8 * page_size, generator=g)[:40] + page * page_size).tolist()
    slots += extra
    positions += [int(x) % 300 for x in extra]
    page += 9
    T = len(slots)
    assert T >= 256 and T % 4 != 0
    qkv = _rand((T, width), dtype, 12)
    qg, kg = (1 + 0.1 * _rand((hd,), torch.float32, 13)), (1 + 0.1 * _rand((hd,), torch.float32, 14))
    cos, sin = rotary_tables(hd, 10000.0, 400)
    slots_t = torch.tensor(slots, dtype=torch.int32)
    pos_t = torch.tensor(positions, dtype=torch.int32)
    row = nKV * page_size * hd
    pools = [torch.zeros((page, row), dtype=dtype) for _ in range(4)]
    q_want = torch.empty((T, nH * hd), dtype=dtype)
    ref.qk_norm_rope_kv_write(qkv.clone(), qg, kg, eps, cos, sin, pos_t, slots_t, pools[0],
                              pools[1], q_want, nH, nKV, hd, page_size)
    q_got = torch.full((T, nH * hd), float("nan"), dtype=dtype, device=DEV)
    kp, vp = pools[2].to(DEV), pools[3].to(DEV)
    ops.qk_norm_rope_kv_write(qkv.to(DEV), qg.to(DEV), kg.to(DEV), eps, cos.to(DEV), sin.to(DEV),
                              pos_t.to(DEV), slots_t.to(DEV), kp, vp, q_got, nH, nKV, hd, page_size)
    assert rel_err(q_got, q_want) <= tol(dtype)
    if ops.mfma_attention_covers(dtype, nH, nKV, hd, page_size):
        pools[0] = ref.tile_k_pool(pools[0], nKV, page_size, hd)
        pools[1] = ref.tile_v_pool(pools[1], nKV, page_size, hd)
    assert rel_err(kp, pools[0]) <= tol(dtype)
    assert torch.equal(vp.cpu(), pools[1])
    # the same tokens one at a time give the same bits (the kernel's other path)
    q_one = torch.empty_like(q_got)
    kp1, vp1 = pools[2].to(DEV), pools[3].to(DEV)
    for lo in range(0, T, 100):
        hi = min(T, lo + 100)
        ops.qk_norm_rope_kv_write(qkv[lo:hi].to(DEV), qg.to(DEV), kg.to(DEV), eps, cos.to(DEV),
                                  sin.to(DEV), pos_t[lo:hi].to(DEV), slots_t[lo:hi].to(DEV), kp1,
                                  vp1, q_one[lo:hi], nH, nKV, hd, page_size)
    bits = lambda t: t.view(torch.int16 if dtype == torch.bfloat16 else torch.int32)
    assert torch.equal(bits(q_one), bits(q_got)) and torch.equal(bits(kp1), bits(kp))
    assert torch.equal(bits(vp1), bits(vp))


@pytest.mark.parametrize("nH,nKV,hd,page_size,window,use_norm,use_rope", [
    (32, 8, 128, 16, 0, True, True), (8, 2, 32, 16, 0, True, True), (6, 6, 64, 32, 0, True, False),
    (16, 1, 64, 16, 37, False, True), (9, 3, 256, 16, 0, True, True), (10, 2, 128, 48, 300, True, True),
    (36, 4, 32, 16, 0, False, False), (32, 2, 128, 16, 0, True, True), (9, 1, 256, 32, 0, True, True)])
def test_decode_attention_fused_equals_the_two_kernels(nH, nKV, hd, page_size, window, use_norm,
                                                       use_rope):
    """The decode attention that norms and rotates q and k and stores the token's key and
    value itself, against qk_norm_rope_kv_write followed by paged_attention: the same bits in
    the output and in both pools.  Contexts end at, before and after a split's (256) and a
    page's edge; the slot of the token's own position holds NaN beforehand, as a page that is
    used again may; 16 query heads to a kv head and head size 256 take two rounds of the
    workgroup's lanes; the rotation's positions are not the cache's (they come from their own
    array)."""
    from zinfer_amd.parts.position import rotary_tables
    dtype, ops = torch.bfloat16, _ops()
    _fused_against_two_kernels(ops, nH, nKV, hd, page_size, window, use_norm, use_rope,
                               [1, 15, 16, 17, 255, 256, 257, 600, 1025, 512, 513])
    # no context beyond one split: the attention kernels write the output themselves
    _fused_against_two_kernels(ops, nH, nKV, hd, page_size, window, use_norm, use_rope,
                               [1, 2, 16, 17, 100, 255, 256])


@pytest.mark.parametrize("M,nH,nKV,hd,page_size,H", [(64, 32, 8, 128, 16, 4096), (40, 8, 2, 64, 16, 2560), (60, 8, 2, 64, 16, 2048),
                                                     (33, 4, 4, 128, 32, 4096), (128, 16, 2, 128, 16, 5120)])
def test_qk_norm_rope_kv_write_from_a_split_products_partials(M, nH, nKV, hd, page_size, H):
    """17 to 128 tokens: the q/k/v product runs split along K.  Its partials handed to the
    kernel that norms, rotates and stores give the bits of the usual way (a kernel adds the
    partials into bfloat16 rows, then that kernel): q and both pools."""
    from zinfer_amd.parts.position import rotary_tables
    ops, dtype = _ops(), torch.bfloat16
    N = (nH + 2 * nKV) * hd
    w = ops.pretile_weight((_rand((N, H), dtype, 41) * 0.05).to(DEV))
    ks = ops.gemm_partials_plan(M, N, H, w, True)
    assert ks is not None and ks > 1, "the test means a product that is split along K"
    a = _rand((M, H), dtype, 42).to(DEV)
    qg = (1 + 0.1 * _rand((hd,), torch.float32, 43)).to(DEV)
    kg = (1 + 0.1 * _rand((hd,), torch.float32, 44)).to(DEV)
    cos, sin = (t.to(DEV) for t in rotary_tables(hd, 10000.0, 400))
    positions = torch.arange(M, dtype=torch.int32, device=DEV) * 3 % 400
    num_pages = (M + page_size - 1) // page_size + 2
    slots = torch.randperm(num_pages * page_size, generator=torch.Generator().manual_seed(2))[:M]
    slots = slots.int().to(DEV)
    row = nKV * page_size * hd
    outs = []
    for way in ("usual", "partials"):
        kp = torch.zeros((num_pages, row), dtype=dtype, device=DEV)
        vp = torch.zeros((num_pages, row), dtype=dtype, device=DEV)
        q = torch.full((M, nH * hd), float("nan"), dtype=dtype, device=DEV)
        if way == "usual":
            qkv = torch.empty((M, N), dtype=dtype, device=DEV)
            ops.gemm(a, w, qkv, w_tiled=True)
        else:
            qkv = ops.gemm_partials(a, w, ks)
            assert qkv.shape == (ks, M, N)
        ops.qk_norm_rope_kv_write(qkv, qg, kg, 1e-6, cos, sin, positions, slots, kp, vp, q, nH, nKV,
                                  hd, page_size)
        outs.append((q, kp, vp))
    torch.cuda.synchronize()
    bits = lambda t: t.view(torch.int16)
    assert not torch.isnan(outs[0][0].float()).any()
    for x, y in zip(*outs):
        assert torch.equal(bits(x), bits(y))


@pytest.mark.parametrize("nH,nKV,hd,page_size,window", [(32, 8, 128, 16, 0), (6, 2, 64, 32, 20),
                                                        (16, 1, 32, 16, 0), (6, 3, 256, 16, 0)])
def test_decode_attention_one_split_writes_what_the_merge_would(nH, nKV, hd, page_size, window):
    """No context beyond 256 keys: the decode attention writes its output itself and the merge
    kernel is not launched.  The same batch with a context bound of two splits (as a wider
    block table gives it) goes through the merge kernel: the same bits."""
    dtype, ops = torch.bfloat16, _ops()
    ctx_lens = [1, 2, 16, 17, 100, 255, 256]
    n = len(ctx_lens)
    s = _paged_setup(dtype, nH, nKV, hd, page_size, ctx_lens, [1] * n, seed=31)
    d = {k: v.to(DEV) for k, v in s.items() if isinstance(v, torch.Tensor)}
    d["k_pool"] = ref.tile_k_pool(d["k_pool"], nKV, page_size, hd)
    d["v_pool"] = ref.tile_v_pool(d["v_pool"], nKV, page_size, hd)
    wide = torch.full((n, 512 // page_size + 1), -1, dtype=torch.int32, device=DEV)
    wide[:, :d["block_table"].shape[1]] = d["block_table"]
    outs = []
    for table, bound in ((d["block_table"], 256), (wide, 512)):
        out = torch.full((n, nH * hd), float("nan"), dtype=dtype, device=DEV)
        ops.paged_attention(d["q"], d["k_pool"], d["v_pool"], table, d["q_start"], d["ctx_len"],
                            d["seq_index"], out, 1.0 / math.sqrt(hd), window, nH, nKV, hd,
                            page_size, 1, bound, n_single=n)
        outs.append(out)
    assert not torch.isnan(outs[0].float()).any()
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))
    want = torch.empty((n, nH * hd), dtype=dtype)
    ref.paged_attention(s["q"], s["k_pool"], s["v_pool"], s["block_table"], s["q_start"],
                        s["ctx_len"], s["seq_index"], want, 1.0 / math.sqrt(hd), window, nH, nKV,
                        hd, page_size, 1, 256)
    assert rel_err(outs[0], want) <= 2 * tol(dtype)


def _fused_against_two_kernels(ops, nH, nKV, hd, page_size, window, use_norm, use_rope, ctx_lens):
    from zinfer_amd.parts.position import rotary_tables
    dtype = torch.bfloat16
    n = len(ctx_lens)
    s = _paged_setup(dtype, nH, nKV, hd, page_size, ctx_lens, [1] * n, seed=21)
    num_pages = s["k_pool"].shape[0]
    k_pool = s["k_pool"].view(num_pages, nKV, page_size, hd).clone()
    v_pool = s["v_pool"].view(num_pages, nKV, hd, page_size).clone()
    slots = []
    for i, c in enumerate(ctx_lens):
        pg, r = int(s["block_table"][i, (c - 1) // page_size]), (c - 1) % page_size
        k_pool[pg, :, r] = float("nan")
        v_pool[pg, :, :, r] = float("nan")
        slots.append(pg * page_size + r)
    k_tiled = ref.tile_k_pool(k_pool.view(num_pages, -1).to(DEV), nKV, page_size, hd)
    v_tiled = ref.tile_v_pool(v_pool.view(num_pages, -1).to(DEV), nKV, page_size, hd)
    qkv = _rand((n, (nH + 2 * nKV) * hd), dtype, 22).to(DEV)
    qg = (1 + 0.1 * _rand((hd,), torch.float32, 23)).to(DEV) if use_norm else None
    kg = (1 + 0.1 * _rand((hd,), torch.float32, 24)).to(DEV) if use_norm else None
    cos, sin = (t.to(DEV) for t in rotary_tables(hd, 10000.0, max(1100, max(ctx_lens) + 8))) \
        if use_rope else (None, None)
    positions = torch.tensor([c - 1 + 5 for c in ctx_lens], dtype=torch.int32, device=DEV)
    slot_mapping = torch.tensor(slots, dtype=torch.int32, device=DEV)
    d = {k: s[k].to(DEV) for k in ("block_table", "q_start", "ctx_len", "seq_index")}
    scale, eps = 1.0 / math.sqrt(hd), 1e-6

    kp_a, vp_a = k_tiled.clone(), v_tiled.clone()
    q = torch.empty((n, nH * hd), dtype=dtype, device=DEV)
    ops.qk_norm_rope_kv_write(qkv.clone(), qg, kg, eps, cos, sin, positions, slot_mapping, kp_a,
                              vp_a, q, nH, nKV, hd, page_size)
    want = torch.full((n, nH * hd), float("nan"), dtype=dtype, device=DEV)
    ops.paged_attention(q, kp_a, vp_a, d["block_table"], d["q_start"], d["ctx_len"],
                        d["seq_index"], want, scale, window, nH, nKV, hd, page_size, 1,
                        max(ctx_lens), n_single=n)

    kp_b, vp_b = k_tiled.clone(), v_tiled.clone()
    before = qkv.clone()
    got = torch.full((n, nH * hd), float("nan"), dtype=dtype, device=DEV)
    ops.decode_attention_fused(qkv, qg, kg, eps, cos, sin, positions, slot_mapping, kp_b, vp_b,
                               d["block_table"], d["q_start"], d["ctx_len"], got, scale, window,
                               nH, nKV, hd, page_size, max(ctx_lens))
    torch.cuda.synchronize()
    assert not torch.isnan(want.float()).any() and not torch.isnan(got.float()).any()
    bits = lambda t: t.view(torch.int16)
    assert torch.equal(bits(got), bits(want))
    assert torch.equal(bits(kp_b), bits(kp_a)) and torch.equal(bits(vp_b), bits(vp_a))
    assert torch.equal(bits(qkv), bits(before)), "the product's rows are only read"
    # and what both write is what the plain implementation writes
    kc, vc = k_pool.view(num_pages, -1).clone(), v_pool.view(num_pages, -1).clone()
    ref.qk_norm_rope_kv_write(before.cpu(), None if qg is None else qg.cpu(),
                              None if kg is None else kg.cpu(), eps,
                              None if cos is None else cos.cpu(), None if sin is None else sin.cpu(),
                              positions.cpu(), slot_mapping.cpu(), kc, vc,
                              torch.empty((n, nH * hd), dtype=dtype), nH, nKV, hd, page_size)
    kc = ref.tile_k_pool(kc, nKV, page_size, hd)
    live = ~torch.isnan(kc.float())
    assert torch.equal(live, ~torch.isnan(kp_b.float().cpu()))
    assert rel_err(torch.where(live, kp_b.cpu().float(), 0.0), torch.where(live, kc.float(), 0.0)) <= tol(dtype)


def test_rope_reference_vector():
    """[1, 2, 3, 4] at position 1, theta 1e4: h0 = cos1 - 3 sin1, h1 = 2 cos(.01) - 4 sin(.01),
    h2 = 3 cos1 + sin1, h3 = 4 cos(.01) + 2 sin(.01) (src/kernel/attention/rope.zig:174-190)."""
    from zinfer_amd.parts.position import rotary_tables
    cos, sin = rotary_tables(4, 10000.0, 4)
    qkv = torch.tensor([[1.0, 2.0, 3.0, 4.0] * 3], device=DEV)   # one q, one k, one v head
    pos = torch.tensor([1], dtype=torch.int32, device=DEV)
    dummy = torch.zeros((1, 16), device=DEV)
    _ops().qk_norm_rope_kv_write(qkv, None, None, 0.0, cos.to(DEV), sin.to(DEV), pos, None, dummy,
                                 dummy, None, 1, 1, 4, 4)
    a = 1.0 / math.sqrt(10000.0)
    want = [math.cos(1) - 3 * math.sin(1), 2 * math.cos(a) - 4 * math.sin(a),
            3 * math.cos(1) + math.sin(1), 4 * math.cos(a) + 2 * math.sin(a)]
    assert torch.allclose(qkv.cpu()[0, :4], torch.tensor(want), atol=1e-6)
    assert torch.allclose(qkv.cpu()[0, 4:8], torch.tensor(want), atol=1e-6)
    assert torch.equal(qkv.cpu()[0, 8:], torch.tensor([1.0, 2.0, 3.0, 4.0]))


def test_gather_rows_and_argmax():
    x = _rand((9, 130), torch.float32, 15)
    idx = torch.tensor([8, 0, 3, 3], dtype=torch.int32)
    out = torch.empty((4, 130), device=DEV)
    _ops().gather_rows(x.to(DEV), idx.to(DEV), out)
    assert torch.equal(out.cpu(), x[idx.long()])
    logits = _rand((6, 1000), torch.float32, 16)
    logits[0, 17] = logits[0, 900] = 50.0      # a tie: the first maximum wins
    logits[1, 999] = 60.0
    logits[2, 0] = 60.0
    logits[3] = -float("inf")
    got = torch.empty((6,), dtype=torch.int32, device=DEV)
    _ops().argmax(logits.to(DEV), got)
    want = torch.argmax(logits, dim=-1).int()
    want[3] = 0
    assert torch.equal(got.cpu(), want)
    assert got[0].item() == 17


def test_cpu_tensor_is_refused():
    """There is no CPU path: a tensor that is not on the GPU is an error, not a fallback."""
    from zinfer_amd.errors import KernelUnavailable
    with pytest.raises(KernelUnavailable):
        _ops().rmsnorm(torch.zeros((1, 4)), torch.ones(4), 1e-6, torch.zeros((1, 4)))


@pytest.mark.parametrize("V", [1000, 151936, 7])
def test_sample_topk_against_the_host_sampler(V):
    """The device sampler draws the token the host sampler (the reference's semantics) draws
    for the same uniform number.  Device and host exponentials may differ in the last bit,
    which can only matter when u * sum falls within that rounding of a boundary between two
    candidates: then the neighbouring candidate is accepted."""
    import numpy as np
    import zinfer_amd.ops as ops
    from zinfer_amd.sampling import SamplingParams, Xoshiro256pp, adjust_logits, count_history, \
        sample_token, top_k_candidates

    class FixedU:
        def __init__(self, u):
            self.u = u

        def float64(self):
            return self.u
    rs = np.random.RandomState(5)
    cases = []
    for trial in range(40):
        sp = SamplingParams(temperature=float(rs.choice([0.6, 0.8, 1.0, 1.7])),
                            top_k=int(rs.choice([1, 2, 20, 50, 1024])) if V > 7 else int(rs.choice([1, 3, 7])),
                            top_p=float(rs.choice([1.0, 0.95, 0.8, 0.3])),
                            min_p=float(rs.choice([0.0, 0.05, 0.5])),
                            repetition_penalty=float(rs.choice([1.0, 1.1, 2.0])),
                            presence_penalty=float(rs.choice([0.0, 0.7])),
                            frequency_penalty=float(rs.choice([0.0, 0.2])))
        logits = (rs.randn(V) * 2.5).astype(np.float32)
        if trial % 5 == 0:
            logits[rs.randint(0, V, 4)] = logits.max() + 1.0      # exact ties at the top
        history = rs.randint(0, V, size=rs.randint(0, 60)).tolist()
        cases.append((sp, logits, history, float(rs.rand())))
    n = len(cases)
    lg = torch.from_numpy(np.stack([c[1] for c in cases])).to(DEV)
    rec = np.zeros((n,), dtype=ops.SAMPLE_ROW_DTYPE)
    rows, toks, cnts = [], [], []
    params = np.zeros((n, 3), np.float32)
    for i, (sp, logits, history, u) in enumerate(cases):
        rec[i] = (sp.temperature, sp.top_p, sp.min_p, sp.top_k, u)
        counts = count_history(history, V)
        rows += [i] * len(counts); toks += list(counts.keys()); cnts += list(counts.values())
        params[i] = (sp.repetition_penalty, sp.presence_penalty, sp.frequency_penalty)
    t = lambda a: torch.from_numpy(np.asarray(a, np.int32)).to(DEV)
    if rows:
        ops.apply_penalties(lg, t(rows), t(toks), t(cnts), torch.from_numpy(params).to(DEV))
    for i, (sp, logits, history, u) in enumerate(cases):      # the penalties alone
        adj = adjust_logits(logits, count_history(history, V), sp)
        assert np.allclose(lg[i].cpu().numpy(), adj, rtol=1e-6, atol=1e-6)
    out = torch.empty((n,), dtype=torch.int32, device=DEV)
    ops.sample_topk(lg, torch.from_numpy(rec.view(np.uint8).reshape(-1).copy()).to(DEV), out)
    got = out.cpu().tolist()
    exact = 0
    for i, (sp, logits, history, u) in enumerate(cases):
        want = sample_token(logits, history, sp, FixedU(u))
        if got[i] == want:
            exact += 1
            continue
        adj = adjust_logits(logits, count_history(history, V), sp)
        ids, _ = top_k_candidates(adj, min(sp.top_k, V))
        pos = {int(t): j for j, t in enumerate(ids)}
        assert got[i] in pos and abs(pos[got[i]] - pos[want]) == 1, \
            f"case {i}: device {got[i]}, host {want}"
    assert exact >= n - 2


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["normal", "gain", "zeros"])
def test_randinit_is_the_numpy_draw_bit_for_bit(dtype, kind):
    """The device's counter-based draw and its numpy twin: the same bits for every element,
    from any starting index (2^20 + 77 elements: every octant of the cosine, both branches of
    the logarithm's range reduction, mantissas next to the rounding boundary)."""
    import numpy as np
    from zinfer_amd.weights import counter_rng
    key = counter_rng.tensor_key(12345, "model.layers.3.self_attn.o_proj.weight")
    for start, n in ((0, (1 << 20) + 77), (3_000_000_019, 4099)):
        got = torch.empty((n,), dtype=dtype, device=DEV)
        _ops().randinit(got, key, start, kind, 0.02)
        want = counter_rng.draw(key, start, n, kind, 0.02)
        if dtype == torch.bfloat16:
            want_bits = counter_rng.to_bfloat16_bits(want).astype(np.int32)
            got_bits = got.cpu().view(torch.int16).numpy().astype(np.int32) & 0xFFFF
        else:
            want_bits = want.view(np.int32)
            got_bits = got.cpu().numpy().view(np.int32)
        assert np.array_equal(got_bits, want_bits), \
            f"{int((got_bits != want_bits).sum())} of {n} elements differ"


def test_random_model_on_the_device_is_the_folder_written_on_the_host(tmp_path):
    """``random_model`` (drawn tensor by tensor on the GPU) binds the values that
    ``write_model_dir`` stores from numpy's draw."""
    import tiny
    from zinfer_amd.models.build import load_model, random_model
    from zinfer_amd.weights import write_model_dir
    path = write_model_dir(str(tmp_path / "m"), tiny.config_of("C"), 9, torch.float32, device=None)
    _, a = load_model(path, "float32", DEV)
    _, b = random_model(tiny.config_of("C"), 9, "float32", DEV)
    assert torch.equal(a.embedding, b.embedding)
    assert torch.equal(a.head.weight, b.head.weight)
    for x, y in zip(a.blocks, b.blocks):
        assert torch.equal(x.mixer.qkv.weight, y.mixer.qkv.weight)
        assert torch.equal(x.mixer.q_gain, y.mixer.q_gain)
        assert torch.equal(x.feed_forward.down.weight, y.feed_forward.down.weight)
        assert torch.equal(x.ff_norm.gain, y.ff_norm.gain)


def test_embed_multiplier_and_logit_scale_cap():
    table = _rand((50, 96), torch.bfloat16, 1)
    ids = torch.tensor([3, 49, 0], dtype=torch.int32)
    want = torch.empty((3, 96))
    ref.embed(table, ids, want, 2.5)
    got = torch.empty((3, 96), device=DEV)
    _ops().embed(table.to(DEV), ids.to(DEV), got, 2.5)
    assert torch.equal(got.cpu(), want)
    x = _rand((5, 1003), torch.float32, 2, 4.0)
    for scale, cap in ((0.25, 0.0), (1.0, 3.0), (30.0, 2.5)):
        want = x.clone()
        ref.scale_cap(want, scale, cap)
        got = x.to(DEV)
        _ops().scale_cap(got, scale, cap)
        assert rel_err(got, want) <= 1e-6


def test_device_sampler_order_vectors():
    """The device's penalties and sampler on the cases in which the order of the reference's
    operations decides the token."""
    import numpy as np
    import sampler_vectors as sv
    import zinfer_amd.ops as ops
    for logits, history, params, us, want, why in sv.ORDER_CASES:
        V = 64                               # the cases' logits first, the rest far below
        for u in us:
            row = np.full((1, V), -1e4, np.float32)
            row[0, :len(logits)] = logits
            lg = torch.from_numpy(row).to(DEV)
            counts = {}
            for t in history:
                counts[t] = counts.get(t, 0) + 1
            if counts:
                t32 = lambda a: torch.tensor(a, dtype=torch.int32, device=DEV)
                pen = torch.tensor([[params.get("repetition_penalty", 1.0),
                                     params.get("presence_penalty", 0.0),
                                     params.get("frequency_penalty", 0.0)]], device=DEV)
                ops.apply_penalties(lg, t32([0] * len(counts)), t32(list(counts)),
                                    t32(list(counts.values())), pen)
            rec = np.zeros((1,), dtype=ops.SAMPLE_ROW_DTYPE)
            greedy = params["temperature"] <= 0.0
            rec[0] = (1.0, 1.0, 0.0, 1, 0.0) if greedy else \
                (params["temperature"], params.get("top_p", 1.0), params.get("min_p", 0.0),
                 params["top_k"], u)
            out = torch.empty((1,), dtype=torch.int32, device=DEV)
            ops.sample_topk(lg, torch.from_numpy(rec.view(np.uint8).reshape(-1).copy()).to(DEV), out)
            assert int(out[0]) == want, f"{why}: u = {u}: token {int(out[0])}, not {want}"


def _stand_out(s, nKV, ps, hd, seq, position, query_row, q_head, dtype, nH):
    """Makes the key at ``position`` of sequence ``seq`` take all the weight of query row
    ``query_row``, head ``q_head``: aligned with that query and scaled up."""
    G = nH // nKV
    q = s["q"].view(-1, nH, hd).float()
    kp = s["k_pool"].view(-1, nKV, ps, hd)
    page = int(s["block_table"][seq, position // ps])
    direction = q[query_row, q_head] / q[query_row, q_head].norm()
    kp[page, q_head // G, position % ps] = (direction * 400.0).to(dtype)


@pytest.mark.parametrize("hd", [64, 128])
def test_mfma_decode_window_edge_and_far_key(hd):
    """The MFMA decode kernel (bfloat16, pages of 16) with a key that stands out: just outside
    the window it must have no influence, just inside it takes all the weight; the window's
    first key is put at a page's edge, across a 64-key wave chunk and across a 256-key split."""
    dtype, nH, nKV, ps = torch.bfloat16, 8, 2, 16
    assert _ops().mfma_attention_covers(dtype, nH, nKV, hd, ps)
    for ctx, window in ((700, 0), (700, 188), (700, 189), (700, 445), (1030, 262), (1030, 7),
                        (300, 300), (300, 299), (513, 257)):
        pos = ctx - 1
        targets = [(0, True), (ctx - 1, True), (255, True), (256, True)] if window == 0 else \
            [(pos - window, False), (pos - window + 1, True)]
        for target, inside in targets:
            if target < 0:
                continue
            s = _paged_setup(dtype, nH, nKV, hd, ps, [ctx, 40], [1, 1], seed=21)
            _stand_out(s, nKV, ps, hd, 0, target, 0, 5, dtype, nH)
            got, want = _run_attention(s, dtype, nH, nKV, hd, ps, window, [1, 1], [ctx, 40])
            v_row = s["Vs"][0][target, 5 // (nH // nKV)].float()
            close = torch.allclose(got.cpu().float()[0, 5 * hd:6 * hd], v_row, atol=3e-2)
            assert close == inside, f"ctx {ctx}, window {window}, key {target}"
            assert rel_err(got, want) <= 2 * tol(dtype), f"ctx {ctx}, window {window}, key {target}"


@pytest.mark.parametrize("variant", [1, 2])
@pytest.mark.parametrize("hd", [64, 128])
def test_mfma_prefill_window_edge_and_far_key(hd, variant):
    """Both MFMA prefill kernels (1: every wave fetches its keys and values, 2: they are staged
    in LDS in tiles of 64 keys) on a portion that starts mid-context: for the first and the last
    query of a 32-query tile, a key that stands out at p - window (no influence) and at
    p - window + 1 (all the weight); windows whose first key falls on and beside the edges of a
    32- and a 64-key tile; without a window, a far key at the very start, at the tiles' edges
    and in a later tile that needs no mask (where the exponent the sums are held against has
    to move)."""
    dtype, nH, nKV, ps = torch.bfloat16, 4, 2, 16
    ctx, q_len = 420, 100                       # the portion is positions 320 .. 419
    start = ctx - q_len
    for window in (0, 33, 64, 65, 97, 129, 200, 330):
        for row in (0, 31, 32, 63, 99):         # rows of the portion: tile edges and the last
            p = start + row
            cases = [(0, True), (31, True), (32, True), (63, True), (64, True), (127, True),
                     (200, True), (p, True)] if window == 0 else \
                [(p - window, False), (p - window + 1, True)]
            for target, inside in cases:
                if target < 0:
                    continue
                s = _paged_setup(dtype, nH, nKV, hd, ps, [ctx, 70], [q_len, 70], seed=23)
                _stand_out(s, nKV, ps, hd, 0, target, row, 3, dtype, nH)
                got, want = _run_attention(s, dtype, nH, nKV, hd, ps, window, [q_len, 70],
                                           [ctx, 70], variant=variant)
                v_row = s["Vs"][0][target, 3 // (nH // nKV)].float()
                close = torch.allclose(got.cpu().float()[row, 3 * hd:4 * hd], v_row, atol=3e-2)
                assert close == inside, f"window {window}, query {p}, key {target}"
                assert rel_err(got, want) <= 2 * tol(dtype), \
                    f"window {window}, query {p}, key {target}"


def test_stream_read_reads_every_byte_once():
    """The measurement kernel's xor over the buffer is the xor of all its words, for sizes
    that are and are not a multiple of what one round of the grid takes."""
    ops = _ops()
    for n_words, wgs in ((4 * 1000, 7), (4 * 512 * 8 * 3, 3), (4 * 123457, 64), (1 << 22, 2048)):
        g = torch.Generator().manual_seed(n_words)
        buf = torch.randint(-2 ** 31, 2 ** 31 - 1, (n_words,), generator=g, dtype=torch.int32)
        want = int(np.bitwise_xor.reduce(buf.numpy().view(np.uint32)))
        sink = torch.zeros((wgs,), dtype=torch.int32, device=DEV)
        ops.stream_read(buf.to(DEV), sink, wgs)
        got = int(np.bitwise_xor.reduce(sink.cpu().numpy().view(np.uint32)))
        assert got == want, (n_words, wgs)
    assert ops.measure_read_bandwidth(DEV, nbytes=1 << 28, repeats=2) > 1e12


def test_mfma_loop_sums_its_products():
    """The measurement kernel's accumulators are its rounds times the products of the operands
    it was given, as the lanes of a wave hold them; its rate on zeros is the clock's, on random
    operands what the power limit leaves."""
    ops = _ops()
    g = torch.Generator().manual_seed(9)
    operands = torch.randn((6, 64, 8), generator=g).to(torch.bfloat16)
    # operand f as a matrix [32, 16]: lane l holds row l % 32, k 8 (l / 32) .. + 8
    mats = operands.double().reshape(6, 2, 32, 8).permute(0, 2, 1, 3).reshape(6, 32, 16)
    out = torch.full((8, 32, 32), float("nan"), dtype=torch.float32, device=DEV)
    iters = 37
    ops.mfma_loop(operands.to(DEV), out, 5, iters)
    for n in range(8):
        want = iters * (mats[n % 4] @ mats[4 + n // 4].T)
        assert rel_err(out[n], want) <= 1e-5, n
    rate_zeros = ops.measure_mfma_rate(DEV, random_operands=False, seconds=0.02)
    rate_random = ops.measure_mfma_rate(DEV, seconds=0.02)
    assert 1.0e15 < rate_random <= rate_zeros * 1.02 < 2.6e15, (rate_random, rate_zeros)


def test_check_tables_reports_and_never_traps():
    """The debugging check of a step's tables: a page beyond the pool, a page that is not held
    (-1) inside a context, a context longer than the row, a slot beyond the pool are reported;
    entries beyond a context are not looked at."""
    ops = _ops()
    ps, num_pages = 16, 10
    bt = torch.tensor([[3, 9, -1, -1], [0, 1, 2, -1]], dtype=torch.int32)
    ctx = torch.tensor([20, 48], dtype=torch.int32)
    slots = torch.tensor([3 * 16 + 4, 2 * 16 + 15], dtype=torch.int32)

    def run(bt, ctx, slots):
        rep = torch.zeros(4, dtype=torch.int32, device=DEV)
        ops.check_tables(bt.to(DEV), ctx.to(DEV), None if slots is None else slots.to(DEV), ps,
                         num_pages, rep)
        return rep.tolist()
    assert run(bt, ctx, slots) == [0, 0, 0, 0]
    assert run(bt, ctx, None) == [0, 0, 0, 0]
    bad = bt.clone(); bad[0, 1] = 10
    assert run(bad, ctx, slots) == [1, 0, 1, 10]
    bad = bt.clone(); bad[1, 2] = -1
    assert run(bad, ctx, slots) == [1, 1, 2, -1]
    assert run(bt, torch.tensor([20, 65], dtype=torch.int32), slots)[:2] == [1, 1]
    assert run(bt, ctx, torch.tensor([5, 160], dtype=torch.int32)) == [2, 1, 0, 160]


def test_only_the_kernels_of_a_class_are_launched():
    """Under `only_classes` a launcher of another class leaves its output alone."""
    ops = _ops()
    x = _rand((3, 64), torch.float32, 1).to(DEV)
    gain = torch.ones(64, device=DEV)
    out = torch.full((3, 64), 7.0, device=DEV)
    with ops.only_classes({"attention"}):
        ops.rmsnorm(x, gain, 1e-6, out)
        assert float(out.min()) == 7.0
        with ops.kernel_class("attention"):            # a caller's label wins
            ops.rmsnorm(x, gain, 1e-6, out)
        assert float(out.abs().max()) < 7.0
    out.fill_(7.0)
    ops.rmsnorm(x, gain, 1e-6, out)
    assert float(out.abs().max()) < 7.0
    with pytest.raises(Exception, match="unknown kernel classes"):
        ops.only_classes({"nonsense"})


def test_cast_and_poison_pages():
    x = _rand((37, 101), torch.float32, 5, 3.0)
    out = torch.empty((37, 101), dtype=torch.bfloat16, device=DEV)
    _ops().cast(x.to(DEV), out)
    assert torch.equal(out.cpu(), x.to(torch.bfloat16))           # nearest even, as torch rounds
    back = torch.empty((37, 101), dtype=torch.float32, device=DEV)
    _ops().cast(out, back)
    assert torch.equal(back.cpu(), x.to(torch.bfloat16).float())  # widening is exact
    for dtype in DTYPES:
        pool = torch.ones((3, 9, 50), dtype=dtype, device=DEV)
        _ops().poison_pages(pool, torch.tensor([7, 0, 4], dtype=torch.int32, device=DEV))
        bad = torch.isnan(pool.float()).cpu()
        assert bad[:, [0, 4, 7]].all() and not bad[:, [1, 2, 3, 5, 6, 8]].any()


@pytest.mark.parametrize("variant", [1, 2, 3])
@pytest.mark.parametrize("nH,nKV,hd,ps,window", [
    (8, 2, 128, 16, 0), (10, 2, 128, 16, 0), (16, 2, 64, 32, 0), (3, 1, 128, 48, 0),
    (2, 2, 64, 16, 0), (18, 2, 128, 16, 0), (8, 2, 128, 16, 150), (5, 1, 64, 16, 64),
    (4, 2, 128, 16, 0), (6, 2, 64, 16, 90)])
def test_both_prefill_kernels_on_portions_and_whole_prompts(nH, nKV, hd, ps, window, variant):
    """Each MFMA prefill kernel, chosen by hand (1: every wave fetches its own keys and values;
    2: staged in LDS, with two groups of waves on the even and the odd key tiles where four
    heads or fewer share a kv head and the prompts are whole; 3: staged, one group), over
    groups of 1, 2, 3, 4, 5, 8 and 9 query heads (9: two blocks of heads per kv head):
    portions whose keys end at, before and after the edges of 64-key tiles, and whole prompts
    with odd and even numbers of key tiles; pages of 16, 32 and 48 rows in a shuffled pool
    whose unwritten rows are NaN, with and without the engine's list of tiles."""
    dtype = torch.bfloat16
    for ctx_lens, q_lens in (([64, 65, 127, 128, 129, 300, 1000, 40, 2],
                              [64, 65, 127, 64, 2, 237, 130, 7, 2]),
                             ([64, 65, 128, 129, 192, 193, 300, 700, 2],
                              [64, 65, 128, 129, 192, 193, 300, 700, 2])):
        s = _paged_setup(dtype, nH, nKV, hd, ps, ctx_lens, q_lens, seed=41)
        for hint in (False, True):
            got, want = _run_attention(s, dtype, nH, nKV, hd, ps, window, q_lens, ctx_lens,
                                       tiles_hint=hint, variant=variant)
            assert not torch.isnan(got.float()).any(), "a row outside the context was read"
            assert rel_err(got, want) <= 2 * tol(dtype)


@pytest.mark.parametrize("nH,nKV,hd,window", [(10, 2, 128, 0), (8, 1, 64, 0), (4, 1, 128, 0),
                                              (10, 2, 128, 700), (6, 2, 64, 33)])
@pytest.mark.parametrize("variant", [1, 2])
def test_prefill_attention_splits_keys_over_workgroups(nH, nKV, hd, window, variant):
    """Portions behind long contexts, few query tiles: the keys are split over workgroups and
    a second kernel merges the partials.  Portions that start at 0, mid-page and at a split's
    edge, a short prompt whose keys lie in one split, single tokens beside them; and a key
    that stands out at a split's last and first position."""
    dtype, ps = torch.bfloat16, 16
    ops = _ops()
    ctx_lens = [2300, 1024 + 40, 70, 1500, 1]
    q_lens = [100, 40, 70, 33, 1]
    tiles = sum((n + 31) // 32 for n in q_lens if n > 1)
    split = ops._prefill_key_split(tiles, nKV, max(ctx_lens))
    assert split is not None and split[1] >= 2
    s = _paged_setup(dtype, nH, nKV, hd, ps, ctx_lens, q_lens, seed=31)
    got, want = _run_attention(s, dtype, nH, nKV, hd, ps, window, q_lens, ctx_lens, tiles_hint=True,
                               variant=variant)
    assert not torch.isnan(got.float()).any(), "a slot outside the context was read"
    assert rel_err(got, want) <= 2 * tol(dtype)
    # the same without the hint (one workgroup walks all keys): equal up to rounding
    plain, _ = _run_attention(s, dtype, nH, nKV, hd, ps, window, q_lens, ctx_lens, variant=variant)
    assert rel_err(got, plain) <= 2 * tol(dtype)
    if window == 0:
        keys = split[0]
        for target in (keys - 1, keys, 2 * keys - 1, 0):
            s = _paged_setup(dtype, nH, nKV, hd, ps, ctx_lens, q_lens, seed=32)
            row = 57                     # a query of the first sequence (position 2257)
            _stand_out(s, nKV, ps, hd, 0, target, row, nH - 1, dtype, nH)
            got, want = _run_attention(s, dtype, nH, nKV, hd, ps, 0, q_lens, ctx_lens,
                                       tiles_hint=True, variant=variant)
            v_row = s["Vs"][0][target, (nH - 1) // (nH // nKV)].float()
            assert torch.allclose(got.cpu().float()[row, (nH - 1) * hd:nH * hd], v_row, atol=3e-2), target
            assert rel_err(got, want) <= 2 * tol(dtype)


# ---------------------------------------------------------------- the served decode regime
# Contexts of thousands of keys at the served head shapes: more than 8 splits of 256 keys (where
# a lane of the merge kernel takes a second, third, ... load) and more than 64 (where it goes
# round its loop again), which the short contexts above never reach.
SERVED_HEADS = [(32, 8, 128, 16), (40, 8, 128, 16), (64, 8, 128, 16)]
LONG_CONTEXTS = [2048, 2049, 2304, 4097, 8192, 32768]


def _long_pools(nKV, hd, ps, ctx_lens, seed):
    """Pools made on the device (rows [page, kv head, row, hd], values [page, kv head, hd,
    row]) with pages dealt in a shuffled order and NaN in every row beyond a context."""
    g = torch.Generator(device=DEV).manual_seed(seed)
    pages_per = [(c + ps - 1) // ps for c in ctx_lens]
    num_pages = sum(pages_per) + 5
    perm = torch.randperm(num_pages, generator=g, device=DEV)
    k = torch.randn((num_pages, nKV, ps, hd), generator=g, device=DEV).to(torch.bfloat16)
    v = torch.randn((num_pages, nKV, hd, ps), generator=g, device=DEV).to(torch.bfloat16)
    bt = torch.full((len(ctx_lens), max(pages_per)), -1, dtype=torch.int32, device=DEV)
    held = torch.zeros((num_pages,), dtype=torch.bool, device=DEV)
    cur = 0
    for i, (c, n) in enumerate(zip(ctx_lens, pages_per)):
        pages = perm[cur:cur + n]
        cur += n
        bt[i, :n] = pages.int()
        held[pages] = True
        if c % ps:
            k[pages[-1], :, c % ps:] = float("nan")
            v[pages[-1], :, :, c % ps:] = float("nan")
    k[~held] = float("nan")
    v[~held] = float("nan")
    return k, v, bt


def _long_reference(q, k, v, bt, ctx_lens, nH, nKV, hd, ps, scale):
    """softmax(q K^T scale) V of every sequence's one query over its whole context, in 64-bit."""
    G = nH // nKV
    out = torch.empty((len(ctx_lens), nH * hd), dtype=torch.float64, device=DEV)
    for i, c in enumerate(ctx_lens):
        pages = bt[i, :(c + ps - 1) // ps].long()
        K = k[pages].permute(1, 0, 2, 3).reshape(nKV, -1, hd)[:, :c].double()
        V = v[pages].permute(1, 0, 3, 2).reshape(nKV, -1, hd)[:, :c].double()
        qi = q[i].view(nKV, G, hd).double()
        a = torch.softmax(torch.einsum("kgd,knd->kgn", qi, K) * scale, dim=-1)
        out[i] = torch.einsum("kgn,knd->kgd", a, V).reshape(-1)
    return out


def _long_decode(nH, nKV, hd, ps, ctx_lens, seed, stand_out=()):
    """The decode attention kernels (splits + merge) against the 64-bit reference.
    ``stand_out``: (sequence, position, query head) triples whose key is aligned with the query
    and scaled up; returns output and reference."""
    ops = _ops()
    n = len(ctx_lens)
    k, v, bt = _long_pools(nKV, hd, ps, ctx_lens, seed)
    g = torch.Generator(device=DEV).manual_seed(seed + 1)
    q = torch.randn((n, nH * hd), generator=g, device=DEV).to(torch.bfloat16)
    G = nH // nKV
    for i, pos, head in stand_out:
        qv = q[i].view(nH, hd)[head].float()
        k[bt[i, pos // ps].long(), head // G, pos % ps] = (qv / qv.norm() * 400.0).to(torch.bfloat16)
    scale = 1.0 / math.sqrt(hd)
    want = _long_reference(q, k, v, bt, ctx_lens, nH, nKV, hd, ps, scale)
    num_pages = k.shape[0]
    kt = ref.tile_k_pool(k.view(num_pages, -1), nKV, ps, hd)
    vt = ref.tile_v_pool(v.view(num_pages, -1), nKV, ps, hd)
    got = torch.full((n, nH * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    q_start = torch.arange(n + 1, dtype=torch.int32, device=DEV)
    ctx = torch.tensor(ctx_lens, dtype=torch.int32, device=DEV)
    ops.paged_attention(q, kt, vt, bt, q_start, ctx, q_start[:n].contiguous(), got, scale, 0, nH,
                        nKV, hd, ps, 1, max(ctx_lens), n_single=n)
    torch.cuda.synchronize()
    return got, want, v, bt


@pytest.mark.parametrize("nH,nKV,hd,ps", SERVED_HEADS)
@pytest.mark.parametrize("batch", [1, 8, 64])
def test_decode_attention_at_served_contexts(nH, nKV, hd, ps, batch):
    """One token per sequence over 2048 to 32768 keys (9 to 128 splits): contexts that end at
    a split's edge, one key beyond it, and deep in the merge kernel's second round."""
    if batch == 1:
        cases = [[c] for c in LONG_CONTEXTS]
    elif batch == 8:
        cases = [LONG_CONTEXTS + [1, 300], [16385, 16384, 20000, 257, 2047, 2050, 16640, 5]]
    else:
        cases = [[LONG_CONTEXTS[i % 5] + 7 * i for i in range(60)] + [32768, 16385, 1, 256]]
    for ctx_lens in cases:
        got, want, _, _ = _long_decode(nH, nKV, hd, ps, ctx_lens, seed=5 + len(ctx_lens))
        assert not torch.isnan(got.float()).any(), f"contexts {ctx_lens[:8]}: NaN was read"
        err = (got.double() - want).abs().amax(dim=1) / want.abs().amax(dim=1)
        bad = torch.nonzero(err > 2 * tol(torch.bfloat16)).flatten().tolist()
        assert not bad, f"sequences {bad} of contexts {ctx_lens}: error {err[bad[0]]:.3g}"


@pytest.mark.parametrize("nH,nKV,hd,ps", SERVED_HEADS)
def test_decode_attention_far_key_in_late_splits(nH, nKV, hd, ps):
    """A key that takes all the weight at the first and at the last key of splits 8, 9 and 127
    (the ninth and tenth partial of a lane's first round of loads, the last of its second):
    the output is that position's value row."""
    G = nH // nKV
    for pos in (8 * 256, 9 * 256 - 1, 9 * 256, 10 * 256 - 1, 127 * 256, 128 * 256 - 1):
        ctx_lens = [32768, max(pos + 1, 2305)]
        head = (pos // 256 * 5) % nH
        got, want, v, bt = _long_decode(nH, nKV, hd, ps, ctx_lens, seed=pos,
                                        stand_out=[(0, pos, head), (1, pos, head)])
        for i in (0, 1):
            row = v[bt[i, pos // ps].long(), head // G, :, pos % ps].float()
            mine = got[i].view(nH, hd)[head].float()
            assert torch.allclose(mine, row, atol=3e-2), f"key {pos}, context {ctx_lens[i]}"
        err = (got.double() - want).abs().max() / want.abs().max()
        assert err <= 2 * tol(torch.bfloat16), f"key {pos}: error {err:.3g}"


@pytest.mark.parametrize("nH,nKV,hd,ps", SERVED_HEADS)
def test_decode_attention_fused_at_served_contexts(nH, nKV, hd, ps):
    """The fused decode attention (steps of up to 32 sequences) against the two kernels it
    replaces, bit for bit in output and pools, at 2048 to 32768 keys; alone (batch 1) and
    eight together."""
    ops = _ops()
    _fused_against_two_kernels(ops, nH, nKV, hd, ps, 0, True, True,
                               [2048, 2049, 2304, 4097, 8192, 32768, 16385, 300])
    for c in (2049, 32768):
        _fused_against_two_kernels(ops, nH, nKV, hd, ps, 0, True, True, [c])
