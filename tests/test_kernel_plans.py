"""Which kernel serves which size: the pure decisions of `zinfer_amd.ops`, without a GPU."""
import pytest

from zinfer_amd import ops

SHAPES = [(6144, 4096), (4096, 4096), (24576, 4096), (4096, 12288), (151936, 4096), (192, 64),
          (1024, 320), (4160, 1088)]


@pytest.mark.parametrize("N,K", SHAPES)
def test_products_of_17_to_128_tokens(N, K):
    for M in range(1, 200):
        plan = ops._mid_plan(M, N, K, True)
        if plan is None:
            continue
        assert 16 < M <= 128 and N % 16 == 0 and K % (256 if M <= 32 else 128) == 0
        assert 1 <= plan <= K // (256 if M <= 32 else 128), "more splits than k-tiles"
        assert ops._mid_plan(M, N, K, True, swiglu=True) == 1, "SwiGLU is never split along K"
        assert ops._mid_plan(M, N, K, False) is None, "only pre-tiled weights"
    # the served sizes do take this kernel at 64 and 128 tokens (and the wide one from 17 on)
    if K % 128 == 0 and N % 16 == 0:
        assert ops._mid_plan(64, N, K, True) is not None
        assert ops._mid_plan(128, N, K, True) is not None and ops._mid_plan(129, N, K, True) is None
    if K % 256 == 0 and N >= 16384:
        assert ops._mid_plan(17, N, K, True) is not None


@pytest.mark.parametrize("N,K", SHAPES)
def test_tiled_products(N, K):
    for M in (65, 100, 128, 300, 512, 1024, 2048, 8192):
        ks = ops._tile_ksplit(M, N, K)
        assert 1 <= ks <= 16
        if ks > 1:
            assert K // 64 // ks >= 8, "every workgroup keeps at least 8 k-tiles"
            tiles = ((M + 127) // 128) * ((N + 127) // 128)
            # a split fills the chip's places (256, or 512 with two workgroups to a CU) more
            # evenly than the tiles alone do
            places = lambda n: 256 if n <= 256 else (n + 511) // 512 * 512
            assert tiles < 384 and places(tiles * ks) / (tiles * ks) < places(tiles) / tiles
        assert ops._tile_variant(M, N, True, False, K) in (6, 10, 16)
        if ops._tile_variant(M, N, True, False, K) == 16:
            assert K % 128 == 0
        assert ops._tile_variant(M, N, False) in (0, 4)
    # 2048 tokens at the served widths: 128 x 256 tiles, except where they would fill the chip
    # one and a half times
    assert ops._tile_variant(2048, 24576, True) == 10 and ops._tile_variant(2048, 4096, True) == 10
    assert ops._tile_variant(2048, 6144, True) == 6
    # measured choices at a few hundred tokens (Qwen3-8B and 14B widths)
    for (M, n, k), want in {(512, 5120, 5120): 3, (512, 5120, 17408): 3, (512, 7168, 5120): 1,
                            (512, 4096, 4096): 2, (512, 4096, 12288): 2, (512, 6144, 4096): 1,
                            (256, 4096, 4096): 4, (256, 6144, 4096): 2, (1024, 5120, 17408): 3,
                            (1024, 4096, 12288): 1}.items():
        assert ops._tile_ksplit(M, n, k) == want, (M, n, k)
    assert ops._tile_variant(512, 24576, True, False, 4096) == 10


def test_weight_streaming_plans():
    for N, K in SHAPES:
        for M in (1, 8, 16, 17, 64):
            for tiled in (True, False):
                rg, ks = ops._skinny_plan(M, N, K, tiled)
                assert rg in (1, 2, 4) and 1 <= ks <= 16


def test_the_flat_kernel_table_is_complete_and_its_references_exist():
    """Every function of `zinfer_amd.ops` that launches a kernel is in the table once, its
    module is one the build knows, and the reference it names exists."""
    import importlib
    import inspect
    import os
    import re
    from zinfer_amd.ops import build, table
    launchers = {name for name, fn in vars(ops).items()
                 if inspect.isfunction(fn) and fn.__module__ == "zinfer_amd.ops"
                 and not name.startswith("_") and "build.load(" in inspect.getsource(fn)}
    assert launchers == set(table.KERNELS), launchers ^ set(table.KERNELS)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for name, entry in table.KERNELS.items():
        assert entry.launch is getattr(ops, name)
        assert entry.module in build.MODULES
        path, fn = entry.reference.split(":")
        with open(os.path.join(root, path)) as f:
            assert re.search(rf"^def {fn}\(", f.read(), re.M), entry.reference
        source = inspect.getsource(entry.launch)
        assert f'build.load("{entry.module}")' in source, name
