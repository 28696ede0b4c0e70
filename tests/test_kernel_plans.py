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
        assert ops._tile_variant(M, N, True, False, K) in (6, 10, 12, 16)
        if ops._tile_variant(M, N, True, False, K) == 16:
            assert K % 128 == 0
        if ops._tile_variant(M, N, True, False, K) == 12:      # two groups of waves over K
            assert K % 256 == 0 and ((M + 127) // 128) * ((N + 255) // 256) <= 256
        assert ops._tile_variant(M, N, False) in (0, 4)
    # 2048 tokens at the served widths: 128 x 256 tiles
    assert ops._tile_variant(2048, 24576, True) == 10 and ops._tile_variant(2048, 4096, True) == 10
    assert ops._tile_variant(2048, 4096, True, True, 4096) == 12
    assert ops._tile_variant(2048, 4096, True, True, 4096 + 128) == 10
    assert ops._tile_variant(2048, 24576, True, False, 4096) == 10
    # between one and two large tiles a CU, many rows of them: 128 x 128 tiles, the waves side
    # by side where k-tiles of 128 divide K
    assert ops._tile_variant(2048, 6144, True) == 6
    assert ops._tile_variant(2048, 6144, True, False, 4096) == 16
    assert ops._tile_variant(2048, 5120, True, True, 5120 + 64) == 6
    assert ops._tile_variant(512, 20480, True, False, 5120) == 10        # 320 tiles in 4 rows
    assert ops._tile_variant(192, 19456, True, False, 2560) == 10        # 152 tiles
    # measured choices at a few hundred tokens (Qwen3-8B and 14B widths)
    for (M, n, k), want in {(512, 5120, 5120): 3, (512, 5120, 17408): 3, (512, 7168, 5120): 1,
                            (512, 4096, 4096): 2, (512, 4096, 12288): 2, (512, 6144, 4096): 1,
                            (256, 4096, 4096): 4, (256, 6144, 4096): 2, (1024, 5120, 17408): 3,
                            (1024, 4096, 12288): 1}.items():
        assert ops._tile_ksplit(M, n, k) == want, (M, n, k)
    # a stored product whose tiles need a second round anyway stays whole; a residual sum splits
    assert ops._tile_ksplit(768, 6144, 4096, False) == 1 and ops._tile_ksplit(768, 6144, 4096) > 1
    assert ops._tile_ksplit(384, 6144, 4096, False) == 3
    # one round of large tiles with two groups of waves needs no partials: over a short K it is
    # taken instead of a split, over a long K the split stays
    assert ops._tile_ksplit(1280, 4096, 4096) == 1 and ops._tile_variant(1280, 4096, True, True, 4096) == 12
    assert ops._tile_ksplit(2048, 2560, 4096) == 1
    assert ops._tile_ksplit(1024, 5120, 17408) == 3
    assert ops._tile_variant(512, 24576, True, False, 4096) == 10


def test_64_token_tiles_for_a_few_hundred_tokens_on_a_narrow_output():
    """Measured on MI355X with weights from HBM: where one round of the chip holds the 64 x 128
    tiles (qkv of the 8B shape up to 320 tokens), or where the 128-token tiles would need a
    second round (qkv of the 14B shape at 513 to 576 tokens); not against a single round of
    128-token tiles, not gate/up, not down (long K), not a residual sum, not 128 tokens and
    fewer (the kernels for those), not 768 and more."""
    assert ops._tile64_covers(272, 6144, 4096, False) and ops._tile64_covers(160, 6144, 4096, False)
    assert ops._tile64_covers(384, 6144, 4096, False)          # 288 tiles
    assert ops._tile64_covers(544, 7168, 5120, False)          # 128-token tiles: 280
    assert ops._tile64_covers(384, 5120, 8192, False)
    assert not ops._tile64_covers(512, 6144, 4096, False)      # 384 against 192 in one round
    assert not ops._tile64_covers(384, 7168, 5120, False)
    assert not ops._tile64_covers(768, 6144, 4096, False)
    assert not ops._tile64_covers(512, 24576, 4096, False)
    assert not ops._tile64_covers(512, 4096, 12288, False)
    assert not ops._tile64_covers(512, 4096, 4096, True)
    assert not ops._tile64_covers(128, 6144, 4096, False)
    assert not ops._tile64_covers(272, 6144, 4096 + 64, False)


def test_256_token_tiles_are_chosen_where_they_fill_the_chip_evenly():
    """Measured on MI355X (Qwen3-8B widths): 2048 tokens into 6144 outputs are 256 tiles of
    256 x 192 (101 -> 83 us); 3072 into 4096 (384 tiles of 128 x 256, 192 of 256 x 256: 108
    against 113 us, with 12288 inputs 283 against 277) and 2048 into 4096 stay with 128 x 256
    tiles, gate/up with its many tiles too (the two kinds run it equally fast), and a residual
    sum that is split along K keeps its split."""
    assert ops._tile256_variant(2048, 6144, 4096) == 21
    assert ops._tile256_variant(3072, 4096, 4096, True) == 20
    assert ops._tile256_variant(3072, 4096, 12288, True) == 20
    # up to 256 tokens too, where one row of tiles fills the chip better than two of 128 tokens
    # (192 tokens into the 14B shape's 34816 gate and up outputs: 139 -> 118 us)
    assert ops._tile256_variant(192, 34816, 5120) == 21
    assert ops._tile256_variant(2048, 24576, 4096) is None and ops._tile256_variant(8192, 24576, 4096) is None
    assert ops._tile256_variant(2048, 4096, 4096, True) is None
    assert ops._tile256_variant(2048, 4096, 12288, True) is None
    assert ops._tile256_variant(1024, 24576, 4096) is None
    for M, N, K in [(512, 5120, 5120), (1024, 5120, 17408), (256, 6144, 4096), (200, 24576, 4096)]:
        assert ops._tile256_variant(M, N, K, True) is None
    # a K that the ring of four k-tiles of 32 does not divide, or rows that are no multiple of 16
    assert ops._tile256_variant(2048, 6144, 4096 + 64) is None
    assert ops._tile256_variant(2048, 6144 + 8, 4096) is None


def test_weight_streaming_plans():
    for N, K in SHAPES:
        for M in (1, 8, 16, 17, 64):
            for tiled in (True, False):
                rg, ks = ops._skinny_plan(M, N, K, tiled)
                assert rg in (1, 2, 4) and 1 <= ks <= 16


# which plain function (or, for kernels that are compared with other kernels or through the
# engine, which test) each kernel of the table is checked against
TESTED_AGAINST = {
    "embed": "kernel_refs.py:embed", "rmsnorm": "kernel_refs.py:rmsnorm",
    "qk_norm_rope_kv_write": "kernel_refs.py:qk_norm_rope_kv_write",
    "swiglu": "kernel_refs.py:swiglu", "gather_rows": "kernel_refs.py:gather_rows",
    "argmax": "kernel_refs.py:argmax", "argmax_no_alloc": "kernel_refs.py:argmax",
    "scale_cap": "kernel_refs.py:scale_cap",
    "advance_decode": "test_engine_gpu.py:test_decode_steps_in_a_row_equal_single_steps",
    "cast": "test_kernels_gpu.py:test_cast_and_poison_pages",
    "poison_pages": "test_kernels_gpu.py:test_cast_and_poison_pages",
    "gemm": "kernel_refs.py:gemm", "gemm_partials": "kernel_refs.py:gemm",
    "gemm_swiglu": "kernel_refs.py:gemm_swiglu", "norm_gemm": "kernel_refs.py:rmsnorm",
    "gemm_emit": "kernel_refs.py:gemm", "gemm_given": "kernel_refs.py:rmsnorm",
    "gemm_sum_norm": "kernel_refs.py:rmsnorm", "paged_attention": "kernel_refs.py:paged_attention",
    "decode_attention_fused":
        "test_kernels_gpu.py:test_decode_attention_fused_equals_the_two_kernels",
    "apply_penalties": "plain.py:adjusted_logit", "sample_topk": "plain.py:sample_token",
    "randinit": "test_kernels_gpu.py:test_randinit_is_the_numpy_draw_bit_for_bit",
    "stream_read": "test_kernels_gpu.py:test_stream_read_reads_every_byte_once",
    "mfma_loop": "test_kernels_gpu.py:test_mfma_loop_sums_its_products",
    "check_tables": "test_kernels_gpu.py:test_check_tables_reports_and_never_traps",
}


def test_the_flat_kernel_table_is_complete_and_every_kernel_has_a_reference():
    """Every function of `zinfer_amd.ops` that launches a kernel is in the table once, its
    module is one the build knows, it cites the reference's formula or says that it has
    none, and the plain function or test it is checked against exists."""
    import inspect
    import os
    import re
    from zinfer_amd.ops import build, table
    launchers = {name for name, fn in vars(ops).items()
                 if inspect.isfunction(fn) and fn.__module__ == "zinfer_amd.ops"
                 and not name.startswith("_") and "build.load(" in inspect.getsource(fn)}
    assert launchers == set(table.KERNELS) == set(TESTED_AGAINST), \
        launchers ^ set(table.KERNELS) ^ set(TESTED_AGAINST)
    here = os.path.dirname(os.path.abspath(__file__))
    for name, entry in table.KERNELS.items():
        assert entry.launch is getattr(ops, name)
        assert entry.launch.kernel_class in ops.KERNEL_CLASSES, name
        assert entry.module in build.MODULES
        assert entry.formula.startswith(("src/", "own: ")), name
        path, fn = TESTED_AGAINST[name].split(":")
        with open(os.path.join(here, path)) as f:
            assert re.search(rf"^def {fn}\(", f.read(), re.M), TESTED_AGAINST[name]
        source = inspect.getsource(entry.launch)
        assert f'build.load("{entry.module}")' in source, name
        assert "tests/" not in entry.formula


def test_measured_plans_are_plans_the_kernels_take():
    """Every entry of the measured table names a kernel configuration that exists: row groups
    of 1, 2 or 4 that divide the outputs, splits that leave each workgroup k-tiles, the
    SwiGLU products unsplit and with whole gate/up pairs."""
    plans = ops._measured_plans()
    for key, entry in plans["plans"].items():
        shape, _, kind = key.partition(":")
        N, K = (int(x) for x in shape.split("x"))
        for bucket, plan in entry.items():
            M = int(bucket)
            assert 16 < M <= 64
            if plan[0] == "mid":
                ks = plan[1]
                assert K % ((256 if M <= 32 else 128) * ks) == 0 and N % 16 == 0
            else:
                assert plan[0] == "skinny"
                rg, ks = plan[1:]
                assert rg in (1, 2, 4) and N % (16 * rg) == 0 and 1 <= ks <= 16 and K % 64 == 0
            if kind == "swiglu":
                assert plan[-1] == 1 and (plan[0] == "mid" or plan[1] >= 2) and N % 32 == 0
            for m in range(17, 65):
                got = ops._small_plan(m, N, K, True, swiglu=(kind == "swiglu"))
                assert got is not None and got[0] in ("mid", "skinny")
                if got[0] == "mid":
                    assert K % ((256 if m <= 32 else 128) * got[1]) == 0
    for key, plan in plans["decode_acc"].items():
        if key == "_":
            continue
        N, K = (int(x) for x in key.split("x"))
        assert plan[0] == "skinny" and plan[1] in (1, 2, 4) and N % (16 * plan[1]) == 0
        assert 2 <= plan[2] <= 16 and N <= 8192
        assert ops._decode_acc_plan(8, N, K) == tuple(plan) and ops._decode_acc_plan(17, N, K) is None
    # widths without an entry follow the rules
    assert ops._small_plan(40, 4160, 1088, True) is not None
    assert ops._skinny_plan(8, 5120, 5120, True) == (2, 1) and ops._skinny_plan(8, 4096, 4096, True) == (1, 1)
    assert ops._skinny_plan(8, 10240, 5120, True) == (4, 1) and ops._skinny_plan(8, 6144, 4096, True) == (2, 1)
    assert ops._skinny_plan(1, 151936, 4096, True) == (2, 1)


def test_widths_without_an_entry_get_plans_the_launchers_accept():
    """The measured table is an override, not the rule: for widths it does not list (other
    models' projections, odd multiples of 64) the rules give, for every number of tokens from
    17 to 64, a plan that passes the same check as a table entry."""
    table = ops._measured_plans()["plans"]
    widths = [(2048, 1024), (1024, 2048), (6144, 1024), (2048, 6144), (4096, 2560), (2560, 4096),
              (19456, 2560), (2560, 9728), (4160, 1088), (192, 4096), (8192, 8192), (64, 64)]
    for N, K in widths:
        for swiglu in (False, True):
            key = f"{N}x{K}" + (":swiglu" if swiglu else "")
            assert key not in table, key
            if swiglu and N % 64:
                continue
            for M in range(17, 65):
                plan = ops._small_plan(M, N, K, True, swiglu=swiglu)
                assert plan is not None and plan[0] in ("mid", "skinny"), (key, M)
                if plan[0] == "skinny" and not swiglu:
                    assert N % (16 * plan[1]) == 0 and plan[2] <= 16, (key, M, plan)
                ops.check_plans({"plans": {key: {str(ops.plan_bucket(M)): list(plan)}}})
            # the decode plans of such widths come from the rules as well
            for M in (1, 8, 16):
                rg, ks = ops._skinny_plan(M, N, K, True)
                assert rg in (1, 2, 4) and N % (16 * rg) == 0 and 1 <= ks <= 16
                assert ops._decode_acc_plan(M, N, K) is None


def test_a_model_folders_plans_are_checked_and_override_the_table(tmp_path, monkeypatch):
    import copy
    import json
    monkeypatch.setattr(ops, "_measured", copy.deepcopy(ops._measured_plans()))
    before = ops._small_plan(40, 2048, 1024, True)
    good = {"plans": {"2048x1024": {"48": ["skinny", 2, 4], "17": ["skinny", 2, 1]}},
            "decode_acc": {"2048x6144": ["skinny", 2, 3], "_": "a remark"}}
    p = tmp_path / ops.PLAN_FILE
    p.write_text(json.dumps(good))
    assert ops.load_plans(str(p)) == 2
    assert ops._small_plan(40, 2048, 1024, True) == ("skinny", 2, 4) != before
    assert ops._small_plan(64, 2048, 1024, True) == ("skinny", 2, 4)     # the nearest bucket above 32
    assert ops._small_plan(20, 2048, 1024, True) == ("skinny", 2, 1)
    assert ops._decode_acc_plan(8, 2048, 6144) == ("skinny", 2, 3)
    for bad in ({"plans": {"2048x1024": {"48": ["skinny", 3, 1]}}},
                {"plans": {"2048x1024": {"40": ["mid", 1]}}},
                {"plans": {"2048x1024": {"48": ["mid", 9]}}},
                {"plans": {"2048x1024:swiglu": {"48": ["mid", 2]}}},
                {"plans": {"2048 by 1024": {"48": ["mid", 1]}}},
                {"decode_acc": {"2048x6144": ["skinny", 2, 1]}}):
        p.write_text(json.dumps(bad))
        with pytest.raises(Exception, match="kernel plans"):
            ops.load_plans(str(p))


def test_the_last_round_of_large_tiles_is_split_only_where_it_is_short():
    """`_tile_tail_split`: whole rounds stay whole; a short last round behind one or two whole
    ones goes to workgroups that share its tiles along K, every part an even number of
    k-tiles and no more parts than one round holds; a long last round, a product of under one
    round or of many rounds stays as it is."""
    from zinfer_amd import ops
    for M in range(128, 8193, 128):
        for N, K in ((34816, 5120), (24576, 4096), (5120, 17408), (4096, 12288), (51200, 5120),
                     (6144, 4096), (24576, 2048), (9728 * 2, 2560)):
            tiles = ((M + 127) // 128) * ((N + 255) // 256)
            tail = ops._tile_tail_split(M, N, K)
            if tail is None:
                continue
            whole, split = tail
            assert whole % ops.TILE_PLACES == 0 and 0 < whole <= 2 * ops.TILE_PLACES
            assert 0 < tiles - whole < ops.TILE_PLACES and (tiles - whole) * split <= ops.TILE_PLACES
            assert split >= 2 and (K // 64) % (2 * split) == 0 and K // 64 // split >= 8
    assert ops._tile_tail_split(512, 34816, 5120) == (512, 4)     # 544 tiles
    assert ops._tile_tail_split(544, 34816, 5120) is None         # 680: a third of a round
    assert ops._tile_tail_split(512, 24576, 4096) is None         # 384: under one round
    assert ops._tile_tail_split(2048, 24576, 4096) is None        # three whole rounds
    assert ops._tile_tail_split(2048, 34816, 5120) is None        # a last round behind four


def test_residual_sums_of_several_hundred_tokens_over_a_long_k_take_wide_tiles_split():
    """`_wide_ksplit`: 641 to 1280 tokens over K >= 8192 run through 128 x 256 tiles split two
    to four times along K, every part an even number of k-tiles; other sizes keep their plan."""
    from zinfer_amd import ops
    for M in (641, 768, 1024, 1280):
        for N, K in ((4096, 12288), (5120, 17408), (5120, 25600), (5120, 8192), (2560, 9728)):
            ks = ops._wide_ksplit(M, N, K)
            if K % 128:
                assert ks is None
                continue
            assert ks in (2, 3, 4) and (K // 64) % (2 * ks) == 0, (M, N, K, ks)
    assert ops._wide_ksplit(1280, 4096, 12288) == 3 and ops._wide_ksplit(768, 5120, 17408) == 4
    for M, N, K in ((512, 5120, 17408), (640, 4096, 12288), (1281, 4096, 12288), (2048, 4096, 12288),
                    (1024, 4096, 4096), (1024, 5120, 5120)):
        assert ops._wide_ksplit(M, N, K) is None, (M, N, K)
