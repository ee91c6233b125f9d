"""The host-side rules that pick a kernel and its grid for the products: pure arithmetic on the shape. What is held
here is what must stay true under any tuning (limits the kernels rely on, no dependence on the number of rows), not
the tuned numbers themselves."""
from jllm_serve_amd.kernels import ops

SHAPES = {  # (N, K, gated): qkv, o, gate/up, down
    "8b": ((6144, 4096, False), (4096, 4096, False), (12288, 4096, True), (4096, 12288, False)),
    "14b": ((7168, 5120, False), (5120, 5120, False), (17408, 5120, True), (5120, 17408, False)),
    "32b": ((10240, 5120, False), (5120, 8192, False), (25600, 5120, True), (5120, 25600, False)),
}


def test_k_parts_fill_the_rounds():
    """Whatever the tuning: every part keeps the minimum length, the kernel's rounding of a part's blocks gives back
    the count, and the chosen count never leaves the busiest compute unit with a larger share of the product than
    no cut at all would."""
    cus = ops.compute_units()
    shapes = [s for v in SHAPES.values() for s in v] + [(96, 128, False), (256, 256, False), (384, 1024, True), (5120, 640, False)]
    for n, k, gated in shapes:
        parts = ops._stream_parts(n, k, gated)
        step = 1 if gated else 2
        nblk = k // 128
        per = -(-(-(-nblk // parts)) // step) * step  # whole steps, as the kernel rounds
        assert parts >= 1 and (parts == 1 or per >= ops.STREAM_MIN_BLOCKS), (n, k, gated, parts)
        assert -(-nblk // per) == parts, (n, k, gated, parts)
        tiles = -(-n // 128)
        share = lambda p: -(-(tiles * p) // cus) / (tiles * p)
        assert share(parts) <= share(1) + 1e-12, (n, k, gated, parts)
    assert ops._stream_parts(151936, 4096, False) == 1, "many column tiles: no cut"


def test_k_parts_do_not_depend_on_rows():
    """The rule has no argument for the number of rows: a row's sum is the same bits in any batch."""
    import inspect
    assert list(inspect.signature(ops._stream_parts.__wrapped__).parameters) == ["N", "K", "gated"]
    assert list(inspect.signature(ops._few_rows_prefer_stream.__wrapped__).parameters) == ["N", "K", "gated"]


def test_kernel_for_few_rows():
    assert not ops._few_rows_prefer_stream(96, 512, False), "small products: the second launch costs more than it saves"
    assert not ops._few_rows_prefer_stream(5120, 100, False), "a K the kernels do not take"
    assert not ops._few_rows_prefer_stream(4096, 4096, False), "N / 16 fills the compute units exactly: nothing to gain"


def test_rows_of_a_workgroup_of_the_first_weight_streaming_kernel():
    """Whatever the tuning: the extra rows divide N together with the 16, the gated product never has any (its second
    tile is the up weight), the rule knows nothing of the number of rows, and it only ever raises the share of the
    compute units' rounds that the workgroups fill."""
    import inspect
    assert list(inspect.signature(ops._skinny_second_rows.__wrapped__).parameters) == ["N", "gated"]
    for n in list(range(16, 12288 + 1, 16)) + [151936]:
        rows = ops._skinny_second_rows(n, False)
        assert rows in (0, 4, 8, 12, 16) and n % (16 + rows) == 0, (n, rows)
        assert rows == 0 or ops._round_fill(n // (16 + rows)) > ops._round_fill(n // 16), (n, rows)
        assert ops._skinny_second_rows(n, True) == 0
    assert ops._skinny_second_rows(4096, False) == 0, "N / 16 fills the compute units exactly"
    assert ops._skinny_second_rows(100, False) == 0, "an N the kernel does not take"


def test_k_splits_of_the_tiled_kernel():
    """A cut divides the K steps evenly and leaves every workgroup at least four of them; more rows never mean more
    cuts; the gated product is never cut."""
    assert ops._k_splits(128, 4096, 4096, True) == 1, "the gated epilogue needs both whole sums"
    for n, k in ((6144, 4096), (4096, 4096), (4096, 12288), (5120, 17408), (96, 128), (130, 192), (384, 4096), (192, 136 * 64)):
        last = None
        for rows in (70, 96, 128, 192, 256, 384, 512, 1000, 1024, 2048, 8192):
            s = ops._k_splits(rows, n, k, False)
            assert s >= 1 and (k // 64) % s == 0 and (s == 1 or k // 64 // s >= 4), (rows, n, k, s)
            assert last is None or s <= last, (rows, n, k, s, last)
            last = s
    assert ops._k_splits(8192, 4096, 4096, False) == 1, "enough tiles: no cut"


def test_plan_of_the_two_group_kernel():
    """Whatever the constants of its estimate: the plan names a tile the kernel has (256 rows) or none, a cut divides
    the K stages evenly and leaves every workgroup a range of the minimum length, the gated product is never cut,
    products of a few rows and shapes the kernel cannot take stay with the other kernel, and a product whose tiles
    fill the compute units many times over takes the large tile with K whole."""
    for shapes in SHAPES.values():
        for n, k, gated in shapes:
            for rows in (1, 64, 65, 128, 256, 257, 320, 448, 512, 1000, 1536, 1792, 2048, 3000, 4096, 8192):
                tile, cut = ops._pingpong_plan(rows, n, k, gated)
                assert tile in (0, 256) and cut in (1, 2, 4), (rows, n, k, gated, tile, cut)
                assert tile or cut == 1, "no tile, no cut"
                if cut > 1:
                    assert not gated and k % 64 == 0 and (k // 32) % cut == 0 and k // cut >= ops.PINGPONG_SPLIT_MIN_K
                if not gated and rows < ops.PINGPONG_MIN_ROWS:
                    assert tile == 0, (rows, n, k)
            assert ops._pingpong_plan(16384, n, k, gated) == (256, 1), (n, k, gated)
    assert ops._pingpong_plan(2048, 4096, 4000 + 16, False) == (0, 1), "K must be whole stages of 32"
    assert ops._pingpong_plan(2048, 4096, 64, False) == (0, 1), "too few stages"
    assert ops._pingpong_plan(2048, 8192, 1024 + 32, False)[1] == 1, "a cut needs K % 64 == 0 and long ranges"


def test_the_attention_plan_says_whether_the_runs_of_a_step_differ_much_in_keys():
    """One prompt from its start has runs of 128 to 2,048 keys (the portion kernel then cuts every run's keys over two
    groups of waves); a portion deep inside a long request, or several of them, has runs of about the same length."""
    from jllm_serve_amd.engine.step import Segment, StepBatch
    from jllm_serve_amd.parts.attention import GqaStepPlanner

    def facts(*portions):
        segments, row = [], 0
        for i, (n, pos0) in enumerate(portions):
            segments.append(Segment(f"r{i}", i, row, n, pos0, i))
            row += n
        batch = StepBatch(segments, row, len(segments), max(p + n for n, p in portions), 16, None, False)
        return GqaStepPlanner().plan(batch).facts

    assert facts((2048, 0))["key_groups"] == 2
    assert facts((1024, 0), (1024, 0))["key_groups"] == 2
    assert facts((2048, 6144))["key_groups"] == 1
    assert facts((2048, 2048))["key_groups"] == 1          # 2,176 to 4,096 keys: 1.3 times the average
    assert facts((512, 7680), (300, 0))["key_groups"] == 2  # a late portion beside a new prompt
    assert facts((1, 100), (1, 5000))["key_groups"] == 1   # single rows go to the split-key kernel anyway
    f = facts((2048, 0), (1, 77))
    assert f["key_groups"] == 2 and f["n_tiles_multi"] == 16 and f["single_rows"] == (2048, 1)
