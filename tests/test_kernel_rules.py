"""The host-side rules that pick a kernel and its grid for the weight-streaming products: pure arithmetic on the
shape, pinned here by the shapes they were measured on."""
from jllm_serve_amd.kernels import ops

SHAPES = {  # (N, K, gated): qkv, o, gate/up, down
    "8b": ((6144, 4096, False), (4096, 4096, False), (12288, 4096, True), (4096, 12288, False)),
    "14b": ((7168, 5120, False), (5120, 5120, False), (17408, 5120, True), (5120, 17408, False)),
    "32b": ((10240, 5120, False), (5120, 8192, False), (25600, 5120, True), (5120, 25600, False)),
}


def test_k_parts_fill_the_rounds():
    assert [ops._stream_parts(*s) for s in SHAPES["8b"]] == [4, 8, 5, 8]
    assert [ops._stream_parts(*s) for s in SHAPES["14b"]] == [4, 5, 5, 6]
    assert [ops._stream_parts(*s) for s in SHAPES["32b"]] == [3, 6, 5, 6]
    assert ops._stream_parts(151936, 4096, False) == 1, "many column tiles: no cut"
    for n, k, gated in ((96, 128, False), (256, 256, False), (384, 1024, True), (5120, 640, False)):
        parts = ops._stream_parts(n, k, gated)
        step = 1 if gated else 2
        per = -(-(-(-(k // 128) // parts)) // step) * step  # whole steps, as the kernel rounds
        assert parts >= 1 and (parts == 1 or per >= ops.STREAM_MIN_BLOCKS), (n, k, gated, parts)


def test_k_parts_do_not_depend_on_rows():
    """The rule has no argument for the number of rows: a row's sum is the same bits in any batch."""
    import inspect
    assert list(inspect.signature(ops._stream_parts.__wrapped__).parameters) == ["N", "K", "gated"]
    assert list(inspect.signature(ops._few_rows_prefer_stream.__wrapped__).parameters) == ["N", "K", "gated"]


def test_kernel_for_few_rows():
    assert not any(ops._few_rows_prefer_stream(*s) for s in SHAPES["8b"])
    assert [ops._few_rows_prefer_stream(*s) for s in SHAPES["14b"]] == [False, False, False, True]
    assert [ops._few_rows_prefer_stream(*s) for s in SHAPES["32b"]] == [False, True, False, True]
    assert not ops._few_rows_prefer_stream(96, 512, False), "small products: the second launch costs more than it saves"
    assert not ops._few_rows_prefer_stream(5120, 100, False), "a K the kernels do not take"


def test_k_splits_of_the_tiled_kernel():
    """First a workgroup for every compute unit, then a second one only while the K ranges stay long."""
    qkv, o, down = (6144, 4096), (4096, 4096), (4096, 12288)
    want = {96: (8, 8, 8), 128: (8, 8, 8), 192: (4, 4, 8), 256: (4, 4, 8), 384: (2, 4, 4), 512: (2, 4, 4),
            1024: (1, 2, 2), 2048: (1, 1, 1), 8192: (1, 1, 1)}
    for rows, splits in want.items():
        assert tuple(ops._k_splits(rows, n, k, False) for n, k in (qkv, o, down)) == splits, rows
    assert ops._k_splits(128, 4096, 4096, True) == 1, "the gated epilogue needs both whole sums"
    for rows, n, k in ((70, 96, 128), (100, 130, 192), (300, 384, 4096), (1000, 192, 136 * 64)):
        s = ops._k_splits(rows, n, k, False)
        assert s >= 1 and (k // 64) % s == 0 and (s == 1 or k // 64 // s >= 4), (rows, n, k, s)


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
