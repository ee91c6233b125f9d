"""The entry point that allocates nothing (csrc/no_alloc.h), called through ctypes: the decode attention with its
split-key scratch inside the library's device image, against the entry point that takes the scratch from the
caller. Two calls in a row, the second smaller, so that what the first left in the scratch would show; a call
beyond the scratch's size is refused with an error and launches nothing."""
import ctypes
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

P, I, F = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
SCRATCH_FLOATS = 4 << 20  # JLLM_NO_ALLOC_SCRATCH_FLOATS


@pytest.fixture(scope="module")
def lib():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from jllm_serve_amd.kernels import build
    path = build.ensure_built()
    lib = ctypes.CDLL(path)
    lib.jllm_last_error.restype = ctypes.c_char_p
    head = [P, I, P, I, P, P, P, I, P, P, I, I, I, I, I, I, F, I]
    lib.jllm_decode_attention_bf16.argtypes = head + [P, P, I, I, P]
    lib.jllm_decode_attention_bf16.restype = I
    lib.jllm_decode_attention_bf16_no_alloc.argtypes = head + [I, P]
    lib.jllm_decode_attention_bf16_no_alloc.restype = I
    return lib


def case(rows, ctx_max, H, Hkv, hd, page, seed):
    """Random q and a paged cache with shuffled pages; contexts from 1 key to ctx_max."""
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(seed)
    ctx = [1 + (i * 977 + seed * 131) % ctx_max for i in range(rows)]
    ctx[0], ctx[-1] = ctx_max, 1
    blocks = [-(-c // page) for c in ctx]
    n_pages = sum(blocks) + 2
    perm = torch.randperm(n_pages, generator=g).tolist()
    table = torch.zeros((rows, max(blocks)), dtype=torch.int32)
    at = 0
    for r, b in enumerate(blocks):
        table[r, :b] = torch.tensor(perm[at:at + b], dtype=torch.int32)
        at += b
    kc = torch.randn((n_pages, Hkv, page, hd), generator=g).bfloat16().to(dev)
    vc = torch.randn((n_pages, Hkv, page, hd), generator=g).bfloat16().to(dev)
    q = (torch.randn((rows, H * hd), generator=g) * 1.5).bfloat16().to(dev)
    positions = torch.tensor([c - 1 for c in ctx], dtype=torch.int32, device=dev)
    row_req = torch.arange(rows, dtype=torch.int32, device=dev)
    return dict(q=q, kc=kc, vc=vc, table=table.to(dev), positions=positions, row_req=row_req, rows=rows, H=H, Hkv=Hkv, hd=hd,
                page=page, max_pos=ctx_max - 1, ctx=ctx)


def head_args(c, out, split):
    return [c["q"].data_ptr(), c["q"].stride(0), out.data_ptr(), out.stride(0), c["kc"].data_ptr(), c["vc"].data_ptr(),
            c["table"].data_ptr(), c["table"].shape[1], c["row_req"].data_ptr(), c["positions"].data_ptr(), c["rows"],
            c["H"], c["Hkv"], c["hd"], c["page"], 0, 1.0 / math.sqrt(c["hd"]), c["max_pos"]]


def run_both(lib, c, split):
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    splits = c["max_pos"] // split + 1
    want = torch.full((c["rows"], c["H"] * c["hd"]), float("nan"), dtype=torch.bfloat16, device=c["q"].device)
    got = want.clone()
    n = c["rows"] * c["H"] * splits
    part_acc = torch.full((n * c["hd"],), float("nan"), dtype=torch.float32, device=c["q"].device)
    part_ml = torch.full((n * 2,), float("nan"), dtype=torch.float32, device=c["q"].device)
    rc = lib.jllm_decode_attention_bf16(*head_args(c, want, split), part_acc.data_ptr(), part_ml.data_ptr(), splits, split, stream)
    assert rc == 0, lib.jllm_last_error()
    torch.cuda.synchronize()
    # free memory as the driver sees it: a hipMalloc inside the library would show here (torch's own counters would not
    # see it), and torch itself allocates nothing between the two readings
    free_before, _ = torch.cuda.mem_get_info()
    held_before = torch.cuda.memory_reserved()
    rc = lib.jllm_decode_attention_bf16_no_alloc(*head_args(c, got, split), split, stream)
    assert rc == 0, lib.jllm_last_error()
    torch.cuda.synchronize()
    assert torch.cuda.memory_reserved() == held_before
    assert torch.cuda.mem_get_info()[0] == free_before, "device memory was allocated or freed during the call"
    return want, got


def check_rows_in_float64(c, got, rows, heads):
    """The given rows and heads of ``got`` against softmax(q k / sqrt(hd)) v in float64 over the row's own pages."""
    H, Hkv, hd, page = c["H"], c["Hkv"], c["hd"], c["page"]
    for r in rows:
        pos = c["ctx"][r] - 1
        pages = c["table"][r, :pos // page + 1].long()
        k = c["kc"][pages].permute(0, 2, 1, 3).reshape(-1, Hkv, hd)[:pos + 1].double().cpu()
        v = c["vc"][pages].permute(0, 2, 1, 3).reshape(-1, Hkv, hd)[:pos + 1].double().cpu()
        qr = c["q"][r].view(H, hd).double().cpu()
        for h in heads:
            p = torch.softmax((k[:, h // (H // Hkv)] @ qr[h]) / math.sqrt(hd), 0)
            ref = p @ v[:, h // (H // Hkv)]
            err = (got[r].view(H, hd)[h].double().cpu() - ref).abs().max()
            assert err <= 6e-3 * max(1.0, float(ref.abs().max())), f"row {r} ({pos + 1} keys) head {h}: {err}"


def test_no_alloc_decode_attention_matches_the_allocating_entry_point(lib):
    print("no-alloc decode attention: 24 rows to 1900 keys, then 5 rows to 300 keys", flush=True)
    big = case(rows=24, ctx_max=1900, H=32, Hkv=8, hd=128, page=16, seed=1)
    want, got = run_both(lib, big, split=256)
    assert not torch.isnan(want.float()).any() and not torch.isnan(got.float()).any()
    assert torch.equal(want.view(torch.int16), got.view(torch.int16))
    # both entry points run the same kernels, so equal bits alone would compare a path with itself: the longest row, a
    # middle one and the row with one key, in float64
    check_rows_in_float64(big, got, rows=(0, 11, 23), heads=(0, 13, 31))
    # the second call is smaller (other head shape too): the scratch still holds the first call's partial sums
    small = case(rows=5, ctx_max=300, H=6, Hkv=2, hd=64, page=8, seed=2)
    want2, got2 = run_both(lib, small, split=128)
    assert not torch.isnan(got2.float()).any()
    assert torch.equal(want2.view(torch.int16), got2.view(torch.int16))
    check_rows_in_float64(small, got2, rows=range(5), heads=range(6))  # every row, the one with a single key included
    # and the first once more, after the smaller one
    want3, got3 = run_both(lib, big, split=256)
    assert torch.equal(want3.view(torch.int16), got3.view(torch.int16)) and torch.equal(got3.view(torch.int16), got.view(torch.int16))


def test_no_alloc_decode_attention_refuses_what_its_scratch_cannot_hold(lib):
    print("no-alloc decode attention: a call beyond the scratch", flush=True)
    c = case(rows=4, ctx_max=64, H=32, Hkv=8, hd=128, page=16, seed=3)
    out = torch.zeros((c["rows"], c["H"] * c["hd"]), dtype=torch.bfloat16, device=c["q"].device)
    args = head_args(c, out, 128)
    args[10] = 4096  # rows: 4096 x 32 heads x 1 split x 130 floats > 4 Mi floats; refused before anything is read
    assert 4096 * 32 * 130 > SCRATCH_FLOATS
    rc = lib.jllm_decode_attention_bf16_no_alloc(*args, 128, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == -1
    msg = lib.jllm_last_error().decode()
    assert "scratch" in msg and "4096 rows" in msg
    torch.cuda.synchronize()
    assert float(out.float().abs().max()) == 0.0
