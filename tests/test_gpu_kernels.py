"""Each kernel alone against a plain fp32/fp64 reference of the same operation, at sizes other than the engine's
tiny configurations: sizes that are no power of two, head sizes in steps of 16, any number of heads and groups."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda"


@pytest.fixture(scope="module")
def ops():
    from jllm_serve_amd.kernels import ops
    ops.library()
    return ops


def bf16_close(got, want, ulps=1.0):
    """got (bf16 or f32 tensor) against a float64 reference: within `ulps` bf16 roundings of the reference."""
    want = want.double()
    err = (got.double() - want).abs()
    tol = ulps * (2.0 ** -8) * want.abs() + 1e-6 * want.abs().max()
    return bool((err <= tol).all()), float((err / (want.abs() + 1e-3 * want.abs().max())).max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed(ops, dtype):
    table = torch.randn(301, 80, device=DEV).to(dtype)
    ids = torch.tensor([0, 300, 7, 7, 150], dtype=torch.int32, device=DEV)
    out = ops.embed(table, ids, 1.0)
    assert out.dtype == torch.float32 and torch.equal(out, table[ids.long()].float())
    assert torch.equal(ops.embed(table, ids, 2.0), table[ids.long()].float() * 2.0)


@pytest.mark.parametrize("d", [16, 80, 96, 4096, 5000])
@pytest.mark.parametrize("gdt,odt", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16), (torch.float32, torch.bfloat16)])
def test_rmsnorm(ops, d, gdt, odt):
    x = torch.randn(7, d, device=DEV) * 3
    x[2] = 0  # an all-zero row gives zeros, not NaN
    g = (torch.rand(d, device=DEV) + 0.5).to(gdt)
    eps = 1e-5
    ref = (x.double() * torch.rsqrt((x.double() ** 2).mean(-1, keepdim=True) + eps)) * g.double()
    out = ops.rmsnorm(x, g, eps, odt)
    if odt == torch.float32:
        assert torch.allclose(out.double(), ref, rtol=2e-6, atol=1e-6)
    else:
        assert bf16_close(out, ref)[0]
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
    assert torch.equal(ops.rmsnorm(x, g, eps, odt, rows), out[rows.long()])


GEMM_SHAPES = [(1, 16, 128), (5, 48, 384), (16, 4096, 128), (17, 80, 256), (33, 16, 1024), (64, 304, 640), (50, 144, 2176),
               (20, 4112, 512),
               (8, 6144, 256), (3, 6144, 128), (16, 6144, 1152),  # 24 weight rows per workgroup (N / 24 = 256 of them)
               (8, 5120, 256), (1, 5120, 1152), (13, 7168, 384), (16, 10240, 128),  # 20 weight rows per workgroup for N = 5120
               (5, 32768, 128), (16, 32800, 256),  # thousands of 16-row tiles
               (100, 256, 64), (70, 200, 192), (90, 136, 320),  # one, three and five K steps of the tiled kernel's two-ahead form
               (3, 50, 70), (65, 96, 128), (200, 130, 96), (128, 256, 512), (300, 384, 4096), (1000, 192, 136)]


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gemm_epilogues(ops, M, N, K, dtype):
    torch.manual_seed(M * 7 + N)
    a = torch.randn(M, K, device=DEV).to(dtype)
    w = (torch.randn(N, K, device=DEV) / math.sqrt(K)).to(dtype)
    w2 = (torch.randn(N, K, device=DEV) / math.sqrt(K)).to(dtype)
    bias = torch.randn(N, device=DEV)
    ref = a.double() @ w.double().T
    exact = dtype == torch.float32
    # store, fp32 out (the output head)
    out = ops.gemm(a, w, out_dtype=torch.float32, exact=exact)
    assert torch.allclose(out.double(), ref, rtol=1e-5, atol=2e-5 * ref.abs().max())
    # store in the activations' type with a bias, from a strided input view
    wide = torch.cat([a, a], dim=1)
    out = ops.gemm(wide[:, K:], w, bias=bias, exact=exact)
    assert out.dtype == dtype
    if exact:
        assert torch.allclose(out.double(), ref + bias.double(), rtol=1e-5, atol=2e-5 * ref.abs().max())
    else:
        assert bf16_close(out, ref + bias.double())[0]
    # add into the fp32 residual
    res = torch.randn(M, N, device=DEV)
    want = res.double() + ref
    ops.gemm(a, w, out=res, epilogue=ops.EPI_ADD, exact=exact)
    assert torch.allclose(res.double(), want, rtol=1e-5, atol=2e-5 * want.abs().max())
    # gated: silu(a w^T) * (a w2^T)
    g, u = ref, a.double() @ w2.double().T
    want = (g / (1 + torch.exp(-g))) * u
    out = ops.gemm(a, w, w2=w2, epilogue=ops.EPI_GATED, exact=exact)
    if exact:
        assert torch.allclose(out.double(), want, rtol=1e-5, atol=2e-5 * want.abs().max())
    else:
        assert bf16_close(out, want, ulps=1.01)[0]


def test_gemm_large_tile(ops):
    """Products with at least 512 tiles of 256 x 256 go through the 8-wave tile: all three epilogues at sizes that
    leave partial tiles in both directions, and the same bits as the small tile gives for the same rows."""
    torch.manual_seed(5)
    M, N, K = 530, 43800, 192
    a = torch.randn(M, K, device=DEV).bfloat16()
    w = (torch.randn(N, K, device=DEV) / math.sqrt(K)).bfloat16()
    bias = torch.randn(N, device=DEV)
    ref = a.double() @ w.double().T
    out = ops.gemm(a, w, out_dtype=torch.float32)
    assert torch.allclose(out.double(), ref, rtol=1e-5, atol=2e-5 * ref.abs().max())
    small = ops.gemm(a[:100].contiguous(), w, out_dtype=torch.float32)   # few tiles: the 4-wave kernel
    assert torch.equal(small, out[:100])
    assert bf16_close(ops.gemm(a, w, bias=bias), ref + bias.double())[0]
    res = torch.randn(M, N, device=DEV)
    want = res.double() + ref
    ops.gemm(a, w, out=res, epilogue=ops.EPI_ADD)
    assert torch.allclose(res.double(), want, rtol=1e-5, atol=2e-5 * want.abs().max())
    del out, res, want, ref, small
    N = 21900
    w = (torch.randn(N, K, device=DEV) / math.sqrt(K)).bfloat16()
    w2 = (torch.randn(N, K, device=DEV) / math.sqrt(K)).bfloat16()
    g, u = a.double() @ w.double().T, a.double() @ w2.double().T
    want = (g / (1 + torch.exp(-g))) * u
    out = ops.gemm(a, w, w2=w2, epilogue=ops.EPI_GATED)
    assert bf16_close(out, want, ulps=1.01)[0]
    assert torch.equal(ops.gemm(a[:100].contiguous(), w, w2=w2, epilogue=ops.EPI_GATED), out[:100])
    # 200 large tiles: one round that fills most of the compute units also takes the large tile
    M, N = 1990, 6300
    a = torch.randn(M, K, device=DEV).bfloat16()
    w = (torch.randn(N, K, device=DEV) / math.sqrt(K)).bfloat16()
    ref = a.double() @ w.double().T
    out = ops.gemm(a, w, out_dtype=torch.float32)
    assert torch.allclose(out.double(), ref, rtol=1e-5, atol=2e-5 * ref.abs().max())
    assert torch.equal(ops.gemm(a[:100].contiguous(), w, out_dtype=torch.float32), out[:100])


@pytest.mark.parametrize("M,N,K,plan", [(1500, 8200, 160, (256, 1)), (2048, 6144, 1024, (256, 1)), (300, 25000, 128, (256, 1)),
                                        (520, 16400, 4096, (256, 1)), (2000, 4096, 8192, (256, 2)), (1024, 6140, 8256, (256, 2)),
                                        (1000, 4100, 8192, (256, 2)), (640, 4100, 8192, (256, 4)), (1024, 6144, 4096, (256, 2))])
def test_gemm_two_group_kernel(ops, M, N, K, plan):
    """The tiled kernel whose waves take turns at the matrix cores (direct-to-LDS loads, a ring of stages): every
    epilogue, with a bias, partial tiles in both directions, K from four stages to many, inputs and
    outputs whose rows are not contiguous, K cut in two or four with partial sums (also an odd number of stages per half);
    against float64."""
    assert ops._pingpong_plan(M, N, K, False) == plan
    torch.manual_seed(M + N + K)
    a = torch.randn(M, K, device=DEV).bfloat16()
    w = (torch.randn(N, K, device=DEV) / math.sqrt(K)).bfloat16()
    bias = torch.randn(N, device=DEV)
    ref = a.double() @ w.double().T
    ops.reset_stats()
    out = ops.gemm(a, w, out_dtype=torch.float32)
    assert ops.stats()["ran"].get("jllm_gemm_pingpong_bf16") == 1, ops.stats()
    assert torch.allclose(out.double(), ref, rtol=1e-5, atol=2e-5 * ref.abs().max())
    wide = torch.cat([a, a], dim=1)
    assert bf16_close(ops.gemm(wide[:, K:], w, bias=bias), ref + bias.double())[0]
    res = torch.randn(M, N, device=DEV)
    want = res.double() + ref + bias.double()
    ops.gemm(a, w, bias=bias, out=res, epilogue=ops.EPI_ADD)
    assert torch.allclose(res.double(), want, rtol=1e-5, atol=2e-5 * want.abs().max())
    if ops._pingpong_plan(M, N // 2, K, True)[0]:
        w1, w2 = w[:N // 2], w[N // 2:2 * (N // 2)]
        g, u = ref[:, :N // 2], ref[:, N // 2:2 * (N // 2)]
        want = (g / (1 + torch.exp(-g))) * u
        out = ops.gemm(a, w1.contiguous(), w2=w2.contiguous(), epilogue=ops.EPI_GATED)
        assert bf16_close(out, want, ulps=1.01)[0]
    assert ops.stats()["ran"].get("jllm_gemm_pingpong_bf16") >= 3 and not ops.stats()["general"], ops.stats()


@pytest.mark.parametrize("M,N,K,N2", [(1, 128, 256, 48), (5, 4096, 384, 4112), (8, 640, 4096, 304), (16, 304, 128, 16), (13, 5120, 1024, 640),
                                      (40, 1024, 1024, 512), (64, 2048, 2048, 768), (17, 1024, 4096, 256),
                                      # few rows, N / 16 just above the compute units: 20 weight rows per workgroup
                                      (8, 5120, 3072, 5120), (16, 5120, 4096, 640), (3, 5120, 3072, 5120), (11, 5120, 128, 7168),
                                      # few rows, few columns and a long K: the K-cutting kernel takes them
                                      (8, 1024, 8192, 512), (3, 1280, 8192, 1024),
                                      # the consuming product with 24 weight rows per workgroup, and with thousands of tiles
                                      (8, 1024, 512, 6144), (13, 256, 256, 32768)])
@pytest.mark.parametrize("gdt", [torch.bfloat16, torch.float32])
def test_norm_between_two_products(ops, M, N, K, N2, gdt):
    """residual += a w^T (+ bias); h = RMSNorm(residual) w2^T without a norm launch: the first product leaves
    bf16(residual * gain) and partial sums of squares, the second scales its sums at the end (both weight-streaming
    kernels: up to 16 rows, and 17 to 64 rows with K cut in parts). Against float64, and
    against the same roundings in float64 (only fp32 summation is left). One residual entry is huge, so a norm over
    the wrong columns or rows shows."""
    torch.manual_seed(M * N + K)
    if N == 5120 and M <= 16:
        assert ops._skinny_second_rows(N, False) == 4, "this case is meant for workgroups with 20 weight rows"
    if K == 8192 and M <= 16:
        assert ops._few_rows_prefer_stream(N, K, False), "this case is meant for the K-cutting kernel"
    a = torch.randn(M, K, device=DEV).bfloat16()
    w = (torch.randn(N, K, device=DEV) / math.sqrt(K)).bfloat16()
    bias = torch.randn(N, device=DEV)
    res = torch.randn(M, N, device=DEV) * 2
    res[M // 2, N - 3] = 200.0
    gain = (torch.rand(N, device=DEV) + 0.5).to(gdt)
    w2 = (torch.randn(N2, N, device=DEV) / math.sqrt(N)).bfloat16()
    w3 = (torch.randn(N2, N, device=DEV) / math.sqrt(N)).bfloat16()
    eps = 1e-3
    want_res = res.double() + a.double() @ w.double().T + bias.double()
    promise = ops.gemm_add_then_norm(a, w, res, gain, eps, torch.bfloat16, bias=bias)
    assert promise.scaled is not None and promise.partials is not None, "the few-row product did not prepare the norm"
    assert torch.allclose(res.double(), want_res, rtol=1e-5, atol=2e-5 * want_res.abs().max())
    scale = torch.rsqrt((res.double() ** 2).mean(-1, keepdim=True) + eps)
    assert torch.allclose(promise.partials.double().sum(-1, keepdim=True), (res.double() ** 2).sum(-1, keepdim=True), rtol=1e-5)
    assert torch.equal(promise.scaled, (res * gain.float()).bfloat16())
    xn = res.double() * scale * gain.double()
    rounded = promise.scaled.double()
    fused = N % 128 == 0  # what the consuming kernels take (and partial sums in fours); else the norm is a launch of its own
    ref = xn @ w2.double().T
    tol = 5 * 2.0 ** -9 * torch.sqrt((xn ** 2) @ (w2.double() ** 2).T) + 1e-6
    if fused:
        out = ops.gemm(promise, w2, w2=w3, epilogue=ops.EPI_GATED, out_dtype=torch.float32)
        g_, u_ = (rounded @ w2.double().T) * scale, (rounded @ w3.double().T) * scale
        same = torch.nn.functional.silu(g_) * u_
        assert torch.allclose(out.double(), same, rtol=2e-4, atol=2e-5 * same.abs().max())
    out = ops.gemm(promise, w2, out_dtype=torch.float32)
    if fused:
        same = (rounded @ w2.double().T) * scale
        fp32_sum = 4e-6 * (rounded.abs() @ w2.double().abs().T) * scale + 1e-6
        assert bool(((out.double() - same).abs() <= fp32_sum).all())
    assert bool(((out.double() - ref).abs() <= tol).all())
    assert (promise._rows is None) == fused, "the norm ran as a launch of its own exactly when it had to"
    # the long way gives the same within bf16 rounding; many rows and 32-bit runs take it by themselves
    long_way = ops.gemm(ops.rmsnorm(res, gain, eps, torch.bfloat16), w2, out_dtype=torch.float32)
    assert bool(((out.double() - long_way.double()).abs() <= 2 * tol).all())
    big_a, big_res = torch.randn(100, K, device=DEV).bfloat16(), torch.randn(100, N, device=DEV)
    p2 = ops.gemm_add_then_norm(big_a, w, big_res, gain, eps, torch.bfloat16)
    assert p2.scaled is None
    assert torch.equal(ops.gemm(p2, w2), ops.gemm(ops.rmsnorm(big_res, gain, eps, torch.bfloat16), w2))


def test_gemm_rows_do_not_depend_on_the_batch(ops):
    """The result of a row is the same bits whether it is alone or among others, within one kernel family (the
    bfloat16 path has one kernel for up to 16 rows, one for up to 64 and one for more; between them results differ
    by rounding)."""
    torch.manual_seed(0)
    for dtype, K, full_rows, parts in ((torch.float32, 200, 64, (1, 2, 7, 16, 33)), (torch.float32, 203, 40, (1, 3, 16, 17)),
                                       (torch.bfloat16, 512, 16, (1, 7, 11)),
                                       (torch.bfloat16, 1024, 64, (17, 33, 48)), (torch.bfloat16, 512, 128, (65, 100)),
                                       (torch.bfloat16, 8192, 64, (1, 8, 16, 17, 40)),  # with N = 1024: one kernel up to 64 rows
                                       (torch.bfloat16, 3072, 16, (1, 8, 11)),  # with N = 5120: 20 weight rows per workgroup
                                       (torch.bfloat16, 384, 16, (1, 5, 9))):  # with N = 6144: 24 weight rows per workgroup
        N = {8192: 1024, 3072: 5120, 384: 6144}.get(K, 96)
        if K == 8192:
            assert ops._few_rows_prefer_stream(N, K, False), "this case is meant for the K-cutting kernel at few rows"
        a = torch.randn(full_rows, K, device=DEV).to(dtype)
        w = torch.randn(N, K, device=DEV).to(dtype)
        full = ops.gemm(a, w, out_dtype=torch.float32, exact=dtype == torch.float32)
        for rows in parts:
            part = ops.gemm(a[:rows].contiguous(), w, out_dtype=torch.float32, exact=dtype == torch.float32)
            assert torch.equal(part, full[:rows])
    # the 32-bit path has a kernel of its own for up to 16 rows: every epilogue and operand type gives the same bits
    a = torch.randn(40, 136, device=DEV)
    w, w2, bias = torch.randn(100, 136, device=DEV), torch.randn(100, 136, device=DEV), torch.randn(100, device=DEV)
    for wt in (torch.float32, torch.bfloat16):
        full = ops.gemm(a, w.to(wt), w2=w2.to(wt), epilogue=ops.EPI_GATED, out_dtype=torch.float32, exact=True)
        few = ops.gemm(a[:9].contiguous(), w.to(wt), w2=w2.to(wt), epilogue=ops.EPI_GATED, out_dtype=torch.float32, exact=True)
        assert torch.equal(few, full[:9])
        res_full, res_few = torch.ones(40, 100, device=DEV), torch.ones(9, 100, device=DEV)
        ops.gemm(a, w.to(wt), bias=bias, out=res_full, epilogue=ops.EPI_ADD, exact=True)
        ops.gemm(a[:9].contiguous(), w.to(wt), bias=bias, out=res_few, epilogue=ops.EPI_ADD, exact=True)
        assert torch.equal(res_few, res_full[:9])
    # and between the bfloat16 kernels: rounding only
    a = torch.randn(100, 1024, device=DEV).bfloat16()
    w = (torch.randn(256, 1024, device=DEV) / 32).bfloat16()
    few = ops.gemm(a[:16].contiguous(), w, out_dtype=torch.float32)
    some = ops.gemm(a[:40].contiguous(), w, out_dtype=torch.float32)[:16]
    many = ops.gemm(a, w, out_dtype=torch.float32)[:16]
    assert torch.allclose(few, many, rtol=1e-4, atol=1e-4) and torch.allclose(few, some, rtol=1e-4, atol=1e-4)


def test_gemm_refuses_bad_arguments(ops):
    a = torch.randn(4, 32, device=DEV)
    w = torch.randn(8, 31, device=DEV)
    with pytest.raises(ops.KernelError):
        ops.gemm(a, w)
    with pytest.raises(ops.KernelError):
        ops.gemm(a.cpu(), torch.randn(8, 32))
    with pytest.raises(ops.KernelError):
        ops.gemm(a, torch.randn(8, 32, device=DEV), epilogue=ops.EPI_ADD)
    with pytest.raises(ops.KernelError):
        ops.gemm(a.double(), torch.randn(8, 32, device=DEV).double())


# ------------------------------------------------------------------------------- q/k norm, rotation, cache store


ROPE_CASES = [  # H, Hkv, hd, rotary width (0: none), page, gains (None: no norm)
    (4, 2, 16, 16, 8, torch.bfloat16), (6, 2, 32, 32, 16, torch.float32), (5, 5, 48, 48, 32, torch.bfloat16),
    (3, 3, 24, 12, 4, torch.bfloat16), (8, 1, 64, 32, 4, None), (3, 3, 80, 64, 16, torch.float32),
    (32, 8, 128, 128, 16, torch.bfloat16), (2, 1, 256, 256, 16, torch.bfloat16), (7, 7, 96, 0, 2, torch.bfloat16),
    (2, 2, 20, 10, 8, torch.float32),
]


@pytest.mark.parametrize("H,Hkv,hd,rot,page,gdt", ROPE_CASES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_qk_norm_rope_store(ops, H, Hkv, hd, rot, page, gdt, dtype):
    """Per-head RMSNorm of q and k, rotation of pairs (i, i + rot/2) by the angles of each row's position, k and v
    into their pages, against float64. The angles differ for every position and pair, q and k have different gains,
    some rows store nothing (slot -1): a wrong pairing, sign, gain or row shows."""
    gen = torch.Generator().manual_seed(H * 131 + hd)
    T, n_pages, max_pos, eps = 37, 20, 50, 1e-4
    qkv = (torch.randn(T, (H + 2 * Hkv) * hd, generator=gen) * 1.5).to(dtype)
    positions = torch.randint(0, max_pos, (T,), generator=gen, dtype=torch.int32)
    slots = torch.randperm(n_pages * page, generator=gen)[:T].to(torch.int32)
    slots[5] = -1
    slots[T - 1] = -1
    gq = gk = None
    if gdt is not None:
        gq = (torch.rand(hd, generator=gen) + 0.5).to(gdt if dtype == torch.bfloat16 else torch.float32)
        gk = (torch.rand(hd, generator=gen) + 0.5).to(gdt if dtype == torch.bfloat16 else torch.float32)
    cos = sin = None
    if rot:
        ang = torch.rand(max_pos, rot // 2, generator=gen, dtype=torch.float64) * 6.28
        cos, sin = torch.cos(ang).float(), torch.sin(ang).float()

    def prepared(x, gain):  # [T, heads, hd] float64
        x = x.double()
        if gain is not None:
            x = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * gain.double()
        if rot:
            c, s_ = cos[positions.long()].double()[:, None, :], sin[positions.long()].double()[:, None, :]
            a, b = x[..., :rot // 2].clone(), x[..., rot // 2:rot].clone()
            x[..., :rot // 2] = a * c - b * s_
            x[..., rot // 2:rot] = b * c + a * s_
        return x

    want_q = prepared(qkv[:, :H * hd].view(T, H, hd), gq)
    want_k = prepared(qkv[:, H * hd:(H + Hkv) * hd].view(T, Hkv, hd), gk)
    want_v = qkv[:, (H + Hkv) * hd:].view(T, Hkv, hd)
    dev = lambda x: None if x is None else x.to(DEV)
    for write_kv in (True, False):
        work = qkv.clone().to(DEV)
        kc = torch.full((n_pages, Hkv, page, hd), 7.0).to(dtype).to(DEV)
        vc = torch.full((n_pages, Hkv, page, hd), 7.0).to(dtype).to(DEV)
        ops.qk_norm_rope_store(work, dev(positions), dev(slots), dev(cos), dev(sin), dev(gq), dev(gk), eps, H, Hkv, hd, rot,
                               page, kc, vc, write_kv=write_kv)
        got_q = work[:, :H * hd].view(T, H, hd).cpu()
        if dtype == torch.float32:
            assert torch.allclose(got_q.double(), want_q, rtol=1e-5, atol=1e-5)
        else:
            assert bf16_close(got_q, want_q)[0]
        assert torch.equal(work[:, H * hd:].cpu(), qkv[:, H * hd:]), "k and v of the projection output stay as they are"
        stored = torch.zeros(n_pages, page, dtype=torch.bool)
        for t in range(T):
            sl = int(slots[t])
            if sl < 0 or not write_kv:
                continue
            pg, off = sl // page, sl % page
            stored[pg, off] = True
            gk_, gv_ = kc[pg, :, off].cpu(), vc[pg, :, off].cpu()
            if dtype == torch.float32:
                assert torch.allclose(gk_.double(), want_k[t], rtol=1e-5, atol=1e-5)
            else:
                assert bf16_close(gk_, want_k[t])[0]
            assert torch.equal(gv_, want_v[t])
        untouched = ~stored[:, None, :, None].expand(n_pages, Hkv, page, hd)
        assert bool((kc.cpu()[untouched] == 7.0).all()) and bool((vc.cpu()[untouched] == 7.0).all())


@pytest.mark.parametrize("H,Hkv,hd,rot", [(4, 2, 16, 16), (6, 2, 32, 32), (5, 5, 48, 24), (8, 2, 128, 128), (3, 1, 80, 64)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rotation_comes_after_the_head_norm(ops, H, Hkv, hd, rot, dtype):
    """Scores depend only on the distance between query and key when the rotation is what happens last to q and k:
    with gains that differ within every rotated pair, the products q_i . k_j of the kernel's outputs are the same at
    positions p.. and p + 10.. . A kernel that rotated first and normalised afterwards would fail this by a wide
    margin (shown below on the same numbers in float64), whatever reference it was compared with."""
    gen = torch.Generator().manual_seed(hd + rot)
    T, page, eps, theta = 12, 4, 1e-6, 100.0
    G = H // Hkv
    qkv = (torch.randn(T, (H + 2 * Hkv) * hd, generator=gen) * 1.5).to(dtype)
    gdt = torch.float32 if dtype == torch.float32 else torch.bfloat16
    gq = (torch.rand(hd, generator=gen) * 2.5 + 0.25).to(gdt)
    gk = (torch.rand(hd, generator=gen) * 2.5 + 0.25).to(gdt)
    inv = 1.0 / theta ** (torch.arange(rot // 2, dtype=torch.float64) * 2 / rot)
    ang = torch.arange(64, dtype=torch.float64)[:, None] * inv[None, :]
    cos, sin = torch.cos(ang).float(), torch.sin(ang).float()
    slots = torch.arange(T, dtype=torch.int32)

    def scores(shift):
        work = qkv.clone().to(DEV)
        kc = torch.zeros(T // page, Hkv, page, hd, dtype=dtype, device=DEV)
        vc = torch.zeros_like(kc)
        pos = (torch.arange(T, dtype=torch.int32) + shift).to(DEV)
        ops.qk_norm_rope_store(work, pos, slots.to(DEV), cos.to(DEV), sin.to(DEV), gq.to(DEV), gk.to(DEV), eps, H, Hkv, hd,
                               rot, page, kc, vc)
        q = work[:, :H * hd].view(T, H, hd).cpu().double()
        k = kc.permute(0, 2, 1, 3).reshape(T, Hkv, hd).cpu().double()  # [page, kv head, row, :] -> [position, kv head, :]
        return torch.einsum("ihd,jhd->ijh", q, k.repeat_interleave(G, 1))

    a, b = scores(3), scores(13)
    span = float(a.abs().max())
    assert (a - b).abs().max() <= (2e-5 if dtype == torch.float32 else 3e-2) * span

    def wrong(shift):  # rotate, then normalise
        def prep(x, g):
            x = x.double().clone()
            c, s_ = cos[shift:shift + T].double()[:, None, :], sin[shift:shift + T].double()[:, None, :]
            u, v = x[..., :rot // 2].clone(), x[..., rot // 2:rot].clone()
            x[..., :rot // 2], x[..., rot // 2:rot] = u * c - v * s_, v * c + u * s_
            return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * g.double()
        q = prep(qkv[:, :H * hd].view(T, H, hd), gq)
        k = prep(qkv[:, H * hd:(H + Hkv) * hd].view(T, Hkv, hd), gk)
        return torch.einsum("ihd,jhd->ijh", q, k.repeat_interleave(G, 1))
    assert (wrong(3) - wrong(13)).abs().max() > 0.1 * span, "the case must tell the two orders apart"


def test_fused_decode_rotates_after_the_head_norm(ops):
    """The same invariant for the decode kernel that prepares q and k itself: a row at position p over keys
    p - 15 .. p (a window hides what lies before) gives the same output when the request sits ten positions
    further on, with the keys stored by the kernel for whole portions at their shifted positions."""
    H, Hkv, hd, page, eps, theta, W = 8, 2, 128, 16, 1e-6, 50.0, 16
    gen = torch.Generator().manual_seed(5)
    gq = (torch.rand(hd, generator=gen) * 2.5 + 0.25).bfloat16().to(DEV)
    gk = (torch.rand(hd, generator=gen) * 2.5 + 0.25).bfloat16().to(DEV)
    inv = 1.0 / theta ** (torch.arange(hd // 2, dtype=torch.float64) * 2 / hd)
    ang = torch.arange(64, dtype=torch.float64)[:, None] * inv[None, :]
    cos, sin = torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV)
    rows = (torch.randn(W, (H + 2 * Hkv) * hd, generator=gen) * 1.5).bfloat16()
    scale = 1.0 / math.sqrt(hd)
    outs = []
    for shift in (0, 10):
        n_pages = 3
        kc = torch.full((n_pages, Hkv, page, hd), float("nan")).bfloat16().to(DEV)  # what the window hides is NaN
        vc = kc.clone()
        table = torch.arange(n_pages, dtype=torch.int32, device=DEV).view(1, n_pages)
        pos = (torch.arange(W, dtype=torch.int32) + shift).to(DEV)
        work = rows.clone().to(DEV)
        ops.qk_norm_rope_store(work[:W - 1], pos[:W - 1], pos[:W - 1], cos, sin, gq, gk, eps, H, Hkv, hd, hd, page, kc, vc)
        meta = {"max_context": W + shift, "decode_only": True, "requests": 1}
        out = ops.decode_attention_fused(rows[W - 1:].to(DEV), kc, vc, table, torch.zeros(1, dtype=torch.int32, device=DEV),
                                         pos[W - 1:], pos[W - 1:], cos, sin, gq, gk, eps, H, Hkv, hd, hd, W, scale, meta)
        assert out is not None and not torch.isnan(out.float()).any()
        outs.append(out.float().cpu())
    assert (outs[0] - outs[1]).abs().max() <= 2e-2 * max(1.0, float(outs[0].abs().max()))
    assert outs[0].abs().max() > 0.1


# ------------------------------------------------------------------------------------------------ attention


def make_cache(R, ctx_lens, Hkv, hd, page, dtype, extra_pages=3, seed=0):
    """Random k/v for R requests in shuffled pages of a pool that also holds garbage pages."""
    g = torch.Generator().manual_seed(seed)
    blocks = [-(-c // page) for c in ctx_lens]
    n_pages = sum(blocks) + extra_pages
    perm = torch.randperm(n_pages, generator=g).tolist()
    kc = torch.full((n_pages, Hkv, page, hd), float("nan")).to(dtype)  # unused slots hold NaN: nothing may read them
    vc = torch.full((n_pages, Hkv, page, hd), float("nan")).to(dtype)
    width = max(blocks)
    table = torch.full((R, width), -1, dtype=torch.int32)
    ks, vs = [], []
    it = iter(perm)
    for r, c in enumerate(ctx_lens):
        k = torch.randn(c, Hkv, hd, generator=g).to(dtype)
        v = torch.randn(c, Hkv, hd, generator=g).to(dtype)
        ks.append(k); vs.append(v)
        for b in range(blocks[r]):
            pg = next(it)
            table[r, b] = pg
            n = min(page, c - b * page)
            kc[pg, :, :n] = k[b * page:b * page + n].transpose(0, 1)
            vc[pg, :, :n] = v[b * page:b * page + n].transpose(0, 1)
    return kc.to(DEV), vc.to(DEV), table.to(DEV), ks, vs


def attention_reference(qrow, k, v, pos, H, window, scale):
    """One row in float64: keys [max(0, pos+1-window), pos]."""
    Hkv = k.shape[1]
    first = max(0, pos + 1 - window) if window > 0 else 0
    out = []
    for h in range(H):
        kk, vv = k[first:pos + 1, h // (H // Hkv)].double(), v[first:pos + 1, h // (H // Hkv)].double()
        p = torch.softmax((kk @ qrow[h].double()) * scale, 0)
        out.append(p @ vv)
    return torch.stack(out)


ATT_CASES = [  # H, Hkv, hd, page, window
    (4, 2, 16, 8, 0), (6, 2, 32, 16, 0), (5, 5, 48, 32, 20), (8, 1, 64, 4, 0), (3, 3, 80, 16, 300), (32, 8, 128, 16, 0),
    (16, 2, 128, 16, 100), (2, 1, 256, 16, 0), (9, 1, 64, 16, 0), (7, 7, 96, 1, 0), (4, 2, 192, 16, 0), (2, 2, 112, 8, 50),
    # head size 128 (the matrix-core decode kernel) with every group size it is instantiated for; 40 over 8 is the 14B shape
    (3, 3, 128, 16, 0), (6, 2, 128, 16, 0), (40, 8, 128, 16, 0), (6, 1, 128, 8, 300), (7, 1, 128, 16, 0), (4, 2, 128, 4, 0),
]


@pytest.mark.parametrize("H,Hkv,hd,window", [(12, 3, 32, 0), (10, 2, 48, 70), (6, 3, 64, 0), (8, 8, 16, 0)])
def test_general_attention_gives_a_row_the_same_bits_in_any_step(ops, H, Hkv, hd, window):
    """The general kernel (the 32-bit path) takes up to four query heads of a kv head in one workgroup when the step
    has many rows, and one head per workgroup when it has few: a row's result is the same bits either way, and whatever
    the other rows of the step are (5 heads to a kv head: a workgroup of four and one that is nearly empty)."""
    page, n = 16, 420
    kc, vc, table, ks, vs = make_cache(1, [n], Hkv, hd, page, torch.float32, seed=H + hd)
    g = torch.Generator().manual_seed(2)
    q = (torch.randn(n, H * hd, generator=g) * 1.5).to(DEV)
    scale = 1.0 / math.sqrt(hd)
    positions = torch.arange(n, dtype=torch.int32, device=DEV)
    row_req = torch.zeros(n, dtype=torch.int32, device=DEV)
    whole = ops.paged_attention(q, kc, vc, table, row_req, positions, H, Hkv, hd, window, scale,
                                meta={"max_context": n, "decode_only": False, "requests": 1}, exact=True)
    for t in (0, 63, 64, 300, n - 1):
        alone = ops.paged_attention(q[t:t + 1].contiguous(), kc, vc, table, row_req[:1], positions[t:t + 1].contiguous(), H, Hkv,
                                    hd, window, scale, meta={"max_context": t + 1, "decode_only": True, "requests": 1},
                                    exact=True)
        assert torch.equal(alone[0], whole[t]), t
        ref = attention_reference(q[t].view(H, hd).cpu(), ks[0], vs[0], t, H, window, scale)
        assert torch.allclose(whole[t].view(H, hd).cpu().double(), ref, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("H,Hkv,hd,page,window", ATT_CASES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_decode_rows(ops, H, Hkv, hd, page, window, dtype):
    """One row per request at the end of contexts of very different lengths (1 key, a page's edge, several splits)."""
    ctx = [1, page, page + 1, 255, 256, 257, 700, 1500]
    kc, vc, table, ks, vs = make_cache(len(ctx), ctx, Hkv, hd, page, dtype, seed=H * hd)
    g = torch.Generator().manual_seed(1)
    q = (torch.randn(len(ctx), H, hd, generator=g) * 1.5).to(dtype)
    scale = 1.0 / math.sqrt(hd)
    positions = torch.tensor([c - 1 for c in ctx], dtype=torch.int32, device=DEV)
    row_req = torch.arange(len(ctx), dtype=torch.int32, device=DEV)
    meta = {"max_context": max(ctx), "decode_only": True, "requests": len(ctx)}
    out = ops.paged_attention(q.view(len(ctx), H * hd).to(DEV), kc, vc, table, row_req, positions, H, Hkv, hd, window,
                              scale, meta=meta, exact=dtype == torch.float32)
    assert not torch.isnan(out.float()).any(), "something read an unused cache slot"
    for r, c in enumerate(ctx):
        ref = attention_reference(q[r], ks[r], vs[r], c - 1, H, window, scale)
        got = out[r].view(H, hd).cpu().double()
        tol = 1e-5 if dtype == torch.float32 else 6e-3  # fp32 sums over up to 1500 keys
        assert (got - ref).abs().max() <= tol * max(1.0, ref.abs().max()), f"request {r} (context {c})"


@pytest.mark.parametrize("R", [12, 24, 40])
def test_decode_rows_with_longer_key_ranges(ops, R):
    """More rows make the decode attention cut the keys into ranges of 256 (12 rows here), 512 (24 rows) and 1,024 (40
    rows) instead of 128: contexts around every one of those edges."""
    H, Hkv, hd, page = 16, 8, 64, 16
    assert ops._decode_split(R, Hkv, 1500) == {12: 256, 24: 512, 40: 1024}[R]
    base = [1, 127, 128, 129, 255, 256, 257, 511, 512, 513, 1023, 1024, 1025, 1500]
    ctx = [base[i % len(base)] for i in range(R)]
    ctx[-1] = 1500
    kc, vc, table, ks, vs = make_cache(R, ctx, Hkv, hd, page, torch.bfloat16, seed=R)
    g = torch.Generator().manual_seed(R)
    q = (torch.randn(R, H, hd, generator=g) * 1.5).bfloat16()
    scale = 1.0 / math.sqrt(hd)
    positions = torch.tensor([c - 1 for c in ctx], dtype=torch.int32, device=DEV)
    row_req = torch.arange(R, dtype=torch.int32, device=DEV)
    meta = {"max_context": max(ctx), "decode_only": True, "requests": R}
    out = ops.paged_attention(q.view(R, H * hd).to(DEV), kc, vc, table, row_req, positions, H, Hkv, hd, 0, scale, meta=meta)
    assert not torch.isnan(out.float()).any()
    for r, c in enumerate(ctx):
        ref = attention_reference(q[r], ks[r], vs[r], c - 1, H, 0, scale)
        got = out[r].view(H, hd).cpu().double()
        assert (got - ref).abs().max() <= 6e-3 * max(1.0, ref.abs().max()), f"request {r} (context {c})"


def test_decode_rows_over_a_long_context(ops):
    """64 query heads over 8 key heads of 128 (the 32B shape) at contexts up to 16,500 keys: 17 key ranges of 1,024 to
    merge, and every range's edge."""
    H, Hkv, hd, page = 64, 8, 128, 16
    ctx = [16500, 16384, 16385, 9000, 1]
    R = len(ctx)
    kc, vc, table, ks, vs = make_cache(R, ctx, Hkv, hd, page, torch.bfloat16, seed=11)
    g = torch.Generator().manual_seed(12)
    q = (torch.randn(R, H, hd, generator=g) * 1.5).bfloat16()
    scale = 1.0 / math.sqrt(hd)
    positions = torch.tensor([c - 1 for c in ctx], dtype=torch.int32, device=DEV)
    row_req = torch.arange(R, dtype=torch.int32, device=DEV)
    meta = {"max_context": max(ctx), "decode_only": True, "requests": R}
    ops.reset_stats()
    out = ops.paged_attention(q.view(R, H * hd).to(DEV), kc, vc, table, row_req, positions, H, Hkv, hd, 0, scale, meta=meta)
    assert ops.stats()["ran"].get("jllm_decode_attention_bf16") == 1 and not ops.stats()["general"]
    assert not torch.isnan(out.float()).any()
    for r, c in enumerate(ctx):
        ref = attention_reference(q[r], ks[r], vs[r], c - 1, H, 0, scale)
        got = out[r].view(H, hd).cpu().double()
        assert (got - ref).abs().max() <= 6e-3 * max(1.0, ref.abs().max()), f"request {r} (context {c})"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_cache_addresses_beyond_four_gigabytes(ops, dtype):
    """A layer's cache of more than 2^32 bytes with the request's pages at its far end: the store of keys and
    values, the decode kernels (plain and fused), the portion kernel, the general kernel and the page copy all
    compute addresses in 64 bits (the reference checks the same arithmetic past 2^31 elements,
    cpu/LongContextTest.java:8-16)."""
    H, Hkv, hd, page = 8, 2, 128, 16
    esize = 4 if dtype == torch.float32 else 2
    page_bytes = Hkv * page * hd * esize
    n_pages = (5 << 30) // page_bytes
    assert (n_pages - 40) * page_bytes > 1 << 32
    storage = torch.empty((2, n_pages, Hkv, page, hd), dtype=dtype, device=DEV)  # keys and values as two runs of one tensor
    kc, vc = storage[0], storage[1]
    ctx, n_new = 300, 45  # 255 positions are in the cache, the step brings 45 more (it crosses pages)
    blocks = -(-ctx // page)
    gen = torch.Generator().manual_seed(3)
    pages = (n_pages - 1 - torch.randperm(blocks + 8, generator=gen)[:blocks]).to(torch.int32)
    kc[pages.long().to(DEV)] = float("nan")
    vc[pages.long().to(DEV)] = float("nan")
    table = pages.view(1, -1).to(DEV)
    k = torch.randn(ctx, Hkv, hd, generator=gen).to(dtype)
    v = torch.randn(ctx, Hkv, hd, generator=gen).to(dtype)
    old = ctx - n_new
    for b in range(-(-old // page)):
        n = min(page, old - b * page)
        kc[int(pages[b]), :, :n] = k[b * page:b * page + n].transpose(0, 1).to(DEV)
        vc[int(pages[b]), :, :n] = v[b * page:b * page + n].transpose(0, 1).to(DEV)
    q = (torch.randn(n_new, H, hd, generator=gen) * 1.5).to(dtype)
    qkv = torch.cat([q.view(n_new, -1), k[old:].reshape(n_new, -1), v[old:].reshape(n_new, -1)], dim=1).to(DEV)
    positions = torch.arange(old, ctx, dtype=torch.int32, device=DEV)
    slots = torch.tensor([int(pages[p // page]) * page + p % page for p in range(old, ctx)], dtype=torch.int32, device=DEV)
    row_req = torch.zeros(n_new, dtype=torch.int32, device=DEV)
    scale = 1.0 / math.sqrt(hd)
    tol = 1e-5 if dtype == torch.float32 else 8e-3
    # the store (no norm, no rotation: the bytes must arrive as they are) of all but the last new position
    ops.qk_norm_rope_store(qkv[:-1], positions[:-1], slots[:-1], None, None, None, None, 1e-6, H, Hkv, hd, 0, page, kc, vc)
    got_k = torch.stack([kc[int(pages[p // page]), :, p % page] for p in range(old, ctx - 1)]).cpu()
    assert torch.equal(got_k, k[old:ctx - 1]), "keys did not arrive at their far pages"
    # portions through the tiles
    meta = {"max_context": ctx - 1, "decode_only": False, "requests": 1, "n_tiles": 1,
            "segments_dev": torch.tensor([0, 0, n_new - 1, old], dtype=torch.int32, device=DEV)}
    ops.reset_stats()
    out = ops.paged_attention(qkv[:-1, :H * hd], kc, vc, table, row_req, positions, H, Hkv, hd, 0, scale, meta=meta,
                              exact=dtype == torch.float32)
    for t in (0, 17, n_new - 2):
        ref = attention_reference(q[t], k, v, old + t, H, 0, scale)
        assert (out[t].view(H, hd).cpu().double() - ref).abs().max() <= tol * max(1.0, ref.abs().max()), f"portion row {t}"
    # the last position as a decode step: fused (bf16) or store + single row
    meta = {"max_context": ctx, "decode_only": True, "requests": 1}
    last = None
    if dtype == torch.bfloat16:
        last = ops.decode_attention_fused(qkv[-1:], kc, vc, table, row_req[:1], positions[-1:], slots[-1:], None, None, None,
                                          None, 1e-6, H, Hkv, hd, 0, 0, scale, meta)
        assert last is not None
        assert not ops.stats()["general"], ops.stats()
    else:
        ops.qk_norm_rope_store(qkv[-1:], positions[-1:], slots[-1:], None, None, None, None, 1e-6, H, Hkv, hd, 0, page, kc, vc)
    again = ops.paged_attention(qkv[-1:, :H * hd], kc, vc, table, row_req[:1], positions[-1:], H, Hkv, hd, 0, scale, meta=meta,
                                exact=dtype == torch.float32)
    ref = attention_reference(q[-1], k, v, ctx - 1, H, 0, scale)
    for o in (last, again):
        if o is not None:
            assert (o.view(H, hd).cpu().double() - ref).abs().max() <= tol * max(1.0, ref.abs().max())
    # the page copy between two far pages
    src, dst = int(pages[0]), n_pages - 1 - (blocks + 8)
    ops.copy_page_rows(storage, src, dst, 5)
    assert torch.equal(kc[dst, :, :5], kc[src, :, :5]) and torch.equal(vc[dst, :, :5], vc[src, :, :5])
    del storage, kc, vc
    torch.cuda.empty_cache()


FUSED_CASES = [  # H, Hkv, hd, rotary width (0: no rotation), page, window, q/k norm gains (None: no norm)
    (4, 2, 16, 16, 8, 0, torch.bfloat16), (6, 2, 32, 32, 16, 0, torch.float32), (5, 5, 48, 48, 32, 20, torch.bfloat16),
    (8, 1, 64, 32, 4, 0, None), (3, 3, 80, 64, 16, 300, torch.bfloat16), (32, 8, 128, 128, 16, 0, torch.bfloat16),
    (16, 2, 128, 0, 16, 100, torch.float32), (2, 1, 256, 256, 16, 0, torch.bfloat16), (7, 7, 96, 96, 2, 0, torch.bfloat16),
    # head size 128, group sizes 1, 3, 5 (the 14B shape), 6, 7, 2
    (3, 3, 128, 128, 16, 0, torch.bfloat16), (6, 2, 128, 64, 16, 0, torch.bfloat16), (40, 8, 128, 128, 16, 0, torch.bfloat16),
    (6, 1, 128, 128, 8, 300, torch.float32), (7, 1, 128, 128, 16, 0, None), (4, 2, 128, 128, 4, 0, torch.bfloat16),
]


@pytest.mark.parametrize("H,Hkv,hd,rot,page,window,gdt", FUSED_CASES)
def test_decode_fused(ops, H, Hkv, hd, rot, page, window, gdt):
    """The fused decode attention (q/k norm, rotation, store of the new key and value and attention in one launch)
    against float64 and against the separate launches it replaces; and without the store, for a layer that reads
    another layer's cache."""
    ctx = [1, page, page + 1, 255, 256, 257, 700, 1500]
    R = len(ctx)
    kc0, vc0, table, ks, vs = make_cache(R, ctx, Hkv, hd, page, torch.bfloat16, seed=H * hd + 1)
    eps = 1e-4
    scale = 1.0 / math.sqrt(hd)
    gen = torch.Generator().manual_seed(7)
    positions = torch.tensor([c - 1 for c in ctx], dtype=torch.int32, device=DEV)
    row_req = torch.arange(R, dtype=torch.int32, device=DEV)
    slots = torch.tensor([int(table[r, (c - 1) // page]) * page + (c - 1) % page for r, c in enumerate(ctx)],
                         dtype=torch.int32, device=DEV)
    gq = gk = None
    if gdt is not None:
        gq = (torch.rand(hd, generator=gen) + 0.5).to(gdt).to(DEV)
        gk = (torch.rand(hd, generator=gen) + 0.5).to(gdt).to(DEV)
    cos = sin = None
    if rot:
        ang = torch.rand(max(ctx), rot // 2, generator=gen, dtype=torch.float64) * 6.28
        cos, sin = torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV)
    meta = {"max_context": max(ctx), "decode_only": True, "requests": R}

    def prepared(x, gain, pos):  # [heads, hd] float64: norm, rotation (half pairing), rounded to bf16 like the kernels
        x = x.double()
        if gain is not None:
            x = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * gain.double().cpu()
        if rot:
            c, s_ = cos[pos].double().cpu(), sin[pos].double().cpu()
            a, b = x[:, :rot // 2].clone(), x[:, rot // 2:rot].clone()
            x[:, :rot // 2] = a * c - b * s_
            x[:, rot // 2:rot] = b * c + a * s_
        return x.float().bfloat16()

    for attempt in range(2):
        qkv = (torch.randn(R, (H + 2 * Hkv) * hd, generator=gen) * 1.5).bfloat16()
        kc, vc = kc0.clone(), vc0.clone()
        for r, c in enumerate(ctx):  # the new token's place holds NaN until the kernel stores it
            pg, off = int(slots[r]) // page, int(slots[r]) % page
            kc[pg, :, off] = float("nan")
            vc[pg, :, off] = float("nan")
        kc3, vc3, q3 = kc.clone(), vc.clone(), qkv.clone().to(DEV)
        out = ops.decode_attention_fused(qkv.to(DEV), kc, vc, table, row_req, positions, slots, cos, sin, gq, gk, eps, H,
                                         Hkv, hd, rot, window, scale, meta)
        assert out is not None, "the fused kernel declined a case it is meant to take"
        ops.qk_norm_rope_store(q3, positions, slots, cos, sin, gq, gk, eps, H, Hkv, hd, rot, page, kc3, vc3)
        out3 = ops.paged_attention(q3[:, :H * hd], kc3, vc3, table, row_req, positions, H, Hkv, hd, window, scale, meta=meta)
        assert not torch.isnan(out.float()).any()
        assert torch.equal(vc.view(torch.int16), vc3.view(torch.int16))
        kd = (kc.float() - kc3.float()).abs()
        assert not torch.isnan(kd[~torch.isnan(kc3.float())]).any()
        assert bool((kd[~torch.isnan(kc3.float())] <= 2.0 ** -7 * kc3.float().abs()[~torch.isnan(kc3.float())] + 1e-30).all())
        for r, c in enumerate(ctx):
            q = prepared(qkv[r, :H * hd].view(H, hd), gq, c - 1)
            k, v = ks[r].clone(), vs[r].clone()
            k[c - 1] = prepared(qkv[r, H * hd:(H + Hkv) * hd].view(Hkv, hd), gk, c - 1)
            v[c - 1] = qkv[r, (H + Hkv) * hd:].view(Hkv, hd)
            ref = attention_reference(q, k, v, c - 1, H, window, scale)
            got = out[r].view(H, hd).cpu().double()
            assert (got - ref).abs().max() <= 6e-3 * max(1.0, ref.abs().max()), f"request {r} (context {c}), attempt {attempt}"
            assert (got - out3[r].view(H, hd).cpu().double()).abs().max() <= 1.2e-2 * max(1.0, ref.abs().max())
    # a layer that reads another layer's cache: nothing is stored, the (complete) cache is only read
    before_k, before_v = kc3.clone(), vc3.clone()
    again = ops.decode_attention_fused(qkv.to(DEV), kc3, vc3, table, row_req, positions, slots, cos, sin, gq, gk, eps, H,
                                       Hkv, hd, rot, window, scale, meta, write_kv=False)
    assert torch.equal(kc3.view(torch.int16), before_k.view(torch.int16)) and torch.equal(vc3.view(torch.int16), before_v.view(torch.int16))
    assert (again.float() - out3.float()).abs().max() <= 1.2e-2 * max(1.0, float(out3.float().abs().max()))


def _crafted_cache(ks, vs, table, ctx, page, dtype):
    """A cache tensor pair holding exactly the given keys and values of one request, NaN elsewhere."""
    n_pages = int(table.max()) + 2
    Hkv, hd = ks.shape[1], ks.shape[2]
    kc = torch.full((n_pages, Hkv, page, hd), float("nan")).to(dtype)
    vc = torch.full((n_pages, Hkv, page, hd), float("nan")).to(dtype)
    for b in range(-(-ctx // page)):
        pg = int(table[0, b])
        n = min(page, ctx - b * page)
        kc[pg, :, :n] = ks[b * page:b * page + n].transpose(0, 1).to(dtype)
        vc[pg, :, :n] = vs[b * page:b * page + n].transpose(0, 1).to(dtype)
    return kc.to(DEV), vc.to(DEV)


# how the rows of the crafted request reach the attention: one decoding row; the same through the fused decode kernel;
# a tile of 128 rows whose last row is the crafted one; a portion of two rows; a single row riding beside a portion of
# another request (a mixed step, which takes the single rows through the decode kernel)
FAR_FORMS = ["decode", "fused", "tile", "two", "mixed"]


@pytest.mark.parametrize("form", FAR_FORMS)
@pytest.mark.parametrize("hd,H,Hkv", [(64, 4, 2), (128, 8, 2), (128, 5, 1)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_far_key_and_window_edge(ops, dtype, hd, H, Hkv, form):
    """Keys made so that a fault shows: one far key among 1200 carries all the weight; with a window, the key just
    outside it would dominate if it were read and the key just inside does dominate. The window's first key is put
    on a split's edge (a multiple of 128, 256 and 512), on a page's edge, and one key before and after them."""
    if form == "fused" and dtype == torch.float32:
        pytest.skip("the fused decode kernel is a bfloat16 kernel")
    page = 16
    ctx = 1200
    G = H // Hkv
    gen = torch.Generator().manual_seed(hd + H)
    blocks = -(-ctx // page)
    perm = torch.randperm(blocks + 3, generator=gen)
    table = perm[:blocks].to(torch.int32).view(1, -1)
    k = torch.randn(ctx, Hkv, hd, generator=gen) * 0.05
    v = torch.randn(ctx, Hkv, hd, generator=gen)
    scale = 1.0
    pos = ctx - 1

    def run(window, special, other=None):
        kk = k.clone()
        kk[special, :, 0] = 4.0  # score 32 against about 0 elsewhere
        if other is not None:
            kk[other, :, 0] = 6.0  # would win if it were visible
        kc, vc = _crafted_cache(kk, v, table, ctx, page, dtype)
        tab = table.to(DEV)
        qrow = torch.zeros(H, hd)
        qrow[:, 0] = 8.0
        if form in ("decode", "fused"):
            n, p0 = 1, pos
        elif form == "tile":
            n, p0 = 128, pos - 127
        elif form == "two":
            n, p0 = 2, pos - 1
        else:
            n, p0 = 1, pos
        q = torch.zeros(n, H, hd)
        q[-1] = qrow
        positions = torch.arange(p0, p0 + n, dtype=torch.int32)
        row_req = torch.zeros(n, dtype=torch.int32)
        meta = {"max_context": ctx, "decode_only": form in ("decode", "fused"), "requests": 1}
        if form == "fused":
            qkv = torch.zeros(1, (H + 2 * Hkv) * hd)
            qkv[0, :H * hd] = qrow.view(-1)
            qkv[0, H * hd:(H + Hkv) * hd] = kk[pos].view(-1)
            qkv[0, (H + Hkv) * hd:] = v[pos].view(-1)
            slot = int(table[0, pos // page]) * page + pos % page
            out = ops.decode_attention_fused(qkv.bfloat16().to(DEV), kc, vc, tab, row_req.to(DEV), positions.to(DEV),
                                             torch.tensor([slot], dtype=torch.int32, device=DEV), None, None, None, None,
                                             1e-6, H, Hkv, hd, 0, window, scale, meta)
            assert out is not None
            return out.view(H, hd).cpu().float()
        if form == "mixed":
            # another request brings a portion of 40 rows in the same step; its pages follow in the table's second row
            n2, ctx2 = 40, 40
            k2 = torch.randn(ctx2, Hkv, hd, generator=torch.Generator().manual_seed(5)) * 0.05
            tab2 = torch.zeros(2, table.shape[1], dtype=torch.int32)
            tab2[0] = table[0]
            extra = [int(perm[blocks]), int(perm[blocks + 1]), int(perm[blocks + 2])]
            tab2[1, :3] = torch.tensor(extra, dtype=torch.int32)
            for b in range(3):
                m = min(page, ctx2 - b * page)
                kc[extra[b], :, :m] = k2[b * page:b * page + m].transpose(0, 1).to(dtype).to(DEV)
                vc[extra[b], :, :m] = k2[b * page:b * page + m].transpose(0, 1).to(dtype).to(DEV)
            q = torch.cat([torch.randn(n2, H, hd, generator=torch.Generator().manual_seed(6)), qrow[None]])
            positions = torch.cat([torch.arange(n2, dtype=torch.int32), torch.tensor([pos], dtype=torch.int32)])
            row_req = torch.cat([torch.ones(n2, dtype=torch.int32), torch.zeros(1, dtype=torch.int32)])
            tiles = [1, 0, n2, 0, 0, n2, 1, pos]
            meta.update(requests=2, n_tiles=2, n_tiles_multi=1, single_rows=(n2, 1),
                        segments_dev=torch.tensor(tiles, dtype=torch.int32, device=DEV))
            tab = tab2.to(DEV)
        elif form in ("tile", "two"):
            meta.update(n_tiles=1, segments_dev=torch.tensor([0, 0, n, p0], dtype=torch.int32, device=DEV))
        out = ops.paged_attention(q.view(-1, H * hd).to(dtype).to(DEV), kc, vc, tab, row_req.to(DEV), positions.to(DEV), H,
                                  Hkv, hd, window, scale, meta=meta, exact=dtype == torch.float32)
        return out[-1].view(H, hd).cpu().float()

    ops.reset_stats()
    far = run(0, 37)
    for h in range(H):
        assert torch.allclose(far[h], v[37, h // G].float(), atol=2e-2), "the far key's value must come through"
    for first in (pos + 1 - 100, 1024, 1023, 1025, 512, 768, 1168, 1167, pos - 1, pos):
        w = pos + 1 - first  # the window whose oldest visible key, for the last row, is `first`
        edge = run(w, first, other=first - 1)
        for h in range(H):
            assert torch.allclose(edge[h], v[first, h // G].float(), atol=2e-2), \
                f"window edge at key {first}: the key inside must win, the one outside is unseen (head {h})"
    if dtype == torch.bfloat16:
        assert not ops.stats()["general"], f"a matrix-core or split-key kernel declined: {ops.stats()}"


@pytest.mark.parametrize("H,Hkv,hd,page,window", ATT_CASES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_portions(ops, H, Hkv, hd, page, window, dtype):
    """A batch of portions at different places of their requests (a whole prompt, a portion deep inside a long
    context, two tokens, one token) beside each other."""
    ctx = [130, 900, 40, 513, 7]        # keys held after this step
    ns = [130, 200, 2, 1, 7]            # rows of this step (the last ns positions of each request)
    R = len(ctx)
    kc, vc, table, ks, vs = make_cache(R, ctx, Hkv, hd, page, dtype, seed=hd + page)
    g = torch.Generator().manual_seed(2)
    T = sum(ns)
    q = (torch.randn(T, H, hd, generator=g) * 1.5).to(dtype)
    scale = 1.0 / math.sqrt(hd)
    pos, req, tiles = [], [], []
    row = 0
    for r in range(R):
        p0 = ctx[r] - ns[r]
        pos += list(range(p0, ctx[r]))
        req += [r] * ns[r]
        for a in range(0, ns[r], 128):
            tiles += [r, row + a, min(128, ns[r] - a), p0 + a]
        row += ns[r]
    positions = torch.tensor(pos, dtype=torch.int32, device=DEV)
    row_req = torch.tensor(req, dtype=torch.int32, device=DEV)
    meta = {"max_context": max(ctx), "decode_only": False, "requests": R,
            "segments_dev": torch.tensor(tiles, dtype=torch.int32, device=DEV), "n_tiles": len(tiles) // 4}
    wide = torch.zeros(T, H * hd + 2 * Hkv * hd, dtype=dtype)
    wide[:, :H * hd] = q.view(T, H * hd)
    wide = wide.to(DEV)
    out = ops.paged_attention(wide[:, :H * hd], kc, vc, table, row_req, positions, H, Hkv, hd, window, scale,
                              meta=meta, exact=dtype == torch.float32)
    assert not torch.isnan(out.float()).any(), "something read an unused cache slot"
    tol = 1e-5 if dtype == torch.float32 else 8e-3  # fp32 sums over hundreds of keys; the reference's 2e-6 is for 40
    for t in range(T):
        r = req[t]
        ref = attention_reference(q[t], ks[r], vs[r], pos[t], H, window, scale)
        got = out[t].view(H, hd).cpu().double()
        assert (got - ref).abs().max() <= tol * max(1.0, ref.abs().max()), f"row {t} (request {r}, position {pos[t]})"


@pytest.mark.parametrize("window", [0, 200])
def test_portions_in_a_small_and_in_a_large_step(ops, window):
    """The matrix-core kernel for portions has two forms: with few tiles in the step a workgroup cuts a tile's keys
    over two groups of waves and merges them, with many it does not. The same 300 rows deep inside a request, alone
    (3 tiles) and beside a 4,200-token prompt (36 tiles at 16 heads: more workgroups than two per compute unit),
    against the reference, and the two against each other."""
    H, Hkv, hd, page = 16, 4, 128, 16
    assert H * 36 > 2 * ops.compute_units() >= H * 3, "the sizes of this test assume about 256 compute units"
    ctx, ns = [900, 4200], [300, 4200]
    kc, vc, table, ks, vs = make_cache(2, ctx, Hkv, hd, page, torch.bfloat16, seed=77)
    g = torch.Generator().manual_seed(3)
    q = (torch.randn(sum(ns), H, hd, generator=g) * 1.5).bfloat16()
    scale = 1.0 / math.sqrt(hd)

    def run(requests):
        pos, req, tiles, rows = [], [], [], []
        row = 0
        for i, r in enumerate(requests):
            p0 = ctx[r] - ns[r]
            pos += list(range(p0, ctx[r]))
            req += [i] * ns[r]
            rows += list(range(sum(ns[:r]), sum(ns[:r]) + ns[r]))
            for a in range(0, ns[r], 128):
                tiles += [i, row + a, min(128, ns[r] - a), p0 + a]
            row += ns[r]
        order = sorted(range(len(tiles) // 4), key=lambda t: -(tiles[4 * t + 3] + tiles[4 * t + 2]))  # most keys first
        tiles = [x for t in order for x in tiles[4 * t:4 * t + 4]]
        meta = {"max_context": max(ctx[r] for r in requests), "decode_only": False, "requests": len(requests),
                "segments_dev": torch.tensor(tiles, dtype=torch.int32, device=DEV), "n_tiles": len(tiles) // 4}
        return ops.paged_attention(q[rows].view(len(rows), H * hd).to(DEV), kc, vc, table[requests].contiguous(),
                                   torch.tensor(req, dtype=torch.int32, device=DEV),
                                   torch.tensor(pos, dtype=torch.int32, device=DEV), H, Hkv, hd, window, scale, meta=meta)

    ops.reset_stats()
    small = run([0])[:300].float().cpu()
    large = run([0, 1])[:300].float().cpu()
    assert ops.stats()["ran"].get("jllm_prefill_attention_bf16") == 2 and not ops.stats()["general"], ops.stats()
    assert not torch.equal(small, large), "the two forms add in different orders: equal bits mean one form ran twice"
    for t in range(0, 300, 7):
        ref = attention_reference(q[t], ks[0], vs[0], ctx[0] - 300 + t, H, window, scale)
        for got in (small[t], large[t]):
            assert (got.view(H, hd).double() - ref).abs().max() <= 8e-3 * max(1.0, ref.abs().max()), f"row {t}"
    assert (small - large).abs().max() <= 8e-3 * max(1.0, small.abs().max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_copy_page_rows(ops, dtype):
    storage = torch.randn(3, 7, 2, 8, 48, device=DEV).to(dtype)  # [runs, pages, heads, page size, head size]
    before = storage.clone()
    ops.copy_page_rows(storage, 5, 2, 3)
    want = before.clone()
    want[:, 2, :, :3, :] = before[:, 5, :, :3, :]
    assert torch.equal(storage, want), "rows 0..2 of page 5 go to page 2 in every run and head; nothing else moves"
    odd = torch.randint(0, 255, (2, 4, 1, 4, 7), device=DEV).to(torch.uint8)  # 7 bytes per position: the byte path
    before = odd.clone()
    ops.copy_page_rows(odd, 0, 3, 2)
    want = before.clone()
    want[:, 3, :, :2] = before[:, 0, :, :2]
    assert torch.equal(odd, want)
    with pytest.raises(ops.KernelError):
        ops.copy_page_rows(storage, 5, 9, 3)
    with pytest.raises(ops.KernelError):
        ops.copy_page_rows(storage, 5, 2, 9)
