"""rtp_gemm through the C ABI: every operand layout, both dtypes, ragged sizes, batching by strides and
the fused epilogue, against float64 matmul on the CPU."""
import pytest
import torch

from gpu_util import DEV, TOL, rel_err

pytestmark = pytest.mark.gpu


def _ops():
    from rtp_amd import ops
    return ops


def _rand(shape, dtype, gen):
    return (torch.randn(shape, generator=gen) * 0.5).to(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("akc,bkc", [(True, True), (True, False), (False, True), (False, False)])
@pytest.mark.parametrize("m,n,k", [(8, 8, 8), (33, 65, 17), (100, 36, 70), (256, 192, 128), (1024, 256, 520), (1000, 200, 136)])
def test_gemm_layouts(dtype, akc, bkc, m, n, k):
    ops = _ops()
    gen = torch.Generator().manual_seed(m * 31 + n * 7 + k)
    a = _rand((m, k) if akc else (k, m), dtype, gen)
    b = _rand((n, k) if bkc else (k, n), dtype, gen)
    A = a.double() if akc else a.double().t()
    B = b.double() if bkc else b.double().t()
    ref = A @ B.t()
    ad, bd = a.to(DEV), b.to(DEV)
    out = torch.full((m, n), float("nan"), dtype=dtype, device=DEV)
    ops.gemm_raw(dtype, a=ad.data_ptr(), b=bd.data_ptr(), c_out=out.data_ptr(), m=m, n=n, k=k,
                 lda=ad.stride(0), ldb=bd.stride(0), ldc=n, a_kcontig=akc, b_kcontig=bkc)
    torch.cuda.synchronize()
    assert rel_err(out, ref) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gemm_big_tile_path(dtype):
    """Enough 128x128 tiles to take the large-tile kernel, with ragged edges."""
    ops = _ops()
    gen = torch.Generator().manual_seed(5)
    m, n, k = 1900, 1700, 300
    a, b = _rand((m, k), dtype, gen), _rand((n, k), dtype, gen)
    ref = a.double() @ b.double().t()
    ad, bd = a.to(DEV), b.to(DEV)
    out = torch.empty(m, n, dtype=dtype, device=DEV)
    ops.linear_fwd(ad, bd, out)
    assert rel_err(out, ref) <= TOL[dtype]
    # weight-gradient and input-gradient layouts on the same path
    dy = _rand((m, n), dtype, gen).to(DEV)
    dx = torch.empty(m, k, dtype=dtype, device=DEV)
    ops.linear_dgrad(dy, bd, dx)
    assert rel_err(dx, dy.double().cpu() @ b.double()) <= TOL[dtype]
    dw = torch.empty(n, k, dtype=dtype, device=DEV)
    ops.linear_wgrad(dy, ad, dw)
    assert rel_err(dw, dy.double().cpu().t() @ a.double()) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gemm_epilogue(dtype):
    ops = _ops()
    gen = torch.Generator().manual_seed(9)
    m, n, k = 70, 50, 40
    x, w = _rand((m, k), dtype, gen), _rand((n, k), dtype, gen)
    bias, cin, gate = _rand((n,), dtype, gen), _rand((m, n), dtype, gen), _rand((m, n), dtype, gen)
    base = x.double() @ w.double().t()
    xd, wd = x.to(DEV), w.to(DEV)
    out = torch.empty(m, n, dtype=dtype, device=DEV)
    ops.linear_fwd(xd, wd, out, bias=bias.to(DEV), relu=True)
    assert rel_err(out, torch.relu(base + bias.double())) <= TOL[dtype]
    # accumulate in place, fp32 accumulator, strided output block
    wide = torch.zeros(m, 3 * n, dtype=torch.float32, device=DEV)
    blk = wide[:, n:2 * n]
    blk.copy_(cin.float())
    ops.linear_fwd(xd, wd, blk, c_in=blk)
    assert rel_err(blk, base + cin.double()) <= TOL[dtype]
    assert wide[:, :n].abs().max() == 0 and wide[:, 2 * n:].abs().max() == 0
    # relu-mask epilogue of the input-gradient GEMM
    dy = _rand((m, n), dtype, gen)
    gk = _rand((m, k), dtype, gen)
    dx = torch.empty(m, k, dtype=dtype, device=DEV)
    ops.linear_dgrad(dy.to(DEV), wd, dx, gate=gk.to(DEV))
    assert rel_err(dx, (dy.double() @ w.double()) * (gk.double() > 0)) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gemm_batched_by_strides(dtype):
    """(batch, head) pairs addressed inside a packed [L, N, 3*E_s] projection, as attention does."""
    ops = _ops()
    gen = torch.Generator().manual_seed(13)
    L, N, h, d = 20, 3, 2, 16
    e_s = h * d
    qkv = _rand((L, N, 3 * e_s), dtype, gen)
    q = qkv[..., :e_s].reshape(L, N, h, d).permute(1, 2, 0, 3).double()
    k = qkv[..., e_s:2 * e_s].reshape(L, N, h, d).permute(1, 2, 0, 3).double()
    ref = q @ k.transpose(-1, -2)
    qd = qkv.to(DEV)
    out = torch.empty(N * h, L, L, dtype=torch.float32, device=DEV)
    esz = qd.element_size()
    ops.gemm_raw(dtype, a=qd.data_ptr(), b=qd.data_ptr() + e_s * esz, c_out=out.data_ptr(), m=L, n=L, k=d,
                 lda=N * 3 * e_s, ldb=N * 3 * e_s, ldc=L, a_kcontig=True, b_kcontig=True, batch=N * h, zdiv=h,
                 a_s=(3 * e_s, d), b_s=(3 * e_s, d), c_s=(h * L * L, L * L), out_f32=True)
    assert rel_err(out.view(N, h, L, L), ref) <= TOL[dtype]


def test_colsum_and_errors():
    ops = _ops()
    from rtp_amd._lib import RtpError
    x = torch.randn(300, 70)
    out = torch.empty(70, device=DEV)
    ops.colsum(x.to(DEV), out)
    assert rel_err(out, x.double().sum(0)) <= 1e-5
    ops.colsum(x.to(DEV), out, accumulate=True)
    assert rel_err(out, 2 * x.double().sum(0)) <= 1e-5
    xb = x.bfloat16()
    outb = torch.empty(70, dtype=torch.bfloat16, device=DEV)
    ops.colsum(xb.to(DEV)[:, 10:40], outb[:30].clone().contiguous())
    with pytest.raises(RtpError):
        ops.linear_fwd(torch.randn(4, 4), torch.randn(4, 4), torch.empty(4, 4))  # CPU tensors: no fallback
    with pytest.raises(ValueError):
        ops.linear_fwd(x.to(DEV), torch.randn(5, 71, device=DEV), torch.empty(300, 5, device=DEV))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gemm_groups_and_k_segments(dtype):
    """Several shards in one launch: groups (column-parallel forward) and K segments (sum over shards)."""
    ops = _ops()
    gen = torch.Generator().manual_seed(17)
    ws, m, k, n_s = 4, 150, 96, 40
    numel = n_s * k + n_s  # flat shard: [weight, bias]
    home = _rand((ws, numel), dtype, gen)
    x = _rand((m, k), dtype, gen)
    hd, xd = home.to(DEV), x.to(DEV)
    y = torch.full((m, ws * n_s), float("nan"), dtype=dtype, device=DEV)
    ops.gemm_raw(dtype, a=xd.data_ptr(), b=hd.data_ptr(), c_out=y.data_ptr(), bias=hd.data_ptr() + n_s * k * hd.element_size(),
                 m=m, n=n_s, k=k, lda=k, ldb=k, ldc=ws * n_s, a_kcontig=True, b_kcontig=True, groups=ws,
                 b_sg=numel, bias_sg=numel, c_sg=n_s)
    w = home[:, :n_s * k].reshape(ws * n_s, k).double()
    b = home[:, n_s * k:].reshape(-1).double()
    assert rel_err(y, x.double() @ w.t() + b) <= TOL[dtype]
    # input gradient of the same layer: dX = sum_s dY[:, s-block] @ W_s, contraction segmented over shards
    dy = _rand((m, ws * n_s), dtype, gen)
    dyd = dy.to(DEV)
    dx = torch.empty(m, k, dtype=dtype, device=DEV)
    ops.gemm_raw(dtype, a=dyd.data_ptr(), b=hd.data_ptr(), c_out=dx.data_ptr(), m=m, n=k, k=n_s, lda=ws * n_s, ldb=k,
                 ldc=k, a_kcontig=True, b_kcontig=False, ksegs=ws, a_sk=n_s, b_sk=numel)
    assert rel_err(dx, dy.double() @ w) <= TOL[dtype]
    # weight gradients of all shards: group g writes dW_g = dY[:, g-block]^T @ X into its flat gradient row
    grads = torch.zeros(ws, numel, dtype=dtype, device=DEV)
    ops.gemm_raw(dtype, a=dyd.data_ptr(), b=xd.data_ptr(), c_out=grads.data_ptr(), m=n_s, n=k, k=m, lda=ws * n_s, ldb=k,
                 ldc=k, a_kcontig=False, b_kcontig=False, groups=ws, a_sg=n_s, c_sg=numel)
    ops.colsum(dyd, grads[0, n_s * k:], seg=n_s, seg_stride=numel)
    assert rel_err(grads[:, :n_s * k].reshape(ws * n_s, k), dy.double().t() @ x.double()) <= TOL[dtype]
    assert rel_err(grads[:, n_s * k:].reshape(-1), dy.double().sum(0)) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", [(1024, 2048, 2048), (2048, 2048, 1024), (512, 640, 300)])
def test_gemm_mid_tile_path(dtype, m, n, k):
    """Shapes that select the 128x64 tile (and its three-slab register ring)."""
    ops = _ops()
    gen = torch.Generator().manual_seed(m + n)
    a, b = _rand((m, k), dtype, gen), _rand((n, k), dtype, gen)
    out = torch.empty(m, n, dtype=dtype, device=DEV)
    ops.linear_fwd(a.to(DEV), b.to(DEV), out)
    assert rel_err(out, a.double() @ b.double().t()) <= TOL[dtype]
    dy = _rand((m, n), dtype, gen).to(DEV)
    dw = torch.empty(n, k, dtype=dtype, device=DEV)
    ops.linear_wgrad(dy, a.to(DEV), dw)
    assert rel_err(dw, dy.double().cpu().t() @ a.double()) <= TOL[dtype]


def test_gemm_huge_leading_dimension_takes_guarded_kernel():
    """A tile's byte offsets must fit 32 bits in the wave-specialised kernel; a leading dimension beyond that
    (here 16 MiB per row) is served by the guarded kernel with the same result."""
    ops = _ops()
    m, n, k, lda = 16, 64, 64, 1 << 23
    gen = torch.Generator().manual_seed(3)
    a = _rand((m, k), torch.bfloat16, gen)
    b = _rand((n, k), torch.bfloat16, gen)
    big = torch.zeros(m * lda, dtype=torch.bfloat16, device=DEV)
    big.view(m, lda)[:, :k] = a.to(DEV)
    bd = b.to(DEV)
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.gemm_raw(torch.bfloat16, a=big.data_ptr(), b=bd.data_ptr(), c_out=out.data_ptr(), m=m, n=n, k=k,
                 lda=lda, ldb=k, ldc=n, a_kcontig=True, b_kcontig=True)
    torch.cuda.synchronize()
    assert rel_err(out, a.double() @ b.double().t()) <= TOL[torch.bfloat16]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("accumulate", [False, True])
@pytest.mark.parametrize("m,n,k,groups", [(256, 2048, 1024, 8), (72, 136, 200, 3), (768, 64, 520, 1), (8, 128, 72, 2)])
def test_gemm_fused_row_sums_of_a(dtype, accumulate, m, n, k, groups):
    """a_rowsum: the bias gradient of dW = dY^T X from the same launch, per group, against an fp64 column sum."""
    ops = _ops()
    gen = torch.Generator().manual_seed(m + n + k + groups)
    dy = _rand((k, groups * m), dtype, gen)           # [tokens, out features of all groups]
    x = _rand((k, n), dtype, gen)
    numel = m * n + m + 8                             # flat gradient row: weight, bias, padding
    grads = _rand((groups, numel), dtype, gen)
    before = grads.clone()
    dyd, xd, gd = dy.to(DEV), x.to(DEV), grads.to(DEV)
    es = gd.element_size()
    fused = ops.gemm_raw(dtype, a=dyd.data_ptr(), b=xd.data_ptr(), c_out=gd.data_ptr(), m=m, n=n, k=k,
                         lda=groups * m, ldb=n, ldc=n, a_kcontig=False, b_kcontig=False, groups=groups, a_sg=m,
                         c_sg=numel, c_in=gd.data_ptr() if accumulate else None, ld_cin=n, cin_sg=numel,
                         rowsum=gd.data_ptr() + m * n * es, rowsum_sg=numel, rowsum_accum=accumulate)
    torch.cuda.synchronize()
    assert fused
    got = gd.cpu()
    for g in range(groups):
        blk = dy[:, g * m:(g + 1) * m].double()
        w_ref = blk.t() @ x.double()
        b_ref = blk.sum(0)
        if accumulate:
            w_ref = w_ref + before[g, :m * n].double().view(m, n)
            b_ref = b_ref + before[g, m * n:m * n + m].double()
        assert rel_err(got[g, :m * n].view(m, n), w_ref) <= TOL[dtype]
        assert rel_err(got[g, m * n:m * n + m], b_ref) <= TOL[dtype]
        assert torch.equal(got[g, m * n + m:], before[g, m * n + m:])   # padding untouched


def test_gemm_row_sums_fall_back_when_not_fusable():
    """A K-contiguous A (or unaligned operands) cannot carry the row sums: gemm_raw says so and leaves them alone."""
    ops = _ops()
    gen = torch.Generator().manual_seed(9)
    a = _rand((128, 256), torch.float32, gen).to(DEV)
    b = _rand((64, 256), torch.float32, gen).to(DEV)
    c = torch.empty(128, 64, device=DEV)
    rs = torch.full((128,), 7.0, device=DEV)
    fused = ops.gemm_raw(torch.float32, a=a.data_ptr(), b=b.data_ptr(), c_out=c.data_ptr(), m=128, n=64, k=256,
                         lda=256, ldb=256, ldc=64, a_kcontig=True, b_kcontig=True, rowsum=rs.data_ptr())
    torch.cuda.synchronize()
    assert not fused
    assert torch.equal(rs, torch.full((128,), 7.0, device=DEV))
    assert rel_err(c, a.double() @ b.double().t()) <= TOL[torch.float32]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("akc", [True, False])
@pytest.mark.parametrize("m,n,k", [(1024, 6144, 256), (1000, 6000, 136)])
def test_gemm_wide_tile_shapes(dtype, akc, m, n, k):
    """Problems whose tile count fills the 256 CUs exactly with 128 x 192 tiles (the packed q/k/v projection of the
    LM: 1024 x 6144), ragged in every extent in the second case; B must be K-contiguous for that shape."""
    ops = _ops()
    gen = torch.Generator().manual_seed(m + n + k)
    a = _rand((m, k) if akc else (k, m), dtype, gen)
    b = _rand((n, k), dtype, gen)
    bias = _rand((n,), dtype, gen)
    A = a.double() if akc else a.double().t()
    ref = A @ b.double().t() + bias.double()
    ad, bd, biasd = a.to(DEV), b.to(DEV), bias.to(DEV)
    out = torch.full((m, n), float("nan"), dtype=dtype, device=DEV)
    ops.gemm_raw(dtype, a=ad.data_ptr(), b=bd.data_ptr(), c_out=out.data_ptr(), m=m, n=n, k=k, lda=ad.stride(0),
                 ldb=k, ldc=n, a_kcontig=akc, b_kcontig=True, bias=biasd.data_ptr())
    torch.cuda.synchronize()
    assert rel_err(out, ref) <= TOL[dtype]


@pytest.mark.parametrize("m,n,k,groups,akc,bkc", [
    (3072, 1536, 256, 1, True, True),      # 12 x 12 tiles of 256 x 128 (or 24 x 12 of 128 x 128): odd divisors
    (1280, 3840, 192, 1, True, False),     # 5 / 10 tile rows
    (2048, 1152, 1024, 2, False, False),   # 2 groups, 9 tile columns of 128: panels of 1 x 9 or 3 x 3
    (4096, 2048, 2048, 4, False, False),   # long K: a strip of B tiles must fit the L2, narrow panels
    (1792, 2560, 64, 3, True, True),       # 3 groups: no even split over the 8 XCDs
])
def test_gemm_many_rounds_tile_order(m, n, k, groups, akc, bkc):
    """Launches of several rounds of tiles per CU: the order in which an XCD's tiles are handed out (bricks, panels of
    prow x pcol tiles walked down strips of tile columns) must cover every tile exactly once whatever the divisors of
    the tile counts are.  Output starts as NaN, so a tile that is never written shows; bf16 against fp64."""
    ops = _ops()
    dtype = torch.bfloat16
    gen = torch.Generator().manual_seed(m + n + k + groups)
    a = _rand((groups, m, k) if akc else (groups, k, m), dtype, gen)
    b = _rand((groups, n, k) if bkc else (groups, k, n), dtype, gen)
    A = a.double() if akc else a.double().transpose(1, 2)
    B = b.double() if bkc else b.double().transpose(1, 2)
    ref = A @ B.transpose(1, 2)
    ad, bd = a.to(DEV), b.to(DEV)
    out = torch.full((groups, m, n), float("nan"), dtype=dtype, device=DEV)
    ops.gemm_raw(dtype, a=ad.data_ptr(), b=bd.data_ptr(), c_out=out.data_ptr(), m=m, n=n, k=k, lda=ad.stride(1),
                 ldb=bd.stride(1), ldc=n, a_kcontig=akc, b_kcontig=bkc, groups=groups, a_sg=ad.stride(0),
                 b_sg=bd.stride(0), c_sg=m * n)
    torch.cuda.synchronize()
    assert not torch.isnan(out).any()
    assert rel_err(out, ref) <= TOL[dtype]


@pytest.mark.parametrize("akc,bkc", [(True, True), (True, False), (False, True)])
def test_gemm_256x256_tile_path(akc, bkc):
    """A product with at least 256 tiles of 256 x 256 and K >= 1024 takes the eight-wave kernel (checked by its
    name in the launch records); ragged on every edge, with bias, ReLU and an addend in the epilogue.  The yardstick
    is torch's fp32 product of the same bf16 values on the device (float64 on the CPU would take minutes)."""
    from rtp_amd import _lib
    ops = _ops()
    dtype = torch.bfloat16
    gen = torch.Generator().manual_seed(77)
    m, n, k = 8104, 8200, 2056  # leading dimensions stay multiples of 16 bytes in every layout
    a = _rand((m, k) if akc else (k, m), dtype, gen).to(DEV)
    b = _rand((n, k) if bkc else (k, n), dtype, gen).to(DEV)
    bias, cin = _rand((n,), dtype, gen).to(DEV), _rand((m, n), dtype, gen).to(DEV)
    A = a.float() if akc else a.float().t()
    B = b.float() if bkc else b.float().t()
    ref = torch.relu(A @ B.t() + bias.float() + cin.float())
    out = torch.full((m, n), float("nan"), dtype=dtype, device=DEV)
    _lib.profile_enable(1)
    try:
        ops.gemm_raw(dtype, a=a.data_ptr(), b=b.data_ptr(), c_out=out.data_ptr(), m=m, n=n, k=k, lda=a.stride(0),
                     ldb=b.stride(0), ldc=n, a_kcontig=akc, b_kcontig=bkc, bias=bias.data_ptr(), c_in=cin.data_ptr(),
                     ld_cin=n, relu=True)
        torch.cuda.synchronize()
        names = list(_lib.profile_collect())
    finally:
        _lib.profile_enable(0)
    assert any("256x256" in nm for nm in names), names
    assert rel_err(out, ref) <= TOL[dtype]


@pytest.mark.parametrize("akc,bkc", [(True, True), (True, False), (False, False)])
@pytest.mark.parametrize("k,ksegs", [(1024, 1), (1096, 1), (520, 2), (136, 8)])
def test_gemm_256x256_tile_path_groups_segments_and_short_contractions(akc, bkc, k, ksegs):
    """The eight-wave kernel's two-stage pipeline at its edges: a grouped launch (16 groups of 4 x 4 tiles fill the
    256 CUs once), contraction lengths of 2 to 17 slabs with and without a ragged last slab, and a contraction cut
    into K segments that sit apart in memory (every segment starts a new run of slabs and may end in a ragged one)."""
    from rtp_amd import _lib
    ops = _ops()
    dtype = torch.bfloat16
    gen = torch.Generator().manual_seed(91)
    groups, m, n = 16, 1000, 1024
    # operand of segment s, group g: a[s, g] is [m, k] (or [k, m]); the product sums over s
    a = _rand((ksegs, groups) + ((m, k) if akc else (k, m)), dtype, gen).to(DEV)
    b = _rand((ksegs, groups) + ((n, k) if bkc else (k, n)), dtype, gen).to(DEV)
    A = a.float() if akc else a.float().transpose(2, 3)
    B = b.float() if bkc else b.float().transpose(2, 3)
    ref = torch.einsum("sgmk,sgnk->gmn", A, B)
    out = torch.full((groups, m, n), float("nan"), dtype=dtype, device=DEV)
    _lib.profile_enable(1)
    try:
        ops.gemm_raw(dtype, a=a.data_ptr(), b=b.data_ptr(), c_out=out.data_ptr(), m=m, n=n, k=k, lda=a.stride(2),
                     ldb=b.stride(2), ldc=n, a_kcontig=akc, b_kcontig=bkc, groups=groups, a_sg=a.stride(1),
                     b_sg=b.stride(1), c_sg=m * n, ksegs=ksegs, a_sk=a.stride(0), b_sk=b.stride(0))
        torch.cuda.synchronize()
        names = list(_lib.profile_collect())
    finally:
        _lib.profile_enable(0)
    assert any("256x256" in nm for nm in names), names
    assert not torch.isnan(out).any()
    assert rel_err(out, ref) <= TOL[dtype]


@pytest.mark.parametrize("warm_bytes", [16, 1024, 3 * 1024 + 16, 1 << 20, 80 << 20])
def test_gemm_carries_a_warm_ahead_hint(warm_bytes):
    """rtp_gemm_warm_next: the next product reads the hinted region at its start and its result is what it is without
    the hint, bit for bit; regions that are no multiple of the 1 KiB request size, smaller than one request and larger
    than a launch can take are all fine.  The hint ends with that launch: a second product runs without it."""
    from rtp_amd import _lib
    ops = _ops()
    lib = _lib.load()
    dtype = torch.bfloat16
    gen = torch.Generator().manual_seed(3)
    m, n, k = 300, 520, 200
    x, w = _rand((m, k), dtype, gen).to(DEV), _rand((n, k), dtype, gen).to(DEV)
    region = torch.ones(warm_bytes, dtype=torch.uint8, device=DEV)
    plain = torch.empty(m, n, dtype=dtype, device=DEV)
    ops.linear_fwd(x, w, plain)
    hinted = torch.full((m, n), float("nan"), dtype=dtype, device=DEV)
    _lib.check(lib.rtp_gemm_warm_next(region.data_ptr(), warm_bytes))
    ops.linear_fwd(x, w, hinted)
    del region  # the hint is gone with the launch: the next product must not touch the freed region
    torch.cuda.empty_cache()
    again = torch.empty(m, n, dtype=dtype, device=DEV)
    ops.linear_fwd(x, w, again)
    torch.cuda.synchronize()
    assert torch.equal(plain, hinted) and torch.equal(plain, again)
    # a launch that cannot carry the hint (the one-wavefront kernel for tiny products) ends it as well
    region = torch.ones(4096, dtype=torch.uint8, device=DEV)
    _lib.check(lib.rtp_gemm_warm_next(region.data_ptr(), 4096))
    tiny = torch.empty(8, 8, dtype=dtype, device=DEV)
    ops.linear_fwd(x[:8, :8].contiguous(), w[:8, :8].contiguous(), tiny)
    del region
    torch.cuda.empty_cache()
    ops.linear_fwd(x, w, again)
    torch.cuda.synchronize()
    assert torch.equal(plain, again)
    with pytest.raises(_lib.RtpError):
        _lib.check(lib.rtp_gemm_warm_next(x.data_ptr() + 2, 64))


def test_cache_warm_reads_and_changes_nothing():
    from rtp_amd import _lib
    lib = _lib.load()
    t = torch.arange(1 << 20, dtype=torch.int32, device=DEV)
    want = t.clone()
    for nbytes in (0, 16, 4096 + 48, t.numel() * 4):
        _lib.check(lib.rtp_cache_warm(torch.cuda.current_stream().cuda_stream, t.data_ptr(), nbytes, 0))
    torch.cuda.synchronize()
    assert torch.equal(t, want)


def test_gemm_random_shapes_layouts_and_epilogues():
    """A seeded sweep over shapes that no test picked by hand: sizes that are not multiples of anything (the guarded
    kernel), multiples of 8 (every fast tile shape the cost model may take, the 256 x 256 kernel included), both
    dtypes, all four operand layouts, with and without bias / addend / ReLU.  Yardstick: the fp32 product of the same
    values on the device."""
    import random
    ops = _ops()
    rng = random.Random(20240607)
    gen = torch.Generator().manual_seed(99)
    for case in range(72):
        dtype = torch.bfloat16 if case % 3 else torch.float32
        akc, bkc = bool(rng.getrandbits(1)), bool(rng.getrandbits(1))
        if case % 4 == 0:      # ragged: not even vector-aligned
            m, n, k = rng.randint(1, 700), rng.randint(1, 700), rng.randint(1, 900)
        elif case % 4 == 3:    # large enough for the biggest tiles
            m, n, k = 8 * rng.randint(200, 520), 8 * rng.randint(200, 520), 8 * rng.randint(100, 330)
        else:
            m, n, k = 8 * rng.randint(1, 160), 8 * rng.randint(1, 160), 8 * rng.randint(1, 300)
        a = _rand((m, k) if akc else (k, m), dtype, gen).to(DEV)
        b = _rand((n, k) if bkc else (k, n), dtype, gen).to(DEV)
        use_bias, use_cin, relu = bool(rng.getrandbits(1)), bool(rng.getrandbits(1)), bool(rng.getrandbits(1))
        bias = _rand((n,), dtype, gen).to(DEV) if use_bias else None
        cin = _rand((m, n), dtype, gen).to(DEV) if use_cin else None
        A = a.float() if akc else a.float().t()
        B = b.float() if bkc else b.float().t()
        ref = A @ B.t()
        if use_bias:
            ref = ref + bias.float()
        if use_cin:
            ref = ref + cin.float()
        if relu:
            ref = torch.relu(ref)
        out = torch.full((m, n), float("nan"), dtype=dtype, device=DEV)
        ops.gemm_raw(dtype, a=a.data_ptr(), b=b.data_ptr(), c_out=out.data_ptr(), m=m, n=n, k=k, lda=a.stride(0),
                     ldb=b.stride(0), ldc=n, a_kcontig=akc, b_kcontig=bkc, bias=bias.data_ptr() if use_bias else None,
                     c_in=cin.data_ptr() if use_cin else None, ld_cin=n, relu=relu)
        torch.cuda.synchronize()
        what = f"case {case}: {dtype} m {m} n {n} k {k} akc {akc} bkc {bkc} bias {use_bias} cin {use_cin} relu {relu}"
        assert not torch.isnan(out).any(), what
        assert rel_err(out, ref) <= TOL[dtype], what


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("akc", [True, False])
@pytest.mark.parametrize("m,k,ksegs", [(1024, 2048, 1), (1000, 520, 1), (1024, 264, 2)])
def test_gemm_128x160_tile_path(akc, dtype, m, k, ksegs):
    """Shards 1280 columns wide (the LM's logits layer) take 128 x 160 tiles -- 4 x 1 wave tiles of 32 x 160 -- for a
    K-contiguous second operand: 8 groups of 8 x 8 tiles fill the CUs in two even rounds (checked by the kernel's name
    in the launch records).  Grouped, with bias, ReLU and an addend, ragged rows, a ragged last slab and K segments."""
    from rtp_amd import _lib
    ops = _ops()
    gen = torch.Generator().manual_seed(m + k)
    groups, n_s = 8, 1280
    n = groups * n_s
    a = _rand((m, k * ksegs) if akc else (k * ksegs, m), dtype, gen).to(DEV)
    b = _rand((n, k * ksegs), dtype, gen).to(DEV)
    bias, cin = _rand((n,), dtype, gen).to(DEV), _rand((m, n), dtype, gen).to(DEV)
    A = a.float() if akc else a.float().t()
    ref = torch.relu(A @ b.float().t() + bias.float() + cin.float())
    out = torch.full((m, n), float("nan"), dtype=dtype, device=DEV)
    es = a.element_size()
    _lib.profile_enable(1)
    try:
        ops.gemm_raw(dtype, a=a.data_ptr(), b=b.data_ptr(), c_out=out.data_ptr(), m=m, n=n_s, k=k, lda=a.stride(0),
                     ldb=b.stride(0), ldc=n, a_kcontig=akc, b_kcontig=True, bias=bias.data_ptr(), c_in=cin.data_ptr(),
                     ld_cin=n, relu=True, groups=groups, b_sg=n_s * k * ksegs, c_sg=n_s, cin_sg=n_s, bias_sg=n_s,
                     ksegs=ksegs, a_sk=k if akc else k * m, b_sk=k)
        torch.cuda.synchronize()
        names = list(_lib.profile_collect())
    finally:
        _lib.profile_enable(0)
    assert any("128x160" in nm for nm in names), names
    assert rel_err(out, ref) <= TOL[dtype]
