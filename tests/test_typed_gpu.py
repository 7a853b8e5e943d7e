"""Typed GEMM (MFMA), relation segmentation, pad_rel and the fused RGCN op
through cxgnncomp_backend vs the oracle.

Every fp32 test runs four times: with the fp32 MFMA kernel ("fp32"), with the
default three-product split of scaled fp16 parts ("split_f16", 2^-21 per product) and
with the six-product bf16 split ("split6", 2^-24) at 1e-4 relative /
1e-5 absolute at O(1) output scale, and with the three-product bf16 split ("split3":
operands keep 16 significant bits and the lo*lo product is dropped, so each
product is off by at most 3 * 2^-18 = 1.1e-5 relative; over K <= 256 terms of
an O(1) row that is 1e-4 relative / 4e-5 absolute, stated here and checked
below).
bf16 MFMA path (stated tolerance): operands are rounded to bf16 (8 significant
bits), products accumulate in fp32; against the oracle run on the same
bf16-rounded operands the bound is the fp32 one, against the unrounded fp32
oracle it is 2e-2 relative to the row scale."""
import numpy as np
import pytest
import torch

import oracle
from conftest import announce, assert_close

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-4, 1e-5


@pytest.fixture(autouse=True, params=["fp32", "split_f16", "split6", "split3"])
def gemm_precision(request):
    """Runs every test of this file under both multiplication modes; ATOL follows."""
    from cxgnncomp_backend import _typed
    global ATOL
    old = _typed.GEMM_PRECISION
    _typed.GEMM_PRECISION = request.param
    ATOL = 4e-5 if request.param == "split3" else 1e-5
    yield request.param
    _typed.GEMM_PRECISION = old
    ATOL = 1e-5


def _np(t):
    return t.detach().cpu().numpy()


@pytest.mark.parametrize("dtype", [torch.int32, torch.int64])
@pytest.mark.parametrize("n,R", [(0, 3), (1, 1), (1000, 7), (50000, 16), (777, 40)])
def test_rel_segment_bit_exact(dtype, n, R):
    from cxgnncomp_backend import _typed
    g = torch.Generator().manual_seed(n + R)
    types = torch.randint(0, R + 1, (n,), generator=g).to(dtype)   # value R = padding sentinel
    announce("rel_segment n=%d R=%d %s" % (n, R, dtype))
    perm, seg = _typed.rel_segment(types.cuda(), R)
    t = types.numpy().astype(np.int64)
    want_perm = np.argsort(t, kind="stable")
    want_seg = np.searchsorted(t[want_perm], np.arange(R + 1), side="left")
    assert np.array_equal(_np(perm), want_perm)
    assert np.array_equal(_np(seg), want_seg)


SHAPES = [(128, 128, 16, 5000), (64, 64, 3, 1000), (32, 40, 4, 700), (96, 47, 5, 900),
          (128, 256, 2, 300), (256, 128, 7, 2000), (64, 200, 1, 130), (128, 16, 6, 999)]


def _typed_problem(K, N, R, M, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g) / K ** 0.5
    w = torch.randn(R, K, N, generator=g)
    p = torch.arange(1, R + 1, dtype=torch.float64) ** -1.2
    types = torch.multinomial(p, M, replacement=True, generator=g).to(torch.int32)
    if R > 2:
        types[types == 1] = 0                     # one empty relation
    return x, w, types


@pytest.mark.parametrize("K,N,R,M", SHAPES)
def test_typed_linear_f32(K, N, R, M):
    import cxgnncomp_backend as B
    x, w, types = _typed_problem(K, N, R, M, K + N + R)
    base = torch.randn(M, N) / 8
    out = base.clone().cuda()
    announce("typed_linear K=%d N=%d R=%d M=%d" % (K, N, R, M))
    B.typed_linear(x.cuda(), w.cuda(), out, types.cuda(), 32)
    torch.cuda.synchronize()
    ref = oracle.typed_linear(x.numpy(), w.numpy(), types.numpy(), out=base.numpy())
    assert_close(_np(out), ref, RTOL, 2 * ATOL, "typed_linear")


@pytest.mark.parametrize("K,N,R,M", SHAPES[:4])
def test_typed_linear_s2e_s2d(K, N, R, M):
    import cxgnncomp_backend as B
    x, w, types = _typed_problem(K, N, R, M, 3 * K + N)
    n_src, n_dst = 300, 150
    g = torch.Generator().manual_seed(1)
    xs = torch.randn(n_src, K, generator=g) / K ** 0.5
    src = torch.randint(0, n_src, (M,), generator=g)
    dst = torch.randint(0, n_dst, (M,), generator=g)
    out = torch.zeros(M, N).cuda()
    announce("typed_linear_s2e K=%d N=%d R=%d M=%d" % (K, N, R, M))
    B.typed_linear_s2e(xs.cuda(), w.cuda(), out, src.cuda(), types.cuda(), 32)
    ref = oracle.typed_linear(xs.numpy(), w.numpy(), types.numpy(), src=src.numpy(), n_out=M)
    assert_close(_np(out), ref, RTOL, ATOL, "s2e")
    out2 = torch.zeros(n_dst, N).cuda()
    announce("typed_linear_s2d K=%d N=%d R=%d M=%d" % (K, N, R, M))
    B.typed_linear_s2d(xs.cuda(), w.cuda(), out2, src.cuda(), dst.cuda(), types.cuda(), 32)
    ref2 = oracle.typed_linear(xs.numpy(), w.numpy(), types.numpy(), src=src.numpy(), dst=dst.numpy(),
                               n_out=n_dst)
    scale = max(1.0, float(np.abs(ref2).max()))
    assert_close(_np(out2) / scale, ref2 / scale, RTOL, ATOL, "s2d")


@pytest.mark.parametrize("K,N,R,M", [(128, 128, 16, 5000), (64, 64, 3, 1000), (96, 40, 4, 700),
                                     (256, 128, 7, 2000)])
def test_typed_gemm_bf16(K, N, R, M):
    from cxgnncomp_backend import _typed
    x, w, types = _typed_problem(K, N, R, M, 5 * K + N)
    perm, seg = _typed.rel_segment(types.cuda(), R)
    announce("typed_gemm bf16 K=%d N=%d R=%d M=%d" % (K, N, R, M))
    out = _typed.typed_gemm(x.cuda(), w.cuda(), seg, M, src_idx=perm, dst_idx=perm, bf16=True)
    torch.cuda.synchronize()
    xr = x.to(torch.bfloat16).float().numpy()
    wr = w.to(torch.bfloat16).float().numpy()
    ref_rounded = oracle.typed_linear(xr, wr, types.numpy())
    assert_close(_np(out), ref_rounded, RTOL, 2 * ATOL, "bf16 vs oracle on bf16-rounded operands")
    ref = oracle.typed_linear(x.numpy(), w.numpy(), types.numpy())
    scale = np.abs(ref).max()
    assert np.abs(_np(out) - ref).max() <= 2e-2 * scale, "bf16 vs fp32 oracle"


@pytest.mark.parametrize("thres", [256, 32, 2])
def test_pad_rel_bit_exact(thres):
    import cxgnncomp_backend as B
    R, n = 9, 5000
    g = torch.Generator().manual_seed(thres)
    types = torch.randint(0, R - 1, (n,), generator=g)          # highest id absent
    count = torch.bincount(types, minlength=R)
    new_types = torch.full((n + R * (thres - 1),), -7, dtype=torch.int64)
    new_types[:n] = types
    new_idx = torch.full_like(new_types, -9)
    new_idx[:n] = torch.arange(n)
    a = new_types.clone().cuda()
    announce("pad_rel thres=%d" % thres)
    B.pad_rel(a, count.cuda(), thres, R, n)
    want = oracle.pad_rel(new_types.numpy(), count.numpy(), thres, R, n)
    assert np.array_equal(_np(a), want)
    a2, i2 = new_types.clone().cuda(), new_idx.clone().cuda()
    announce("pad_rel_idx thres=%d" % thres)
    B.pad_rel_idx(a2, i2, count.cuda(), thres, R, n)
    want_r, want_i = oracle.pad_rel(new_types.numpy(), count.numpy(), thres, R, n, idx=new_idx.numpy())
    assert np.array_equal(_np(a2), want_r) and np.array_equal(_np(i2), want_i)
    # each relation's padded count is a multiple of thres (what the padding is for)
    padded = np.bincount(_np(a), minlength=R + 1)[:R]
    assert (padded % thres == 0).all()


def test_rgcn_fused_toy_all_ones():
    """example/prof_rgcn.py:22-51: x = ones[128,128], W = ones, one row with 31
    neighbours -> every output element is 31 * 128 = 3968."""
    import cxgnncomp_backend as B
    ptr = torch.tensor([0, 31])
    idx = torch.arange(1, 32)
    rel = (torch.arange(31) % 7).int()
    x = torch.ones(128, 128)
    w = torch.ones(7, 128, 128)
    announce("rgcn fused toy")
    out = B.aggr_rgcn_direct_func(x.cuda(), ptr.cuda(), idx.cuda(), w.cuda(), rel.cuda(), 1)
    assert out.shape == (1, 128)
    assert torch.all(out.cpu() == 3968.0)


@pytest.mark.parametrize("strategy", ["transform_first", "pair_rows", "per_edge_rows", "gather_gemm_scatter"])
@pytest.mark.parametrize("K,N,R", [(128, 128, 16), (64, 32, 3)])
def test_rgcn_fused_forward_backward(K, N, R, strategy, monkeypatch):
    """The four strategies of the fused relational layer: dense transform of every (node,
    relation) pair, transform of the pairs that own an edge, one GEMM row per edge summed per
    destination, atomic scatter."""
    import cxgnncomp_backend as B
    from cxgnncomp import synthetic as S
    from cxgnncomp_backend import _typed
    if strategy not in ("transform_first", "pair_rows"):
        monkeypatch.setattr(_typed, "RGCN_DENSE_MAX_BYTES", 0)    # rules the transform-first paths out
    if strategy == "gather_gemm_scatter":
        monkeypatch.setattr(_typed, "RGCN_EDGE_ROWS_MAX_BYTES", 0)   # and the per-edge rows
    # the share of pairs that own an edge decides between the dense table and the compacted one
    monkeypatch.setattr(_typed, "RGCN_PAIR_FILL_MAX", 2.0 if strategy == "pair_rows" else -1.0)
    assert _typed._use_dense(40000, 3000, R, N) == (strategy in ("transform_first", "pair_rows"))
    ptr, idx, etype, _ = S.hetero_graph(3000, 40000, num_rel=R, seed=4)
    n = ptr.shape[0] - 1
    torch.manual_seed(14)
    x = torch.randn(n, K) / (K ** 0.5 * 4)
    w = torch.randn(R, K, N) * 0.5
    g = torch.randn(n, N) / 4
    xg = x.cuda().requires_grad_(True)
    wg = w.cuda().requires_grad_(True)
    rel = etype.int()
    announce("aggr_rel_direct K=%d N=%d R=%d %s" % (K, N, R, strategy))
    out = B.aggr_rel_direct(xg, ptr.cuda(), idx.cuda(), wg, rel.cuda(), n, R)
    out.backward(g.cuda())
    torch.cuda.synchronize()
    ref = oracle.rgcn_fused(x.numpy(), ptr.numpy(), idx.numpy(), w.numpy(), rel.numpy(), n)
    assert_close(_np(out), ref, RTOL, 2 * ATOL, "rgcn fused fwd")
    # gradients from autograd through the pure-torch restatement in float64
    from oracle import pyref
    x64 = x.double().requires_grad_(True)
    w64 = w.double().requires_grad_(True)
    o64 = pyref.typed_linear_s2d_sort(x64, w64, ptr, idx, etype, n)
    o64.backward(g.double())
    # absolute bounds are stated at O(1) output scale: rows here sum ~13 edge terms of size ~1.4
    scx = max(1.0, float(x64.grad.abs().max()))
    assert_close(_np(xg.grad) / scx, x64.grad.numpy() / scx, RTOL, 2 * ATOL, "grad x")
    sc = float(w64.grad.abs().max())
    assert_close(_np(wg.grad) / sc, w64.grad.numpy() / sc, RTOL, 2 * ATOL, "grad w")
    announce("seastar fwd/bwd K=%d" % K)
    so = B.seastar_forward(x.cuda(), ptr.cuda(), idx.cuda(), w.cuda(), etype.cuda())
    assert_close(_np(so), ref, RTOL, 2 * ATOL, "seastar fwd")
    sgx, sgw = B.seastar_backward(x.cuda(), ptr.cuda(), idx.cuda(), w.cuda(), etype.cuda(), g.cuda())
    assert_close(_np(sgx) / scx, x64.grad.numpy() / scx, RTOL, 2 * ATOL, "seastar grad x")


@pytest.mark.parametrize("K,N,R,M", [(128, 128, 16, 5000), (64, 48, 3, 1000), (4, 256, 1, 3000), (128, 2048, 1, 700),
                                     (32, 40, 4, 70000), (12, 20, 5, 1), (256, 128, 5, 3000), (200, 64, 1, 900),
                                     (256, 47, 1, 1024), (64, 5, 3, 2000)])
def test_typed_gemm_wgrad(K, N, R, M):
    """gw[r] = sum over the rows of relation r of a[src]^T (x) g[dst], against per-relation
    float64 products; covers several column tiles (N = 2048), K far below one tile (K = 4),
    K above one launch's 128 (in slices, one and several relations), many row chunks (M = 70000),
    N that is not a multiple of 4 (padded copy of g) and relations without rows."""
    from cxgnncomp_backend import _typed
    gen = torch.Generator().manual_seed(K + N + M)
    n_a, n_g = max(1, M // 2), max(1, M // 3)
    a = torch.randn(n_a, K, generator=gen)
    g = torch.randn(n_g, N, generator=gen) / max(1.0, (M / R) ** 0.5)
    src = torch.randint(0, n_a, (M,), generator=gen)
    dst = torch.randint(0, n_g, (M,), generator=gen)
    types = torch.randint(0, R, (M,), generator=gen).int()
    if R > 2:
        types[types == 1] = 0
    perm, seg = _typed.rel_segment(types.cuda(), R)
    announce("typed_gemm_wgrad K=%d N=%d R=%d M=%d" % (K, N, R, M))
    gw = _typed.typed_gemm_wgrad(a.cuda(), g.cuda(), seg, M, R, src_idx=src.cuda()[perm], dst_idx=dst.cuda()[perm])
    assert gw is not None and gw.shape == (R, K, N)
    want = torch.zeros(R, K, N, dtype=torch.float64)
    for r in range(R):
        m = types == r
        want[r] = a[src[m]].double().t() @ g[dst[m]].double()
    assert_close(_np(gw), want.numpy(), RTOL, 2 * ATOL, "wgrad")
    again = _typed.typed_gemm_wgrad(a.cuda(), g.cuda(), seg, M, R, src_idx=src.cuda()[perm], dst_idx=dst.cuda()[perm])
    assert torch.equal(gw, again)                                   # deterministic
    assert _typed.typed_gemm_wgrad(torch.zeros(4, 130).cuda(), g.cuda(), seg, 0, R) is None   # K not a multiple of 4: not taken


@pytest.mark.parametrize("K,N", [(128, 128), (64, 96), (20, 40)])
def test_typed_gemm_scaled_fp16_dynamic_range(K, N):
    """The three-product form on scaled fp16 parts keeps fp32-grade accuracy whatever the scale of
    a row or of a weight column: rows spread over e^+-9, elements inside a row over e^+-4.5, rows
    at 1e-30 and 1e+15, all-zero rows, weight columns over e^+-9.  The error of every output is
    bounded against sum_k |x||w| of its dot product -- what the rounding of an fp32 product chain is
    relative to -- with 2e-6 (fp32 MFMA: 9e-7 on this input, six bf16 products: 6e-7, three bf16
    products: 2e-5).  An infinity in a row makes that row non-finite, as in fp32."""
    from cxgnncomp_backend import _typed
    M, R = 6000, 3
    gen = torch.Generator().manual_seed(K * N)
    x = torch.randn(M, K, generator=gen)
    x *= torch.exp(torch.randn(M, 1, generator=gen) * 3)
    x *= torch.exp(torch.randn(M, K, generator=gen) * 1.5)
    x[:50] = 0
    x[50:100] *= 1e-30
    x[100:150] *= 1e15
    w = torch.randn(R, K, N, generator=gen) * torch.exp(torch.randn(R, 1, N, generator=gen) * 3)
    w[1, :, 3] = 0                                                  # an all-zero weight column
    seg = torch.tensor([0, 2500, 2501, M], dtype=torch.int64)
    announce("typed_gemm split_f16 dynamic range K=%d N=%d" % (K, N))
    out = _typed.typed_gemm(x.cuda(), w.cuda(), seg.cuda(), M, precision="split_f16").cpu().double()
    ref = torch.empty(M, N, dtype=torch.float64)
    mag = torch.empty(M, N, dtype=torch.float64)
    for r in range(R):
        b, e = int(seg[r]), int(seg[r + 1])
        ref[b:e] = x[b:e].double() @ w[r].double()
        mag[b:e] = x[b:e].double().abs() @ w[r].double().abs()
    assert torch.isfinite(out).all()
    assert torch.equal(out[:50], torch.zeros(50, N, dtype=torch.float64))
    # rows whose largest magnitude is an fp32 denormal (below 2^-112 here: the 1e-30 rows times
    # e^-9) are treated as zero rows; everything else obeys the bound
    err = (out - ref).abs()
    ok = err <= 2e-6 * mag + 1e-33
    assert ok.all(), "worst error / sum|x||w| = %.3e" % float((err / mag.clamp_min(1e-300))[~ok].max())
    xi = x.clone()
    xi[7, 5] = float("inf")
    bad = _typed.typed_gemm(xi.cuda(), w.cuda(), seg.cuda(), M, precision="split_f16").cpu()
    assert not torch.isfinite(bad[7]).any() or (w[0, 5] == 0).any()
    assert torch.isfinite(bad[8]).all()


@pytest.mark.parametrize("K,N,M", [(128, 128, 30000), (64, 96, 9000), (20, 40, 5000)])
def test_typed_gemm_wgrad_scaled_fp16_dynamic_range(K, N, M):
    """The weight gradient on scaled fp16 parts: its scales depend on the column group only and
    follow the largest magnitude met so far in the chunk, so rows of very different size share a
    scale.  Rows spread over e^+-9 (both operands, independently), elements over e^+-3, blocks of
    all-zero rows, the first rows tiny (the scales have to grow inside a chunk): the error of
    every gw element is bounded against sum_i |a||g| of its reduction with 4e-6 (measured 6e-7;
    six bf16 products: 5e-7, three bf16 products: 2e-5 on this input)."""
    from cxgnncomp_backend import _typed
    R = 3
    gen = torch.Generator().manual_seed(K + N + M)
    a = torch.randn(M, K, generator=gen) * torch.exp(torch.randn(M, 1, generator=gen) * 3)
    a *= torch.exp(torch.randn(M, K, generator=gen))
    g = torch.randn(M, N, generator=gen) * torch.exp(torch.randn(M, 1, generator=gen) * 3)
    g *= torch.exp(torch.randn(M, N, generator=gen))
    a[:300] *= 1e-12
    g[:300] *= 1e-9
    a[1000:1400] = 0
    g[1200:1500] = 0
    seg = torch.tensor([0, M // 2, M // 2 + 1, M], dtype=torch.int64)
    announce("typed_gemm_wgrad split_f16 dynamic range K=%d N=%d M=%d" % (K, N, M))
    gw = _typed.typed_gemm_wgrad(a.cuda(), g.cuda(), seg.cuda(), M, R, precision="split_f16")
    assert gw is not None and bool(torch.isfinite(gw).all())
    gw = gw.cpu().double()
    for r in range(R):
        b, e = int(seg[r]), int(seg[r + 1])
        want = a[b:e].double().t() @ g[b:e].double()
        mag = a[b:e].double().abs().t() @ g[b:e].double().abs()
        err = (gw[r] - want).abs()
        ok = err <= 4e-6 * mag + 1e-30
        assert ok.all(), "relation %d: worst error / sum|a||g| = %.3e" % (r, float((err / mag.clamp_min(1e-300))[~ok].max()))


def test_typed_gemm_wgrad_scaled_fp16_columns_of_different_scale():
    """The weight gradient's fp16 parts share one power-of-two scale per group of 32 columns, so a
    column far below the largest column of its group keeps fewer significant bits: the two parts
    of a scaled value resolve 2^-24 absolute, i.e. 2^-37 of the group's largest magnitude with the
    three bits of headroom.  Columns at 1, 2^-10, 2^-20 and 2^-30 of their group's scale, in
    either operand: down to 2^-20 every gw element stays within 4e-6 of sum_i |a||g| of its own
    reduction (measured 1.5e-7); at 2^-30 the bound is 2^-37 / 2^-30 = 8e-3 per product and 5e-4
    is asserted on the sum (measured 1.4e-4).  The six-product bf16 form carries no shared scale
    and stays at 2e-8 for every column (asserted at 4e-7)."""
    from cxgnncomp_backend import _typed
    K, N, M, R = 128, 128, 30000, 2
    gen = torch.Generator().manual_seed(1)
    ea = torch.tensor([0, 10, 20, 30])[torch.arange(K) % 4]
    eg = torch.tensor([0, 10, 20, 30])[(torch.arange(N) // 2) % 4]
    a = torch.randn(M, K, generator=gen) * torch.exp2(-ea.float())
    g = torch.randn(M, N, generator=gen) * torch.exp2(-eg.float())
    seg = torch.tensor([0, M // 2, M], dtype=torch.int64)
    low = torch.maximum(ea[:, None], eg[None, :])
    for precision, bound_near, bound_far in (("split_f16", 4e-6, 5e-4), ("split6", 4e-7, 4e-7)):
        announce("typed_gemm_wgrad %s, columns at 2^0..2^-30 of their group's scale" % precision)
        gw = _typed.typed_gemm_wgrad(a.cuda(), g.cuda(), seg.cuda(), M, R, precision=precision).cpu().double()
        for r in range(R):
            b, e = int(seg[r]), int(seg[r + 1])
            want = a[b:e].double().t() @ g[b:e].double()
            mag = a[b:e].double().abs().t() @ g[b:e].double().abs()
            rel = (gw[r] - want).abs() / mag
            assert float(rel[low <= 20].max()) <= bound_near, (precision, float(rel[low <= 20].max()))
            assert float(rel[low == 30].max()) <= bound_far, (precision, float(rel[low == 30].max()))


@pytest.mark.parametrize("M", [1, 63, 64, 65, 1100])
@pytest.mark.parametrize("K,N", [(128, 128), (4, 4), (36, 72), (256, 96)])
def test_typed_gemm_small_shapes_and_skipped_rows(M, K, N):
    """Row counts around one 64-row tile and past one block's 16 mapped tiles, K and N far below
    and above a tile, and row maps with negative entries (a negative source or destination skips
    the row, which is how the reference's padded layouts are accepted): forward product into
    scattered rows and the weight gradient, against float64."""
    from cxgnncomp_backend import _typed
    R = 3
    gen = torch.Generator().manual_seed(M * 1000 + K + N)
    n_a = 2 * M + 3
    a = torch.randn(n_a, K, generator=gen) / K ** 0.5
    w = torch.randn(R, K, N, generator=gen)
    types = torch.sort(torch.randint(0, R, (M,), generator=gen))[0]
    seg = torch.zeros(R + 1, dtype=torch.int64)
    seg[1:] = torch.bincount(types, minlength=R).cumsum(0)
    src = torch.randint(0, n_a, (M,), generator=gen)
    dst = torch.randperm(M + 5, generator=gen)[:M]                  # unique destinations
    skip = torch.rand(M, generator=gen) < 0.2
    src_m = torch.where(skip & (torch.arange(M) % 2 == 0), torch.full_like(src, -1), src)
    dst_m = torch.where(skip & (torch.arange(M) % 2 == 1), torch.full_like(dst, -7), dst)
    announce("typed_gemm M=%d K=%d N=%d with skipped rows" % (M, K, N))
    out = torch.full((M + 5, N), 3.0).cuda()
    _typed.typed_gemm(a.cuda(), w.cuda(), seg.cuda(), M, src_idx=src_m.cuda(), dst_idx=dst_m.cuda(), out=out)
    want = torch.full((M + 5, N), 3.0, dtype=torch.float64)
    for i in range(M):
        if not bool(skip[i]):
            want[dst[i]] = a[src[i]].double() @ w[types[i]].double()
    assert_close(_np(out), want.numpy(), RTOL, 2 * ATOL, "typed_gemm with skipped rows")
    # the same rows added to what is there (the read-add-store paths), twice in a row
    acc = torch.full((M + 5, N), 3.0).cuda()
    for _ in range(2):
        _typed.typed_gemm(a.cuda(), w.cuda(), seg.cuda(), M, src_idx=src_m.cuda(), dst_idx=dst_m.cuda(), out=acc,
                          accumulate=True)
    want_acc = torch.full((M + 5, N), 3.0, dtype=torch.float64)      # 3 + 2 * product on the rows that exist
    for i in range(M):
        if not bool(skip[i]):
            want_acc[dst[i]] += 2 * want[dst[i]]
    assert_close(_np(acc), want_acc.numpy(), RTOL, 4 * ATOL, "typed_gemm accumulate with skipped rows")
    g = torch.randn(M + 5, N, generator=gen)
    gw = _typed.typed_gemm_wgrad(a.cuda(), g.cuda(), seg.cuda(), M, R, src_idx=src_m.cuda(), dst_idx=dst_m.cuda())
    want_gw = torch.zeros(R, K, N, dtype=torch.float64)
    for i in range(M):
        if not bool(skip[i]):
            want_gw[types[i]] += torch.outer(a[src[i]].double(), g[dst[i]].double())
    scale = max(1.0, float(want_gw.abs().max()))
    assert_close(_np(gw) / scale, want_gw.numpy() / scale, RTOL, 2 * ATOL, "wgrad with skipped rows")


@pytest.mark.parametrize("M,K,N,R", [(5000, 128, 128, 1), (4097, 64, 200, 1), (9000, 36, 72, 3), (70, 128, 256, 2),
                                     (120000, 256, 128, 1), (6000, 200, 96, 2)])
@pytest.mark.parametrize("with_bias,with_addend", [(True, False), (False, True), (True, True)])
def test_typed_gemm_epilogue_bias_and_addend(M, K, N, R, with_bias, with_addend, gemm_precision):
    """cxg_typed_gemm_epilogue_f32 through the C ABI: per-relation bias rows and an addend with
    a row stride wider than N are added before the store; against float64, and against the
    plain entry point followed by the two additions (same products, so the same bits up to the
    order of the last two additions)."""
    from cxgnncomp_backend import _lib, _typed
    if gemm_precision != "split_f16":
        pytest.skip("the entry point takes its form from its flags: runs once")
    lib = _lib.load()
    gen = torch.Generator().manual_seed(M + K + N + R)
    a = (torch.randn(M, K, generator=gen) / K ** 0.5).cuda()
    w = torch.randn(R, K, N, generator=gen).cuda()
    cuts = torch.sort(torch.randint(0, M + 1, (R - 1,), generator=gen))[0]
    seg = torch.cat([torch.zeros(1, dtype=torch.int64), cuts, torch.tensor([M])]).cuda()
    bias = torch.randn(R, N, generator=gen).cuda() if with_bias else None
    ldd = N + 12
    addend_buf = torch.randn(M, ldd, generator=gen).cuda() if with_addend else None
    out = torch.full((M, N), 7.0).cuda()
    announce("typed_gemm_epilogue M=%d K=%d N=%d R=%d bias=%s addend=%s" % (M, K, N, R, with_bias, with_addend))
    st = lib.cxg_typed_gemm_epilogue_f32(a.data_ptr(), K, w.data_ptr(), _lib.ptr(bias), _lib.ptr(addend_buf), ldd,
                                         out.data_ptr(), N, None, None, seg.data_ptr(), M, K, N, R,
                                         _typed.GEMM_SPLIT_F16X3, _lib.current_stream(a.device))
    _lib.check(st)
    torch.cuda.synchronize()
    seg_h = seg.cpu().tolist()
    want = torch.empty(M, N, dtype=torch.float64)
    for r in range(R):
        lo, hi = seg_h[r], seg_h[r + 1]
        want[lo:hi] = a[lo:hi].double().cpu() @ w[r].double().cpu()
        if with_bias:
            want[lo:hi] += bias[r].double().cpu()
    if with_addend:
        want += addend_buf[:, :N].double().cpu()
    assert_close(_np(out), want.numpy(), RTOL, 2 * ATOL, "typed_gemm_epilogue")
    plain = _typed.typed_gemm(a, w, seg, M, precision="split_f16")
    if with_bias:
        plain = plain + bias[torch.bucketize(torch.arange(M, device="cuda"), seg[1:], right=True)]
    if with_addend:
        plain = plain + addend_buf[:, :N]
    assert float((plain - out).abs().max()) <= 4e-6 * float(want.abs().max())


def test_typed_gemm_epilogue_rejects_what_it_does_not_take(gemm_precision):
    """Row maps, the atomic flag, precisions other than the fp16 split and a short addend stride
    are refused with an error code and nothing is written."""
    from cxgnncomp_backend import _lib, _typed
    lib = _lib.load()
    M, K, N = 256, 64, 64
    a = torch.randn(M, K).cuda()
    w = torch.randn(1, K, N).cuda()
    seg = torch.tensor([0, M], dtype=torch.int64).cuda()
    idx = torch.arange(M, dtype=torch.int64).cuda()
    bias = torch.randn(1, N).cuda()
    out = torch.full((M, N), 7.0).cuda()

    def call(flags, src=None, dst=None, addend=None, ldd=N):
        return lib.cxg_typed_gemm_epilogue_f32(a.data_ptr(), K, w.data_ptr(), bias.data_ptr(), _lib.ptr(addend), ldd,
                                               out.data_ptr(), N, _lib.ptr(src), _lib.ptr(dst), seg.data_ptr(),
                                               M, K, N, 1, flags, _lib.current_stream(a.device))
    if gemm_precision != "fp32":
        pytest.skip("independent of the default precision: runs once")
    announce("typed_gemm_epilogue argument checks")
    assert call(_typed.GEMM_SPLIT_F16X3, src=idx) != 0
    assert call(_typed.GEMM_SPLIT_F16X3, dst=idx) != 0
    assert call(0) != 0
    assert call(_typed.GEMM_SPLIT_F16X3 | 1) != 0
    assert call(_typed.GEMM_SPLIT_F16X3 | 2) != 0
    assert call(_typed.GEMM_SPLIT_F16X3, addend=out, ldd=N - 4) != 0
    torch.cuda.synchronize()
    assert bool((out == 7.0).all())
    assert call(_typed.GEMM_SPLIT_F16X3) == 0


@pytest.mark.parametrize("M,K,N", [(5000, 128, 256), (4096, 100, 64), (130000, 256, 256)])
def test_dense_linear_helpers_match_library(M, K, N):
    """dense_linear / dense_linear_add_ (what LinearOP, SageLayerOP and GatLayerOP call) against
    float64 F.linear; shapes they do not take return None / False and write nothing."""
    from cxgnncomp_backend import _typed
    gen = torch.Generator().manual_seed(M + K)
    x = (torch.randn(M, K, generator=gen) / K ** 0.5).cuda()
    w = torch.randn(N, K, generator=gen).cuda()                    # nn.Linear layout [out, in]
    b = torch.randn(N, generator=gen).cuda()
    add = torch.randn(M, N, generator=gen).cuda()
    announce("dense_linear M=%d K=%d N=%d" % (M, K, N))
    want = x.double() @ w.double().t() + b.double()
    got = _typed.dense_linear(x, w.t(), b)
    if _typed.GEMM_PRECISION != "split_f16":             # only the default form has the epilogue
        assert got is None and not _typed.dense_linear_add_(add.clone(), x, w.t())
        return
    assert got is not None
    assert_close(_np(got), _np(want), RTOL, 2 * ATOL, "dense_linear bias")
    got = _typed.dense_linear(x, w.t(), b, add)
    assert_close(_np(got), _np(want + add.double()), RTOL, 2 * ATOL, "dense_linear bias addend")
    acc = add.clone()
    assert _typed.dense_linear_add_(acc, x, w.t())
    assert_close(_np(acc), _np(want - b.double() + add.double()), RTOL, 2 * ATOL, "dense_linear_add_")
    acc = add[:100].clone()
    assert not _typed.dense_linear_add_(acc, x[:100], w.t())         # too few rows: nothing written
    assert torch.equal(acc, add[:100])
    assert _typed.dense_linear(x[:100], w.t(), b) is None
    assert _typed.dense_linear(x.double(), w.t().double(), b.double()) is None


@pytest.mark.parametrize("M,H,K,C", [(70001, 4, 128, 64), (5003, 2, 100, 32), (8192, 8, 24, 16), (9000, 4, 36, 20),
                                     (300, 4, 128, 64), (6000, 4, 132, 64)])
def test_dense_linear_heads(M, H, K, C):
    """dense_linear_heads (the per-head products after GatLayerOP's aggregation of the input rows):
    out[:, h*C:(h+1)*C] = x[:, h, :] @ W_h^T (+ bias) against float64, on shapes the split GEMM
    takes (one launch per head over strided rows) and on shapes that go through torch.bmm."""
    from cxgnncomp_backend import _typed
    gen = torch.Generator().manual_seed(M + K)
    x = (torch.randn(M, H, K, generator=gen) / K ** 0.5).cuda()
    w = torch.randn(H * C, K, generator=gen).cuda()
    b = torch.randn(H * C, generator=gen).cuda()
    want = torch.einsum("mhk,hck->mhc", x.double(), w.double().view(H, C, K)).reshape(M, H * C)
    announce("dense_linear_heads M=%d H=%d K=%d C=%d" % (M, H, K, C))
    got = _typed.dense_linear_heads(x, w, b)
    assert got.shape == (M, H * C)
    assert_close(_np(got), _np(want + b.double()), RTOL, 2 * ATOL, "per-head products with bias")
    got = _typed.dense_linear_heads(x, w)
    assert_close(_np(got), _np(want), RTOL, 2 * ATOL, "per-head products")


def test_linear_op_gradients_through_typed_gemm():
    """LinearOP on a shape dense_linear takes: output and the three gradients against float64
    autograd of F.linear."""
    from cxgnncomp.graph_conv import LinearOP
    gen = torch.Generator().manual_seed(5)
    M, K, N = 6000, 128, 64
    x = (torch.randn(M, K, generator=gen) / K ** 0.5).cuda().requires_grad_()
    w = torch.randn(N, K, generator=gen).cuda().requires_grad_()
    b = torch.randn(N, generator=gen).cuda().requires_grad_()
    g = torch.randn(M, N, generator=gen).cuda()
    announce("LinearOP fwd+bwd M=%d K=%d N=%d" % (M, K, N))
    y = LinearOP.apply(x, w, b)
    y.backward(g)
    xd, wd, bd = (t.detach().double().requires_grad_() for t in (x, w, b))
    yd = torch.nn.functional.linear(xd, wd, bd)
    yd.backward(g.double())
    assert_close(_np(y), _np(yd), RTOL, 2 * ATOL, "LinearOP forward")
    for name, got, want in (("x", x.grad, xd.grad), ("w", w.grad, wd.grad), ("b", b.grad, bd.grad)):
        scale = max(1.0, float(want.abs().max()))
        assert_close(_np(got) / scale, _np(want) / scale, RTOL, 2 * ATOL, "LinearOP grad " + name)


def test_typed_gemm_random_shapes_all_store_paths(gemm_precision):
    """120 seeded random shapes (M up to 5000, K up to 256, N up to 300, 1 - 5 relations) through
    every way a row can leave the kernel: plain, accumulating, with row maps and skipped rows,
    with bias and / or addend through the epilogue entry point; each against float64."""
    import random
    from cxgnncomp_backend import _lib, _typed
    if gemm_precision != "split_f16":
        pytest.skip("the store paths are those of the default form: runs once")
    lib = _lib.load()
    rnd = random.Random(1)
    gen = torch.Generator().manual_seed(1)
    announce("typed_gemm random shapes")
    for case in range(120):
        M = rnd.choice([1, 7, 63, 64, 65, 200, 1023, 1100, 2049, 5000])
        K = rnd.choice([4, 8, 36, 64, 100, 128, 176, 200, 256])
        N = rnd.choice([4, 32, 40, 64, 96, 100, 128, 132, 200, 256, 300])
        R = rnd.choice([1, 1, 2, 5])
        mode = rnd.choice(["plain", "acc", "bias", "addend", "bias+addend", "mapped", "mapped_acc"])
        if mode in ("bias", "addend", "bias+addend") and K > 128 and not (K >= 176 and N >= 96):
            continue
        n_a = M + 3
        a = (torch.randn(n_a, K, generator=gen) / K ** 0.5).cuda()
        w = torch.randn(R, K, N, generator=gen).cuda()
        cuts = sorted(rnd.randint(0, M) for _ in range(R - 1))
        seg = torch.tensor([0] + cuts + [M], dtype=torch.int64).cuda()
        rel = torch.bucketize(torch.arange(M, device="cuda"), seg[1:], right=True)
        base = torch.randn(M + 2, N, generator=gen).cuda()
        out = base.clone()
        src = dst = None
        if mode.startswith("mapped"):
            src = torch.randint(0, n_a, (M,), generator=gen).cuda()
            dst = torch.randperm(M + 2, generator=gen)[:M].cuda()
            src = torch.where((torch.rand(M, generator=gen) < 0.15).cuda(), torch.full_like(src, -1), src)
        s_eff = src if src is not None else torch.arange(M, device="cuda")
        d_eff = dst if dst is not None else torch.arange(M, device="cuda")
        live = s_eff >= 0
        prod = torch.zeros(M, N, dtype=torch.float64, device="cuda")
        prod[live] = torch.bmm(a[s_eff[live]].double().unsqueeze(1), w[rel[live]].double()).squeeze(1)
        want = base.double().clone()
        if mode in ("plain", "mapped"):
            want[d_eff[live]] = prod[live]
            _typed.typed_gemm(a, w, seg, M, src_idx=src, dst_idx=dst, out=out)
        elif mode in ("acc", "mapped_acc"):
            want[d_eff[live]] += prod[live]
            _typed.typed_gemm(a, w, seg, M, src_idx=src, dst_idx=dst, out=out, accumulate=True)
        else:
            bias = torch.randn(R, N, generator=gen).cuda() if "bias" in mode else None
            addend = torch.randn(M, N + 4, generator=gen).cuda() if "addend" in mode else None
            want[:M] = prod
            if bias is not None:
                want[:M] += bias[rel].double()
            if addend is not None:
                want[:M] += addend[:, :N].double()
            st = lib.cxg_typed_gemm_epilogue_f32(a.data_ptr(), K, w.data_ptr(), _lib.ptr(bias), _lib.ptr(addend), N + 4,
                                                 out.data_ptr(), N, None, None, seg.data_ptr(), M, K, N, R,
                                                 _typed.GEMM_SPLIT_F16X3, _lib.current_stream(a.device))
            _lib.check(st)
        torch.cuda.synchronize()
        assert_close(_np(out), want.cpu().numpy(), RTOL, 2 * ATOL,
                     "case %d: M=%d K=%d N=%d R=%d %s" % (case, M, K, N, R, mode))
