"""The typed GEMM for wide operands (cxg_typed_gemm_wide_f32: K >= 160, both operand tiles in
LDS, three fp16 partial products of power-of-two-scaled parts) against float64.

Tolerance: the fp32 aggregation bar, 1e-4 relative / 1e-5 absolute at O(1) output scale; the
dynamic-range test bounds every output against sum_k |x||w| of its own dot product (2e-6, the
bound the register-resident fp16 form is held to)."""
import numpy as np
import pytest
import torch

from conftest import announce, assert_close

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-4, 1e-5


def _np(t):
    return t.detach().cpu().numpy()


def _segments(M, R, gen, empty=True):
    types = torch.sort(torch.randint(0, R, (M,), generator=gen))[0]
    if empty and R > 2:
        types[types == 1] = 0                      # one relation without rows
    seg = torch.zeros(R + 1, dtype=torch.int64)
    seg[1:] = torch.bincount(types, minlength=R).cumsum(0)
    return types, seg


def _ref(a, w, types, src=None):
    rows = a if src is None else a[src]
    out = torch.empty(rows.shape[0], w.shape[2], dtype=torch.float64)
    for r in range(w.shape[0]):
        sel = types == r
        out[sel] = rows[sel].double() @ w[r].double()
    return out


SHAPES = [(512, 512, 7, 3000), (160, 64, 3, 1000), (320, 300, 4, 2500), (256, 40, 2, 700), (1024, 96, 1, 500),
          (164, 520, 3, 1300), (512, 256, 2, 1), (172, 257, 5, 129), (260, 128, 1, 4100)]


@pytest.mark.parametrize("K,N,R,M", SHAPES)
def test_wide_form_plain_rows(K, N, R, M):
    """Plain rows (no maps): column tiles that are full, partly filled and a single column past a
    tile, K on and off the 32-wide chunks, segment tails inside a 128-row tile, an empty relation."""
    from cxgnncomp_backend import _typed
    gen = torch.Generator().manual_seed(K * 7 + N)
    a = torch.randn(M, K, generator=gen) / K ** 0.5
    w = torch.randn(R, K, N, generator=gen)
    types, seg = _segments(M, R, gen)
    assert _typed._takes_wide_form(K, N, _typed.GEMM_SPLIT_F16X3)
    announce("wide typed GEMM plain M=%d K=%d N=%d R=%d" % (M, K, N, R))
    out = _typed.typed_gemm(a.cuda(), w.cuda(), seg.cuda(), M, precision="split_f16")
    assert_close(_np(out), _ref(a, w, types).numpy(), RTOL, ATOL, "wide plain")
    again = _typed.typed_gemm(a.cuda(), w.cuda(), seg.cuda(), M, precision="split_f16")
    assert torch.equal(out, again)


@pytest.mark.parametrize("K,N,R,M", [(512, 512, 7, 3000), (160, 64, 3, 1000), (320, 300, 4, 2500), (288, 96, 2, 131)])
def test_wide_form_row_maps_accumulate_atomic(K, N, R, M):
    """Gathered A rows, scattered C rows, negative map entries (the row is skipped), accumulation
    onto what is there twice in a row, and fp32 atomics for rows that share a destination."""
    from cxgnncomp_backend import _typed
    gen = torch.Generator().manual_seed(K + 31 * N)
    n_a = M // 2 + 7
    a = torch.randn(n_a, K, generator=gen) / K ** 0.5
    w = torch.randn(R, K, N, generator=gen)
    types, seg = _segments(M, R, gen)
    src = torch.randint(0, n_a, (M,), generator=gen)
    dst = torch.randperm(M + 5, generator=gen)[:M]
    skip = torch.rand(M, generator=gen) < 0.2
    src_m = torch.where(skip & (torch.arange(M) % 2 == 0), torch.full_like(src, -1), src)
    dst_m = torch.where(skip & (torch.arange(M) % 2 == 1), torch.full_like(dst, -7), dst)
    prod = _ref(a, w, types, src)
    announce("wide typed GEMM with row maps M=%d K=%d N=%d" % (M, K, N))
    out = torch.full((M + 5, N), 3.0).cuda()
    _typed.typed_gemm(a.cuda(), w.cuda(), seg.cuda(), M, src_idx=src_m.cuda(), dst_idx=dst_m.cuda(), out=out,
                      precision="split_f16")
    want = torch.full((M + 5, N), 3.0, dtype=torch.float64)
    want[dst[~skip]] = prod[~skip]
    assert_close(_np(out), want.numpy(), RTOL, ATOL, "wide with row maps")
    acc = torch.full((M + 5, N), 3.0).cuda()
    for _ in range(2):
        _typed.typed_gemm(a.cuda(), w.cuda(), seg.cuda(), M, src_idx=src_m.cuda(), dst_idx=dst_m.cuda(), out=acc,
                          accumulate=True, precision="split_f16")
    want_acc = torch.full((M + 5, N), 3.0, dtype=torch.float64)
    want_acc[dst[~skip]] += 2 * prod[~skip]
    assert_close(_np(acc), want_acc.numpy(), RTOL, 3 * ATOL, "wide accumulate")
    # several rows per destination: atomic adds
    n_dst = max(1, M // 6)
    dst2 = torch.randint(0, n_dst, (M,), generator=gen)
    at = torch.zeros(n_dst, N).cuda()
    _typed.typed_gemm(a.cuda(), w.cuda(), seg.cuda(), M, src_idx=src.cuda(), dst_idx=dst2.cuda(), out=at, atomic=True,
                      precision="split_f16")
    want_at = torch.zeros(n_dst, N, dtype=torch.float64).index_add_(0, dst2, prod)
    sc = max(1.0, float(want_at.abs().max()))
    assert_close(_np(at) / sc, want_at.numpy() / sc, RTOL, 2 * ATOL, "wide atomic")


def test_wide_form_many_tiles_per_block():
    """Enough rows that a block walks its full eight 128-row tiles (row tables and inverse scales
    alternate between two LDS slots from tile to tile), with a gather map."""
    from cxgnncomp_backend import _typed
    M, K, N, R = 300000, 160, 64, 3
    gen = torch.Generator().manual_seed(5)
    a = torch.randn(50000, K, generator=gen) / K ** 0.5
    w = torch.randn(R, K, N, generator=gen)
    types, seg = _segments(M, R, gen, empty=False)
    src = torch.randint(0, 50000, (M,), generator=gen)
    announce("wide typed GEMM, 300k gathered rows")
    out = _typed.typed_gemm(a.cuda(), w.cuda(), seg.cuda(), M, src_idx=src.cuda(), precision="split_f16")
    assert_close(_np(out), _ref(a, w, types, src).numpy(), RTOL, ATOL, "wide, eight tiles per block")


@pytest.mark.parametrize("K,N", [(512, 128), (200, 96 + 256)])
def test_wide_form_dynamic_range_along_k(K, N):
    """The row scale follows the largest magnitude met so far along K and is lowered when a later
    value outgrows its three bits of headroom: rows that grow geometrically along K (the scale
    moves in nearly every chunk), rows that shrink, a spike of 1e6 in the last chunk, a spike in
    the first, rows spread over e^+-9 with elements over e^+-4.5, zero rows, rows at 1e-30 and
    1e+15, zero prefixes (the scale is first set deep inside K), weight columns over e^+-9 and an
    all-zero column.  Every output within 2e-6 of sum_k |x||w| of its own dot product; an infinity
    makes its own row non-finite and no other."""
    from cxgnncomp_backend import _typed
    M, R = 3000, 3
    gen = torch.Generator().manual_seed(K + N)
    x = torch.randn(M, K, generator=gen)
    x *= torch.exp(torch.randn(M, 1, generator=gen) * 3)
    x *= torch.exp(torch.randn(M, K, generator=gen) * 1.5)
    ramp = torch.arange(K, dtype=torch.float32)
    x[0:200] = torch.randn(200, K, generator=gen) * torch.exp2(ramp / 6)          # grows by 2^85 along K = 512
    x[200:400] = torch.randn(200, K, generator=gen) * torch.exp2(-ramp / 6)
    x[400:500, K - 3] *= 1e6
    x[500:600, 1] *= 1e6
    x[600:650] = 0
    x[650:700] *= 1e-30
    x[700:750] *= 1e15
    x[750:850, :K - 40] = 0
    x[850:900, :100] = 0
    w = torch.randn(R, K, N, generator=gen) * torch.exp(torch.randn(R, 1, N, generator=gen) * 3)
    w[1, :, 3] = 0
    seg = torch.tensor([0, 1300, 1301, M], dtype=torch.int64)
    types = torch.repeat_interleave(torch.arange(R), seg[1:] - seg[:-1])
    announce("wide typed GEMM dynamic range along K, K=%d N=%d" % (K, N))
    out = _typed.typed_gemm(x.cuda(), w.cuda(), seg.cuda(), M, precision="split_f16").cpu().double()
    ref = _ref(x, w, types)
    mag = torch.empty(M, N, dtype=torch.float64)
    for r in range(R):
        b, e = int(seg[r]), int(seg[r + 1])
        mag[b:e] = x[b:e].double().abs() @ w[r].double().abs()
    assert torch.isfinite(out).all()
    assert torch.equal(out[600:650], torch.zeros(50, N, dtype=torch.float64))
    err = (out - ref).abs()
    ok = err <= 2e-6 * mag + 1e-33
    assert ok.all(), "worst error / sum|x||w| = %.3e at row %d" % (
        float((err / mag.clamp_min(1e-300))[~ok].max()), int(torch.nonzero(~ok)[0, 0]))
    xi = x.clone()
    xi[7, K - 5] = float("inf")
    bad = _typed.typed_gemm(xi.cuda(), w.cuda(), seg.cuda(), M, precision="split_f16").cpu()
    assert not torch.isfinite(bad[7]).any() or (w[0, K - 5] == 0).any()
    assert torch.isfinite(bad[8]).all() and torch.isfinite(bad[6]).all()


def test_wide_entry_point_rejects_what_it_does_not_take():
    from cxgnncomp_backend import _lib
    lib = _lib.load()
    a = torch.zeros(256, 512, device="cuda")
    w = torch.zeros(1, 512, 64, device="cuda")
    c = torch.zeros(256, 64, device="cuda")
    seg = torch.tensor([0, 256], device="cuda")
    need = lib.cxg_typed_gemm_wide_workspace_bytes(512, 64, 1)
    assert need == 1 * 1 * 16 * 2 * 256 * 32 * 2 + 256 * 4
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    st = _lib.current_stream(a.device)
    args = (a.data_ptr(), 512, w.data_ptr(), c.data_ptr(), 64, None, None, seg.data_ptr(), 256)
    assert lib.cxg_typed_gemm_wide_f32(*args, 512, 64, 1, 0, ws.data_ptr(), need - 1, st) == -3
    assert lib.cxg_typed_gemm_wide_f32(*args, 512, 64, 1, 0, None, 0, st) == -3
    assert lib.cxg_typed_gemm_wide_f32(*args, 128, 64, 1, 0, ws.data_ptr(), need, st) == -2
    assert lib.cxg_typed_gemm_wide_f32(*args, 512, 64, 1, 4, ws.data_ptr(), need, st) == -1   # bf16 split flag
    assert lib.cxg_typed_gemm_wide_f32(*args, 512, 64, 1, 16, ws.data_ptr(), need, st) == 0
    torch.cuda.synchronize()


@pytest.mark.parametrize("K,N", [(256, 256), (512, 384), (300, 72)])
def test_dense_products_without_an_epilogue_take_the_tiled_kernel(K, N):
    """dense_linear(x, W) without bias and addend from 10^5 rows on: 176 <= K <= 256 with more than 128
    columns and any K above 256 run on the tiled kernel (one relation); against float64 on sampled
    rows, and linear in x on every row."""
    from cxgnncomp_backend import _typed
    M = 120000
    gen = torch.Generator().manual_seed(K + N)
    x = (torch.randn(M, K, generator=gen) / K ** 0.5).cuda()
    x2 = (torch.randn(M, K, generator=gen) / K ** 0.5).cuda()
    w = torch.randn(K, N, generator=gen).cuda()
    announce("dense_linear on the tiled kernel M=%d K=%d N=%d" % (M, K, N))
    got = _typed.dense_linear(x, w)
    if K <= 256 and N <= 128:
        assert got is None or got.shape == (M, N)          # shapes the rule leaves to other kernels or the library
        return
    assert got is not None and got.shape == (M, N)
    rows = torch.randint(0, M, (3000,), generator=gen).cuda()
    want = x[rows].double() @ w.double()
    assert_close(_np(got[rows]), _np(want), RTOL, ATOL, "dense product rows")
    both = _typed.dense_linear(x + x2, w)
    sep = got + _typed.dense_linear(x2, w)
    assert float((both - sep).abs().max()) <= 1e-4 * max(1.0, float(sep.abs().max()))
