"""HIP SpMM family vs the CPU oracle, through the C ABI (cxgnncomp_backend).

Tolerance for fp32 aggregation: 1e-4 relative / 1e-5 absolute against the
double-accumulated oracle.  Features are drawn so that a row sum keeps a scale
of O(1) (x ~ N(0,1)/sqrt(max_degree) on heavy-tailed graphs): the absolute
rounding error of an fp32 sum grows with the magnitude of its partial sums, so
the absolute tolerance is only meaningful at a fixed output scale.
"""
import numpy as np
import pytest
import torch

import oracle
from conftest import announce, assert_close

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-4, 1e-5


def _graph(kind, seed=0):
    from cxgnncomp import synthetic as S
    if kind == "uniform":
        return S.uniform_graph(10000, 100000, seed=seed)
    if kind == "powerlaw":
        return S.powerlaw_directed_symmetrised(20000, 150000, max_degree=6000, seed=seed)
    if kind == "empty_rows":
        ptr, idx = S.uniform_graph(3000, 2000, seed=seed)   # most rows empty
        return ptr, idx
    if kind == "no_edges":
        return torch.zeros(501, dtype=torch.int64), torch.zeros(0, dtype=torch.int64)
    if kind == "one_hub":
        n = 300
        deg = torch.zeros(n, dtype=torch.int64)
        deg[7] = 5000
        deg[299] = 3
        ptr = torch.zeros(n + 1, dtype=torch.int64)
        ptr[1:] = torch.cumsum(deg, 0)
        g = torch.Generator().manual_seed(seed)
        idx = torch.randint(0, n, (int(ptr[-1]),), generator=g)
        return ptr, idx
    raise KeyError(kind)


def _scale(ptr):
    deg = (ptr[1:] - ptr[:-1]).max().item() if ptr.shape[0] > 1 else 1
    return 1.0 / max(1.0, float(deg)) ** 0.5


@pytest.mark.parametrize("kind", ["uniform", "powerlaw", "empty_rows", "no_edges", "one_hub"])
@pytest.mark.parametrize("feat", [64, 128, 256, 32, 40, 100, 1, 600])
def test_spmm_sum(kind, feat):
    import cxgnncomp_backend as B
    ptr, idx = _graph(kind)
    n = ptr.shape[0] - 1
    torch.manual_seed(0)
    x = torch.randn(n, feat) * _scale(ptr)
    announce("spmm_sum kind=%s feat=%d n=%d E=%d" % (kind, feat, n, idx.shape[0]))
    out = B.run_spmm_configurable(ptr.cuda(), idx.cuda(), x.cuda(), n, 0, 0, 0, 0, 0, 0, 0, 0, 0)
    torch.cuda.synchronize()
    ref = oracle.spmm(ptr.numpy(), idx.numpy(), x.numpy(), n)
    assert_close(out.cpu().numpy(), ref, RTOL, ATOL, "spmm_sum %s F=%d" % (kind, feat))


@pytest.mark.parametrize("kind", ["uniform", "powerlaw", "empty_rows"])
def test_spmm_mean_and_prefix_rows(kind):
    import cxgnncomp_backend as B
    ptr, idx = _graph(kind)
    n = ptr.shape[0] - 1
    torch.manual_seed(1)
    x = torch.randn(n, 128) * _scale(ptr)
    for rows in (n, n // 3, 1):
        announce("spmm_mean kind=%s rows=%d" % (kind, rows))
        out = B.sage_mean_forward(x.cuda(), ptr.cuda(), idx.cuda(), rows)
        torch.cuda.synchronize()
        ref = oracle.spmm(ptr.numpy(), idx.numpy(), x.numpy(), rows, mean=True)
        assert out.shape == (rows, 128)
        assert_close(out.cpu().numpy(), ref, RTOL, ATOL, "mean %s rows=%d" % (kind, rows))


# Row widths that reach every (vector width, lanes per edge) form of the grouped-lane
# kernel (F <= 32 vector lanes) plus the first widths past it.
WIDTHS = [2, 3, 4, 6, 7, 8, 12, 16, 20, 24, 30, 31, 33, 48, 52, 62, 64, 66, 96, 124, 126, 128, 130, 132]


@pytest.mark.parametrize("feat", WIDTHS)
def test_spmm_width_sweep(feat):
    """Sum, mean, accumulate and a row prefix at every width, on a graph whose 2.33M edges
    give spans of several 64-edge steps, hub rows that cross spans, and empty rows."""
    from cxgnncomp import synthetic as S
    from cxgnncomp_backend import _ops
    ptr, idx = S.powerlaw_directed_symmetrised(169343, 1166243, seed=3)
    n = ptr.shape[0] - 1
    torch.manual_seed(feat)
    x = torch.randn(n, feat) * _scale(ptr)
    pc, ic, xc = ptr.cuda(), idx.cuda(), x.cuda()
    announce("spmm width sweep F=%d" % feat)
    got = _ops.spmm(pc, ic, xc, n)
    want = oracle.spmm(ptr.numpy(), idx.numpy(), x.numpy(), n)
    assert_close(got.cpu().numpy(), want, RTOL, ATOL, "sum F=%d" % feat)
    assert torch.equal(got, _ops.spmm(pc, ic, xc, n))                       # deterministic
    rows = n // 7
    got = _ops.spmm(pc, ic, xc, rows, mean=True)
    want = oracle.spmm(ptr.numpy(), idx.numpy(), x.numpy(), rows, mean=True)
    assert_close(got.cpu().numpy(), want, RTOL, ATOL, "mean prefix F=%d" % feat)
    base = torch.randn(n, feat) / 4
    out = base.clone().cuda()
    _ops.spmm(pc, ic, xc, n, out=out, accumulate=True)
    want = oracle.spmm(ptr.numpy(), idx.numpy(), x.numpy(), n) + base.numpy()
    assert_close(out.cpu().numpy(), want, RTOL, ATOL, "accumulate F=%d" % feat)
    # one weight per edge, also read through a permutation
    val = torch.rand(idx.shape[0]) + 0.5
    got = _ops.spmm(pc, ic, xc, n, val=val.cuda())
    want = oracle.spmm(ptr.numpy(), idx.numpy(), x.numpy(), n, val=val.numpy())
    sc = max(1.0, float(np.abs(want).max()))
    assert_close(got.cpu().numpy() / sc, want / sc, RTOL, ATOL, "weighted F=%d" % feat)
    perm = torch.randperm(idx.shape[0])
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(idx.shape[0])
    got2 = _ops.spmm(pc, ic, xc, n, val=val[perm].cuda(), val_perm=inv.cuda())
    assert torch.equal(got, got2)


@pytest.mark.parametrize("kind", ["uniform", "powerlaw", "empty_rows", "no_edges", "one_hub", "c2", "empty_runs"])
@pytest.mark.parametrize("heads,feat", [(4, 128), (2, 128), (8, 128), (4, 100), (4, 64), (2, 40), (8, 24), (4, 20)])
def test_spmm_one_gathered_row_under_several_weights(kind, heads, feat):
    """cxg_spmm_weighted_heads_f32: out[r, h, :] = sum_e val[e, h] x[idx[e], :].  Every head against
    the oracle's weighted SpMM with that head's column of weights (1e-4 / 1e-5), bit for bit
    against the single-weight kernel (the same additions in the same order), rows of x with a
    stride, a row prefix, and run-to-run equality."""
    from cxgnncomp import synthetic as S
    from cxgnncomp_backend import _ops
    if kind == "c2":
        if (heads, feat) not in ((4, 128), (2, 40)):
            pytest.skip("the large graph runs two shapes")
        ptr, idx = S.powerlaw_directed_symmetrised(169343, 1166243, seed=3)
    elif kind == "empty_runs":
        ptr, idx, _ = _graph_with_empty_runs(5)
    else:
        ptr, idx = _graph(kind)
    n = ptr.shape[0] - 1
    E = idx.shape[0]
    assert _ops.spmm_heads_supported(heads, feat)
    torch.manual_seed(heads * 1000 + feat)
    wide = torch.randn(n, feat + 4) * _scale(ptr)
    x = wide[:, :feat]
    val = torch.rand(E, heads) + 0.25
    pc, ic = ptr.cuda(), idx.cuda()
    announce("spmm several weights kind=%s H=%d F=%d n=%d E=%d" % (kind, heads, feat, n, E))
    got = _ops.spmm_weighted_heads(pc, ic, val.cuda(), wide.cuda()[:, :feat], n)
    torch.cuda.synchronize()
    assert got.shape == (n, heads, feat)
    xc = x.contiguous().cuda()
    assert torch.equal(got, _ops.spmm_weighted_heads(pc, ic, val.cuda(), xc, n))
    for h in range(heads):
        vh = val[:, h].contiguous()
        want = oracle.spmm(ptr.numpy(), idx.numpy(), x.contiguous().numpy(), n, val=vh.numpy())
        sc = max(1.0, float(np.abs(want).max()))
        assert_close(got[:, h].cpu().numpy() / sc, want / sc, RTOL, ATOL, "head %d" % h)
        if E > 0:
            assert torch.equal(got[:, h], _ops.spmm(pc, ic, xc, n, val=vh.cuda())), "head %d against the single-weight kernel" % h
    rows = n // 3
    if rows > 0:
        part = _ops.spmm_weighted_heads(pc, ic, val.cuda(), xc, rows)
        assert torch.equal(part, got[:rows])


def test_spmm_several_weights_rejects_other_shapes():
    from cxgnncomp_backend import _ops
    ptr, idx = _graph("uniform")
    n, E = ptr.shape[0] - 1, idx.shape[0]
    for heads, feat in [(3, 128), (4, 132), (4, 16), (16, 64), (4, 30)]:
        assert not _ops.spmm_heads_supported(heads, feat)
        with pytest.raises(RuntimeError):
            _ops.spmm_weighted_heads(ptr.cuda(), idx.cuda(), torch.zeros(E, heads).cuda(), torch.zeros(n, feat).cuda(), n)


def _graph_with_empty_runs(seed):
    """Long runs of rows without edges at the start, in the middle (two of them inside one
    64-edge span, one across a span boundary) and at the end, between rows of 1-3 edges and
    one row long enough to cross spans."""
    rng = np.random.default_rng(seed)
    blocks = [np.zeros(1000), rng.integers(1, 4, 20), np.zeros(70), rng.integers(1, 3, 5), np.zeros(300),
              rng.integers(1, 4, 15), [400], np.zeros(129), rng.integers(0, 3, 2000), np.zeros(64),
              rng.integers(1, 4, 30), np.zeros(2500)]
    deg = np.concatenate(blocks).astype(np.int64)
    ptr = np.concatenate([[0], np.cumsum(deg)])
    n = deg.shape[0]
    idx = rng.integers(0, n, int(ptr[-1]))
    return torch.from_numpy(ptr), torch.from_numpy(idx), n


@pytest.mark.parametrize("feat", [8, 47, 128, 256, 330])
def test_spmm_runs_of_rows_without_edges(feat):
    """Runs of empty rows are not walked row by row: every variant of the row store (plain,
    mean, bias, accumulate, int32 indices, a row prefix) still leaves the right values in
    them and around them."""
    import cxgnncomp_backend as B
    from cxgnncomp_backend import _ops
    ptr, idx, n = _graph_with_empty_runs(feat)
    torch.manual_seed(feat)
    x = torch.randn(n, feat) / 20
    pc, ic, xc = ptr.cuda(), idx.cuda(), x.cuda()
    pn, in_, xn = ptr.numpy(), idx.numpy(), x.numpy()
    announce("spmm empty runs F=%d n=%d E=%d" % (feat, n, idx.shape[0]))
    want = oracle.spmm(pn, in_, xn, n)
    got = _ops.spmm(pc, ic, xc, n, out=torch.full((n, feat), 7.0, device="cuda"))
    assert_close(got.cpu().numpy(), want, RTOL, ATOL, "sum")
    got = _ops.spmm(pc, ic, xc, n, mean=True, out=torch.full((n, feat), 7.0, device="cuda"))
    assert_close(got.cpu().numpy(), oracle.spmm(pn, in_, xn, n, mean=True), RTOL, ATOL, "mean")
    got = B.run_spmm_configurable_int32(pc.int(), ic.int(), xc, n, 0, 0, 0, 0, 0, 0, 0, 0, 0)
    assert_close(got.cpu().numpy(), want, RTOL, ATOL, "int32")
    base = torch.randn(n, feat)
    out = base.clone().cuda()
    _ops.spmm(pc, ic, xc, n, out=out, accumulate=True)
    assert_close(out.cpu().numpy(), want + base.numpy(), RTOL, ATOL, "accumulate")
    val = torch.rand(idx.shape[0]) + 0.5
    bias = torch.randn(feat)
    wantw = oracle.spmm(pn, in_, xn, n, val=val.numpy())
    got = _ops.spmm(pc, ic, xc, n, val=val.cuda(), bias=bias.cuda(), out=torch.full((n, feat), 7.0, device="cuda"))
    assert_close(got.cpu().numpy(), wantw + bias.numpy(), RTOL, ATOL, "weighted + bias")
    out = base.clone().cuda()
    _ops.spmm(pc, ic, xc, n, val=val.cuda(), bias=bias.cuda(), out=out, accumulate=True)
    assert_close(out.cpu().numpy(), wantw + bias.numpy() + base.numpy(), RTOL, ATOL, "weighted + bias + accumulate")
    for rows in (1500, 3700, n - 2400):      # prefixes that end inside runs of empty rows
        got = _ops.spmm(pc, ic, xc, rows, out=torch.full((rows, feat), 7.0, device="cuda"))
        assert_close(got.cpu().numpy(), want[:rows], RTOL, ATOL, "prefix %d" % rows)


def test_spmm_multihead_runs_of_rows_without_edges():
    from cxgnncomp_backend import _ops
    ptr, idx, n = _graph_with_empty_runs(5)
    torch.manual_seed(5)
    x = torch.randn(n, 4, 64) / 20
    val = torch.rand(idx.shape[0], 4) + 0.5
    announce("spmm multihead empty runs")
    got = _ops.spmm(ptr.cuda(), idx.cuda(), x.cuda(), n, val=val.cuda(), out=torch.full((n, 4, 64), 7.0, device="cuda"))
    want = oracle.spmm(ptr.numpy(), idx.numpy(), x.numpy(), n, val=val.numpy())
    assert_close(got.cpu().numpy(), want, RTOL, ATOL, "multihead")
