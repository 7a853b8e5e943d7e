"""GSpMM_u / GSpMM_u_e (generalised int32-CSR SpMM, every REDUCEOP x COMPUTEOP)
through cxgnncomp_backend against the oracle.  max / min are exact; sum / mean
use the fp32 aggregation bound (1e-4 relative, 1e-5 absolute at O(1) scale)."""
import numpy as np
import pytest
import torch

import oracle
from conftest import announce, assert_close

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-4, 1e-5


def _np(t):
    return t.detach().cpu().numpy()


def _graph(n_dst, n_src, e, seed, hub=False):
    rng = np.random.default_rng(seed)
    dst = rng.integers(0, n_dst, e)
    dst = np.where(dst % 7 == 0, np.minimum(dst + 1, n_dst - 1), dst)     # empty rows
    if hub:
        dst[: e // 3] = 3                                                  # one row with > 64 edges
    src = rng.integers(0, n_src, e)
    ptr, idx = oracle.coo_to_csr(src, dst, n_dst)
    return ptr.astype(np.int32), idx.astype(np.int32)


CASES = [(50, 40, 300, 7, False), (300, 200, 5000, 64, True), (1000, 1000, 20000, 100, True), (1, 3, 0, 5, False)]


@pytest.mark.parametrize("n_dst,n_src,e,feat,hub", CASES)
@pytest.mark.parametrize("red", ["SUM", "MAX", "MIN", "MEAN"])
def test_gspmm_u(n_dst, n_src, e, feat, hub, red):
    import cxgnncomp_backend as B
    ptr, idx = _graph(n_dst, n_src, e, e + feat, hub)
    rng = np.random.default_rng(1)
    scale = 1.0 / max(1.0, float(np.sqrt(np.diff(ptr).max()))) if red == "SUM" else 1.0
    b = (rng.standard_normal((n_src, feat)) * scale).astype(np.float32)
    op = getattr(B.REDUCEOP, red)
    announce("GSpMM_u %s n=%d e=%d F=%d" % (red, n_dst, e, feat))
    got = B.GSpMM_u(torch.from_numpy(ptr).cuda(), torch.from_numpy(idx).cuda(), torch.from_numpy(b).cuda(), op)
    want = oracle.gspmm(ptr, idx, b, int(op))
    if red in ("MAX", "MIN"):
        assert np.array_equal(_np(got), want)
    else:
        assert_close(_np(got), want, RTOL, ATOL, "GSpMM_u " + red)


@pytest.mark.parametrize("n_dst,n_src,e,feat,hub", CASES[:3])
@pytest.mark.parametrize("red", ["SUM", "MAX", "MIN", "MEAN"])
@pytest.mark.parametrize("comp", ["ADD", "SUB", "MUL", "DIV"])
def test_gspmm_u_e(n_dst, n_src, e, feat, hub, red, comp):
    import cxgnncomp_backend as B
    ptr, idx = _graph(n_dst, n_src, e, e + feat + 1, hub)
    rng = np.random.default_rng(2)
    scale = 1.0 / max(1.0, float(np.sqrt(np.diff(ptr).max()))) if red == "SUM" else 1.0
    b = (rng.standard_normal((n_src, feat)) * scale).astype(np.float32)
    val = ((rng.random(idx.shape[0]) + 0.5) * rng.choice([-1.0, 1.0], idx.shape[0])).astype(np.float32)
    if red == "SUM" and comp in ("ADD", "SUB"):
        val = (val * scale).astype(np.float32)
    rop, cop = getattr(B.REDUCEOP, red), getattr(B.COMPUTEOP, comp)
    announce("GSpMM_u_e %s %s n=%d e=%d F=%d" % (red, comp, n_dst, e, feat))
    got = B.GSpMM_u_e(torch.from_numpy(ptr).cuda(), torch.from_numpy(idx).cuda(), torch.from_numpy(val).cuda(),
                      torch.from_numpy(b).cuda(), rop, cop)
    want = oracle.gspmm(ptr, idx, b, int(rop), int(cop), val=val)
    if red in ("MAX", "MIN"):
        # one fp32 operation per term on both sides; division may differ in the last bit
        assert_close(_np(got), want, 1e-6 if comp == "DIV" else 0.0, 0.0, "GSpMM_u_e %s %s" % (red, comp))
    else:
        sc = max(1.0, float(np.abs(want).max()))
        assert_close(_np(got) / sc, want / sc, RTOL, ATOL, "GSpMM_u_e %s %s" % (red, comp))


def _long_row_graph(n_src, lead, rng):
    """Rows of more than 512 edges next to each other, at both ends of the edge array, with
    lengths at and around the piece size, short and empty rows in between; `lead` unused
    column ids in front of the first row (rowptr[0] = lead)."""
    degs = [1300, 513, 512, 0, 0, 2049, 3, 511, 1024, 1025, 0, 7, 700]
    ptr = (np.concatenate([[0], np.cumsum(degs)]) + lead).astype(np.int32)
    idx = rng.integers(0, n_src, int(ptr[-1])).astype(np.int32)
    return ptr, idx


@pytest.mark.parametrize("feat", [4, 7, 100, 300])
@pytest.mark.parametrize("lead", [0, 37])
@pytest.mark.parametrize("red,comp", [("MAX", None), ("MIN", "SUB"), ("SUM", "ADD"), ("MEAN", "DIV"), ("SUM", "MUL")])
def test_gspmm_rows_cut_into_pieces(feat, lead, red, comp):
    """Rows above 512 edges go through per-piece partial rows: same answers as the oracle,
    max / min exactly, and the same bits on a second call."""
    import cxgnncomp_backend as B
    rng = np.random.default_rng(feat + lead)
    n_src = 500
    ptr, idx = _long_row_graph(n_src, lead, rng)
    scale = 1.0 / np.sqrt(2049.0) if red == "SUM" else 1.0
    b = (rng.standard_normal((n_src, feat)) * scale).astype(np.float32)
    val = None
    if comp is not None:
        val = ((rng.random(idx.shape[0]) + 0.5) * rng.choice([-1.0, 1.0], idx.shape[0])).astype(np.float32)
        if red == "SUM" and comp == "ADD":
            val = (val * scale).astype(np.float32)
    rop = getattr(B.REDUCEOP, red)
    announce("GSpMM long rows %s %s F=%d lead=%d" % (red, comp, feat, lead))
    tp, ti, tb = torch.from_numpy(ptr).cuda(), torch.from_numpy(idx).cuda(), torch.from_numpy(b).cuda()
    if comp is None:
        run = lambda: B.GSpMM_u(tp, ti, tb, rop)
        want = oracle.gspmm(ptr, idx, b, int(rop))
    else:
        cop = getattr(B.COMPUTEOP, comp)
        tv = torch.from_numpy(val).cuda()
        run = lambda: B.GSpMM_u_e(tp, ti, tv, tb, rop, cop)
        want = oracle.gspmm(ptr, idx, b, int(rop), int(cop), val=val)
    got = run()
    if red in ("MAX", "MIN"):
        assert np.array_equal(_np(got), want)
    else:
        sc = max(1.0, float(np.abs(want).max()))
        assert_close(_np(got) / sc, want / sc, RTOL, ATOL, "GSpMM long rows %s %s" % (red, comp))
    assert torch.equal(run(), got)


def test_gspmm_enum_values_and_errors():
    import cxgnncomp_backend as B
    assert [int(B.REDUCEOP.SUM), int(B.REDUCEOP.MAX), int(B.REDUCEOP.MIN), int(B.REDUCEOP.MEAN)] == [0, 1, 2, 3]
    assert [int(B.COMPUTEOP.ADD), int(B.COMPUTEOP.SUB), int(B.COMPUTEOP.MUL), int(B.COMPUTEOP.DIV)] == [0, 1, 2, 3]
    assert B.SUM is B.REDUCEOP.SUM and B.MUL is B.COMPUTEOP.MUL
    p = torch.tensor([0, 1]).cuda()
    with pytest.raises(ValueError):
        B.GSpMM_u(p, p, torch.zeros(2, 2).cuda(), B.REDUCEOP.MAX)          # int64 indices
