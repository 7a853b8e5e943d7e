"""Masked, targeted and relational aggregation through cxgnncomp_backend vs the oracle."""
import numpy as np
import pytest
import torch

import oracle
from conftest import announce, assert_close
from test_spmm_gpu import ATOL, RTOL, _graph, _scale

pytestmark = pytest.mark.gpu


def _np(t):
    return t.detach().cpu().numpy()


@pytest.mark.parametrize("kind", ["uniform", "powerlaw", "one_hub"])
@pytest.mark.parametrize("feat", [128, 40])
def test_selective_aggr_forward_backward(kind, feat):
    import cxgnncomp_backend as B
    ptr, idx = _graph(kind)
    n = ptr.shape[0] - 1
    E = idx.shape[0]
    torch.manual_seed(11)
    sc = _scale(ptr)
    x = torch.randn(n, feat) * sc
    rel = torch.randint(0, 3, (E,))
    base = torch.randn(n, feat) * sc
    for r in range(3):
        mask = rel == r
        out = base.clone().cuda()
        announce("selective_aggr kind=%s F=%d rel=%d" % (kind, feat, r))
        B.selective_aggr(x.cuda(), ptr.cuda(), idx.cuda(), mask.cuda(), out, n)
        ref = oracle.selective_aggr_fwd(x.numpy(), ptr.numpy(), idx.numpy(), mask.numpy(), base.numpy(), n)
        assert_close(_np(out), ref, RTOL, 2 * ATOL, "selective fwd")
        g = torch.randn(n, feat) * sc
        gx = base.clone().cuda()
        announce("selective_aggr_bwd kind=%s F=%d rel=%d" % (kind, feat, r))
        B.selective_aggr_bwd(g.cuda(), ptr.cuda(), idx.cuda(), mask.cuda(), gx, n)
        ref = oracle.selective_aggr_bwd(g.numpy(), ptr.numpy(), idx.numpy(), mask.numpy(), base.numpy(), n)
        assert_close(_np(gx), ref, RTOL, 2 * ATOL, "selective bwd")


@pytest.mark.parametrize("kind", ["uniform", "powerlaw", "one_hub"])
def test_target_aggr_recombines_neighbor_groups(kind):
    """neighbor_grouping + target_aggr == plain aggregation (cxgnncomp/schedule.py:20-35)."""
    import cxgnncomp_backend as B
    ptr, idx = _graph(kind)
    n = ptr.shape[0] - 1
    torch.manual_seed(12)
    sc = _scale(ptr)
    x = torch.randn(n, 64) * sc
    new_ptr, new_target = oracle.neighbor_grouping(ptr.numpy(), 32)
    gp, gt = torch.from_numpy(new_ptr), torch.from_numpy(new_target)
    out = torch.zeros(n, 64).cuda()
    announce("target_aggr kind=%s groups=%d" % (kind, gt.shape[0]))
    B.target_aggr(x.cuda(), gp.cuda(), idx.cuda(), gt.cuda(), out, gt.shape[0])
    ref = oracle.target_aggr_fwd(x.numpy(), new_ptr, idx.numpy(), new_target, np.zeros((n, 64), np.float32),
                                 gt.shape[0])
    assert_close(_np(out), ref, RTOL, ATOL, "target fwd")
    assert_close(_np(out), oracle.spmm(ptr.numpy(), idx.numpy(), x.numpy(), n), RTOL, ATOL, "== plain spmm")
    g = torch.randn(n, 64) * sc
    gx = torch.zeros(n, 64).cuda()
    announce("target_aggr_backward kind=%s" % kind)
    B.target_aggr_backward(g.cuda(), gp.cuda(), idx.cuda(), gt.cuda(), gx, gt.shape[0])
    ref = oracle.target_aggr_bwd(g.numpy(), new_ptr, idx.numpy(), new_target, np.zeros((n, 64), np.float32),
                                 gt.shape[0])
    assert_close(_np(gx), ref, RTOL, ATOL, "target bwd")


@pytest.mark.parametrize("kind", ["uniform", "powerlaw"])
def test_aggr_rel_forward_backward(kind):
    import cxgnncomp_backend as B
    ptr, idx = _graph(kind)
    n = ptr.shape[0] - 1
    E = idx.shape[0]
    R, F = 4, 64
    torch.manual_seed(13)
    sc = _scale(ptr)
    x = (torch.randn(R * n, F) * sc)
    etype = torch.randint(0, R, (E,), dtype=torch.int32)
    xg = x.cuda().requires_grad_(True)
    announce("aggr_rel kind=%s" % kind)
    out = B.aggr_rel(xg, ptr.cuda(), idx.cuda(), etype.cuda(), n, R)
    g = torch.randn(n, F) * sc
    out.backward(g.cuda())
    torch.cuda.synchronize()
    assert_close(_np(out), oracle.aggr_rel_fwd(x.numpy(), ptr.numpy(), idx.numpy(), etype.numpy(), n, R),
                 RTOL, ATOL, "aggr_rel fwd")
    assert_close(_np(xg.grad), oracle.aggr_rel_bwd(g.numpy(), ptr.numpy(), idx.numpy(), etype.numpy(), n, R, n),
                 RTOL, ATOL, "aggr_rel bwd")
