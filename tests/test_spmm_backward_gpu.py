"""Backward / weighted / multi-head SpMM through cxgnncomp_backend vs the oracle.

fp32 aggregation tolerance: 1e-4 relative / 1e-5 absolute (see test_spmm_gpu.py
for why features are scaled by 1/sqrt(max degree))."""
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
@pytest.mark.parametrize("mean", [False, True])
def test_sage_backward(kind, mean):
    import cxgnncomp_backend as B
    ptr, idx = _graph(kind)
    n = ptr.shape[0] - 1
    torch.manual_seed(2)
    sc = _scale(ptr)
    x = (torch.randn(n, 96) * sc).cuda().requires_grad_(True)
    g = torch.randn(n, 96) * sc
    announce("sage backward kind=%s mean=%s" % (kind, mean))
    fn = B.sage_mean_forward if mean else B.sage_sum_forward
    out = fn(x, ptr.cuda(), idx.cuda(), n)
    out.backward(g.cuda())
    torch.cuda.synchronize()
    ref_out = oracle.spmm(ptr.numpy(), idx.numpy(), _np(x), n, mean=mean)
    ref_gx = oracle.spmm_bwd(ptr.numpy(), idx.numpy(), g.numpy(), n, n, mean=mean)
    assert_close(_np(out), ref_out, RTOL, ATOL, "forward")
    assert_close(_np(x.grad), ref_gx, RTOL, ATOL, "grad_x")


def test_sage_num_node_zero_means_all_rows():
    import cxgnncomp_backend as B
    ptr, idx = _graph("uniform")
    n = ptr.shape[0] - 1
    x = torch.randn(n, 32).cuda()
    announce("sage num_node=0")
    out = B.sage_sum_forward(x, ptr.cuda(), idx.cuda(), 0)
    assert out.shape == (n, 32)


def test_sampled_prefix_layers():
    """CSR_Layer use: one CSR, each layer passes a smaller num_node (rows are a prefix)."""
    import cxgnncomp_backend as B
    from cxgnncomp import synthetic as S
    ptr, idx, nn, ne = S.sampled_batch(num_seeds=64, fanouts=(5, 4, 3), id_space=100000, seed=5)
    n_src = nn[-1]
    torch.manual_seed(3)
    x = (torch.randn(n_src, 128) / 3).cuda().requires_grad_(True)
    for layer_rows in (nn[2], nn[1], nn[0]):
        announce("sampled prefix rows=%d of %d" % (layer_rows, ptr.shape[0] - 1))
        x.grad = None
        out = B.sage_mean_forward(x, ptr.cuda(), idx.cuda(), layer_rows)
        g = torch.randn(layer_rows, 128)
        out.backward(g.cuda())
        torch.cuda.synchronize()
        assert_close(_np(out), oracle.spmm(ptr.numpy(), idx.numpy(), _np(x), layer_rows, mean=True),
                     RTOL, ATOL, "fwd rows=%d" % layer_rows)
        assert_close(_np(x.grad), oracle.spmm_bwd(ptr.numpy(), idx.numpy(), g.numpy(), layer_rows, n_src,
                                                   mean=True), RTOL, ATOL, "bwd rows=%d" % layer_rows)


@pytest.mark.parametrize("kind", ["uniform", "powerlaw"])
def test_run_spmm_configurable_bwd_and_int32(kind):
    import cxgnncomp_backend as B
    ptr, idx = _graph(kind)
    n = ptr.shape[0] - 1
    torch.manual_seed(4)
    sc = _scale(ptr)
    x = torch.randn(n, 64) * sc
    g = torch.randn(n, 64) * sc
    z = (0,) * 9
    announce("run_spmm_configurable_bwd kind=%s" % kind)
    gx = B.run_spmm_configurable_bwd(ptr.cuda(), idx.cuda(), x.cuda(), g.cuda(), n, *z)
    assert_close(_np(gx), oracle.spmm_bwd(ptr.numpy(), idx.numpy(), g.numpy(), n, n), RTOL, ATOL, "bwd")
    announce("run_spmm_configurable_int32 kind=%s" % kind)
    out32 = B.run_spmm_configurable_int32(ptr.int().cuda(), idx.int().cuda(), x.cuda(), n, *z)
    out64 = B.run_spmm_configurable(ptr.cuda(), idx.cuda(), x.cuda(), n, *z)
    assert torch.equal(out32, out64)          # same kernel, same order of additions


@pytest.mark.parametrize("kind", ["uniform", "powerlaw", "one_hub"])
@pytest.mark.parametrize("shape", [(1, 128), (1, 40), (4, 64), (2, 24), (3, 100), (8, 16), (8, 8), (4, 4), (1, 256), (2, 128),
                                   (8, 32), (1, 512)])
def test_weighted_spmm_forward_backward(kind, shape):
    import cxgnncomp_backend as B
    H, C = shape
    ptr, idx = _graph(kind)
    n = ptr.shape[0] - 1
    E = idx.shape[0]
    torch.manual_seed(5)
    sc = _scale(ptr)
    if H == 1:
        x = torch.randn(n, C) * sc
        val = torch.rand(E)
        g = torch.randn(n, C) * sc
    else:
        x = torch.randn(n, H, C) * sc
        val = torch.rand(E, H)
        g = torch.randn(n, H, C) * sc
    xg = x.cuda().requires_grad_(True)
    vg = val.cuda().requires_grad_(True)
    announce("weighted spmm kind=%s H=%d C=%d" % (kind, H, C))
    out = B.sage_sum_forward_edge_value(xg, ptr.cuda(), idx.cuda(), vg, n)
    out.backward(g.cuda())
    torch.cuda.synchronize()
    p, i = ptr.numpy(), idx.numpy()
    assert_close(_np(out), oracle.spmm(p, i, x.numpy(), n, val=val.numpy()), RTOL, ATOL, "fwd")
    assert_close(_np(xg.grad), oracle.spmm_bwd(p, i, g.numpy(), n, n, val=val.numpy()), RTOL, ATOL, "grad_x")
    # edge gradient: values are O(sc^2 * C); compare at that scale
    ref_gv = oracle.edge_grad(p, i, x.numpy(), g.numpy(), n)
    assert_close(_np(vg.grad), ref_gv, RTOL, ATOL, "grad_val")


def test_weighted_mean_is_refused():
    import cxgnncomp_backend as B
    ptr, idx = _graph("uniform")
    n = ptr.shape[0] - 1
    x = torch.randn(n, 16).cuda()
    val = torch.rand(idx.shape[0]).cuda()
    with pytest.raises(ValueError, match="DO NOT use mean with edge value"):
        B.sage_mean_forward_edge_value(x, ptr.cuda(), idx.cuda(), val, n)


@pytest.mark.parametrize("kind", ["uniform", "powerlaw"])
def test_spmm_multihead_schedules_and_bwd(kind):
    import cxgnncomp_backend as B
    H, C = 4, 64
    ptr, idx = _graph(kind)
    n = ptr.shape[0] - 1
    E = idx.shape[0]
    torch.manual_seed(6)
    sc = _scale(ptr)
    x = torch.randn(n, H, C) * sc
    val = torch.rand(E, H)
    p, i = ptr.numpy(), idx.numpy()
    announce("spmm_multihead Naive kind=%s" % kind)
    naive = B.spmm_multihead(ptr.cuda(), idx.cuda(), val.cuda(), x.cuda(), n,
                             B.SPMM_MULTIHEAD_SCHEDULE.Naive)
    assert naive.shape == (n, H, C)
    assert_close(_np(naive), oracle.spmm(p, i, x.numpy(), n, val=val.numpy()), RTOL, ATOL, "naive")
    announce("spmm_multihead Optimal kind=%s" % kind)
    pre = B.spmm_multihead(ptr.cuda(), idx.cuda(), val.cuda(), x.cuda(), n)
    assert pre.shape == (n, C)
    assert_close(_np(pre), oracle.spmm_prereduce(p, i, val.numpy(), x.numpy(), n), RTOL, ATOL, "prereduce")
    pre2 = B.run_spmm_multihead_configurable(ptr.cuda(), idx.cuda(), val.cuda(), x.cuda(), n, *(0,) * 9)
    assert torch.equal(pre, pre2)
    # backward accumulates into the caller's buffer
    g = torch.randn(n, H, C) * sc
    base = torch.randn(n, H, C) * sc
    gx = base.clone().cuda()
    announce("spmm_multihead_bwd kind=%s" % kind)
    B.spmm_multihead_bwd(ptr.cuda(), idx.cuda(), val.cuda(), g.cuda(), gx, n)
    ref = oracle.spmm_bwd(p, i, g.numpy(), n, n, val=val.numpy()).astype(np.float64) + base.numpy()
    assert_close(_np(gx), ref, RTOL, 2 * ATOL, "multihead bwd accumulate")


def test_gather_forward_backward():
    import cxgnncomp_backend as B
    torch.manual_seed(7)
    E, N, F = 5000, 700, 48
    dest = torch.randint(0, N, (E,))
    x = (torch.randn(E, F) / 4).cuda().requires_grad_(True)
    announce("gather E=%d N=%d F=%d" % (E, N, F))
    out = B.gather(x, dest.cuda(), N)
    g = torch.randn(N, F)
    out.backward(g.cuda())
    torch.cuda.synchronize()
    assert_close(_np(out), oracle.gather_fwd(_np(x), dest.numpy(), N), RTOL, ATOL, "gather fwd")
    assert np.array_equal(_np(x.grad), oracle.gather_bwd(g.numpy(), dest.numpy()))


def test_bad_arguments_raise_instead_of_exiting():
    import cxgnncomp_backend as B
    ptr, idx = _graph("uniform")
    n = ptr.shape[0] - 1
    x = torch.randn(n, 16)
    with pytest.raises(ValueError):
        B.run_spmm_configurable(ptr.cuda(), idx.cuda(), x, n)            # CPU tensor
    with pytest.raises(ValueError):
        B.run_spmm_configurable(ptr.cuda(), idx.cuda(), x.double().cuda(), n)   # wrong dtype
    with pytest.raises(ValueError):
        B.run_spmm_configurable(ptr.cuda(), idx.cuda(), x.cuda(), n + 5)  # more rows than ptr holds
    with pytest.raises(ValueError):
        B.run_spmm_configurable(ptr.cuda(), idx.cuda(), x.cuda().unsqueeze(0), n)  # vin must be 2D


@pytest.mark.parametrize("kind", ["uniform", "powerlaw", "empty_rows", "one_hub"])
@pytest.mark.parametrize("shape", [(4, 64), (8, 32), (2, 128), (2, 64), (4, 32), (2, 32), (8, 8), (16, 16), (4, 40), (3, 64), (4, 128)])
def test_spmm_multihead_head_sum_inside_the_kernel(kind, shape):
    """spmm_multihead(PreReduce / Optimal): out[N, C] summed over the heads.  Rows of heads x channels
    = 64, 128 or 256 floats with a power-of-two head count are summed by the gathering wave itself
    (cxg_spmm_prereduce_f32: rows inside a span, rows completed by the fix-up kernel in 'one_hub' and
    'powerlaw', rows without edges); the other shapes aggregate per head and sum afterwards.  Both
    against the oracle, deterministic, and a row prefix."""
    import cxgnncomp_backend as B
    H, C = shape
    ptr, idx = _graph(kind)
    n = ptr.shape[0] - 1
    E = idx.shape[0]
    torch.manual_seed(H * 100 + C)
    x = torch.randn(n, H, C) * _scale(ptr)
    val = torch.rand(E, H) - 0.3
    p, i = ptr.numpy(), idx.numpy()
    announce("spmm_multihead PreReduce kind=%s H=%d C=%d" % (kind, H, C))
    pc, ic, vc, xc = ptr.cuda(), idx.cuda(), val.cuda(), x.cuda()
    pre = B.spmm_multihead(pc, ic, vc, xc, n, B.SPMM_MULTIHEAD_SCHEDULE.PreReduce)
    assert pre.shape == (n, C)
    want = oracle.spmm_prereduce(p, i, val.numpy(), x.numpy(), n)
    assert_close(_np(pre), want, RTOL, ATOL, "prereduce")
    assert torch.equal(pre, B.spmm_multihead(pc, ic, vc, xc, n, B.SPMM_MULTIHEAD_SCHEDULE.Optimal))
    rows = n // 3
    part = B.spmm_multihead(pc, ic, vc, xc, rows, B.SPMM_MULTIHEAD_SCHEDULE.PreReduce)
    assert_close(_np(part), oracle.spmm_prereduce(p, i, val.numpy(), x.numpy(), rows), RTOL, ATOL, "prereduce prefix")


def test_prereduce_entry_point_rejects_other_shapes():
    from cxgnncomp_backend import _lib
    lib = _lib.load()
    ptr = torch.tensor([0, 2, 3], device="cuda")
    idx = torch.tensor([0, 1, 1], device="cuda")
    ws = torch.empty(lib.cxg_spmm_workspace_bytes(3, 512), dtype=torch.uint8, device="cuda")
    st = _lib.current_stream(ptr.device)

    def call(H, C):
        x = torch.zeros(2, H, C, device="cuda")
        val = torch.zeros(3, H, device="cuda")
        out = torch.zeros(2, C, device="cuda")
        return lib.cxg_spmm_prereduce_f32(ptr.data_ptr(), idx.data_ptr(), val.data_ptr(), None, x.data_ptr(), H * C,
                                          out.data_ptr(), C, 2, 3, H, C, 0, ws.data_ptr(), ws.numel(), st)
    assert call(4, 64) == 0 and call(2, 32) == 0
    assert call(3, 64) == -2 and call(4, 128) == -2 and call(4, 40) == -2      # CXG_ERR_UNSUPPORTED
    assert call(1, 64) == -1                                                   # one head: nothing to sum
    torch.cuda.synchronize()
