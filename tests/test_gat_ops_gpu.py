"""SDDMM, fused edge softmax and spmv through cxgnncomp_backend vs the oracle.

Tolerances: SDDMM is an fp32 dot product (1e-4 rel / 1e-5 abs at O(1) scale).
The softmax uses the hardware exponential (__expf, as the reference does,
src/cpp/src/edge_softmax.cu:25); its outputs lie in [0,1] and are compared at
2e-4 relative / 1e-6 absolute against the double-precision oracle."""
import numpy as np
import pytest
import torch

import oracle
from conftest import announce, assert_close
from test_spmm_gpu import ATOL, RTOL, _graph

pytestmark = pytest.mark.gpu


def _np(t):
    return t.detach().cpu().numpy()


def _coo(ptr, idx):
    n = ptr.shape[0] - 1
    dst = torch.repeat_interleave(torch.arange(n), ptr[1:] - ptr[:-1])
    return idx.clone(), dst


@pytest.mark.parametrize("kind", ["uniform", "powerlaw", "empty_rows", "one_hub"])
@pytest.mark.parametrize("shape", [(4, 64), (1, 128), (1, 64), (2, 32), (3, 40), (1, 300), (8, 8), (1, 4), (1, 8),
                                   (2, 4), (1, 16), (1, 32), (4, 8), (4, 16), (4, 32), (8, 16), (2, 64), (1, 12)])
@pytest.mark.parametrize("dst_heads", [True, False])
def test_sddmm_coo_and_csr(kind, shape, dst_heads):
    import cxgnncomp_backend as B
    H, C = shape
    ptr, idx = _graph(kind)
    n = ptr.shape[0] - 1
    E = idx.shape[0]
    torch.manual_seed(8)
    a = torch.randn(n, H, C) / C ** 0.5
    b = torch.randn(n, H, C) if dst_heads else torch.randn(n, C)
    src, dst = _coo(ptr, idx)
    ref = oracle.sddmm(src.numpy(), dst.numpy(), a.numpy(), b.numpy())
    out = torch.zeros(E, H).cuda()
    announce("run_sddmm kind=%s H=%d C=%d dst_heads=%s" % (kind, H, C, dst_heads))
    B.run_sddmm(src.cuda(), dst.cuda(), a.cuda(), b.cuda(), out, E)
    torch.cuda.synchronize()
    assert_close(_np(out), ref, RTOL, ATOL, "sddmm coo")
    announce("run_sddmm_vertex_centric kind=%s H=%d C=%d dst_heads=%s" % (kind, H, C, dst_heads))
    out2 = B.run_sddmm_vertex_centric(ptr.cuda(), idx.cuda(), a.cuda(), b.cuda(), n, *(0,) * 9)
    torch.cuda.synchronize()
    assert out2.shape == (E, H)
    assert_close(_np(out2), ref, RTOL, ATOL, "sddmm csr")


def test_sddmm_toy_coo():
    """Hand-computable case: 3 edges, 2 heads, 2 channels."""
    import cxgnncomp_backend as B
    src = torch.tensor([0, 1, 1])
    dst = torch.tensor([1, 0, 1])
    a = torch.tensor([[[1., 2.], [3., 4.]], [[5., 6.], [7., 8.]]])      # [2,2,2]
    b = torch.tensor([[1., 10.], [100., 1000.]])                         # [2,2], shared by heads
    out = torch.zeros(3, 2).cuda()
    announce("sddmm toy")
    B.run_sddmm(src.cuda(), dst.cuda(), a.cuda(), b.cuda(), out, 3)
    want = [[1 * 100 + 2 * 1000, 3 * 100 + 4 * 1000], [5 + 60, 7 + 80], [500 + 6000, 700 + 8000]]
    assert _np(out).tolist() == want


@pytest.mark.parametrize("kind", ["uniform", "powerlaw", "empty_rows", "one_hub"])
@pytest.mark.parametrize("heads", [1, 4, 3, 8])
def test_edge_softmax_forward_backward(kind, heads):
    import cxgnncomp_backend as B
    ptr, idx = _graph(kind)
    n = ptr.shape[0] - 1
    E = idx.shape[0]
    torch.manual_seed(9)
    att_dst = torch.randn(n, heads)
    att_src = torch.randn(n, heads)
    slope = 0.2
    ad = att_dst.cuda().requires_grad_(True)
    asr = att_src.cuda().requires_grad_(True)
    announce("edge_attention kind=%s H=%d" % (kind, heads))
    out = B.edge_attention(ptr=ptr.cuda(), idx=idx.cuda(), att_dst=ad, att_src=asr, num_edge=E,
                           relu_l=slope)
    g = torch.randn(E, heads)
    out.backward(g.cuda())
    torch.cuda.synchronize()
    p, i = ptr.numpy(), idx.numpy()
    ref, mask = oracle.edge_softmax_fwd(p, i, att_dst.numpy(), att_src.numpy(), E, slope)
    assert out.shape == (E, heads)
    assert_close(_np(out), ref, 2e-4, 1e-6, "softmax fwd")
    # backward of the oracle on the oracle's own forward output
    gd, gs = oracle.edge_softmax_bwd(p, i, g.numpy(), mask, ref, n, n, slope)
    assert_close(_np(ad.grad), gd, 1e-3, 2e-5, "grad att_dst")
    assert_close(_np(asr.grad), gs, 1e-3, 2e-5, "grad att_src")
    # rows sum to one
    if E:
        sums = oracle.spmv(p, np.arange(E), _np(out)[:, 0], n)
        deg = p[1:] - p[:-1]
        assert np.allclose(sums[deg > 0], 1.0, atol=1e-5)


@pytest.mark.parametrize("kind", ["uniform", "powerlaw", "empty_rows", "one_hub"])
def test_spmv_and_edge_value_degree(kind):
    import cxgnncomp_backend as B
    ptr, idx = _graph(kind)
    n = ptr.shape[0] - 1
    E = idx.shape[0]
    torch.manual_seed(10)
    v = torch.randn(n) / 70
    announce("spmv kind=%s" % kind)
    out = B.spmv(ptr.cuda(), idx.cuda(), v.cuda(), n)
    assert_close(_np(out), oracle.spmv(ptr.numpy(), idx.numpy(), v.numpy(), n), RTOL, ATOL, "spmv")
    announce("edge_value_degree kind=%s" % kind)
    ev = B.edge_value_degree(ptr.cuda(), n, E)
    assert np.array_equal(_np(ev), oracle.edge_value_degree(ptr.numpy(), n, E))


@pytest.mark.parametrize("kind", ["uniform", "powerlaw", "empty_rows", "one_hub"])
@pytest.mark.parametrize("width", [1, 2, 4, 8])
@pytest.mark.parametrize("with_sel", [True, False])
def test_segment_gather_sum(kind, width, with_sel):
    """Edge-parallel segmented row sums (the softmax source-gradient kernel) against the
    oracle's SpMM on the same rows; rows cross 64-edge steps and edge spans in 'one_hub'
    and 'powerlaw', 'empty_rows' has rows that must come out as 0."""
    from cxgnncomp_backend import _ops
    ptr, idx = _graph(kind)
    n = ptr.shape[0] - 1
    E = idx.shape[0]
    torch.manual_seed(11 + width)
    scale = 1.0 / max(1.0, float((ptr[1:] - ptr[:-1]).max()) ** 0.5)
    if with_sel:
        table = torch.randn(int(idx.max()) + 1, width) * scale
        sel = idx
    else:
        table = torch.randn(E, width) * scale
        sel = None
    inp = table[:, 0].contiguous() if width == 1 else table
    announce("segment_gather_sum kind=%s W=%d sel=%s" % (kind, width, with_sel))
    rows32 = _ops.csr_row_ids32(ptr.cuda(), n, E)
    want_rows = np.repeat(np.arange(n), np.diff(ptr.numpy()))
    assert rows32.dtype == torch.int32 and np.array_equal(_np(rows32), want_rows)
    got = _ops.narrow_gather_sum(ptr.cuda(), None if sel is None else sel.cuda(), inp.cuda(), n, rows32=rows32)
    src = idx.numpy() if with_sel else np.arange(E)
    want = oracle.spmm(ptr.numpy(), src, table.numpy(), n)
    assert_close(_np(got).reshape(n, width), want, RTOL, ATOL, "segment_gather_sum")
    old = _ops.narrow_gather_sum(ptr.cuda(), None if sel is None else sel.cuda(), inp.cuda(), n)
    assert_close(_np(old).reshape(n, width), want, RTOL, ATOL, "narrow_gather_sum")
    again = _ops.narrow_gather_sum(ptr.cuda(), None if sel is None else sel.cuda(), inp.cuda(), n, rows32=rows32)
    assert torch.equal(got, again)                      # deterministic


def test_segment_gather_sum_multi_step_spans():
    """2.33M edges: spans of 192 edges = three 64-edge steps per wave, so rows are carried
    from step to step inside a span as well as across spans."""
    from cxgnncomp import synthetic as S
    from cxgnncomp_backend import _ops
    ptr, idx = S.powerlaw_directed_symmetrised(169343, 1166243, seed=2)
    n, E = ptr.shape[0] - 1, idx.shape[0]
    torch.manual_seed(5)
    table = torch.randn(n, 4) / float((ptr[1:] - ptr[:-1]).max()) ** 0.5
    announce("segment_gather_sum 2.33M edges W=4")
    pc, ic = ptr.cuda(), idx.cuda()
    rows32 = _ops.csr_row_ids32(pc, n, E)
    got = _ops.narrow_gather_sum(pc, ic, table.cuda(), n, rows32=rows32)
    want = oracle.spmm(ptr.numpy(), idx.numpy(), table.numpy(), n)
    assert_close(_np(got), want, RTOL, ATOL, "segment_gather_sum, multi-step spans")
