"""SDDMM, fused edge softmax and spmv through cxgnncomp_backend vs the oracle.

Tolerances: SDDMM is an fp32 dot product (1e-4 rel / 1e-5 abs at O(1) scale).
The softmax uses the hardware exponential (__expf, as the reference does,
src/cpp/src/edge_softmax.cu:25); its outputs lie in [0,1] and are compared at
2e-4 relative / 1e-6 absolute against the double-precision oracle.  The softmax
backward is plain fp32 arithmetic on the saved output: 1e-4 / 1e-5, the bar of
every fp32 aggregation, against the oracle's backward of that same output."""
import numpy as np
import pytest
import torch

import oracle
from conftest import announce, assert_close
from test_spmm_gpu import ATOL, RTOL, _graph

pytestmark = pytest.mark.gpu
SM_BWD_RTOL, SM_BWD_ATOL = 1e-4, 1e-5


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
    # The backward consumes the saved forward output (edge_softmax.cu:134-177), so the oracle's
    # backward is run on the kernel's own output: the hardware exp of the forward (2e-4) then does
    # not enter, and both gradients are held to the fp32 aggregation bar, 1e-4 / 1e-5.
    gd, gs = oracle.edge_softmax_bwd(p, i, g.numpy(), mask, _np(out), n, n, slope)
    assert_close(_np(ad.grad), gd, SM_BWD_RTOL, SM_BWD_ATOL, "grad att_dst")
    assert_close(_np(asr.grad), gs, SM_BWD_RTOL, SM_BWD_ATOL, "grad att_src")
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


@pytest.mark.parametrize("heads", [1, 2, 4, 8])
def test_edge_softmax_degrees_at_the_step_boundaries(heads):
    """Rows whose lengths sit on either side of what the kernels switch on: 64 edges (one
    step of a wave), 512 edges (rows handed to the whole block), empty rows between them,
    a long row first and last in a wave's 64 rows, and a row count that fills neither the
    last wave nor the last block."""
    import cxgnncomp_backend as B
    pattern = [64, 0, 63, 1, 65, 512, 513, 0, 0, 128, 511, 2, 127, 129, 0, 700, 3, 64, 64, 1, 0, 0, 31, 33]
    deg = torch.tensor((pattern * 15)[:331], dtype=torch.int64)
    deg[0] = 900        # a row left to the block, first of its wave
    deg[63] = 600       # ... and last of its wave
    deg[64] = 0
    deg[330] = 1500     # the very last row
    n = deg.shape[0]
    ptr = torch.zeros(n + 1, dtype=torch.int64)
    ptr[1:] = torch.cumsum(deg, 0)
    E = int(ptr[-1])
    g0 = torch.Generator().manual_seed(5)
    idx = torch.randint(0, n, (E,), generator=g0)
    att_dst = torch.randn(n, heads, generator=g0) * 3
    att_src = torch.randn(n, heads, generator=g0) * 3
    slope = 0.2
    ad = att_dst.cuda().requires_grad_(True)
    asr = att_src.cuda().requires_grad_(True)
    announce("edge_attention boundary degrees H=%d" % heads)
    out = B.edge_attention(ptr=ptr.cuda(), idx=idx.cuda(), att_dst=ad, att_src=asr, num_edge=E, relu_l=slope)
    g = torch.randn(E, heads, generator=g0)
    out.backward(g.cuda())
    torch.cuda.synchronize()
    p, i = ptr.numpy(), idx.numpy()
    ref, mask = oracle.edge_softmax_fwd(p, i, att_dst.numpy(), att_src.numpy(), E, slope)
    assert_close(_np(out), ref, 2e-4, 1e-6, "softmax fwd")
    gd, gs = oracle.edge_softmax_bwd(p, i, g.numpy(), mask, _np(out), n, n, slope)
    assert_close(_np(ad.grad), gd, SM_BWD_RTOL, SM_BWD_ATOL, "grad att_dst")
    assert_close(_np(asr.grad), gs, SM_BWD_RTOL, SM_BWD_ATOL, "grad att_src")
    # a second run gives the same bits
    ad2 = att_dst.cuda().requires_grad_(True)
    out2 = B.edge_attention(ptr=ptr.cuda(), idx=idx.cuda(), att_dst=ad2, att_src=asr.detach(), num_edge=E, relu_l=slope)
    out2.backward(g.cuda())
    assert torch.equal(out, out2) and torch.equal(ad.grad, ad2.grad)


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


ATT_SHAPES = [(4, 64), (1, 128), (8, 16), (3, 40), (2, 7), (1, 1), (4, 256), (16, 64), (8, 512), (2, 6)]


@pytest.mark.parametrize("shape", ATT_SHAPES)
@pytest.mark.parametrize("n_src,n_dst", [(1, 1), (1000, 0), (1000, 333), (70001, 70001), (70001, 12345)])
def test_attention_logits_forward_backward(shape, n_src, n_dst):
    """Both per-node GAT logits and their three gradients against the upstream expressions
    ``(x * att).sum(-1)`` differentiated in double precision.  Tolerance: 1e-4 relative /
    1e-5 absolute on values scaled to O(1); the parameter gradients are sums over all
    nodes and are compared relative to their largest entry."""
    from cxgnncomp_backend import _ops
    H, C = shape
    if H * C >= 1024 and n_src > 1000:
        n_src, n_dst = 5003, min(n_dst, 5003)
    torch.manual_seed(H * 1000 + C + n_src)
    x = (torch.randn(n_src, H, C) / C ** 0.5)
    a_s, a_d = torch.randn(1, H, C), torch.randn(1, H, C)
    gs, gd = torch.randn(n_src, H), torch.randn(n_dst, H)
    xd = x.double().requires_grad_(True)
    asd, add = a_s.double().requires_grad_(True), a_d.double().requires_grad_(True)
    ref_s = (xd * asd).sum(-1)
    ref_d = (xd[:n_dst] * add).sum(-1)
    (ref_s * gs.double()).sum().backward(retain_graph=True)
    (ref_d * gd.double()).sum().backward()
    announce("attention_logits H=%d C=%d n_src=%d n_dst=%d" % (H, C, n_src, n_dst))
    out_s, out_d = _ops.attention_logits(x.cuda(), a_s.cuda(), a_d.cuda(), n_dst)
    torch.cuda.synchronize()
    assert out_s.shape == (n_src, H) and out_d.shape == (n_dst, H)
    assert_close(_np(out_s), ref_s.detach().numpy(), RTOL, ATOL, "logits src")
    assert_close(_np(out_d), ref_d.detach().numpy(), RTOL, ATOL, "logits dst")
    announce("attention_logits_bwd H=%d C=%d n_src=%d n_dst=%d" % (H, C, n_src, n_dst))
    gx, ga_s, ga_d = _ops.attention_logits_bwd(x.cuda(), a_s.cuda(), a_d.cuda(), gs.cuda(), gd.cuda())
    gx2, ga_s2, ga_d2 = _ops.attention_logits_bwd(x.cuda(), a_s.cuda(), a_d.cuda(), gs.cuda(), gd.cuda())
    torch.cuda.synchronize()
    assert_close(_np(gx), xd.grad.numpy(), RTOL, ATOL, "grad x")
    for got, ref, name in ((ga_s, asd.grad, "grad att_src"), (ga_d, add.grad, "grad att_dst")):
        ref = ref.numpy().reshape(H, C)
        scale = max(1.0, float(np.abs(ref).max()))
        assert_close(_np(got) / scale, ref / scale, RTOL, ATOL, name)
    assert torch.equal(ga_s, ga_s2) and torch.equal(ga_d, ga_d2) and torch.equal(gx, gx2)
    # adding into an existing gradient of x
    base = torch.randn(n_src, H, C, generator=torch.Generator().manual_seed(8))
    acc = base.cuda()
    gx3, ga_s3, _ = _ops.attention_logits_bwd(x.cuda(), a_s.cuda(), a_d.cuda(), gs.cuda(), gd.cuda(), add_to=acc)
    assert gx3.data_ptr() == acc.data_ptr() and torch.equal(ga_s3, ga_s)
    assert_close(_np(acc), base.numpy() + xd.grad.numpy(), RTOL, ATOL, "grad x added in place")


PROJ_SHAPES = [(128, 4), (100, 4), (64, 8), (256, 2), (4, 1), (8, 4), (16, 8), (36, 1), (128, 8), (252, 4)]


@pytest.mark.parametrize("shape", PROJ_SHAPES)
@pytest.mark.parametrize("n_src,n_dst", [(1, 1), (1000, 0), (1000, 333), (70001, 70001), (70001, 12345)])
def test_attention_logits_from_the_layer_input(shape, n_src, n_dst):
    """The logits taken from the layer's input, ``x @ m[:H].T`` and ``x[:n_dst] @ m[H:].T``, and
    their gradients against the same expressions differentiated in double precision (same
    tolerances as the test above); rows of x with a stride, adding into an existing
    gradient, and the call that skips grad_x."""
    from cxgnncomp_backend import _ops
    n_in, H = shape
    assert _ops.logits_proj_supported(n_in, H)
    torch.manual_seed(n_in * 100 + H + n_src)
    wide = torch.randn(n_src, n_in + 4) / n_in ** 0.5
    x = wide[:, :n_in]
    m = torch.randn(2 * H, n_in)
    gs, gd = torch.randn(n_src, H), torch.randn(n_dst, H)
    xd, md = x.double().requires_grad_(True), m.double().requires_grad_(True)
    ref_s, ref_d = xd @ md[:H].t(), xd[:n_dst] @ md[H:].t()
    ((ref_s * gs.double()).sum() + (ref_d * gd.double()).sum()).backward()
    announce("attention_logits_proj in=%d H=%d n_src=%d n_dst=%d" % (n_in, H, n_src, n_dst))
    xg = wide.cuda()[:, :n_in]                       # row stride n_in + 4
    out_s, out_d = _ops.attention_logits_proj(xg, m.cuda(), n_dst, H)
    torch.cuda.synchronize()
    assert out_s.shape == (n_src, H) and out_d.shape == (n_dst, H)
    assert_close(_np(out_s), ref_s.detach().numpy(), RTOL, ATOL, "logits src")
    assert_close(_np(out_d), ref_d.detach().numpy(), RTOL, ATOL, "logits dst")
    out_s2, _ = _ops.attention_logits_proj(x.contiguous().cuda(), m.cuda(), n_dst, H)
    assert torch.equal(out_s, out_s2)
    announce("attention_logits_proj_bwd in=%d H=%d n_src=%d n_dst=%d" % (n_in, H, n_src, n_dst))
    gx, gm = _ops.attention_logits_proj_bwd(xg, m.cuda(), gs.cuda(), gd.cuda(), H)
    gx2, gm2 = _ops.attention_logits_proj_bwd(xg, m.cuda(), gs.cuda(), gd.cuda(), H)
    none, gm3 = _ops.attention_logits_proj_bwd(xg, m.cuda(), gs.cuda(), gd.cuda(), H, need_x=False)
    torch.cuda.synchronize()
    assert none is None and torch.equal(gm, gm2) and torch.equal(gm, gm3) and torch.equal(gx, gx2)
    assert_close(_np(gx), xd.grad.numpy(), RTOL, ATOL, "grad x")
    ref_m = md.grad.numpy()
    scale = max(1.0, float(np.abs(ref_m).max()))
    assert_close(_np(gm) / scale, ref_m / scale, RTOL, ATOL, "grad m")
    base = torch.randn(n_src, n_in, generator=torch.Generator().manual_seed(8))
    acc = base.cuda()
    gx3, gm4 = _ops.attention_logits_proj_bwd(xg, m.cuda(), gs.cuda(), gd.cuda(), H, add_to=acc)
    assert gx3.data_ptr() == acc.data_ptr() and torch.equal(gm4, gm)
    assert_close(_np(acc), base.numpy() + xd.grad.numpy(), RTOL, ATOL, "grad x added in place")


def test_attention_logits_from_the_layer_input_rejects_other_shapes():
    from cxgnncomp_backend import _ops
    for n_in, H in [(130, 4), (260, 4), (128, 3), (128, 16), (2, 1)]:
        assert not _ops.logits_proj_supported(n_in, H)
    x, m = torch.zeros(8, 130, device="cuda"), torch.zeros(8, 130, device="cuda")
    with pytest.raises(RuntimeError):
        _ops.attention_logits_proj(x, m, 8, 4)


def test_attention_logits_op_autograd():
    """The autograd wrapper used by MyGATConv: gradients flow to x and both parameters."""
    import cxgnncomp
    from cxgnncomp.graph_conv import AttentionLogitsOP
    torch.manual_seed(3)
    n, H, C, nd = 4097, 4, 32, 1500
    x = torch.randn(n, H, C, device="cuda", requires_grad=True)
    a_s = torch.randn(1, H, C, device="cuda", requires_grad=True)
    a_d = torch.randn(1, H, C, device="cuda", requires_grad=True)
    gs, gd = torch.randn(n, H, device="cuda"), torch.randn(nd, H, device="cuda")
    announce("AttentionLogitsOP autograd")
    s, d = AttentionLogitsOP.apply(x, a_s, a_d, nd)
    ((s * gs).sum() + (d * gd).sum()).backward()
    got = [x.grad.clone(), a_s.grad.clone(), a_d.grad.clone()]
    x.grad = a_s.grad = a_d.grad = None
    (((x * a_s).sum(-1) * gs).sum() + ((x[:nd] * a_d).sum(-1) * gd).sum()).backward()
    for g, r in zip(got, [x.grad, a_s.grad, a_d.grad]):
        assert g.shape == r.shape
        scale = max(1.0, float(r.abs().max()))
        assert_close(_np(g) / scale, _np(r) / scale, 1e-4, 2e-5, "autograd")


@pytest.mark.parametrize("kind", ["uniform", "powerlaw", "empty_rows", "one_hub"])
@pytest.mark.parametrize("shape", [(4, 64), (8, 32), (2, 128), (1, 256), (8, 64)])
def test_spmm_with_edge_dot_products(kind, shape):
    """cxg_spmm_weighted_dot_f32 on the transposed graph: the aggregation equals the plain
    weighted SpMM bit for bit, and the per-edge products equal the CSR SDDMM of the original
    graph (the oracle's), written at the original edge positions."""
    from cxgnncomp_backend import _ops
    H, C = shape
    ptr, idx = _graph(kind)
    n = ptr.shape[0] - 1
    E = idx.shape[0]
    torch.manual_seed(11)
    xs = torch.randn(n, H, C) / 8
    g = torch.randn(n, H, C) / 8
    ev = torch.rand(E, H)
    pc, ic = ptr.cuda(), idx.cuda()
    tg = _ops.transposed(pc, ic, n, n)
    announce("spmm_dot kind=%s H=%d C=%d" % (kind, H, C))
    dot = torch.full((E, H), float("nan"), device="cuda")
    gx, dot = _ops.spmm_dot(tg.ptr_t, tg.idx_t, g.cuda(), n, ev.cuda(), tg.perm, xs.cuda(), dot)
    want_gx = _ops.spmm(tg.ptr_t, tg.idx_t, g.cuda(), n, val=ev.cuda(), val_perm=tg.perm)
    torch.cuda.synchronize()
    assert torch.equal(gx, want_gx)
    rows = np.repeat(np.arange(n), np.diff(ptr.numpy()))
    ref = oracle.sddmm(idx.numpy(), rows, xs.numpy(), g.numpy())
    assert_close(_np(dot), ref.reshape(E, H), RTOL, ATOL, "edge dot products")
    # untransposed form (no permutation): products land at the edge's own position
    dot2 = torch.empty(E, H, device="cuda")
    out2, dot2 = _ops.spmm_dot(pc, ic, xs.cuda(), n, ev.cuda(), None, g.cuda(), dot2)
    assert torch.equal(out2, _ops.spmm(pc, ic, xs.cuda(), n, val=ev.cuda()))
    assert_close(_np(dot2), ref.reshape(E, H), RTOL, ATOL, "edge dot products, CSR order")
    # products left in the transposed graph's edge order (contiguous stores): the same values,
    # row k of this result is row perm[k] of the first
    dot3 = torch.full((E, H), float("nan"), device="cuda")
    gx3, dot3 = _ops.spmm_dot(tg.ptr_t, tg.idx_t, g.cuda(), n, ev.cuda(), tg.perm, xs.cuda(), dot3, dot_at_edge=True)
    assert torch.equal(gx3, want_gx)
    assert torch.equal(dot3, dot[tg.perm])
    inv = _ops.inverse_perm_transposed(tg)
    assert torch.equal(inv[tg.perm], torch.arange(E, device="cuda"))
    assert torch.equal(dot3[inv], dot)


@pytest.mark.parametrize("kind", ["uniform", "powerlaw", "empty_rows", "one_hub", "c2", "empty_runs"])
@pytest.mark.parametrize("feat", [128, 64, 100, 36, 24, 16])
def test_spmm_with_edge_dot_products_on_narrow_rows(kind, feat):
    """cxg_spmm_weighted_dot_f32 for one head of 16 .. 128 channels (weights through the
    transposition's permutation, products left at the edge's own position in the reversed graph):
    the aggregation equals the plain weighted SpMM bit for bit, the products equal the oracle's
    SDDMM of the original graph read through the permutation; rows of the reversed graph that
    cross spans, hubs, rows without edges."""
    from cxgnncomp import synthetic as S
    from cxgnncomp_backend import _ops
    from test_spmm_gpu import _graph_with_empty_runs
    if kind == "c2":
        if feat not in (128, 36):
            pytest.skip("the large graph runs two widths")
        ptr, idx = S.powerlaw_directed_symmetrised(169343, 1166243, seed=3)
    elif kind == "empty_runs":
        ptr, idx, _ = _graph_with_empty_runs(5)
    else:
        ptr, idx = _graph(kind)
    n = ptr.shape[0] - 1
    E = idx.shape[0]
    assert _ops.spmm_dot_supported(1, feat, at_edge=True) and (feat == 256 or not _ops.spmm_dot_supported(1, feat))
    torch.manual_seed(feat)
    xs = torch.randn(n, 1, feat) / 8
    g = torch.randn(n, 1, feat) / 8
    ev = torch.rand(E, 1)
    pc, ic = ptr.cuda(), idx.cuda()
    tg = _ops.transposed(pc, ic, n, n)
    announce("spmm_dot narrow rows kind=%s F=%d n=%d E=%d" % (kind, feat, n, E))
    dot = torch.full((E, 1), float("nan"), device="cuda")
    gx, dot = _ops.spmm_dot(tg.ptr_t, tg.idx_t, g.cuda(), n, ev.cuda(), tg.perm, xs.cuda(), dot, dot_at_edge=True)
    want_gx = _ops.spmm(tg.ptr_t, tg.idx_t, g.cuda().view(n, feat), n, val=ev.cuda().view(-1), val_perm=tg.perm)
    torch.cuda.synchronize()
    assert torch.equal(gx.view(n, feat), want_gx)
    rows = np.repeat(np.arange(n), np.diff(ptr.numpy()))
    ref = oracle.sddmm(idx.numpy(), rows, xs.numpy(), g.numpy()).reshape(E, 1)
    perm = tg.perm.cpu().numpy()
    assert_close(_np(dot), ref[perm], RTOL, ATOL, "edge dot products in the reversed graph's edge order")
    gx2, dot2 = _ops.spmm_dot(tg.ptr_t, tg.idx_t, g.cuda(), n, ev.cuda(), tg.perm, xs.cuda(), torch.empty_like(dot),
                              dot_at_edge=True)
    assert torch.equal(gx2, gx) and torch.equal(dot2, dot)
    with pytest.raises(ValueError):
        _ops.spmm_dot(tg.ptr_t, tg.idx_t, g.cuda(), n, ev.cuda(), tg.perm, xs.cuda(), dot)      # not at the edge


@pytest.mark.parametrize("kind", ["uniform", "powerlaw", "empty_rows", "one_hub"])
@pytest.mark.parametrize("heads", [1, 2, 4, 8, 3])
def test_edge_softmax_backward_reads_the_gradient_through_positions(kind, heads):
    """cxg_edge_softmax_bwd_at_f32: with the gradient rows stored in another edge order and the
    position of every edge's row handed over, the result is bit for bit that of
    cxg_edge_softmax_bwd_f32 on the gradient in CSR order (the walk kernels of 1, 2, 4, 8 heads
    and the row kernel for other head counts)."""
    from cxgnncomp_backend import _ops
    ptr, idx = _graph(kind)
    n = ptr.shape[0] - 1
    E = idx.shape[0]
    gen = torch.Generator().manual_seed(heads + 17)
    pc, ic = ptr.cuda(), idx.cuda()
    out, mask = _ops.edge_softmax_fwd(pc, ic, torch.randn(n, heads, generator=gen).cuda(),
                                      torch.randn(n, heads, generator=gen).cuda(), E, 0.2)
    grad = torch.randn(E, heads, generator=gen).cuda()
    where = torch.randperm(E, generator=gen).cuda()            # edge k's row sits at where[k]
    moved = torch.empty_like(grad)
    moved[where] = grad
    announce("edge_softmax_bwd with gradient positions kind=%s H=%d" % (kind, heads))
    gd, te = _ops.edge_softmax_bwd(pc, out, mask, grad, n, 0.2)
    gd2, te2 = _ops.edge_softmax_bwd(pc, out, mask, moved, n, 0.2, grad_pos=where)
    torch.cuda.synchronize()
    assert torch.equal(gd, gd2) and torch.equal(te, te2)


@pytest.mark.parametrize("feat", [1, 2, 4, 8, 3, 16, 100])
def test_gather_rows_all_widths(feat):
    """out[e] = in[sel[e]]: the one-thread-per-row path for rows of 1, 2, 4, 8 floats and the
    wave-per-row path for the others, bit-exact."""
    from cxgnncomp_backend import _ops
    g0 = torch.Generator().manual_seed(feat)
    inp = torch.randn(5000, feat, generator=g0)
    sel = torch.randint(0, 5000, (70001,), generator=g0)
    announce("gather_rows feat=%d" % feat)
    out = _ops.gather_rows(inp.cuda(), sel.cuda())
    assert torch.equal(out.cpu(), inp[sel])
    assert _ops.gather_rows(inp.cuda(), sel[:0].cuda()).shape == (0, feat)


@pytest.mark.parametrize("kind", ["uniform", "powerlaw", "empty_rows", "one_hub"])
@pytest.mark.parametrize("shape", [(4, 64), (2, 32), (1, 40), (8, 64)])
def test_weighted_spmm_with_bias(kind, shape):
    """cxg_spmm_weighted_bias_f32: the bias reaches every row exactly once -- rows that end
    inside a span, rows completed by the fix-up kernel (one_hub) and empty rows -- so the result
    equals the plain weighted SpMM plus the bias bit for bit."""
    from cxgnncomp_backend import _ops
    H, C = shape
    ptr, idx = _graph(kind)
    n = ptr.shape[0] - 1
    E = idx.shape[0]
    torch.manual_seed(13)
    x = (torch.randn(n, H, C) / 8).cuda()
    ev = torch.rand(E, H).cuda()
    bias = torch.randn(H * C).cuda()
    announce("spmm weighted + bias kind=%s H=%d C=%d" % (kind, H, C))
    got = _ops.spmm(ptr.cuda(), idx.cuda(), x, n, val=ev, bias=bias)
    want = _ops.spmm(ptr.cuda(), idx.cuda(), x, n, val=ev) + bias.view(1, H, C)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
