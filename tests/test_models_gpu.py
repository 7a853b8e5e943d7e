"""The layer stacks of cxgnncomp.model (SAGE / GCN / GIN / GAT / RGCN) on the GPU.

SAGE (sampled nested CSR, "CSR_Layer") and GCN (full graph, "CSR") are compared,
logits and input gradient, with a float64 restatement of the same stack built from the
oracle's PyTorch SpMM; GIN / GAT / RGCN are compared with their own layers applied by
hand over the per-layer row / edge prefixes (the layers themselves are checked in
test_package_gpu.py)."""
import copy

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from conftest import announce, assert_close
from oracle import pyref

pytestmark = pytest.mark.gpu
RTOL, ATOL = 2e-4, 2e-5


def _np(t):
    return t.detach().cpu().numpy()


def _batch(seed=0, feat=16):
    import cxgnncomp
    from cxgnncomp import synthetic as S
    ptr, idx, nn, ne = S.sampled_batch(num_seeds=64, fanouts=(5, 4, 3), id_space=4000, seed=seed)
    torch.manual_seed(seed)
    x = torch.randn(nn[-1], feat)
    return cxgnncomp.Batch(x, ptr, idx, torch.tensor(nn), torch.tensor(ne))


def _sum64(x, ptr, idx, rows):
    return pyref.spmm_torch(x, ptr, idx, rows, torch.ones(idx.shape[0], dtype=x.dtype))


def _mean64(x, ptr, idx, rows):
    s = _sum64(x, ptr, idx, rows)
    deg = (ptr[1:rows + 1] - ptr[:rows]).double().unsqueeze(1)
    return torch.where(deg > 0, s / deg.clamp(min=1), torch.zeros_like(s))


def _bn_relu(x, bn):
    return F.relu(F.batch_norm(x, None, None, bn.weight.double(), bn.bias.double(), True, 0.0, bn.eps))


def test_sage_model_on_sampled_batch():
    import cxgnncomp
    b = _batch(1)
    torch.manual_seed(3)
    model = cxgnncomp.SAGE(16, 32, 7, 3, 0.0, "CSR_Layer")
    ref = copy.deepcopy(model).double()
    x64 = b.x.double().requires_grad_(True)
    h = x64
    nn = [int(v) for v in b.num_node_in_layer]
    for i, conv in enumerate(ref.convs):
        rows = nn[2 - i]
        if conv.in_channels > conv.hidden_channels:
            out = _mean64(conv.lin_l(h), b.ptr, b.idx, rows)
        else:
            out = conv.lin_l(_mean64(h, b.ptr, b.idx, rows))
        h = out + conv.lin_r(h[:rows])
        if i < 2:
            h = _bn_relu(h, ref.bns[i])
    want = h.log_softmax(-1)
    g = torch.randn(nn[0], 7, dtype=torch.float64) / 8
    want.backward(g)
    announce("SAGE model, CSR_Layer")
    model = model.cuda()
    gb = copy.copy(b).to("cuda")
    gb.x = b.x.cuda().requires_grad_(True)
    got = model(gb)
    got.backward(g.float().cuda())
    assert got.shape == (nn[0], 7)
    assert_close(_np(got), want.detach().numpy(), RTOL, ATOL, "SAGE logits")
    assert_close(_np(gb.x.grad), x64.grad.numpy(), RTOL, ATOL, "SAGE grad x")
    w_got = model.convs[0].lin_l.weight.grad
    assert_close(_np(w_got), ref.convs[0].lin_l.weight.grad.numpy(), RTOL, ATOL, "SAGE grad lin_l")


def test_gcn_model_on_full_graph():
    import cxgnncomp
    from cxgnncomp import synthetic as S
    cxgnncomp.set_timers()
    ptr, idx = S.uniform_graph(900, 6000, seed=5)
    n = 900
    torch.manual_seed(6)
    x = torch.randn(n, 24) / 4
    model = cxgnncomp.GCN(24, 16, 5, 3, 0.0, "CSR")
    ref = copy.deepcopy(model).double()
    x64 = x.double().requires_grad_(True)
    h = x64
    for i, conv in enumerate(ref.convs):
        before = conv.in_channels > conv.out_channels
        t = conv.lin(h) if before else h
        t = _sum64(t, ptr, idx, n)
        if not before:
            t = conv.lin(t)
        h = t + conv.bias
        if i < 2:
            h = _bn_relu(h, ref.bns[i])
    want = h.log_softmax(-1)
    g = torch.randn(n, 5, dtype=torch.float64) / 8
    want.backward(g)
    announce("GCN model, CSR")
    model = model.cuda()
    b = cxgnncomp.Batch(x.cuda().requires_grad_(True), ptr.cuda(), idx.cuda(), torch.tensor([n, n, n, n]))
    got = model(b)
    got.backward(g.float().cuda())
    assert_close(_np(got), want.detach().numpy(), RTOL, 2 * ATOL, "GCN logits")
    sc = max(1.0, float(x64.grad.abs().max()))
    assert_close(_np(b.x.grad) / sc, x64.grad.numpy() / sc, RTOL, 2 * ATOL, "GCN grad x")


@pytest.mark.parametrize("kind", ["GIN", "GAT", "RGCN"])
def test_other_models_apply_their_layers_over_the_layer_prefixes(kind):
    import cxgnncomp
    cxgnncomp.set_timers()
    b = _batch(2).to("cuda")
    nn = [int(v) for v in b.num_node_in_layer]
    ne = [int(v) for v in b.num_edge_in_layer]
    torch.manual_seed(9)
    if kind == "GIN":
        model = cxgnncomp.GIN(16, 32, 7, 3, 0.0, "CSR_Layer").cuda()
    elif kind == "GAT":
        model = cxgnncomp.GAT(16, 32, 8, 3, 0.0, "CSR_Layer", heads=4, concat=True).cuda()
    else:
        model = cxgnncomp.RGCN(16, 32, 7, 3, 0.0, "CSR_Layer", num_rel=3, dataset_name="synthetic").cuda()
        b.etypes = torch.randint(0, 3, (ne[2],), device="cuda")
    announce("%s model, CSR_Layer" % kind)
    got = model(b)
    h = b.x
    for i, conv in enumerate(model.convs):
        k = 2 - i
        if kind == "GAT":
            h = conv(h, b.ptr, b.idx, num_dst=nn[k], num_src=nn[k + 1], num_edge=ne[k])
        elif kind == "RGCN":
            h = conv(h, b.ptr, b.idx, b.etypes[:ne[k]], nn[k])
        else:
            h = conv(h, b.ptr, b.idx, nn[k])
        if i < 2:
            h = F.relu(model.bns[i](h))
    want = h.log_softmax(-1)
    assert got.shape == want.shape == (nn[0], model.out_channels)
    assert torch.isfinite(got).all()
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-6)
    got.sum().backward()
    # every parameter the forward uses gets a finite gradient (MyRGCNConv keeps upstream's unused
    # single_linear, which gets none)
    used = [p for name, p in model.named_parameters() if "single_linear" not in name]
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in used)


def test_models_reject_other_graph_types():
    import cxgnncomp
    with pytest.raises(NotImplementedError):
        cxgnncomp.SAGE(4, 4, 2, 2, 0.0, "DGL")
