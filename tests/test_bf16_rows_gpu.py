"""bf16 rows on the gathered and / or stored side of the single-head aggregation, bf16 result
rows of the bf16-operand typed GEMM, bf16 A rows of the weight gradient: what the bf16 variant of
the relational layer keeps its pair-row tables in.

Stated tolerances: a value rounded to bf16 is off by at most 2^-9 relative; sums are formed in
fp32.  With bf16 INPUT rows the kernel is compared with the oracle on the same rounded inputs at
the fp32 bar (1e-4 / 1e-5); bf16 OUTPUT rows are compared with the correctly rounded oracle result,
allowing one bf16 unit in the last place (2^-8 relative) for sums that fall next to a rounding
boundary."""
import numpy as np
import pytest
import torch

import oracle
from conftest import announce, assert_close
from test_spmm_gpu import _graph, _scale

pytestmark = pytest.mark.gpu


def _np(t):
    return t.detach().float().cpu().numpy()


@pytest.mark.parametrize("kind", ["uniform", "powerlaw", "empty_rows", "one_hub"])
@pytest.mark.parametrize("feat", [128, 64, 100, 16, 4])
@pytest.mark.parametrize("weighted", [False, True])
def test_spmm_bf16_rows(kind, feat, weighted):
    from cxgnncomp_backend import _ops
    ptr, idx = _graph(kind)
    n, E = ptr.shape[0] - 1, idx.shape[0]
    torch.manual_seed(feat + 7 * weighted)
    x = torch.randn(n, feat) * _scale(ptr)
    val = (torch.rand(E) + 0.5) if weighted else None
    xb = x.to(torch.bfloat16)
    p, i = ptr.numpy(), idx.numpy()
    pc, ic = ptr.cuda(), idx.cuda()
    vc = None if val is None else val.cuda()
    vn = None if val is None else val.numpy()
    announce("spmm bf16 rows kind=%s F=%d weighted=%s" % (kind, feat, weighted))
    # bf16 gathered rows, fp32 sums
    got = _ops.spmm_bf16_rows(pc, ic, xb.cuda(), n, val=vc)
    assert got.dtype == torch.float32
    want = oracle.spmm(p, i, xb.float().numpy(), n, val=vn)
    assert_close(_np(got), want, 1e-4, 1e-5, "bf16 in, fp32 out")
    # fp32 gathered rows, bf16 stored rows: the correctly rounded fp32 result, one unit in the last place allowed
    got = _ops.spmm_bf16_rows(pc, ic, x.cuda(), n, val=vc, out_bf16=True)
    assert got.dtype == torch.bfloat16
    want = oracle.spmm(p, i, x.numpy(), n, val=vn)
    assert_close(_np(got), want, 2.0 ** -8, 1e-6, "fp32 in, bf16 out")
    exact = torch.from_numpy(want).to(torch.bfloat16).float().numpy()
    assert (np.abs(_np(got) - exact) > 0).mean() < 0.02        # nearly every element is the correctly rounded one
    # both, through a permutation of the weights and a row prefix
    rows = max(1, n // 3)
    if weighted:
        perm = torch.randperm(E)
        inv = torch.empty_like(perm)
        inv[perm] = torch.arange(E)
        got = _ops.spmm_bf16_rows(pc, ic, xb.cuda(), rows, val=val[perm].cuda(), val_perm=inv.cuda(), out_bf16=True)
    else:
        got = _ops.spmm_bf16_rows(pc, ic, xb.cuda(), rows, out_bf16=True, mean=True)
    want = oracle.spmm(p, i, xb.float().numpy(), rows, val=vn, mean=not weighted)
    assert_close(_np(got), want, 2.0 ** -8, 1e-6, "bf16 in, bf16 out, row prefix")


@pytest.mark.parametrize("K,N,R,M", [(128, 128, 16, 5000), (64, 96, 3, 1000), (96, 40, 4, 700), (128, 2, 1, 130)])
def test_typed_gemm_bf16_result_rows(K, N, R, M):
    """bf16 result rows of the bf16-operand typed GEMM, from bf16 A rows and from fp32 A rows rounded
    as they are staged (with a gather map), against the fp32-accumulated product of the same rounded
    operands rounded to bf16."""
    from cxgnncomp_backend import _typed
    gen = torch.Generator().manual_seed(K + N)
    a = torch.randn(M, K, generator=gen) / K ** 0.5
    w = torch.randn(R, K, N, generator=gen)
    types = torch.sort(torch.randint(0, R, (M,), generator=gen))[0]
    seg = torch.zeros(R + 1, dtype=torch.int64)
    seg[1:] = torch.bincount(types, minlength=R).cumsum(0)
    ab, wb = a.to(torch.bfloat16), w.to(torch.bfloat16)
    want = torch.bmm(ab.double().unsqueeze(1), wb.double()[types]).squeeze(1).numpy()
    announce("typed GEMM bf16 result rows K=%d N=%d" % (K, N))
    got = _typed.typed_gemm(ab.cuda(), w.cuda(), seg.cuda(), M, bf16=True, out_bf16=True)
    assert got.dtype == torch.bfloat16 and got.shape == (M, N)
    assert_close(_np(got), want, 2.0 ** -8, 1e-5, "bf16 A, bf16 C")
    src = torch.randint(0, M, (M,), generator=gen)
    got = _typed.typed_gemm(a.cuda(), w.cuda(), seg.cuda(), M, src_idx=src.cuda(), bf16=True, out_bf16=True)
    want = torch.bmm(ab[src].double().unsqueeze(1), wb.double()[types]).squeeze(1).numpy()
    assert_close(_np(got), want, 2.0 ** -8, 1e-5, "fp32 A rounded while staged, gathered, bf16 C")
    with pytest.raises(ValueError):
        _typed.typed_gemm(a.cuda(), w.cuda(), seg.cuda(), M, out_bf16=True)           # not with fp32 products


@pytest.mark.parametrize("K,N,R,M", [(128, 128, 16, 5000), (64, 48, 3, 1000)])
def test_weight_gradient_from_bf16_rows(K, N, R, M):
    from cxgnncomp_backend import _typed
    gen = torch.Generator().manual_seed(K * N)
    a = (torch.randn(M, K, generator=gen) / 8).to(torch.bfloat16)
    g = torch.randn(M + 3, N, generator=gen) / 8
    types = torch.sort(torch.randint(0, R, (M,), generator=gen))[0]
    seg = torch.zeros(R + 1, dtype=torch.int64)
    seg[1:] = torch.bincount(types, minlength=R).cumsum(0)
    dst = torch.randint(0, M + 3, (M,), generator=gen)
    src = torch.randperm(M, generator=gen)
    announce("weight gradient with bf16 A rows K=%d N=%d" % (K, N))
    got = _typed.typed_gemm_wgrad(a.cuda(), g.cuda(), seg.cuda(), M, R, src_idx=src.cuda(), dst_idx=dst.cuda(),
                                  precision="split6")
    want = torch.zeros(R, K, N, dtype=torch.float64)
    want.index_add_(0, types, torch.einsum("mk,mn->mkn", a[src].double(), g[dst].double()))
    sc = max(1.0, float(want.abs().max()))
    assert_close(_np(got) / sc, want.numpy() / sc, 1e-4, 1e-5, "wgrad, bf16 A rows")
    plain = _typed.typed_gemm_wgrad(a.cuda(), g[:M].contiguous().cuda(), seg.cuda(), M, R, precision="split6")
    want = torch.zeros(R, K, N, dtype=torch.float64)
    want.index_add_(0, types, torch.einsum("mk,mn->mkn", a.double(), g[:M].double()))
    assert_close(_np(plain) / sc, want.numpy() / sc, 1e-4, 1e-5, "wgrad, bf16 A rows, no maps")
