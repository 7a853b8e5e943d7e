"""cxg_spmm_sum_f32_noalloc (the entry point that neither allocates nor takes a workspace)
against cxg_spmm_sum_f32, both called through the C ABI.

The two share their kernels, so the results must be bit-identical.  Two calls in a row, the
second on a smaller graph, show that what the first call left in the built-in scratch array
does not leak into the second; a third, oversized request must be rejected.
"""
import numpy as np
import pytest
import torch

import oracle
from conftest import announce, assert_close

pytestmark = pytest.mark.gpu


def _call_workspace(lib, L, ptr, idx, x, n, feat, flags=0):
    out = torch.full((n, feat), float("nan"), device=x.device)
    nbytes = lib.cxg_spmm_workspace_bytes(idx.shape[0], feat)
    ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=x.device)
    L.check(lib.cxg_spmm_sum_f32(ptr.data_ptr(), idx.data_ptr(), x.data_ptr(), feat, out.data_ptr(), feat,
                                 n, idx.shape[0], feat, flags, ws.data_ptr(), ws.numel(),
                                 L.current_stream(x.device)))
    return out


def _call_noalloc(lib, L, ptr, idx, x, n, feat, flags=0):
    out = torch.full((n, feat), float("nan"), device=x.device)
    L.check(lib.cxg_spmm_sum_f32_noalloc(ptr.data_ptr(), idx.data_ptr(), x.data_ptr(), feat, out.data_ptr(),
                                         feat, n, idx.shape[0], feat, flags, L.current_stream(x.device)))
    return out


def test_noalloc_matches_workspace_entry_point_twice():
    from cxgnncomp_backend import _lib as L
    from cxgnncomp import synthetic as S
    lib = L.load()
    dev = torch.device("cuda:0")
    cases = [
        # a heavy-tailed graph whose hub rows cross many spans, then a smaller uniform one
        ("powerlaw", S.powerlaw_directed_symmetrised(60000, 600000, max_degree=9000, seed=5), 128, 0),
        ("uniform", S.uniform_graph(3000, 20000, seed=6), 128, 0),
        ("uniform-mean-narrow", S.uniform_graph(2000, 9000, seed=7), 40, 1),
    ]
    for name, (ptr, idx), feat, flags in cases:
        n = ptr.shape[0] - 1
        deg = int((ptr[1:] - ptr[:-1]).max())
        torch.manual_seed(11)
        x = torch.randn(n, feat) / max(1.0, float(deg)) ** 0.5
        announce("noalloc %s n=%d E=%d feat=%d flags=%d" % (name, n, idx.shape[0], feat, flags))
        ptr_d, idx_d, x_d = ptr.to(dev), idx.to(dev), x.to(dev)
        got = _call_noalloc(lib, L, ptr_d, idx_d, x_d, n, feat, flags)
        torch.cuda.synchronize()
        want = _call_workspace(lib, L, ptr_d, idx_d, x_d, n, feat, flags)
        torch.cuda.synchronize()
        assert torch.equal(got, want), "%s: no-alloc result differs from cxg_spmm_sum_f32" % name
        ref = oracle.spmm(ptr.numpy(), idx.numpy(), x.numpy(), n, mean=bool(flags & 1))
        assert_close(got.cpu().numpy(), ref, 1e-4, 1e-5, "noalloc %s vs oracle" % name)


def test_noalloc_allocates_nothing_and_runs_on_the_callers_stream():
    """A call leaves the device's free memory and torch's allocator counters where they were
    (the property the entry point exists for), and its kernels run on the stream it is given:
    on a side stream the input rows are written behind a long spin kernel, the call follows on
    the same stream and a dependent copy after it; had the kernels run on any other stream
    they would have gathered the zeros the rows held before."""
    from cxgnncomp_backend import _lib as L
    from cxgnncomp import synthetic as S
    lib = L.load()
    dev = torch.device("cuda:0")
    ptr, idx = S.powerlaw_directed_symmetrised(30000, 300000, max_degree=5000, seed=9)
    n, feat = ptr.shape[0] - 1, 128
    torch.manual_seed(3)
    x = torch.randn(n, feat) / 30
    ptr_d, idx_d, x_d = ptr.to(dev), idx.to(dev), x.to(dev)
    out = torch.full((n, feat), float("nan"), device=dev)
    args = (ptr_d.data_ptr(), idx_d.data_ptr(), x_d.data_ptr(), feat, out.data_ptr(), feat, n, idx.shape[0], feat, 0)
    announce("noalloc memory counters around a call, n=%d E=%d" % (n, idx.shape[0]))
    L.check(lib.cxg_spmm_sum_f32_noalloc(*args, L.current_stream(dev)))          # first call: symbol lookup
    torch.cuda.synchronize()

    def counters():
        st = torch.cuda.memory_stats(dev)
        return (st["allocation.all.allocated"], st["allocation.all.freed"], st["segment.all.allocated"],
                st["segment.all.freed"], torch.cuda.mem_get_info(dev)[0])
    before = counters()
    L.check(lib.cxg_spmm_sum_f32_noalloc(*args, L.current_stream(dev)))
    torch.cuda.synchronize()
    assert counters() == before, "the call changed the allocator's counters or the device's free memory"
    want = out.clone()

    announce("noalloc on a side stream behind a spin kernel")
    stale = torch.zeros_like(x_d)
    out2 = torch.full((n, feat), float("nan"), device=dev)
    side = torch.cuda.Stream(device=dev)
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        torch.cuda._sleep(50_000_000)                 # tens of milliseconds of spinning on `side`
        stale.copy_(x_d)                              # the rows arrive behind it
        L.check(lib.cxg_spmm_sum_f32_noalloc(ptr_d.data_ptr(), idx_d.data_ptr(), stale.data_ptr(), feat,
                                             out2.data_ptr(), feat, n, idx.shape[0], feat, 0,
                                             L.current_stream(dev)))
        got = out2.clone()                            # dependent read on the same stream
    side.synchronize()
    assert torch.equal(got, want), "the call did not run in order on the stream it was given"
    torch.cuda.synchronize()


def test_noalloc_rejects_shapes_beyond_the_scratch():
    from cxgnncomp_backend import _lib as L
    lib = L.load()
    dev = torch.device("cuda:0")
    # sizes only: the call must fail before it touches any pointer
    ptr = torch.zeros(2, dtype=torch.int64, device=dev)
    idx = torch.zeros(1, dtype=torch.int64, device=dev)
    x = torch.zeros(1, 128, device=dev)
    out = torch.zeros(1, 128, device=dev)
    too_many = 40_000_000
    assert lib.cxg_spmm_workspace_bytes(too_many, 128) > (64 << 20)
    announce("noalloc oversize request (expects an error status, launches nothing)")
    rc = lib.cxg_spmm_sum_f32_noalloc(ptr.data_ptr(), idx.data_ptr(), x.data_ptr(), 128, out.data_ptr(), 128,
                                      1, too_many, 128, 0, L.current_stream(dev))
    assert rc == -3
    assert b"scratch" in lib.cxg_last_error()
    torch.cuda.synchronize()
