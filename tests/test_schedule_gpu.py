"""Scheduling helpers on the GPU (neighbor grouping, row / edge filters, the
per-relation sub-graphs of rel_schedule, COO -> CSR) against the CPU oracle:
index work, so every comparison is bit-exact.  Edge cases: empty graph, empty
rows, thresholds 1 and larger than any degree, everything removed, nothing
removed, relations that never occur, layer boundaries the reference's walk never
reaches.  A benchmark-sized case checks the invariants the outputs must satisfy."""
import io
from contextlib import redirect_stdout

import numpy as np
import pytest
import torch

import oracle
from conftest import announce
from oracle import pyref

pytestmark = pytest.mark.gpu


def _np(t):
    return t.detach().cpu().numpy()


def _random_ptr(rng, n, hi):
    deg = rng.integers(0, hi, n)
    deg[::6] = 0
    return np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)


@pytest.mark.parametrize("n,hi", [(0, 5), (1, 1), (1, 9), (500, 120), (20000, 40)])
@pytest.mark.parametrize("thres", [1, 4, 32, 1000])
def test_neighbor_grouping_bit_exact(n, hi, thres):
    import cxgnncomp
    rng = np.random.default_rng(n + thres)
    ptr = _random_ptr(rng, n, hi)
    want_ptr, want_target = oracle.neighbor_grouping(ptr, thres)
    announce("neighbor_grouping n=%d thres=%d" % (n, thres))
    got_ptr, got_target = cxgnncomp.neighbor_grouping(torch.from_numpy(ptr).cuda(), thres)
    assert got_ptr.is_cuda and got_ptr.dtype == torch.int64 and got_target.dtype == torch.int64
    assert np.array_equal(_np(got_ptr), want_ptr) and np.array_equal(_np(got_target), want_target)
    assert np.array_equal(_np(cxgnncomp.neighbor_grouping_gpu(torch.from_numpy(ptr).cuda(), thres)), want_ptr)


@pytest.mark.parametrize("n,hi,p", [(0, 3, 0.5), (1, 4, 0.0), (200, 15, 0.3), (200, 15, 1.0), (200, 15, 0.0),
                                    (30000, 30, 0.5)])
def test_row_and_edge_filters_bit_exact(n, hi, p):
    import cxgnncomp
    rng = np.random.default_rng(n + int(10 * p))
    ptr = _random_ptr(rng, n, hi)
    E = int(ptr[-1])
    idx = rng.integers(0, 1000, E)
    tp, ti = torch.from_numpy(ptr).cuda(), torch.from_numpy(idx).cuda()
    flag = rng.random(n) < p
    with redirect_stdout(io.StringIO()):
        want = pyref.remove_from_graph(ptr, idx, flag)
    announce("remove_from_graph n=%d p=%.1f" % (n, p))
    got = cxgnncomp.remove_from_graph(tp, ti, torch.from_numpy(flag).cuda())
    assert np.array_equal(_np(got[0]), want[0]) and np.array_equal(_np(got[1]), want[1])
    eflag = rng.random(E) < p
    want = pyref.remove_from_graph_by_edge(ptr, idx, eflag)
    announce("remove_from_graph_by_edge n=%d p=%.1f" % (n, p))
    got = cxgnncomp.remove_from_graph_by_edge(tp, ti, torch.from_numpy(eflag).cuda())
    assert np.array_equal(_np(got[0]), want[0]) and np.array_equal(_np(got[1]), want[1])


@pytest.mark.parametrize("layers", [[20, 70, 150, 150], [150, 150], [70, 20, 150], [10, 151, 150], [150]])
def test_rel_schedule_bit_exact(layers):
    import cxgnncomp_backend as B
    rng = np.random.default_rng(4)
    ptr = _random_ptr(rng, 150, 12)
    E = int(ptr[-1])
    idx = rng.integers(0, 400, E)
    rel = rng.integers(0, 5, E).astype(np.int32)
    rel[rel == 3] = 2                                   # relation 3 never occurs
    want = oracle.rel_schedule(ptr, idx, rel, layers, 5)
    announce("rel_schedule layers=%s" % layers)
    got = B.rel_schedule(torch.from_numpy(ptr).cuda(), torch.from_numpy(idx).cuda(), torch.from_numpy(rel).cuda(),
                         torch.tensor(layers), 5)
    assert len(got) == len(want) == 16
    for g, w in zip(got, want):
        assert g.is_cuda and g.dtype == torch.int64 and np.array_equal(_np(g), w)


@pytest.mark.parametrize("n,e", [(1, 0), (5, 1), (300, 4000), (100000, 1500000)])
def test_coo_to_csr_bit_exact(n, e):
    from cxgnncomp import synthetic
    from cxgnncomp_backend import _ops
    rng = np.random.default_rng(e)
    src = rng.integers(0, 5 * n, e)
    dst = rng.integers(0, n, e)
    want_ptr, want_idx = oracle.coo_to_csr(src, dst, n)
    announce("coo_to_csr n=%d e=%d" % (n, e))
    ptr, idx, perm = _ops.coo_to_csr(torch.from_numpy(src).cuda(), torch.from_numpy(dst).cuda(), n)
    assert np.array_equal(_np(ptr), want_ptr) and np.array_equal(_np(idx), want_idx)
    assert np.array_equal(_np(perm), np.argsort(dst, kind="stable"))
    p2, i2 = synthetic.csr_from_coo(torch.from_numpy(src).cuda(), torch.from_numpy(dst).cuda(), n)
    assert torch.equal(p2, ptr) and torch.equal(i2, idx)
    with pytest.raises(ValueError):
        _ops.coo_to_csr(torch.tensor([0]).cuda(), torch.tensor([n]).cuda(), n)


def test_schedule_helpers_at_benchmark_size():
    """2.45M rows / 61.9M edges: the outputs' defining invariants, checked on the device."""
    import cxgnncomp
    from cxgnncomp import synthetic
    N = 2449029
    ptr, idx = synthetic.powerlaw_symmetric_graph(N, 30929570, device="cuda")
    E = idx.shape[0]
    deg = ptr[1:] - ptr[:-1]
    announce("neighbor_grouping at 61.9M edges")
    new_ptr, new_target = cxgnncomp.neighbor_grouping(ptr, 32)
    sizes = new_ptr[1:] - new_ptr[:-1]
    groups = torch.clamp((deg + 31) // 32, min=1)
    assert int(new_ptr[0]) == 0 and int(new_ptr[-1]) == E and new_target.shape[0] == int(groups.sum())
    assert int(sizes.max()) <= 32 and int(sizes.min()) >= 0
    assert torch.equal(torch.bincount(new_target, minlength=N), groups)
    assert bool((new_target[1:] >= new_target[:-1]).all())
    assert torch.equal(torch.zeros(N, dtype=torch.int64, device="cuda").index_add_(0, new_target, sizes), deg)
    announce("remove_from_graph_by_edge at 61.9M edges")
    g = torch.Generator(device="cuda").manual_seed(3)
    eflag = torch.rand(E, generator=g, device="cuda") < 0.7
    p2, i2 = cxgnncomp.remove_from_graph_by_edge(ptr, idx, eflag)
    assert torch.equal(i2, idx[~eflag]) and int(p2[-1]) == i2.shape[0]
    assert bool(((p2[1:] - p2[:-1]) > 0).all())
    announce("remove_from_graph at 61.9M edges")
    rflag = torch.rand(N, generator=g, device="cuda") < 0.5
    p3, i3 = cxgnncomp.remove_from_graph(ptr, idx, rflag)
    assert torch.equal(p3[1:] - p3[:-1], deg[~rflag])
    assert torch.equal(i3, idx[torch.repeat_interleave(~rflag, deg)])


@pytest.mark.parametrize("kind", ["uniform", "powerlaw", "empty_rows", "no_edges", "one_hub"])
@pytest.mark.parametrize("prefix", [False, True])
def test_csr_transpose_bit_exact(kind, prefix):
    """Reversed graph of all rows / of a row prefix, with more source nodes than the ids
    that occur (trailing empty columns): ptr_t, idx_t and the stable edge order perm."""
    from cxgnncomp_backend import _ops
    from test_spmm_gpu import _graph
    ptr, idx = _graph(kind)
    n = ptr.shape[0] - 1
    n_rows = n // 3 if prefix else n
    n_src = n + 37
    want_ptr, want_idx, want_perm = oracle.csr_transpose(ptr.numpy(), idx.numpy(), n_rows, n_src)
    announce("csr_transpose kind=%s prefix=%s" % (kind, prefix))
    ptr_t, idx_t, perm, n_edges = _ops.csr_transpose(ptr.cuda(), idx.cuda(), n_rows, n_src)
    torch.cuda.synchronize()
    assert n_edges == int(ptr[n_rows])
    assert np.array_equal(_np(ptr_t), want_ptr)
    assert np.array_equal(_np(idx_t), want_idx)
    assert np.array_equal(_np(perm), want_perm)


def test_csr_transpose_leading_empty_columns():
    """Sources 0..4 never occur, one source takes every edge."""
    from cxgnncomp_backend import _ops
    ptr = torch.tensor([0, 2, 2, 5])
    idx = torch.tensor([7, 5, 9, 5, 5])
    announce("csr_transpose leading empty columns")
    ptr_t, idx_t, perm, n_edges = _ops.csr_transpose(ptr.cuda(), idx.cuda(), 3, 12)
    assert n_edges == 5
    assert _np(ptr_t).tolist() == [0, 0, 0, 0, 0, 0, 3, 3, 4, 4, 5, 5, 5]
    assert _np(idx_t).tolist() == [0, 2, 2, 0, 2]
    assert _np(perm).tolist() == [1, 3, 4, 0, 2]


def _gappy_ptr(rng, n, first=0):
    """Degrees with runs of hundreds of empty rows between occupied ones, and some hubs."""
    deg = np.zeros(n, dtype=np.int64)
    occupied = rng.choice(n, max(1, n // 150), replace=False)
    deg[occupied] = rng.integers(1, 9, occupied.shape[0])
    deg[rng.choice(n, 3)] = 1500
    return first + np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)


@pytest.mark.parametrize("case", ["gappy", "gappy_offset", "dense", "single_row", "degree_one"])
def test_csr_row_ids_bit_exact(case):
    """Row of every edge position, int64 and int32 forms; positions count from ptr[0]."""
    from cxgnncomp_backend import _ops
    rng = np.random.default_rng(len(case))
    if case == "gappy":
        ptr = _gappy_ptr(rng, 40000)
    elif case == "gappy_offset":
        ptr = _gappy_ptr(rng, 40000, first=777)
    elif case == "dense":
        ptr = _random_ptr(rng, 30000, 60)
    elif case == "single_row":
        ptr = np.array([0, 100000], dtype=np.int64)
    else:
        ptr = np.arange(0, 70001, dtype=np.int64)
    n = ptr.shape[0] - 1
    E = int(ptr[-1] - ptr[0])
    want = np.repeat(np.arange(n, dtype=np.int64), np.diff(ptr))
    announce("csr_row_ids case=%s" % case)
    got = _ops.csr_row_ids(torch.from_numpy(ptr).cuda(), n, E)
    got32 = _ops.csr_row_ids32(torch.from_numpy(ptr).cuda(), n, E)
    torch.cuda.synchronize()
    assert np.array_equal(_np(got), want)
    assert got32.dtype == torch.int32 and np.array_equal(_np(got32).astype(np.int64), want)


def test_csr_transpose_far_more_columns_than_edges():
    """A sampled layer whose sources are numbered over all nodes: 600 edges, a million columns."""
    from cxgnncomp_backend import _ops
    rng = np.random.default_rng(5)
    n_rows, n_src = 40, 1000003
    deg = rng.integers(0, 30, n_rows)
    ptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    idx = rng.integers(0, n_src, int(ptr[-1])).astype(np.int64)
    idx[:3] = [n_src - 1, 0, n_src - 1]
    want_ptr, want_idx, want_perm = oracle.csr_transpose(ptr, idx, n_rows, n_src)
    announce("csr_transpose far more columns than edges")
    ptr_t, idx_t, perm, n_edges = _ops.csr_transpose(torch.from_numpy(ptr).cuda(), torch.from_numpy(idx).cuda(),
                                                     n_rows, n_src)
    assert np.array_equal(_np(ptr_t), want_ptr)
    assert np.array_equal(_np(idx_t), want_idx)
    assert np.array_equal(_np(perm), want_perm)


def test_transposed_graphs_of_nested_layers_are_cut_from_the_largest():
    """The layers of a sampled batch are row prefixes of one CSR.  Once a forward pass has
    announced them, the transposed graph of a smaller layer is compacted out of the largest
    layer's instead of sorted again: it must equal the direct transposition bit for bit
    (and both the oracle's)."""
    from cxgnncomp import synthetic as S
    from cxgnncomp_backend import _ops
    ptr, idx, nn, ne = S.sampled_batch(num_seeds=300, fanouts=(7, 5, 3), id_space=200000, seed=9)
    p, i = ptr.cuda(), idx.cuda()
    _ops.clear_graph_cache()
    for k in (2, 1, 0):                                  # forward order: largest layer first
        _ops.note_layer(p, i, nn[k], nn[k + 1])
    before = _ops._C.graph_cache_stats()
    graphs = {}
    for k in (0, 1, 2):                                  # backward order: smallest layer first
        announce("transposed prefix layer %d: rows=%d sources=%d" % (k, nn[k], nn[k + 1]))
        graphs[k] = _ops.transposed(p, i, nn[k], nn[k + 1])
    after = _ops._C.graph_cache_stats()
    # one sort, of the largest layer; the two smaller graphs were cut out of it
    assert after["sorts"] - before["sorts"] == 1 and after["cuts"] - before["cuts"] == 2
    assert graphs[2].n_dst == nn[2] and graphs[0].n_src == nn[1]
    for k in (0, 1, 2):
        g = graphs[k]
        pt, it, pm, n_e = _ops.csr_transpose(p, i, nn[k], nn[k + 1])
        assert g.n_edges == n_e == ne[k]
        assert torch.equal(g.ptr_t, pt) and torch.equal(g.idx_t, it) and torch.equal(g.perm, pm)
        want = oracle.csr_transpose(ptr.numpy(), idx.numpy(), nn[k], nn[k + 1])
        assert np.array_equal(_np(g.ptr_t), want[0]) and np.array_equal(_np(g.idx_t), want[1])
        assert np.array_equal(_np(g.perm), want[2])
    # direct use of the entry point: an empty prefix and the whole graph as its own prefix
    whole = _ops.transposed(p, i, nn[2], nn[3])
    pt, it, pm, n_e = _ops.csr_transpose_prefix(whole, p, nn[2], nn[3])
    assert torch.equal(pt, whole.ptr_t) and torch.equal(it, whole.idx_t) and torch.equal(pm, whole.perm)
    pt, it, pm, n_e = _ops.csr_transpose_prefix(whole, p, 0, 5)
    assert n_e == 0 and it.numel() == 0 and not pt.any()
    _ops.clear_graph_cache()


def test_known_edge_counts_spare_the_read_back():
    """A sampled batch carries its layers' edge counts.  Announced with note_edge_counts, they size
    the reversed graphs, so no transposition reads ptr[num_node] back from the device (the host
    then never waits for the GPU while it enqueues the first backward pass of a new batch); the
    graphs are the same bit for bit."""
    from cxgnncomp import synthetic as S
    from cxgnncomp_backend import _ops
    ptr, idx, nn, ne = S.sampled_batch(num_seeds=300, fanouts=(7, 5, 3), id_space=200000, seed=11)
    p, i = ptr.cuda(), idx.cuda()
    want = {k: _ops.csr_transpose(p, i, nn[k], nn[k + 1]) for k in (0, 1, 2)}
    _ops.clear_graph_cache()
    _ops.note_edge_counts(p, i, nn[:3], ne)
    for k in (2, 1, 0):
        _ops.note_layer(p, i, nn[k], nn[k + 1])
    before = _ops._C.graph_cache_stats()
    announce("transposed graphs of three nested layers with announced edge counts")
    got = {k: _ops.transposed(p, i, nn[k], nn[k + 1]) for k in (0, 1, 2)}
    after = _ops._C.graph_cache_stats()
    assert after["readbacks"] == before["readbacks"]
    assert after["sorts"] - before["sorts"] == 1 and after["cuts"] - before["cuts"] == 2
    for k in (0, 1, 2):
        pt, it, pm, n_e = want[k]
        assert got[k].n_edges == n_e == ne[k]
        assert torch.equal(got[k].ptr_t, pt) and torch.equal(got[k].idx_t, it) and torch.equal(got[k].perm, pm)
    # without the announcement the counts come from the device
    _ops.clear_graph_cache()
    _ops.transposed(p, i, nn[0], nn[1])
    assert _ops._C.graph_cache_stats()["readbacks"] == after["readbacks"] + 1
    # counts that cannot be right are refused
    with pytest.raises((ValueError, RuntimeError)):
        _ops.note_edge_counts(p, i, [nn[0]], [idx.shape[0] + 1])
    with pytest.raises((ValueError, RuntimeError)):
        _ops.note_edge_counts(p, i, [ptr.shape[0]], [0])
    _ops.clear_graph_cache()


def test_sage_layer_with_frozen_input_announces_nothing():
    """The first layer of a batch whose input features need no gradient (the normal training case)
    does not ask for its reversed graph in the backward pass, so it does not announce itself: the
    reversed graphs of the layers above it are cut from the largest layer that needs one, not from
    the largest layer of the batch."""
    import cxgnncomp
    from cxgnncomp import synthetic as S
    from cxgnncomp_backend import _ops
    ptr, idx, nn, ne = S.sampled_batch(num_seeds=200, fanouts=(6, 4, 3), id_space=100000, seed=12)
    p, i = ptr.cuda(), idx.cuda()
    torch.manual_seed(0)
    layers = [cxgnncomp.MySageConv(16, 32).cuda(), cxgnncomp.MySageConv(32, 32).cuda(), cxgnncomp.MySageConv(32, 8).cuda()]
    x = torch.randn(nn[3], 16, device="cuda")                      # no gradient wanted
    _ops.clear_graph_cache()
    before = _ops._C.graph_cache_stats()
    h = x
    for li, layer in enumerate(layers):
        h = torch.relu(layer(h, p, i, nn[2 - li]))
    announce("3 SAGE layers, frozen input features")
    h.sum().backward()
    torch.cuda.synchronize()
    after = _ops._C.graph_cache_stats()
    # layers 2 and 3 need reversed graphs (rows nn[1] and nn[0]); the first layer's (rows nn[2]) is never built
    assert after["sorts"] - before["sorts"] == 1 and after["cuts"] - before["cuts"] == 1
    assert after["graphs"] == 2
    _ops.clear_graph_cache()
