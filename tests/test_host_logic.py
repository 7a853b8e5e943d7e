"""CPU-only checks of the host side: the C ABI loads and exports what the header
declares, index/scheduling helpers are bit-exact against the oracle, the tuner,
timers and harness helpers behave like the reference's, and the synthetic graph
generators produce the shapes the configurations name.  No kernel is launched."""
import ctypes
import io
import json
import os
import re
from contextlib import redirect_stdout

import numpy as np
import pytest
import torch

import oracle
from oracle import pyref

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FX = json.load(open(os.path.join(ROOT, "tests", "golden", "fixtures.json")))


# ----------------------------------------------------------------------------- C ABI
def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "cxgnn_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cxg_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from cxgnncomp_backend import _lib
    names = _declared_symbols()
    assert len(names) >= 25
    assert os.path.exists(_lib.LIB_PATH), "build the library first: python cxgnn-compute_amd/build.py"
    lib = ctypes.CDLL(_lib.LIB_PATH)
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing
    # the ctypes table covers exactly the header
    assert sorted(_lib.SIGNATURES) == names
    assert _lib.load().cxg_version() >= 100
    assert _lib.load().cxg_last_error() is not None


def test_missing_library_fails_loudly(monkeypatch):
    from cxgnncomp_backend import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libcxgnn_hip.so")
    with pytest.raises(RuntimeError, match="libcxgnn_hip.so not found"):
        _lib.load()


def test_argument_errors_come_back_as_status_codes():
    """Size queries and argument checks run on the host; nothing is launched."""
    from cxgnncomp_backend import _lib
    lib = _lib.load()
    assert lib.cxg_spmm_workspace_bytes(-1, 128) == 0
    small = lib.cxg_spmm_workspace_bytes(1000, 128)
    big = lib.cxg_spmm_workspace_bytes(10 ** 7, 128)
    assert 0 < small < big
    st = lib.cxg_spmm_sum_f32(None, None, None, 128, None, 128, 10, 100, 128, 0, None, 0, None)
    assert st == -1 and b"null" in lib.cxg_last_error()
    with pytest.raises(ValueError):
        _lib.check(st)
    st = lib.cxg_spmm_sum_f32(None, None, None, 128, None, 128, 10, 100, 128, 64, None, 0, None)
    assert st == -1 and b"flag" in lib.cxg_last_error()
    assert lib.cxg_spmm_sum_f32(None, None, None, 128, None, 128, 0, 0, 128, 0, None, 0, None) == 0


def test_backend_rejects_cpu_tensors_without_touching_the_gpu():
    import cxgnncomp_backend as B
    ptr = torch.tensor([0, 1, 2])
    idx = torch.tensor([1, 0])
    x = torch.randn(2, 4)
    with pytest.raises(ValueError, match="CUDA"):
        B.run_spmm_configurable(ptr, idx, x, 2)
    with pytest.raises(ValueError, match="CUDA"):
        B.edge_attention(ptr, idx, x, x, 2, 0.2)


def test_compiled_host_layer_exports_the_reference_names():
    """cxgnncomp_backend._C carries the exports the reference writes in C++ (binding.cpp:15-25,
    37-41, 58-78); the module as a whole carries every name of binding.cpp:14-119."""
    import cxgnncomp_backend as B
    from cxgnncomp_backend import _C
    compiled = ["aggr_rel", "sage_sum_forward", "sage_mean_forward", "sage_sum_forward_edge_value", "sage_mean_forward_edge_value",
                "gather", "edge_attention", "edge_value_degree", "spmv", "run_spmm_configurable",
                "run_spmm_configurable_bwd", "run_spmm_configurable_int32", "spmm_multihead", "spmm_multihead_bwd",
                "run_spmm_multihead_configurable", "run_sddmm", "run_sddmm_vertex_centric"]
    for name in compiled:
        assert getattr(B, name) is getattr(_C, name), name
    others = ["target_aggr", "target_aggr_backward", "rel_schedule", "selective_aggr", "selective_aggr_bwd",
              "gen_edge_type_mag240m", "topo_sort", "aggr_rel_direct", "aggr_rgcn_direct_func",
              "typed_linear", "typed_linear_s2e", "typed_linear_s2d", "pad_rel", "pad_rel_idx", "seastar_forward",
              "seastar_backward", "GSpMM_u_e", "GSpMM_u", "REDUCEOP", "COMPUTEOP", "SPMM_MULTIHEAD_SCHEDULE"]
    for name in others:
        assert hasattr(B, name), name
    # export_values(): the enum members are module attributes too, Optimal is the default schedule
    assert int(B.Naive) == 0 and int(B.PreReduce) == 1 and int(B.Optimal) == 2
    assert B.SPMM_MULTIHEAD_SCHEDULE.Optimal == B.Optimal
    assert "schedule" in B.spmm_multihead.__doc__ and "block_size" in B.spmm_multihead.__doc__
    assert _C.lib_version() == B._lib_version()
    assert set(_C.graph_cache_stats()) == {"graphs", "sorts", "cuts", "readbacks"}


def test_missing_host_layer_fails_loudly(monkeypatch):
    import builtins
    from cxgnncomp_backend import _lib
    monkeypatch.setattr(_lib, "_native_mod", None)
    real_import = builtins.__import__

    def no_ext(name, globals=None, locals=None, fromlist=(), level=0):
        if level == 1 and fromlist and "_C" in fromlist:
            raise ImportError("simulated: no _C.so")
        return real_import(name, globals, locals, fromlist, level)
    monkeypatch.setattr(builtins, "__import__", no_ext)
    with pytest.raises(RuntimeError, match="compiled host layer"):
        _lib.native()


def test_compiled_host_layer_checks_arguments_before_any_launch():
    """Argument errors of the C++ layer are ValueErrors raised on the host (the reference exits the
    process, src/cpp/include/common.h:16-26)."""
    import cxgnncomp_backend as B
    from cxgnncomp_backend import _ops
    ptr, idx, x = torch.tensor([0, 1, 2]), torch.tensor([1, 0]), torch.randn(2, 4)
    with pytest.raises(ValueError, match="2D"):
        B.run_spmm_configurable(ptr, idx, torch.randn(2, 2, 2), 2)
    with pytest.raises(ValueError, match="3D"):
        B.spmm_multihead(ptr, idx, torch.rand(2, 2), x, 2)
    with pytest.raises(ValueError, match="num_head mismatch"):
        B.spmm_multihead(ptr, idx, torch.rand(2, 3), torch.randn(2, 2, 4), 2)
    with pytest.raises((ValueError, RuntimeError), match="DO NOT use mean with edge value"):
        B.sage_mean_forward_edge_value(x, ptr, idx, torch.rand(2), 2)      # aggr.cu:158,163 aborts here
    with pytest.raises((ValueError, RuntimeError), match="num_node must be > 0"):
        B.gather(x, idx, 0)
    with pytest.raises(ValueError, match="CUDA"):
        B.run_sddmm(idx, idx, x, x, torch.zeros(2, 1), 2)
    with pytest.raises(ValueError, match="CUDA"):
        _ops.spmm(ptr, idx, x, 2, val=torch.rand(2))
    with pytest.raises(ValueError, match="CUDA"):
        _ops.transposed(ptr, idx, 2, 2)
    # scalars may arrive as 0-d tensors (cxgnncomp/graph_conv.py:41-50): converted, then checked
    with pytest.raises(ValueError, match="CUDA"):
        B.run_spmm_configurable(ptr, idx, x, torch.tensor(2), 0, 0, 0, 0, 0, 0, 0, 0, 0)


# ----------------------------------------------------------------------------- scheduling helpers
def _random_ptr(rng, n, hi):
    deg = rng.integers(0, hi, n)
    deg[::6] = 0
    return np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)


@pytest.mark.parametrize("thres", [1, 4, 32])
def test_neighbor_grouping_bit_exact(thres):
    import cxgnncomp
    rng = np.random.default_rng(thres)
    ptr = _random_ptr(rng, 500, 120)
    want_ptr, want_target = oracle.neighbor_grouping(ptr, thres)
    got_ptr, got_target = cxgnncomp.neighbor_grouping(torch.from_numpy(ptr), thres)
    assert got_ptr.dtype == torch.int64 and got_target.dtype == torch.int64
    assert np.array_equal(got_ptr.numpy(), want_ptr) and np.array_equal(got_target.numpy(), want_target)
    assert np.array_equal(cxgnncomp.neighbor_grouping_gpu(torch.from_numpy(ptr), thres).numpy(), want_ptr)
    f = FX["neighbor_grouping_small"]
    p, t = cxgnncomp.neighbor_grouping(torch.tensor(f["ptr"]), f["thres"])
    assert p.tolist() == f["new_ptr"] and t.tolist() == f["new_target"]


def test_row_filters_and_reorder_bit_exact():
    import cxgnncomp
    rng = np.random.default_rng(2)
    ptr = _random_ptr(rng, 200, 15)
    E = int(ptr[-1])
    idx = rng.integers(0, 1000, E)
    tp, ti = torch.from_numpy(ptr), torch.from_numpy(idx)
    flag = rng.random(200) < 0.3
    with redirect_stdout(io.StringIO()):
        want = pyref.remove_from_graph(ptr, idx, flag)
    got = cxgnncomp.remove_from_graph(tp, ti, torch.from_numpy(flag))
    assert np.array_equal(got[0].numpy(), want[0]) and np.array_equal(got[1].numpy(), want[1])
    eflag = rng.random(E) < 0.5
    want = pyref.remove_from_graph_by_edge(ptr, idx, eflag)
    got = cxgnncomp.remove_from_graph_by_edge(tp, ti, torch.from_numpy(eflag))
    assert np.array_equal(got[0].numpy(), want[0]) and np.array_equal(got[1].numpy(), want[1])
    metric = rng.permutation(200)
    want = pyref.reorder_by(ptr, idx, metric)
    got = cxgnncomp.reorder_by(tp, ti, torch.from_numpy(metric))
    assert np.array_equal(got[0].numpy(), want[0]) and np.array_equal(got[1].numpy(), want[1])
    f = FX["reorder_by_doc"]
    p, i = cxgnncomp.reorder_by(torch.tensor(f["ptr"]), torch.tensor(f["idx"]), torch.tensor(f["metric"]))
    assert p.tolist() == f["new_ptr"] and i.tolist() == f["new_idx"]


def test_partition_2d_conserves_edges():
    """The reference's own check for partitioning (test/1-kernels/test_partition.py:22-51)."""
    import cxgnncomp
    rng = np.random.default_rng(3)
    ptr = _random_ptr(rng, 64, 9)
    E = int(ptr[-1])
    idx = rng.integers(0, 80, E)
    new_ptr, new_idx = cxgnncomp.partition_2d(torch.from_numpy(ptr), torch.from_numpy(idx), 80, 64, num_parts=4)
    assert int(new_ptr[-1]) == E and new_idx.shape[0] == E
    assert sorted(new_idx.tolist()) == sorted(idx.tolist())
    assert (torch.diff(new_ptr) > 0).all()
    # first block = destination part 0 x source part 0
    rows = np.repeat(np.arange(64), np.diff(ptr))
    m = (rows < 16) & (idx < 20)
    assert new_idx[:int(m.sum())].tolist() == idx[m].tolist()


def test_rel_schedule_bit_exact():
    import cxgnncomp_backend as B
    rng = np.random.default_rng(4)
    ptr = _random_ptr(rng, 150, 12)
    E = int(ptr[-1])
    idx = rng.integers(0, 400, E)
    rel = rng.integers(0, 5, E).astype(np.int32)
    layers = [20, 70, 150, 150]
    want = oracle.rel_schedule(ptr, idx, rel, layers, 5)
    got = B.rel_schedule(torch.from_numpy(ptr), torch.from_numpy(idx), torch.from_numpy(rel),
                         torch.tensor(layers), 5)
    assert len(got) == len(want) == 16
    for g, w in zip(got, want):
        assert g.dtype == torch.int64 and np.array_equal(g.numpy(), w)
    f = FX["rel_schedule_small"]
    got = B.rel_schedule(torch.tensor(f["ptr"]), torch.tensor(f["idx"]), torch.tensor(f["rel"], dtype=torch.int32),
                         torch.tensor(f["num_node_in_layer"]), f["num_rel"])
    assert got[0].tolist() == f["rel0"]["ptr"] and got[5].tolist() == f["rel1"]["target"]
    assert got[-1].tolist() == f["table"]


def test_mag240m_edge_types():
    import cxgnncomp_backend as B
    P, PA = 121751666, 244134778
    sub_to_full = torch.tensor([5, P + 3, PA + 1, 7])          # paper, author, institute, paper
    ptr = torch.tensor([0, 2, 4, 5, 5])
    idx = torch.tensor([3, 1, 0, 2, 1])
    assert B.gen_edge_type_mag240m(ptr, idx, sub_to_full).tolist() == [0, 1, 2, 3, 4]
    with pytest.raises(ValueError):
        B.gen_edge_type_mag240m(torch.tensor([0, 1]), torch.tensor([2]), sub_to_full)   # paper<-institute


# ----------------------------------------------------------------------------- pure-torch ops on the CPU
def test_torch_reference_paths_run_on_cpu():
    import cxgnncomp
    f = FX["spmm_small"]
    x = torch.tensor(f["x"])
    out = cxgnncomp.spmm_torch(x, torch.tensor(f["ptr"]), torch.tensor(f["idx"]), 4)
    assert np.allclose(out.numpy(), f["sum"])
    out = cxgnncomp.spmm_torch(x, torch.tensor(f["ptr"]), torch.tensor(f["idx"]), 4, torch.tensor(f["val"]))
    assert np.allclose(out.numpy(), f["weighted"])
    rng = np.random.default_rng(5)
    ptr = _random_ptr(rng, 60, 8)
    E = int(ptr[-1])
    idx = rng.integers(0, 60, E)
    rel = rng.integers(0, 3, E)
    xx = rng.standard_normal((60, 8)).astype(np.float32)
    w = rng.standard_normal((3, 8, 4)).astype(np.float32)
    want = oracle.rgcn_fused(xx, ptr, idx, w, rel, 60)
    args = (torch.from_numpy(xx), torch.from_numpy(w), torch.from_numpy(ptr), torch.from_numpy(idx),
            torch.from_numpy(rel), 60)
    assert np.allclose(cxgnncomp.TypedLinearS2DSort(*args).numpy(), want, rtol=1e-4, atol=1e-5)
    dst = torch.repeat_interleave(torch.arange(60), torch.from_numpy(np.diff(ptr)))
    got = cxgnncomp.TypedLinearNaiveS2D(args[0], args[1], args[4], args[3], dst, 60, E)
    assert np.allclose(got.numpy(), want, rtol=1e-4, atol=1e-5)
    order = torch.sort(args[4], stable=True)[1]
    got = cxgnncomp.RGCNOP_sorted(args[0], args[1], args[3][order], dst[order],
                                  torch.bincount(args[4], minlength=3), 60)
    assert np.allclose(got.numpy(), want, rtol=1e-4, atol=1e-5)
    parts = cxgnncomp.SelectMMS2EOP(args[0], args[1], args[3], args[4])
    assert [p.shape[0] for p in parts] == np.bincount(rel, minlength=3).tolist()
    conv = cxgnncomp.MyGCNConv(8, 4, normalize=True)
    ev = conv.gcn_norm(torch.from_numpy(ptr), torch.from_numpy(idx))
    assert np.array_equal(ev.numpy(), oracle.edge_value_degree(ptr, 60, E))
    assert np.array_equal(ev.numpy(), pyref.gcn_norm(torch.from_numpy(ptr), torch.from_numpy(idx)).numpy())
    gat = cxgnncomp.MyGATConv(8, 4, heads=2)
    gat.edge_softmax_schedule = "opwise"
    a_s, a_d = torch.randn(60, 2), torch.randn(60, 2)
    got = gat.edge_softmax(torch.from_numpy(ptr), torch.from_numpy(idx), a_s, a_d, E, 0.2)
    want_sm, _ = oracle.edge_softmax_fwd(ptr, idx, a_d.numpy(), a_s.numpy(), E, 0.2)
    assert np.allclose(got.numpy(), want_sm, rtol=1e-5, atol=1e-7)


# ----------------------------------------------------------------------------- tuner, timers, harness helpers
def test_tuner_caches_and_forwards_nine_launch_integers():
    import cxgnncomp
    from cxgnncomp.codegen import validate
    calls = []

    def run_spmm_configurable(a, b, *ints):
        calls.append(ints)
        return "out"
    t = cxgnncomp.Tuner(lazy=False)
    assert t.tune_graph(1000, 5000, 128, run_spmm_configurable, ["a", "b"]) == "out"
    assert len(calls[0]) == 9 and all(isinstance(v, int) for v in calls[0])
    grid_x, grid_y, block_x, block_y, rpb, cpb, cpw, grid_map, block_map = calls[0]
    assert validate(cpw, rpb, cpb, block_x * block_y, 128) == 1
    key = t.hash(1000, 5000, 128, run_spmm_configurable, ["a", "b"])
    assert key == "1000_5000_128_run_spmm_configurable_a_b" and key in t.cache
    t.tune_graph(1000, 5000, 128, run_spmm_configurable, ["a", "b"])
    assert calls[1] == calls[0]
    lazy = cxgnncomp.Tuner(lazy=True)
    assert lazy.hash(1, 2, 3, run_spmm_configurable, []) == "run_spmm_configurable_lazy"
    lazy.tune_graph(torch.tensor(64), 10, 64, run_spmm_configurable, ["a", "b"])
    lazy.tune_graph(640, 10, 64, run_spmm_configurable, ["a", "b"])
    assert calls[3][0] == 10 * calls[2][0]        # grid_x follows the row count on lazy replay
    assert cxgnncomp.global_tuner.lazy is True
    assert validate(64, 1, 32, 32, 128) == 0 and validate(512, 1, 512, 32, 512) == 0


def test_timers_follow_the_reference_contract():
    import cxgnncomp
    from cxgnncomp import timer
    timer._GLOBAL_TIMERS = None
    with pytest.raises(AssertionError):
        cxgnncomp.get_timers()
    cxgnncomp.set_timers()
    x = torch.randn(3, requires_grad=True)
    y = cxgnncomp.TimerOP.apply(x, "stage", True)
    z = cxgnncomp.TimerOP.apply(y * 2, "stage", False)
    z.sum().backward()
    assert torch.equal(x.grad, torch.full((3,), 2.0))
    timers = cxgnncomp.get_timers()
    assert set(timers.timers) == {"stage_fwd", "stage_bwd"}
    assert timers("stage_fwd").skip and timers("stage_fwd").elapsed() is None
    lines = []
    timers.log_all(lines.append)
    assert lines and lines[0].startswith("time (ms)")


def test_compare_prints_the_reference_strings():
    import cxgnncomp
    buf = io.StringIO()
    with redirect_stdout(buf):
        cxgnncomp.compare(torch.ones(4), torch.ones(4) + 1e-3)
        cxgnncomp.compare(torch.ones(4), torch.tensor([1.0, 1.0, 2.0, 1.0]))
    text = buf.getvalue()
    assert "CORRECT: match" in text and "ERROR: differ ratio: 0.25" in text
    with pytest.raises(AssertionError):
        cxgnncomp.compare(torch.ones(4), torch.ones(5))


# ----------------------------------------------------------------------------- synthetic inputs and batch files
def test_synthetic_graphs_have_the_configured_shapes():
    from cxgnncomp import synthetic as S
    ptr, idx = S.uniform_graph(10000, 100000, seed=0)
    assert ptr.shape == (10001,) and idx.shape == (100000,) and int(ptr[-1]) == 100000
    ptr2, idx2 = S.uniform_graph(10000, 100000, seed=0)
    assert torch.equal(ptr, ptr2) and torch.equal(idx, idx2)          # seeded
    ptr, idx = S.powerlaw_directed_symmetrised(169343, 1166243, seed=0)
    assert idx.shape[0] == 2332486 and int(ptr[-1]) == 2332486
    deg = ptr[1:] - ptr[:-1]
    assert 9000 < int(deg.max()) < 17000
    # symmetric as a multiset: in-degree == out-degree for every node
    assert torch.equal(torch.bincount(idx, minlength=169343), deg)
    ptr, idx = S.powerlaw_symmetric_graph(50000, 400000, max_degree=3000, seed=1)
    assert idx.shape[0] == 800000
    assert torch.equal(torch.bincount(idx, minlength=50000), ptr[1:] - ptr[:-1])
    ptr, idx, etype, ntype = S.hetero_graph(20000, 400000, num_rel=16, seed=0)
    assert int((ptr[1:] - ptr[:-1]).min()) >= 1 and etype.shape == idx.shape
    cnt = torch.bincount(etype, minlength=16)
    assert int(etype.max()) == 15 and cnt[0] > cnt[3] > cnt[15] > 0
    assert int(ntype.max()) == 3
    ptr, idx, nn, ne = S.sampled_batch(num_seeds=256, fanouts=(15, 10, 5), seed=0)
    assert nn[0] == 256 and ne[0] == 256 * 15 and ptr.shape[0] == nn[2] + 1
    assert int(ptr[nn[0]]) == ne[0] and int(ptr[nn[1]]) == ne[1] and int(ptr[-1]) == ne[2] == idx.shape[0]
    assert int(idx.max()) == nn[3] - 1
    # first-seen numbering: sources referenced by layer l edges are < num_node_in_layer[l+1]
    assert int(idx[:ne[0]].max()) < nn[1] and int(idx[:ne[1]].max()) < nn[2]


def test_batch_round_trip(tmp_path):
    """The reference's container (cxgnncomp/batch.py:7-90): target as the sixth argument,
    x.dat / ptr.dat / idx.dat / target.dat as flat numpy images, an instance fromfile that leaves
    every tensor flat, totype, and the two-argument PyGBatch."""
    import cxgnncomp
    from cxgnncomp import synthetic as S
    ptr, idx, nn, ne = S.sampled_batch(num_seeds=16, fanouts=(3, 2), id_space=5000, seed=2)
    x = torch.randn(nn[-1], 8)
    target = torch.arange(ptr.shape[0] - 1) * 3
    b = cxgnncomp.Batch(x, ptr, idx, nn, ne, target)
    assert b.target is target and b.block is None and b.edge_index is None
    b.tofile(str(tmp_path))
    assert np.array_equal(np.fromfile(str(tmp_path / "ptr.dat"), dtype="<i8"), ptr.numpy())
    assert np.array_equal(np.fromfile(str(tmp_path / "target.dat"), dtype="<i8"), target.numpy())
    assert np.array_equal(np.fromfile(str(tmp_path / "x.dat"), dtype="<f4"), x.numpy().ravel())
    # instance method, as upstream: fills the object, x stays flat
    b2 = cxgnncomp.Batch(None, None, None)
    assert b2.fromfile(str(tmp_path)) is None
    assert torch.equal(b2.x, x.flatten()) and torch.equal(b2.ptr, ptr) and torch.equal(b2.idx, idx)
    assert torch.equal(b2.target, target)
    # the ready-to-use loader
    b3 = cxgnncomp.Batch.load(str(tmp_path), 8)
    assert torch.equal(b3.x, x) and torch.equal(b3.target, target)
    assert b3.num_node_in_layer.tolist() == nn and b3.num_edge_in_layer.tolist() == ne
    b3.totype(torch.int32)
    assert b3.ptr.dtype == b3.idx.dtype == b3.target.dtype == torch.int32
    assert torch.equal(b3.ptr.long(), ptr)
    assert b3.to("cpu") is b3
    with pytest.raises(NotImplementedError):
        b3.todgl(4, 2)
    # a batch without target writes no target.dat, and fromfile leaves target alone
    d2 = tmp_path / "no_target"
    cxgnncomp.Batch(x, ptr, idx).tofile(str(d2))
    assert not (d2 / "target.dat").exists()
    pg = cxgnncomp.PyGBatch(x, torch.stack([idx, idx]))
    assert pg.x is x and pg.edge_index.shape[0] == 2
    with pytest.raises(TypeError):
        cxgnncomp.PyGBatch(x, ptr, idx)


def test_model_factories_build_the_reference_layouts():
    """get_conv_from_str / get_model_from_str / get_model (cxgnncomp/model.py:362-467) for the CSR
    graph types: classes, layer widths and state-dict keys of the reference's modules."""
    import types

    import cxgnncomp
    from cxgnncomp import get_conv_from_str, get_model, get_model_from_str
    for name, cls in (("gat", cxgnncomp.MyGATConv), ("GCN", cxgnncomp.MyGCNConv), ("sage", cxgnncomp.MySageConv),
                      ("rgcn", cxgnncomp.MyRGCNConv)):
        conv = get_conv_from_str(name, 8, 16, num_head=2, num_rel=3)
        assert type(conv) is cls
    with pytest.raises(AssertionError):
        get_conv_from_str("hgt", 8, 16)
    bn = {"bns.0." + k for k in ("weight", "bias", "running_mean", "running_var", "num_batches_tracked")}
    conv_keys = {
        "GCN": {"bias", "lin.weight"},
        "SAGE": {"lin_l.weight", "lin_l.bias", "lin_r.weight"},
        "GAT": {"att_src", "att_dst", "bias", "lin_src"},
        "RGCN": {"linear", "rel_weight", "single_linear.weight", "single_linear.bias"},
    }
    for mtype, keys in conv_keys.items():
        m = get_model_from_str(mtype, 8, 16, 4, "CSR_Layer", 2, num_head=2, num_rel=3, dataset="x")
        assert type(m) is getattr(cxgnncomp, mtype) and m.dropout == 0.5 and len(m.convs) == 2
        want = bn | {"convs.%d.%s" % (i, k) for i in range(2) for k in keys}
        assert set(m.state_dict()) == want, mtype
    assert get_model_from_str("sage", 8, 16, 4, "CSR", 3).convs[2].lin_l.weight.shape == (4, 16)
    with pytest.raises(NotImplementedError):
        get_model_from_str("GCN", 8, 16, 4, "DGL", 2)
    with pytest.raises(NotImplementedError):
        get_model_from_str("LSTM", 8, 16, 4, "CSR_Layer", 2)
    with pytest.raises(AssertionError):
        get_model_from_str("MLP", 8, 16, 4, "CSR_Layer", 2)

    def config(model, train_type="cxg"):
        ns = types.SimpleNamespace
        return ns(dl=ns(dataset=ns(feature_dim=8, num_classes=4, name="Arxiv"),
                        sampler=ns(train=ns(num_layer=3))),
                  train=ns(type=train_type, model=model))
    m = get_model(config({"type": "SAGE", "hidden_dim": 16, "dropout": 0.25}))
    assert type(m) is cxgnncomp.SAGE and m.graph_type == "CSR_Layer" and m.num_layer == 3 and m.dropout == 0.25
    assert m.convs[0].lin_l.weight.shape == (16, 8) and m.convs[2].lin_l.weight.shape == (4, 16)
    m = get_model(config({"type": "gat", "hidden_dim": 16, "dropout": 0.0, "heads": 4, "concat": True}))
    assert type(m) is cxgnncomp.GAT and m.convs[0].heads == 4 and m.convs[0].att_src.shape == (1, 4, 4)
    m = get_model(config({"type": "rgcn", "hidden_dim": 16, "dropout": 0.0, "num_rel": "7"}))
    assert type(m) is cxgnncomp.RGCN and m.convs[0].linear.shape == (7, 8, 16) and m.dataset_name == "arxiv"
    m = get_model(config(types.SimpleNamespace(type="gin", hidden_dim=16, dropout=0.0)))
    assert type(m) is cxgnncomp.GIN
    with pytest.raises(NotImplementedError):
        get_model(config({"type": "gcn", "hidden_dim": 16, "dropout": 0.0}, train_type="dgl"))


def test_topo_sort_matches_restatement(capsys):
    import cxgnncomp_backend as B
    rng = np.random.default_rng(41)
    for n, e, cyclic in ((1, 0, False), (50, 160, False), (300, 1500, False), (60, 200, True), (300, 900, True)):
        if cyclic:
            src, dst = rng.integers(0, n, e), rng.integers(0, n, e)
        else:
            a, b = rng.integers(0, n, e), rng.integers(0, n, e)
            keep = a != b
            relabel = rng.permutation(n)
            src, dst = relabel[np.minimum(a, b)[keep]], relabel[np.maximum(a, b)[keep]]
        ptr, idx = oracle.coo_to_csr(dst, src, n)
        indeg = np.bincount(dst, minlength=n).astype(np.int64)
        want, cnt = pyref.topo_sort(ptr, idx, indeg)
        got = B.topo_sort(torch.from_numpy(ptr), torch.from_numpy(idx), torch.from_numpy(indeg))
        assert got.dtype == torch.int64 and got[:cnt].tolist() == want
        msg = capsys.readouterr().out
        assert ("not a DAG" in msg) == (cnt != n)
    with pytest.raises(ValueError):
        B.topo_sort(torch.tensor([0, 1]), torch.tensor([5]), torch.tensor([0]))
