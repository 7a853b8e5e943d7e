"""CPU oracle -- TEST INFRASTRUCTURE ONLY.

A restatement of the reference's graph-kernel semantics on the CPU, used by
tests/, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py`` to check (and time a baseline for) the HIP kernels.  The shipped
package never imports this module.

Two layers:
  * ``cxg_oracle.c`` (plain C, gcc) -- the CUDA kernels and C++ host functions,
    reached through the numpy wrappers below;
  * ``pyref.py`` -- the reference's pure-Python / PyTorch functions
    (``spmm_torch``, op-wise edge softmax, ``TypedLinearS2DSort``, scheduling
    helpers), restated with numpy / CPU torch.

Which checks pin each function (independent library routines, closed forms,
brute force) is listed in tests/test_oracle_*.py; functions without such a
check are marked "parity unpinned" there and below.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SRC = os.path.join(_HERE, "cxg_oracle.c")
_LIB = os.path.join(_HERE, "_build", "libcxg_oracle.so")


def build(force=False):
    """Compile cxg_oracle.c with gcc into oracle/_build/libcxg_oracle.so."""
    os.makedirs(os.path.dirname(_LIB), exist_ok=True)
    if (not force and os.path.exists(_LIB)
            and os.path.getmtime(_LIB) >= os.path.getmtime(_SRC)):
        return _LIB
    cmd = ["gcc", "-O2", "-fPIC", "-shared", "-std=c99", "-Wall", "-o", _LIB, _SRC, "-lm"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("gcc failed:\n" + r.stdout + r.stderr)
    return _LIB


_lib = None


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            build()
        _lib = ctypes.CDLL(_LIB)
        _lib.orc_neighbor_grouping.restype = ctypes.c_int64
        _lib.orc_rel_schedule_one.restype = ctypes.c_int64
    return _lib


def _i64(a):
    return np.ascontiguousarray(np.asarray(a), dtype=np.int64)


def _i32(a):
    return np.ascontiguousarray(np.asarray(a), dtype=np.int32)


def _f32(a):
    return np.ascontiguousarray(np.asarray(a), dtype=np.float32)


def _u8(a):
    return np.ascontiguousarray(np.asarray(a).astype(np.uint8))


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


_L = ctypes.c_int64
_I = ctypes.c_int
_F = ctypes.c_float


def spmm(ptr, idx, x, n_rows, val=None, mean=False, seq32=False):
    """out[r,h,c] = sum_e val[e,h] x[idx[e],h,c]; x [N,F] or [N,H,C]; val [E] or [E,H]."""
    ptr, idx, x = _i64(ptr), _i64(idx), _f32(x)
    heads, channels = 1, int(np.prod(x.shape[1:]))
    if val is not None:
        val = _f32(val)
        if val.ndim == 2:
            heads = val.shape[1]
            assert x.ndim == 3 and x.shape[1] == heads
            channels = x.shape[2]
    out = np.zeros((n_rows,) + x.shape[1:], dtype=np.float32)
    _load().orc_spmm(_p(ptr), _p(idx), _p(val), _p(x), _p(out), _L(n_rows), _I(heads),
                     _I(channels), _I(int(mean)), _I(int(seq32)))
    return out


def spmm_bwd(ptr, idx, g, n_rows, n_src, val=None, mean=False):
    """gx[idx[e],h,c] += val[e,h] * g[row(e),h,c] (mean: / deg(row))."""
    ptr, idx, g = _i64(ptr), _i64(idx), _f32(g)
    heads, channels = 1, int(np.prod(g.shape[1:]))
    if val is not None:
        val = _f32(val)
        if val.ndim == 2:
            heads = val.shape[1]
            channels = g.shape[2]
    gx = np.zeros((n_src,) + g.shape[1:], dtype=np.float32)
    _load().orc_spmm_bwd(_p(ptr), _p(idx), _p(val), _p(g), _p(gx), _L(n_rows), _L(n_src), _I(heads),
                         _I(channels), _I(int(mean)))
    return gx


def edge_grad(ptr, idx, x, g, n_rows, heads=None):
    """gval[e,h] = <g[row(e),h,:], x[idx[e],h,:]>; returns [E] for 2-D x, else [E,H]."""
    ptr, idx, x, g = _i64(ptr), _i64(idx), _f32(x), _f32(g)
    if x.ndim == 2:
        h, c = 1, x.shape[1]
    else:
        h, c = x.shape[1], x.shape[2]
    E = int(ptr[n_rows])
    out = np.zeros((E, h), dtype=np.float32)
    _load().orc_edge_grad(_p(ptr), _p(idx), _p(x), _p(g), _p(out), _L(n_rows), _I(h), _I(c))
    return out[:, 0] if x.ndim == 2 else out


def spmm_prereduce(ptr, idx, val, x, n_rows):
    ptr, idx, val, x = _i64(ptr), _i64(idx), _f32(val), _f32(x)
    out = np.zeros((n_rows, x.shape[2]), dtype=np.float32)
    _load().orc_spmm_prereduce(_p(ptr), _p(idx), _p(val), _p(x), _p(out), _L(n_rows),
                               _I(x.shape[1]), _I(x.shape[2]))
    return out


def sddmm(src, dst, src_feat, dst_feat, n_edges=None):
    """out[e,h] = <src_feat[src[e],h,:], dst_feat[dst[e],(h,):]>."""
    src, dst, a, b = _i64(src), _i64(dst), _f32(src_feat), _f32(dst_feat)
    n_edges = src.shape[0] if n_edges is None else n_edges
    out = np.zeros((n_edges, a.shape[1]), dtype=np.float32)
    _load().orc_sddmm(_p(src), _p(dst), _p(a), _p(b), _p(out), _L(n_edges), _I(a.shape[1]),
                      _I(a.shape[2]), _I(int(b.ndim == 3)))
    return out


def edge_softmax_fwd(ptr, idx, att_dst, att_src, n_edges, slope):
    ptr, idx, ad, as_ = _i64(ptr), _i64(idx), _f32(att_dst), _f32(att_src)
    H = ad.shape[1]
    out = np.zeros((n_edges, H), dtype=np.float32)
    mask = np.zeros((n_edges, H), dtype=np.uint8)
    _load().orc_edge_softmax_fwd(_p(ptr), _p(idx), _p(ad), _p(as_), _p(out), _p(mask),
                                 _L(ad.shape[0]), _I(H), _F(slope))
    return out, mask.astype(bool)


def edge_softmax_bwd(ptr, idx, grad, mask, out, n_dst, n_src, slope):
    ptr, idx, g, o = _i64(ptr), _i64(idx), _f32(grad), _f32(out)
    m = _u8(mask)
    H = o.shape[1]
    g_dst = np.zeros((n_dst, H), dtype=np.float32)
    g_src = np.zeros((n_src, H), dtype=np.float32)
    _load().orc_edge_softmax_bwd(_p(ptr), _p(idx), _p(g), _p(m), _p(o), _p(g_dst), _p(g_src),
                                 _L(n_dst), _L(n_src), _I(H), _F(slope))
    return g_dst, g_src


def edge_value_degree(ptr, n_dst, n_edges):
    ptr = _i64(ptr)
    out = np.zeros(n_edges, dtype=np.float32)
    _load().orc_edge_value_degree(_p(ptr), _p(out), _L(n_dst))
    return out


def spmv(ptr, idx, x, n_dst):
    ptr, idx, x = _i64(ptr), _i64(idx), _f32(x)
    out = np.zeros(n_dst, dtype=np.float32)
    _load().orc_spmv(_p(ptr), _p(idx), _p(x), _p(out), _L(n_dst))
    return out


def gspmm(rowptr, colind, b, red, comp=2, val=None):
    """dgSPARSE-style generalised SpMM; red 0 sum / 1 max / 2 min / 3 mean,
    comp 0 add / 1 sub / 2 mul / 3 div (the C enum values of dgsparse.h:13-14)."""
    rowptr, colind, b = _i32(rowptr), _i32(colind), _f32(b)
    val = None if val is None else _f32(val)
    n = rowptr.shape[0] - 1
    out = np.zeros((n, b.shape[1]), dtype=np.float32)
    _load().orc_gspmm(_p(rowptr), _p(colind), _p(val), _p(b), _p(out), _L(n), _I(b.shape[1]), _I(int(red)),
                      _I(int(comp)))
    return out


def gather_fwd(x, dest, n_nodes):
    x, dest = _f32(x), _i64(dest)
    out = np.zeros((n_nodes, x.shape[1]), dtype=np.float32)
    _load().orc_gather_fwd(_p(x), _p(dest), _p(out), _L(dest.shape[0]), _L(n_nodes), _I(x.shape[1]))
    return out


def gather_bwd(gout, dest):
    gout, dest = _f32(gout), _i64(dest)
    gin = np.zeros((dest.shape[0], gout.shape[1]), dtype=np.float32)
    _load().orc_gather_bwd(_p(gout), _p(dest), _p(gin), _L(dest.shape[0]), _I(gout.shape[1]))
    return gin


def selective_aggr_fwd(x, ptr, idx, mask, out, n_rows):
    """Returns out + masked aggregation (the reference accumulates in place)."""
    ptr, idx, x = _i64(ptr), _i64(idx), _f32(x)
    out = _f32(out).copy()
    m = _u8(mask)
    _load().orc_selective_aggr_fwd(_p(ptr), _p(idx), _p(m), _p(x), _p(out), _L(n_rows),
                                   _I(x.shape[1]))
    return out


def selective_aggr_bwd(g, ptr, idx, mask, gx, n_rows):
    ptr, idx, g = _i64(ptr), _i64(idx), _f32(g)
    gx = _f32(gx).copy()
    m = _u8(mask)
    _load().orc_selective_aggr_bwd(_p(ptr), _p(idx), _p(m), _p(g), _p(gx), _L(n_rows),
                                   _L(gx.shape[0]), _I(g.shape[1]))
    return gx


def target_aggr_fwd(x, ptr, idx, targets, out, n_rows):
    ptr, idx, t, x = _i64(ptr), _i64(idx), _i64(targets), _f32(x)
    out = _f32(out).copy()
    _load().orc_target_aggr_fwd(_p(ptr), _p(idx), _p(t), _p(x), _p(out), _L(n_rows),
                                _L(out.shape[0]), _I(x.shape[1]))
    return out


def target_aggr_bwd(g, ptr, idx, targets, gx, n_rows):
    ptr, idx, t, g = _i64(ptr), _i64(idx), _i64(targets), _f32(g)
    gx = _f32(gx).copy()
    _load().orc_target_aggr_bwd(_p(ptr), _p(idx), _p(t), _p(g), _p(gx), _L(n_rows),
                                _L(gx.shape[0]), _I(g.shape[1]))
    return gx


def aggr_rel_fwd(x, ptr, idx, rel, n_rows, num_rel):
    ptr, idx, rel, x = _i64(ptr), _i64(idx), _i32(rel), _f32(x)
    out = np.zeros((n_rows, x.shape[1]), dtype=np.float32)
    _load().orc_aggr_rel_fwd(_p(ptr), _p(idx), _p(rel), _p(x), _p(out), _L(n_rows),
                             _L(x.shape[0] // num_rel), _I(x.shape[1]))
    return out


def aggr_rel_bwd(g, ptr, idx, rel, n_rows, num_rel, n_per_rel):
    ptr, idx, rel, g = _i64(ptr), _i64(idx), _i32(rel), _f32(g)
    gx = np.zeros((num_rel * n_per_rel, g.shape[1]), dtype=np.float32)
    _load().orc_aggr_rel_bwd(_p(ptr), _p(idx), _p(rel), _p(g), _p(gx), _L(n_rows), _L(n_per_rel),
                             _I(num_rel), _I(g.shape[1]))
    return gx


def rgcn_fused(x, ptr, idx, w, rel, n_rows):
    ptr, idx, rel, x, w = _i64(ptr), _i64(idx), _i32(rel), _f32(x), _f32(w)
    out = np.zeros((n_rows, w.shape[2]), dtype=np.float32)
    _load().orc_rgcn_fused(_p(ptr), _p(idx), _p(rel), _p(x), _p(w), _p(out), _L(n_rows),
                           _I(w.shape[1]), _I(w.shape[2]))
    return out


def typed_linear(x, w, types, out=None, src=None, dst=None, n_out=None):
    """out[dst_i] += x[src_i] @ w[types[i]] (returns the updated copy of out)."""
    x, w, types = _f32(x), _f32(w), _i32(types)
    n = types.shape[0]
    src = None if src is None else _i64(src)
    dst = None if dst is None else _i64(dst)
    if out is None:
        n_out = n if n_out is None else n_out
        out = np.zeros((n_out, w.shape[2]), dtype=np.float32)
    else:
        out = _f32(out).copy()
    _load().orc_typed_linear(_p(x), _p(w), _p(out), _p(src), _p(dst), _p(types), _L(n),
                             _L(out.shape[0]), _I(w.shape[1]), _I(w.shape[2]))
    return out


def pad_rel(rel, count, thres, num_rel, base, idx=None):
    """In-place on copies; returns rel (and idx if given)."""
    rel = _i64(rel).copy()
    count = _i64(count)
    idx_c = None if idx is None else _i64(idx).copy()
    _load().orc_pad_rel(_p(rel), _p(idx_c), _p(count), _I(thres), _I(num_rel), _L(base))
    return rel if idx is None else (rel, idx_c)


def neighbor_grouping(ptr, thres=32):
    ptr = _i64(ptr)
    n_rows = ptr.shape[0] - 1
    lib = _load()
    n = lib.orc_neighbor_grouping(_p(ptr), _L(n_rows), _L(thres), None, None)
    new_ptr = np.zeros(n + 1, dtype=np.int64)
    new_target = np.zeros(n, dtype=np.int64)
    lib.orc_neighbor_grouping(_p(ptr), _L(n_rows), _L(thres), _p(new_ptr), _p(new_target))
    return new_ptr, new_target


def rel_schedule(ptr, idx, rel, num_node_in_layer, num_rel):
    """Returns [ptr_0, idx_0, target_0, ..., ptr_{R-1}, idx_{R-1}, target_{R-1}, counts[R,L]]
    with L = len(num_node_in_layer) - 1 (src/cpp/src/schedule.cu:9)."""
    ptr, idx, rel, nl = _i64(ptr), _i64(idx), _i32(rel), _i64(num_node_in_layer)
    n_rows = ptr.shape[0] - 1
    L = nl.shape[0] - 1
    lib = _load()
    out = []
    counts = np.zeros((num_rel, max(L, 0)), dtype=np.int64)
    for r in range(num_rel):
        ne = ctypes.c_int64(0)
        rows = lib.orc_rel_schedule_one(_p(ptr), _p(idx), _p(rel), _L(n_rows), _I(r), _p(nl), _I(L),
                                        None, None, None, None, ctypes.byref(ne))
        sp = np.zeros(rows + 1, dtype=np.int64)
        si = np.zeros(ne.value, dtype=np.int64)
        stg = np.zeros(rows, dtype=np.int64)
        lc = np.zeros(max(L, 1), dtype=np.int64)
        lib.orc_rel_schedule_one(_p(ptr), _p(idx), _p(rel), _L(n_rows), _I(r), _p(nl), _I(L), _p(sp),
                                 _p(si), _p(stg), _p(lc), None)
        counts[r, :] = lc[:L]
        out += [sp, si, stg]
    out.append(counts)
    return out


def csr_transpose(ptr, idx, n_rows, n_cols):
    ptr, idx = _i64(ptr), _i64(idx)
    E = int(ptr[n_rows])
    ptr_t = np.zeros(n_cols + 1, dtype=np.int64)
    idx_t = np.zeros(E, dtype=np.int64)
    perm = np.zeros(E, dtype=np.int64)
    _load().orc_csr_transpose(_p(ptr), _p(idx), _L(n_rows), _L(n_cols), _p(ptr_t), _p(idx_t),
                              _p(perm))
    return ptr_t, idx_t, perm


def coo_to_csr(src, dst, n_dst):
    src, dst = _i64(src), _i64(dst)
    ptr = np.zeros(n_dst + 1, dtype=np.int64)
    idx = np.zeros(src.shape[0], dtype=np.int64)
    _load().orc_coo_to_csr(_p(src), _p(dst), _L(src.shape[0]), _L(n_dst), _p(ptr), _p(idx))
    return ptr, idx
