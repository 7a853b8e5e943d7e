"""Tensor-level wrappers over the C ABI: argument checks, output allocation,
workspace, current stream, and the per-graph cache of transposed CSRs.

torch is used for device memory and streams only; all arithmetic happens in
libcxgnn_hip.so.  Every function raises if a tensor is not a contiguous CUDA
tensor of the expected dtype -- the kernels index raw memory.
"""
import collections

import torch

from . import _lib

SPMM_MEAN = 1
SPMM_ACCUMULATE = 2


def as_int(v):
    """Scalars arrive as Python ints or 0-d tensors (cxgnncomp/graph_conv.py:41-50)."""
    if isinstance(v, torch.Tensor):
        return int(v.item())
    return int(v)


def _req(t, name, dtype, ndim=None):
    if not isinstance(t, torch.Tensor):
        raise TypeError("%s must be a tensor" % name)
    if not t.is_cuda:
        raise ValueError("%s must be a CUDA tensor" % name)
    if t.dtype != dtype:
        raise ValueError("%s must be %s, got %s" % (name, dtype, t.dtype))
    if not t.is_contiguous():
        raise ValueError("%s must be contiguous" % name)
    if ndim is not None and t.dim() not in (ndim if isinstance(ndim, tuple) else (ndim,)):
        raise ValueError("%s must have %s dims, got %d" % (name, ndim, t.dim()))


def _workspace(nbytes, device):
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


def _check_graph(ptr, idx, n_rows, dtype=torch.int64):
    _req(ptr, "ptr", dtype, 1)
    _req(idx, "idx", dtype, 1)
    if n_rows < 0 or n_rows + 1 > ptr.shape[0]:
        raise ValueError("num_node=%d does not fit ptr of length %d" % (n_rows, ptr.shape[0]))
    if ptr.device != idx.device:
        raise ValueError("ptr and idx are on different devices")


def spmm(ptr, idx, x, n_rows, *, mean=False, val=None, val_perm=None, out=None, accumulate=False):
    """out[r] = sum_{e in row r} (val[vrow(e)] *) x[idx[e]] for r < n_rows.

    x is [n_src, F] or [n_src, H, C]; val (optional) is [E] or [E, H].  Returns
    a new [n_rows, ...] tensor unless ``out`` is given.
    """
    lib = _lib.load()
    int32 = ptr.dtype == torch.int32
    _check_graph(ptr, idx, n_rows, torch.int32 if int32 else torch.int64)
    _req(x, "x", torch.float32, (2, 3))
    if x.device != ptr.device:
        raise ValueError("x and ptr are on different devices")
    heads = 1
    channels = x.shape[-1]
    if val is not None:
        _req(val, "val", torch.float32, (1, 2))
        if val.dim() == 2:
            heads = val.shape[1]
            if x.dim() != 3 or x.shape[1] != heads:
                raise ValueError("val has %d heads but x has shape %s" % (heads, tuple(x.shape)))
        elif x.dim() == 3:
            if x.shape[1] != 1:
                raise ValueError("1-D val needs x of shape [N, F] or [N, 1, F]")
        need = idx.shape[0] if val_perm is None else 0
        if val.shape[0] < need:
            raise ValueError("val has %d rows, idx has %d" % (val.shape[0], idx.shape[0]))
        if val_perm is not None:
            _req(val_perm, "val_perm", torch.int64, 1)
            if val_perm.shape[0] < idx.shape[0]:
                raise ValueError("val_perm shorter than idx")
    elif x.dim() == 3:
        channels = x.shape[1] * x.shape[2]
    row = heads * channels if val is not None else channels
    out_shape = (n_rows,) + tuple(x.shape[1:])
    if out is None:
        out = torch.empty(out_shape, dtype=torch.float32, device=x.device)
    else:
        _req(out, "out", torch.float32)
        if tuple(out.shape) != out_shape:
            raise ValueError("out has shape %s, expected %s" % (tuple(out.shape), out_shape))
    if n_rows == 0:
        return out
    n_cap = idx.shape[0]
    ws_bytes = lib.cxg_spmm_workspace_bytes(n_cap, row)
    ws = _workspace(ws_bytes, x.device)
    flags = (SPMM_MEAN if mean else 0) | (SPMM_ACCUMULATE if accumulate else 0)
    stream = _lib.current_stream(x.device)
    with torch.cuda.device(x.device):
        if val is None:
            fn = lib.cxg_spmm_sum_f32_i32 if int32 else lib.cxg_spmm_sum_f32
            st = fn(ptr.data_ptr(), _lib.ptr(idx), _lib.ptr(x), row, out.data_ptr(), row, n_rows,
                    n_cap, row, flags, ws.data_ptr(), ws.numel(), stream)
        else:
            if int32:
                raise ValueError("weighted SpMM needs int64 ptr/idx")
            st = lib.cxg_spmm_weighted_f32(ptr.data_ptr(), _lib.ptr(idx), val.data_ptr(),
                                           _lib.ptr(val_perm), _lib.ptr(x), row, out.data_ptr(), row,
                                           n_rows, n_cap, heads, channels, flags, ws.data_ptr(),
                                           ws.numel(), stream)
    _lib.check(st)
    return out


# --------------------------------------------------------------------------- #
# transposed-graph cache
# --------------------------------------------------------------------------- #
class TransposedGraph:
    """CSR of the reversed graph: rows = source nodes, idx_t = destination ids,
    perm = position of each transposed edge in the original idx array."""

    __slots__ = ("ptr_t", "idx_t", "perm", "n_edges", "n_src", "n_dst", "_keep", "_inv_deg_t")

    def __init__(self, ptr_t, idx_t, perm, n_edges, n_src, n_dst, keep):
        self.ptr_t, self.idx_t, self.perm = ptr_t, idx_t, perm
        self.n_edges, self.n_src, self.n_dst = n_edges, n_src, n_dst
        self._keep = keep  # the tensors the key was made from stay alive while cached
        self._inv_deg_t = None


_GRAPH_CACHE = collections.OrderedDict()
_GRAPH_CACHE_CAP = 8


def clear_graph_cache():
    _GRAPH_CACHE.clear()


def set_graph_cache_capacity(n):
    global _GRAPH_CACHE_CAP
    _GRAPH_CACHE_CAP = max(0, int(n))
    while len(_GRAPH_CACHE) > _GRAPH_CACHE_CAP:
        _GRAPH_CACHE.popitem(last=False)


def csr_transpose(ptr, idx, n_rows, n_src):
    """Uncached transposition; returns (ptr_t, idx_t, perm, n_edges)."""
    lib = _lib.load()
    _check_graph(ptr, idx, n_rows)
    n_edges = int(ptr[n_rows].item())
    first = int(ptr[0].item())
    if first != 0:
        raise ValueError("ptr[0] must be 0")
    if n_edges > idx.shape[0]:
        raise ValueError("ptr[num_node]=%d exceeds idx length %d" % (n_edges, idx.shape[0]))
    dev = ptr.device
    ptr_t = torch.empty(n_src + 1, dtype=torch.int64, device=dev)
    idx_t = torch.empty(n_edges, dtype=torch.int64, device=dev)
    perm = torch.empty(n_edges, dtype=torch.int64, device=dev)
    ws_bytes = lib.cxg_csr_transpose_workspace_bytes(n_edges, n_src)
    ws = _workspace(ws_bytes, dev)
    with torch.cuda.device(dev):
        st = lib.cxg_csr_transpose_i64(ptr.data_ptr(), _lib.ptr(idx), n_rows, n_src, n_edges,
                                       ptr_t.data_ptr(), _lib.ptr(idx_t), _lib.ptr(perm),
                                       ws.data_ptr(), ws.numel(), _lib.current_stream(dev))
    _lib.check(st)
    return ptr_t, idx_t, perm, n_edges


def transposed(ptr, idx, n_rows, n_src):
    """Cached TransposedGraph of (ptr[:n_rows+1], idx) with n_src source nodes."""
    key = (ptr.data_ptr(), idx.data_ptr(), ptr.shape[0], idx.shape[0], n_rows, n_src,
           ptr._version, idx._version, ptr.device.index)
    g = _GRAPH_CACHE.get(key)
    if g is not None:
        _GRAPH_CACHE.move_to_end(key)
        return g
    ptr_t, idx_t, perm, n_edges = csr_transpose(ptr, idx, n_rows, n_src)
    g = TransposedGraph(ptr_t, idx_t, perm, n_edges, n_src, n_rows, (ptr, idx))
    if _GRAPH_CACHE_CAP > 0:
        _GRAPH_CACHE[key] = g
        while len(_GRAPH_CACHE) > _GRAPH_CACHE_CAP:
            _GRAPH_CACHE.popitem(last=False)
    return g


def edge_value_degree(ptr, n_rows, n_edges):
    lib = _lib.load()
    _req(ptr, "ptr", torch.int64, 1)
    if n_rows + 1 > ptr.shape[0]:
        raise ValueError("num_dst=%d does not fit ptr" % n_rows)
    out = torch.zeros(n_edges, dtype=torch.float32, device=ptr.device)
    with torch.cuda.device(ptr.device):
        st = lib.cxg_edge_value_degree_f32(ptr.data_ptr(), n_rows, out.data_ptr(),
                                           _lib.current_stream(ptr.device))
    _lib.check(st)
    return out


def inv_degree_transposed(g, ptr, n_rows):
    """1/deg(dst) per edge, in transposed edge order (cached on the graph)."""
    if g._inv_deg_t is None:
        inv = edge_value_degree(ptr, n_rows, g.n_edges)
        g._inv_deg_t = inv[g.perm] if g.n_edges > 0 else inv
    return g._inv_deg_t


def csr_row_ids(ptr, n_rows, n_edges):
    lib = _lib.load()
    _req(ptr, "ptr", torch.int64, 1)
    rows = torch.empty(n_edges, dtype=torch.int64, device=ptr.device)
    with torch.cuda.device(ptr.device):
        st = lib.cxg_csr_row_ids_i64(ptr.data_ptr(), n_rows, n_edges, _lib.ptr(rows),
                                     _lib.current_stream(ptr.device))
    _lib.check(st)
    return rows
