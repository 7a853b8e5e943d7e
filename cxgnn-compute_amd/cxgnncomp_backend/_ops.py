"""Tensor-level wrappers over the C ABI: argument checks, output allocation,
workspace, current stream, and the per-graph cache of transposed CSRs.

torch is used for device memory and streams only; all arithmetic happens in
libcxgnn_hip.so.  Every function raises if a tensor is not a contiguous CUDA
tensor of the expected dtype -- the kernels index raw memory.
"""

import torch

from . import _lib
from ._lib import native as _native

_C = _native()

SPMM_MEAN = 1
SPMM_ACCUMULATE = 2
SPMM_HINT_EXACT_EDGES = 4
SPMM_DOT_AT_EDGE = 8


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


def spmm(ptr, idx, x, n_rows, *, mean=False, val=None, val_perm=None, out=None, accumulate=False, bias=None):
    """out[r] = sum_{e in row r} (val[vrow(e)] *) x[idx[e]] for r < n_rows.

    x is [n_src, F] or [n_src, H, C]; val (optional) is [E] or [E, H].  Returns
    a new [n_rows, ...] tensor unless ``out`` is given.  ``bias`` (with val, without mean:
    one float per column of a row) is added to every output row as it is stored.
    Checks, allocation and the call into the library happen in the compiled host layer.
    """
    return _C.spmm(ptr, idx, x, int(n_rows), mean, val, val_perm, out, accumulate, bias)


def spmm_dot_supported(heads, channels, at_edge=False):
    """Shapes ``spmm_dot`` takes (the others use spmm and sddmm_csr): rows of 256 * k floats, and --
    with the weights read through ``val_perm`` and the products left at the edge's own position
    (``at_edge``) -- single-head rows of 16 .. 128 floats, a multiple of 4."""
    if (heads * channels) % 256 == 0 and channels in (32, 64, 128, 256):
        return True
    return bool(at_edge) and heads == 1 and 16 <= channels <= 128 and channels % 4 == 0


def spmm_dot(ptr, idx, x, n_rows, val, val_perm, dot_b, dot_out, dot_at_edge=False):
    """Weighted multi-head SpMM that also stores, for every edge e of output row r,
    dot_out[vrow(e), h] = <x[idx[e], h, :], dot_b[r, h, :]> (vrow(e) = val_perm[e], or e; with
    ``dot_at_edge`` always e, the position in idx: contiguous stores):
    (out [n_rows, H, C], dot_out).  x [n_src, H, C], val [*, H], dot_b [>= n_rows, H, C],
    dot_out [*, H] (the entries of the edges of the first n_rows rows are written)."""
    lib = _lib.load()
    _check_graph(ptr, idx, n_rows)
    _req(x, "x", torch.float32, 3)
    _req(val, "val", torch.float32, 2)
    _req(dot_b, "dot_b", torch.float32, 3)
    _req(dot_out, "dot_out", torch.float32, 2)
    heads, channels = x.shape[1], x.shape[2]
    if val.shape[1] != heads or dot_out.shape[1] != heads or tuple(dot_b.shape[1:]) != (heads, channels):
        raise ValueError("head / channel counts of x %s, val %s, dot_b %s, dot_out %s differ"
                         % (tuple(x.shape), tuple(val.shape), tuple(dot_b.shape), tuple(dot_out.shape)))
    if dot_b.shape[0] < n_rows:
        raise ValueError("dot_b has %d rows, %d needed" % (dot_b.shape[0], n_rows))
    if val_perm is not None:
        _req(val_perm, "val_perm", torch.int64, 1)
        if val_perm.shape[0] < idx.shape[0]:
            raise ValueError("val_perm shorter than idx")
        if dot_out.shape[0] != val.shape[0]:
            raise ValueError("dot_out must have a row per row of val")
    elif val.shape[0] < idx.shape[0] or dot_out.shape[0] < idx.shape[0]:
        raise ValueError("val / dot_out shorter than idx")
    if not spmm_dot_supported(heads, channels, at_edge=dot_at_edge and val_perm is not None):
        raise ValueError("spmm_dot needs heads*channels %% 256 == 0 and channels in (32, 64, 128, 256), or -- with "
                         "val_perm and dot_at_edge -- one head of 16 .. 128 channels, a multiple of 4")
    row = heads * channels
    out = torch.empty((n_rows, heads, channels), dtype=torch.float32, device=x.device)
    if n_rows == 0:
        return out, dot_out
    ws = _workspace(lib.cxg_spmm_workspace_bytes(idx.shape[0], row), x.device)
    flags = SPMM_HINT_EXACT_EDGES if n_rows == ptr.shape[0] - 1 else 0
    if dot_at_edge:
        flags |= SPMM_DOT_AT_EDGE
    with torch.cuda.device(x.device):
        st = lib.cxg_spmm_weighted_dot_f32(ptr.data_ptr(), _lib.ptr(idx), val.data_ptr(), _lib.ptr(val_perm),
                                           _lib.ptr(x), row, out.data_ptr(), row, _lib.ptr(dot_b), row,
                                           dot_out.data_ptr(), n_rows, idx.shape[0], heads, channels, flags,
                                           ws.data_ptr(), ws.numel(), _lib.current_stream(x.device))
    _lib.check(st)
    return out, dot_out


# --------------------------------------------------------------------------- #
# transposed-graph cache
# --------------------------------------------------------------------------- #
TransposedGraph = _C.TransposedGraph      # ptr_t, idx_t, perm, n_edges, n_src, n_dst (see csrc_ext/backend_ext.cpp)

_GRAPH_CACHE_CAP = 8


def spmm_bf16_rows(ptr, idx, x, n_rows, val=None, val_perm=None, out_bf16=False, mean=False):
    """Single-head aggregation whose gathered rows (x of dtype bfloat16) and / or stored rows
    (``out_bf16``) are bf16, summed in fp32 (cxg_spmm_bf16_rows; rows of 4 .. 128 values, a
    multiple of 4)."""
    lib = _lib.load()
    _check_graph(ptr, idx, n_rows)
    if x.dim() != 2 or not x.is_contiguous() or x.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("x must be a contiguous [N, F] float32 or bfloat16 tensor")
    x_bf16 = x.dtype == torch.bfloat16
    if not (x_bf16 or out_bf16):
        raise ValueError("fp32 rows on both sides: use spmm")
    feat = x.shape[1]
    out = torch.empty((n_rows, feat), dtype=torch.bfloat16 if out_bf16 else torch.float32, device=x.device)
    if n_rows == 0:
        return out
    if val is not None:
        _req(val, "val", torch.float32, 1)
    if val_perm is not None:
        _req(val_perm, "val_perm", torch.int64, 1)
    ws = _workspace(lib.cxg_spmm_workspace_bytes(idx.shape[0], feat), x.device)
    with torch.cuda.device(x.device):
        st = lib.cxg_spmm_bf16_rows(ptr.data_ptr(), _lib.ptr(idx), _lib.ptr(val), _lib.ptr(val_perm), _lib.ptr(x), feat,
                                    int(x_bf16), out.data_ptr(), feat, int(out_bf16), n_rows, idx.shape[0], feat,
                                    SPMM_MEAN if mean else 0, ws.data_ptr(), ws.numel(), _lib.current_stream(x.device))
    _lib.check(st)
    return out


def spmm_heads_supported(heads, feat):
    """Shapes cxg_spmm_weighted_heads_f32 takes."""
    return heads in (2, 4, 8) and 20 <= feat <= 128 and feat % 4 == 0


def spmm_weighted_heads(ptr, idx, val, x, n_rows):
    """out[r, h, :] = sum_e val[e, h] * x[idx[e], :] for val [E, H] and x [n_src, F] (rows may be
    strided): one gathered row per edge under H weights; returns [n_rows, H, F]."""
    lib = _lib.load()
    _check_graph(ptr, idx, n_rows)
    _req(val, "val", torch.float32, 2)
    if x.dim() != 2 or x.dtype != torch.float32 or not x.is_cuda or (x.shape[1] != 1 and x.stride(1) != 1):
        raise ValueError("x must be a [N, F] float32 CUDA tensor with contiguous rows")
    heads, feat = val.shape[1], x.shape[1]
    if val.shape[0] < idx.shape[0]:
        raise ValueError("val has %d rows for %d edges" % (val.shape[0], idx.shape[0]))
    out = torch.empty((n_rows, heads, feat), dtype=torch.float32, device=x.device)
    if n_rows == 0:
        return out
    ldx = x.stride(0) if x.shape[0] > 1 else feat
    ws = _workspace(lib.cxg_spmm_workspace_bytes(idx.shape[0], heads * feat), x.device)
    with torch.cuda.device(x.device):
        st = lib.cxg_spmm_weighted_heads_f32(ptr.data_ptr(), _lib.ptr(idx), _lib.ptr(val), _lib.ptr(x), ldx,
                                             out.data_ptr(), heads * feat, n_rows, idx.shape[0], heads, feat, 0,
                                             ws.data_ptr(), ws.numel(), _lib.current_stream(x.device))
    _lib.check(st)
    return out


def clear_graph_cache():
    _C.clear_graph_cache()


def set_graph_cache_capacity(n):
    global _GRAPH_CACHE_CAP
    _GRAPH_CACHE_CAP = max(0, int(n))
    _C.set_graph_cache_capacity(_GRAPH_CACHE_CAP)


def csr_transpose(ptr, idx, n_rows, n_src):
    """Uncached transposition by a stable sort; returns (ptr_t, idx_t, perm, n_edges)."""
    return _C.csr_transpose(ptr, idx, int(n_rows), int(n_src))


def csr_transpose_prefix(whole, ptr, n_rows, n_src):
    """Transposed graph of the first n_rows rows from the TransposedGraph ``whole`` of more rows of
    the same (ptr, idx): a stable compaction of its entries (see cxg_csr_transpose_prefix_i64).
    Returns (ptr_t, idx_t, perm, n_edges)."""
    return _C.csr_transpose_prefix(whole, ptr, int(n_rows), int(n_src))


def note_layer(ptr, idx, n_rows, n_src):
    """Tell the transposed-graph cache that a layer aggregates rows [0, n_rows) of (ptr, idx)
    over n_src sources (called by the forward passes whose backward needs the transposed graph):
    the layers of a sampled mini-batch work on nested row prefixes of one CSR, and the backward
    pass, which meets the smallest layer first, then sorts the largest once and cuts the others
    out of it."""
    _C.note_layer(ptr, idx, int(n_rows), int(n_src))


def note_edge_counts(ptr, idx, rows, edges):
    """Tell the transposed-graph cache how many edges the first rows[k] rows of (ptr, idx) hold
    (``num_node_in_layer`` / ``num_edge_in_layer`` of a sampled batch): the reversed graphs of
    those row prefixes are then built without reading ptr[rows[k]] back from the device.  The
    counts are trusted."""
    _C.note_edge_counts(ptr, idx, [int(r) for r in rows], [int(e) for e in edges])


def transposed(ptr, idx, n_rows, n_src):
    """Cached TransposedGraph of (ptr[:n_rows+1], idx) with n_src source nodes (LRU of
    ``set_graph_cache_capacity`` graphs, kept in the compiled host layer)."""
    return _C.transposed(ptr, idx, int(n_rows), int(n_src))


class DestGroups:
    """Edge positions grouped by destination: ptr [n+1] and perm [E] (stable)."""

    __slots__ = ("ptr", "perm")

    def __init__(self, ptr, perm):
        self.ptr, self.perm = ptr, perm


def dest_groups(dest, n_rows):
    """DestGroups of an edge -> node destination array (one stable sort, cached in the compiled
    host layer per destination array)."""
    return DestGroups(*_C.dest_groups(dest, int(n_rows)))


def edge_value_degree(ptr, n_rows, n_edges):
    return _C.edge_value_degree_raw(ptr, int(n_rows), int(n_edges))


def inv_degree_transposed(g, ptr, n_rows):
    """1/deg(dst) per edge, in transposed edge order (kept with the graph)."""
    return _C.inv_degree_transposed(g, ptr, int(n_rows))


def csr_row_ids(ptr, n_rows, n_edges):
    lib = _lib.load()
    _req(ptr, "ptr", torch.int64, 1)
    rows = torch.empty(n_edges, dtype=torch.int64, device=ptr.device)
    with torch.cuda.device(ptr.device):
        st = lib.cxg_csr_row_ids_i64(ptr.data_ptr(), n_rows, n_edges, _lib.ptr(rows),
                                     _lib.current_stream(ptr.device))
    _lib.check(st)
    return rows


# --------------------------------------------------------------------------- #
# SDDMM / edge softmax / narrow row sums
# --------------------------------------------------------------------------- #
def sddmm_csr(ptr, idx, src_feat, dst_feat, n_rows, out_shape=None, out=None):
    """out[e,h] = <src_feat[idx[e],h,:], dst_feat[row(e),(h,):]> in CSR edge order.

    src_feat [Ns,H,C] or [Ns,C]; dst_feat [Nd,H,C], or [Nd,C] (shared by all
    heads when H > 1).  Result is [E,H] ([E] when out_shape says so)."""
    res = _C.sddmm_csr(ptr, idx, src_feat, dst_feat, int(n_rows), out)
    return res.reshape(out_shape) if out_shape is not None else res


def sddmm_coo(src, dst, src_feat, dst_feat, out, n_edges):
    return _C.sddmm_coo(src, dst, src_feat, dst_feat, out, int(n_edges))


def edge_softmax_fwd(ptr, idx, att_dst, att_src, n_edges, slope):
    """(out [n_edges, H], mask [n_edges, H] bool)."""
    return _C.edge_softmax_fwd(ptr, idx, att_dst, att_src, int(n_edges), float(slope))


def edge_softmax_bwd(ptr, out, mask, grad, n_dst, slope, grad_pos=None):
    """Returns (g_dst [n_dst,H], t_edge [E,H]); rows of t_edge at or past ptr[n_dst] are not
    written (the transposed gather that consumes t_edge never reads them).  With ``grad_pos``
    (int64 per edge) the gradient row of edge k is grad[grad_pos[k]]: a gradient that was stored
    in the transposed graph's edge order is read through ``inverse_perm_transposed``."""
    return _C.edge_softmax_bwd(ptr, out, mask, grad, int(n_dst), float(slope), grad_pos)


def attention_logits(x, att_src, att_dst, n_dst):
    """(x[:, h, :] . att_src[h], x[:n_dst, h, :] . att_dst[h]) for x [n_src, H, C]: both
    per-node logits of a GAT layer from one pass over x."""
    lib = _lib.load()
    _req(x, "x", torch.float32, 3)
    n_src, heads, channels = x.shape
    att_src = att_src.reshape(heads, channels).contiguous()
    att_dst = att_dst.reshape(heads, channels).contiguous()
    _req(att_src, "att_src", torch.float32, 2)
    _req(att_dst, "att_dst", torch.float32, 2)
    if not 0 <= n_dst <= n_src:
        raise ValueError("n_dst=%d outside [0, %d]" % (n_dst, n_src))
    out_src = torch.empty(n_src, heads, dtype=torch.float32, device=x.device)
    out_dst = torch.empty(n_dst, heads, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        st = lib.cxg_attention_logits_fwd_f32(_lib.ptr(x), att_src.data_ptr(), att_dst.data_ptr(), n_src,
                                              n_dst, heads, channels, _lib.ptr(out_src), _lib.ptr(out_dst),
                                              _lib.current_stream(x.device))
    _lib.check(st)
    return out_src, out_dst


def attention_logits_bwd(x, att_src, att_dst, g_src, g_dst, add_to=None):
    """Gradients of ``attention_logits``: (grad_x, grad_att_src, grad_att_dst), reproducible.
    ``add_to`` (shaped like x) receives grad_x added in place and is returned as grad_x."""
    lib = _lib.load()
    _req(x, "x", torch.float32, 3)
    n_src, heads, channels = x.shape
    n_dst = g_dst.shape[0]
    att_src = att_src.reshape(heads, channels).contiguous()
    att_dst = att_dst.reshape(heads, channels).contiguous()
    _req(g_src, "g_src", torch.float32, 2)
    _req(g_dst, "g_dst", torch.float32, 2)
    if tuple(g_src.shape) != (n_src, heads) or g_dst.shape[1] != heads or n_dst > n_src:
        raise ValueError("gradient shapes %s / %s do not fit x %s"
                         % (tuple(g_src.shape), tuple(g_dst.shape), tuple(x.shape)))
    if add_to is not None:
        _req(add_to, "add_to", torch.float32, 3)
        if add_to.shape != x.shape or add_to.device != x.device:
            raise ValueError("add_to %s does not fit x %s" % (tuple(add_to.shape), tuple(x.shape)))
    grad_x = torch.empty_like(x) if add_to is None else add_to
    ga_src = torch.empty(heads, channels, dtype=torch.float32, device=x.device)
    ga_dst = torch.empty(heads, channels, dtype=torch.float32, device=x.device)
    ws_bytes = lib.cxg_attention_logits_workspace_bytes(n_src, heads, channels)
    ws = _workspace(ws_bytes, x.device)
    with torch.cuda.device(x.device):
        st = lib.cxg_attention_logits_bwd_f32(_lib.ptr(x), att_src.data_ptr(), att_dst.data_ptr(),
                                              _lib.ptr(g_src), _lib.ptr(g_dst), n_src, n_dst, heads, channels,
                                              _lib.ptr(grad_x), int(add_to is not None), ga_src.data_ptr(),
                                              ga_dst.data_ptr(),
                                              ws.data_ptr(), ws.numel(), _lib.current_stream(x.device))
    _lib.check(st)
    return grad_x, ga_src, ga_dst


def logits_proj_supported(n_in, heads):
    """Whether the kernels that take a GAT layer's logits from its input handle this shape."""
    return bool(_lib.load().cxg_attention_logits_proj_supported(int(n_in), int(heads)))


def _proj_rows(x, m, heads):
    _req(m, "m", torch.float32, 2)
    if not isinstance(x, torch.Tensor) or not x.is_cuda or x.dtype != torch.float32 or x.dim() != 2:
        raise ValueError("x must be a 2-d float32 CUDA tensor")
    if x.stride(1) != 1 and x.shape[1] != 1:
        raise ValueError("the rows of x must be contiguous")
    if m.shape != (2 * heads, x.shape[1]) or m.device != x.device:
        raise ValueError("m %s does not fit x %s with %d heads" % (tuple(m.shape), tuple(x.shape), heads))
    return x.shape[0], x.shape[1], (x.stride(0) if x.shape[0] > 1 else x.shape[1])


def attention_logits_proj(x, m, n_dst, heads):
    """(x @ m[:H].T, x[:n_dst] @ m[H:].T) for x [n_src, in] (rows may be strided) and
    m [2H, in]: both per-node logits of a GAT layer taken from the layer's input, where m
    holds att_src / att_dst carried through the layer's weight."""
    lib = _lib.load()
    n_src, n_in, ldx = _proj_rows(x, m, heads)
    if not 0 <= n_dst <= n_src:
        raise ValueError("n_dst=%d outside [0, %d]" % (n_dst, n_src))
    out_src = torch.empty(n_src, heads, dtype=torch.float32, device=x.device)
    out_dst = torch.empty(n_dst, heads, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        st = lib.cxg_attention_logits_proj_fwd_f32(_lib.ptr(x), ldx, m.data_ptr(), n_src, n_dst, n_in, heads,
                                                   _lib.ptr(out_src), _lib.ptr(out_dst),
                                                   _lib.current_stream(x.device))
    _lib.check(st)
    return out_src, out_dst


def attention_logits_proj_bwd(x, m, g_src, g_dst, heads, add_to=None, need_x=True):
    """Gradients of ``attention_logits_proj``: (grad_x, grad_m), reproducible.  ``add_to``
    ([n_src, in], contiguous) receives grad_x added in place and is returned as grad_x;
    with ``need_x=False`` grad_x is None and only grad_m [2H, in] is computed."""
    lib = _lib.load()
    n_src, n_in, ldx = _proj_rows(x, m, heads)
    n_dst = g_dst.shape[0]
    _req(g_src, "g_src", torch.float32, 2)
    _req(g_dst, "g_dst", torch.float32, 2)
    if tuple(g_src.shape) != (n_src, heads) or g_dst.shape[1] != heads or n_dst > n_src:
        raise ValueError("gradient shapes %s / %s do not fit x %s"
                         % (tuple(g_src.shape), tuple(g_dst.shape), tuple(x.shape)))
    grad_x = None
    if add_to is not None:
        _req(add_to, "add_to", torch.float32, 2)
        if tuple(add_to.shape) != (n_src, n_in) or add_to.device != x.device:
            raise ValueError("add_to %s does not fit x %s" % (tuple(add_to.shape), tuple(x.shape)))
        grad_x = add_to
    elif need_x:
        grad_x = torch.empty(n_src, n_in, dtype=torch.float32, device=x.device)
    grad_m = torch.empty_like(m)
    ws = _workspace(lib.cxg_attention_logits_proj_workspace_bytes(n_in, heads), x.device)
    with torch.cuda.device(x.device):
        st = lib.cxg_attention_logits_proj_bwd_f32(_lib.ptr(x), ldx, m.data_ptr(), _lib.ptr(g_src), _lib.ptr(g_dst),
                                                   n_src, n_dst, n_in, heads, _lib.ptr(grad_x), n_in,
                                                   int(add_to is not None), grad_m.data_ptr(), ws.data_ptr(),
                                                   ws.numel(), _lib.current_stream(x.device))
    _lib.check(st)
    return grad_x, grad_m


def _bn_vec(t, name, c, device):
    if t is None:
        return None
    _req(t, name, torch.float32, 1)
    if t.shape[0] != c or t.device != device:
        raise ValueError("%s must hold %d floats on %s" % (name, c, device))
    return t


def batchnorm_stats(x, eps):
    """Column statistics of x [n, c]: (mean, 1/sqrt(biased var + eps), unbiased var)."""
    lib = _lib.load()
    _req(x, "x", torch.float32, 2)
    n, c = x.shape
    if n < 1 or c < 1:
        raise ValueError("batch statistics need at least one row and one column, got %s" % (tuple(x.shape),))
    mean = torch.empty(c, dtype=torch.float32, device=x.device)
    invstd = torch.empty_like(mean)
    var_unbiased = torch.empty_like(mean)
    ws = _workspace(lib.cxg_batchnorm_workspace_bytes(n, c), x.device)
    with torch.cuda.device(x.device):
        st = lib.cxg_batchnorm_stats_f32(_lib.ptr(x), n, c, x.stride(0), float(eps), mean.data_ptr(),
                                         invstd.data_ptr(), var_unbiased.data_ptr(), ws.data_ptr(), ws.numel(),
                                         _lib.current_stream(x.device))
    _lib.check(st)
    return mean, invstd, var_unbiased


def batchnorm_apply(x, mean, invstd, gamma=None, beta=None, relu=False):
    """(x - mean) * invstd * gamma + beta per column of x [n, c], then max(., 0) if relu."""
    lib = _lib.load()
    _req(x, "x", torch.float32, 2)
    n, c = x.shape
    if c < 1:
        raise ValueError("x has no columns")
    mean, invstd = _bn_vec(mean, "mean", c, x.device), _bn_vec(invstd, "invstd", c, x.device)
    gamma, beta = _bn_vec(gamma, "gamma", c, x.device), _bn_vec(beta, "beta", c, x.device)
    y = torch.empty_like(x)
    with torch.cuda.device(x.device):
        st = lib.cxg_batchnorm_apply_f32(_lib.ptr(x), n, c, x.stride(0), mean.data_ptr(), invstd.data_ptr(),
                                         _lib.ptr(gamma), _lib.ptr(beta), _lib.ptr(y), y.stride(0), int(bool(relu)),
                                         _lib.current_stream(x.device))
    _lib.check(st)
    return y


def batchnorm_bwd(x, dy, mean, invstd, gamma=None, beta=None, relu=False):
    """Gradients of batchnorm_apply over batch statistics: (dx, dgamma, dbeta)."""
    lib = _lib.load()
    _req(x, "x", torch.float32, 2)
    _req(dy, "dy", torch.float32, 2)
    n, c = x.shape
    if tuple(dy.shape) != (n, c) or n < 1 or c < 1:
        raise ValueError("dy %s does not fit x %s" % (tuple(dy.shape), tuple(x.shape)))
    mean, invstd = _bn_vec(mean, "mean", c, x.device), _bn_vec(invstd, "invstd", c, x.device)
    gamma, beta = _bn_vec(gamma, "gamma", c, x.device), _bn_vec(beta, "beta", c, x.device)
    dx = torch.empty_like(x)
    dgamma = torch.empty(c, dtype=torch.float32, device=x.device)
    dbeta = torch.empty_like(dgamma)
    ws = _workspace(lib.cxg_batchnorm_workspace_bytes(n, c), x.device)
    with torch.cuda.device(x.device):
        st = lib.cxg_batchnorm_bwd_f32(_lib.ptr(x), _lib.ptr(dy), n, c, x.stride(0), dy.stride(0), mean.data_ptr(),
                                       invstd.data_ptr(), _lib.ptr(gamma), _lib.ptr(beta), int(bool(relu)),
                                       _lib.ptr(dx), dx.stride(0), dgamma.data_ptr(), dbeta.data_ptr(),
                                       ws.data_ptr(), ws.numel(), _lib.current_stream(x.device))
    _lib.check(st)
    return dx, dgamma, dbeta


def column_sum(x):
    """x.sum(0) of a 2-D fp32 tensor, in a fixed order (bias gradients)."""
    lib = _lib.load()
    _req(x, "x", torch.float32, 2)
    n, c = x.shape
    if c < 1:
        raise ValueError("x has no columns")
    out = torch.empty(c, dtype=torch.float32, device=x.device)
    ws = _workspace(lib.cxg_batchnorm_workspace_bytes(n, c), x.device)
    with torch.cuda.device(x.device):
        st = lib.cxg_column_sum_f32(_lib.ptr(x), n, c, x.stride(0), out.data_ptr(), ws.data_ptr(), ws.numel(),
                                    _lib.current_stream(x.device))
    _lib.check(st)
    return out


def csr_row_ids32(ptr, n_rows, n_edges):
    """int32 row id of every edge position (the edge-parallel kernels' row lookup)."""
    lib = _lib.load()
    _req(ptr, "ptr", torch.int64, 1)
    rows = torch.empty(n_edges, dtype=torch.int32, device=ptr.device)
    with torch.cuda.device(ptr.device):
        st = lib.cxg_csr_row_ids_i32(ptr.data_ptr(), n_rows, n_edges, _lib.ptr(rows),
                                     _lib.current_stream(ptr.device))
    _lib.check(st)
    return rows


def rows32_transposed(g):
    """Row (source) id of every edge of a TransposedGraph, built once and kept with it."""
    return _C.rows32_transposed(g)


def inverse_perm_transposed(g):
    """Position in the transposed edge order of every original edge position of a
    TransposedGraph (the inverse of ``g.perm``), built once and kept with it."""
    return _C.inverse_perm_transposed(g)


def narrow_gather_sum(ptr, sel, inp, n_rows, rows32=None):
    """out[r,:] = sum_{k in row r} inp[sel[k],:] (sel None: inp[k,:]); inp [M] or [M,W].
    With ``rows32`` (int32 row id per edge of ptr[:n_rows+1], ptr[0] == 0) and W in
    {1, 2, 4, 8} the edge-parallel segmented kernel is used."""
    return _C.narrow_gather_sum(ptr, sel, inp, int(n_rows), rows32)


def head_sum(x):
    """[N, H, C] -> [N, C], summed over heads."""
    return _C.head_sum(x)


def scatter_add_rows(inp, dest, n_nodes):
    """out[dest[e]] += inp[e] into a fresh zero [n_nodes, F] tensor."""
    lib = _lib.load()
    _req(inp, "input", torch.float32, 2)
    _req(dest, "dest", torch.int64, 1)
    if inp.shape[0] < dest.shape[0]:
        raise ValueError("input has fewer rows than dest")
    out = torch.zeros((n_nodes, inp.shape[1]), dtype=torch.float32, device=inp.device)
    with torch.cuda.device(inp.device):
        st = lib.cxg_scatter_add_rows_f32(_lib.ptr(inp), _lib.ptr(dest), _lib.ptr(out), dest.shape[0],
                                          inp.shape[1], _lib.current_stream(inp.device))
    _lib.check(st)
    return out


def gather_rows(inp, sel):
    """out[e] = inp[sel[e]]."""
    return _C.gather_rows(inp, sel)


# --------------------------------------------------------------------------- #
# scheduling helpers as device index work
# --------------------------------------------------------------------------- #
def _scan_ws(lib, n, dev):
    return _workspace(lib.cxg_scan_workspace_bytes(int(n)), dev)


def neighbor_group(ptr, thres):
    """(new_ptr, new_target) of cxg_neighbor_group_*: rows cut into chunks of ``thres`` edges."""
    lib = _lib.load()
    _req(ptr, "ptr", torch.int64, 1)
    dev, n = ptr.device, ptr.shape[0] - 1
    off = torch.empty(n + 1, dtype=torch.int64, device=dev)
    ws = _scan_ws(lib, n, dev)
    with torch.cuda.device(dev):
        stream = _lib.current_stream(dev)
        _lib.check(lib.cxg_neighbor_group_plan_i64(ptr.data_ptr(), n, int(thres), off.data_ptr(),
                                                   ws.data_ptr(), ws.numel(), stream))
        n_groups = int(off[n].item())
        new_ptr = torch.empty(n_groups + 1, dtype=torch.int64, device=dev)
        new_target = torch.empty(n_groups, dtype=torch.int64, device=dev)
        _lib.check(lib.cxg_neighbor_group_fill_i64(ptr.data_ptr(), off.data_ptr(), n, int(thres), n_groups,
                                                   new_ptr.data_ptr(), _lib.ptr(new_target), stream))
    return new_ptr, new_target


def filter_rows(ptr, idx, remove_flag):
    """Keep the rows whose flag is false: (new_ptr, new_idx)."""
    lib = _lib.load()
    n = ptr.shape[0] - 1
    _check_graph(ptr, idx, n)
    flag = remove_flag.to(torch.uint8).contiguous()
    if flag.shape[0] < n or flag.device != ptr.device:
        raise ValueError("remove_flag must have one entry per row on the graph's device")
    dev = ptr.device
    row_off = torch.empty(n + 1, dtype=torch.int64, device=dev)
    edge_off = torch.empty(n + 1, dtype=torch.int64, device=dev)
    ws = _scan_ws(lib, n, dev)
    with torch.cuda.device(dev):
        stream = _lib.current_stream(dev)
        _lib.check(lib.cxg_filter_rows_plan_i64(ptr.data_ptr(), n, _lib.ptr(flag), row_off.data_ptr(),
                                                edge_off.data_ptr(), ws.data_ptr(), ws.numel(), stream))
        n_rows_out, n_edges_out = int(row_off[n].item()), int(edge_off[n].item())
        new_ptr = torch.empty(n_rows_out + 1, dtype=torch.int64, device=dev)
        new_idx = torch.empty(n_edges_out, dtype=torch.int64, device=dev)
        _lib.check(lib.cxg_filter_rows_fill_i64(ptr.data_ptr(), _lib.ptr(idx), n, row_off.data_ptr(),
                                                edge_off.data_ptr(), n_edges_out, new_ptr.data_ptr(),
                                                _lib.ptr(new_idx), stream))
    return new_ptr, new_idx


def filter_edges(ptr, idx, remove_flag=None, rel=None, keep_rel=0, want_target=False):
    """Keep edge e if ``rel[e] == keep_rel`` (rel given) or ``not remove_flag[e]``, drop the
    rows left empty.  Returns (new_ptr, new_idx, new_target or None, row_off); row_off[i]
    is the number of kept rows among the first i rows."""
    lib = _lib.load()
    n = ptr.shape[0] - 1
    _check_graph(ptr, idx, n)
    dev = ptr.device
    n_edges = int(ptr[n].item())
    if int(ptr[0].item()) != 0:
        raise ValueError("ptr[0] must be 0")
    if idx.shape[0] < n_edges:
        raise ValueError("idx shorter than ptr[-1]")
    flag = None
    if rel is not None:
        _req(rel, "rel", torch.int32, 1)
        if rel.shape[0] < n_edges:
            raise ValueError("rel shorter than the number of edges")
    else:
        flag = remove_flag.to(torch.uint8).contiguous()
        if flag.shape[0] < n_edges or flag.device != dev:
            raise ValueError("remove_flag must have one entry per edge on the graph's device")
    edge_pos = torch.empty(n_edges + 1, dtype=torch.int64, device=dev)
    row_off = torch.empty(n + 1, dtype=torch.int64, device=dev)
    ws = _scan_ws(lib, max(n, n_edges), dev)
    with torch.cuda.device(dev):
        stream = _lib.current_stream(dev)
        _lib.check(lib.cxg_filter_edges_plan_i64(ptr.data_ptr(), n, n_edges, _lib.ptr(flag), _lib.ptr(rel),
                                                 int(keep_rel), edge_pos.data_ptr(), row_off.data_ptr(),
                                                 ws.data_ptr(), ws.numel(), stream))
        n_rows_out, n_edges_out = int(row_off[n].item()), int(edge_pos[n_edges].item())
        new_ptr = torch.empty(n_rows_out + 1, dtype=torch.int64, device=dev)
        new_idx = torch.empty(n_edges_out, dtype=torch.int64, device=dev)
        new_target = torch.empty(n_rows_out, dtype=torch.int64, device=dev) if want_target else None
        _lib.check(lib.cxg_filter_edges_fill_i64(ptr.data_ptr(), _lib.ptr(idx), n, n_edges, edge_pos.data_ptr(),
                                                 row_off.data_ptr(), new_ptr.data_ptr(), _lib.ptr(new_idx),
                                                 _lib.ptr(new_target), stream))
    return new_ptr, new_idx, new_target, row_off


def coo_to_csr(src, dst, n_rows):
    """CSR by destination of the edge list (src, dst), stable: (ptr, idx, perm)."""
    lib = _lib.load()
    _req(src, "src", torch.int64, 1)
    _req(dst, "dst", torch.int64, 1)
    if src.shape != dst.shape or src.device != dst.device:
        raise ValueError("src and dst must have the same length and device")
    dev, e = src.device, src.shape[0]
    if e and (int(dst.min()) < 0 or int(dst.max()) >= n_rows):
        raise ValueError("destination ids must lie in [0, %d)" % n_rows)
    ptr = torch.empty(n_rows + 1, dtype=torch.int64, device=dev)
    idx = torch.empty(e, dtype=torch.int64, device=dev)
    perm = torch.empty(e, dtype=torch.int64, device=dev)
    ws = _workspace(lib.cxg_coo_to_csr_workspace_bytes(e, n_rows), dev)
    with torch.cuda.device(dev):
        _lib.check(lib.cxg_coo_to_csr_i64(_lib.ptr(src), _lib.ptr(dst), e, n_rows, ptr.data_ptr(), _lib.ptr(idx),
                                          _lib.ptr(perm), ws.data_ptr(), ws.numel(), _lib.current_stream(dev)))
    return ptr, idx, perm
