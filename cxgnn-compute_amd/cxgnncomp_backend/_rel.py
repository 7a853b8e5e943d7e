"""Masked / targeted / relational aggregation of the reference backend
(binding.cpp:26-31, 45-47) on top of cxg_spmm_ext_f32 and
cxg_spmm_scatter_atomic_f32."""

import torch

from . import _lib, _ops
from ._ops import _check_graph, _req, _workspace, as_int


def spmm_ext(ptr, idx, x, n_rows, out, *, accumulate=False, mask=None, mask_perm=None, rel=None,
             rel_stride=0, src_map=None, targets=None):
    """out[r or targets[r]] (+)= sum over unmasked edges of x[src_map[rel*stride + idx]]."""
    lib = _lib.load()
    _check_graph(ptr, idx, n_rows)
    _req(x, "input", torch.float32, 2)
    _req(out, "output", torch.float32, 2)
    feat = x.shape[1]
    if out.shape[1] != feat:
        raise ValueError("output has %d columns, input %d" % (out.shape[1], feat))
    if targets is None and out.shape[0] < n_rows:
        raise ValueError("output has fewer rows than num_node")
    if mask is not None:
        _req(mask, "mask", torch.bool, 1)
        if mask_perm is None and mask.shape[0] < idx.shape[0]:
            raise ValueError("mask shorter than idx")
    if mask_perm is not None:
        _req(mask_perm, "mask_perm", torch.int64, 1)
    if rel is not None:
        _req(rel, "etype", torch.int32, 1)
        if rel.shape[0] < idx.shape[0]:
            raise ValueError("etype shorter than idx")
    if src_map is not None:
        _req(src_map, "src_map", torch.int64, 1)
    if targets is not None:
        _req(targets, "targets", torch.int64, 1)
        if targets.shape[0] < n_rows:
            raise ValueError("targets shorter than num_node")
    if n_rows == 0:
        return out
    n_cap = idx.shape[0]
    ws = _workspace(lib.cxg_spmm_workspace_bytes(n_cap, feat), x.device)
    flags = _ops.SPMM_ACCUMULATE if accumulate else 0
    with torch.cuda.device(x.device):
        st = lib.cxg_spmm_ext_f32(ptr.data_ptr(), _lib.ptr(idx), _lib.ptr(x), feat, out.data_ptr(), feat,
                                  n_rows, n_cap, feat, flags, _lib.ptr(mask), _lib.ptr(mask_perm),
                                  _lib.ptr(rel), int(rel_stride), _lib.ptr(src_map), _lib.ptr(targets),
                                  ws.data_ptr(), ws.numel(), _lib.current_stream(x.device))
    _lib.check(st)
    return out


def scatter_atomic(ptr, idx, g, gx, n_rows, *, rel=None, rel_stride=0, val=None, mask=None):
    lib = _lib.load()
    _check_graph(ptr, idx, n_rows)
    _req(g, "grad", torch.float32, 2)
    _req(gx, "grad_input", torch.float32, 2)
    if rel is not None:
        _req(rel, "etype", torch.int32, 1)
    with torch.cuda.device(g.device):
        st = lib.cxg_spmm_scatter_atomic_f32(ptr.data_ptr(), _lib.ptr(idx), _lib.ptr(rel), int(rel_stride),
                                             _lib.ptr(val), _lib.ptr(mask), _lib.ptr(g), _lib.ptr(gx),
                                             n_rows, idx.shape[0], g.shape[1],
                                             _lib.current_stream(g.device))
    _lib.check(st)
    return gx


# --------------------------------------------------------------------------- #
def selective_aggr(input, ptr, idx, mask, output, num_node):
    """output[r] += sum_{e in row r, mask[e]} input[idx[e]] (src/cpp/src/aggr.cu:483-497)."""
    spmm_ext(ptr, idx, input, as_int(num_node), output, accumulate=True, mask=mask)


def selective_aggr_bwd(grad_output, ptr, idx, mask, computed_grad, num_center):
    """computed_grad[idx[e]] += grad_output[r] for masked edges (src/cpp/src/aggr.cu:499-514)."""
    n = as_int(num_center)
    g = _ops.transposed(ptr, idx, n, computed_grad.shape[0])
    spmm_ext(g.ptr_t, g.idx_t, grad_output, computed_grad.shape[0], computed_grad, accumulate=True,
             mask=mask, mask_perm=g.perm)


def target_aggr(input, ptr, idx, targets, output, num_node):
    """output[targets[r]] += sum_{e in row r} input[idx[e]] (src/cpp/src/aggr.cu:450-465)."""
    n = as_int(num_node)
    if n <= 0:
        n = ptr.shape[0] - 1
    spmm_ext(ptr, idx, input, n, output, targets=targets)


def target_aggr_backward(grad_in, ptr, idx, targets, grad_out, num_node):
    """grad_out[idx[e]] += grad_in[targets[r]] (src/cpp/src/aggr.cu:467-481)."""
    n = as_int(num_node)
    if n <= 0:
        n = ptr.shape[0] - 1
    g = _ops.transposed(ptr, idx, n, grad_out.shape[0])
    spmm_ext(g.ptr_t, g.idx_t, grad_in, grad_out.shape[0], grad_out, accumulate=True, src_map=targets)


# aggr_rel(input, ptr, idx, etype, num_node, num_rel): out[r] = sum_e input[etype[e]*N + idx[e]],
# input [num_rel*N, F], etype int32 (AggrRelFunction, src/cpp/src/rel_spmm.cu:37-136, :66-70): autograd
# in the compiled host layer, over the cached combined index and its transposed graph.
aggr_rel = _lib.native().aggr_rel
