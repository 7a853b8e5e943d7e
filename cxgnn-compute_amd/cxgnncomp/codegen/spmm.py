"""``spmm_triton`` / ``spmm_mm_triton`` (cxgnncomp/codegen/triton_spmm.py:137-165)
by name; the work is done by the edge-span SpMM kernels."""
import torch

from cxgnncomp_backend import _ops, _typed


def spmm_triton(x, ptr, idx, num_nodes, val=None):
    assert x.is_cuda and ptr.is_cuda and idx.is_cuda
    return _ops.spmm(ptr, idx, x.contiguous(), int(num_nodes), val=val)


def spmm_mm_triton(x, ptr, idx, weight, num_nodes):
    """Aggregate, then multiply by ``weight`` given transposed ([out, in]) as upstream."""
    agg = _ops.spmm(ptr, idx, x.contiguous(), int(num_nodes))
    out = _typed.dense_linear(agg, weight.t())        # the split GEMM where it takes the shape
    return out if out is not None else torch.mm(agg, weight.t())
