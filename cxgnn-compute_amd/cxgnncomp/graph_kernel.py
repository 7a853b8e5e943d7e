"""``SpMMValOP``: multi-head edge-weighted aggregation with gradients for both the
node features and the edge values (cxgnncomp/graph_kernel.py:5-36).

forward   out[r,h,:] = sum_e val[e,h] * x[idx[e],h,:]
backward  grad_x over the cached transposed CSR (upstream: atomic scatter),
          grad_val[e,h] = <grad_out[row(e),h,:], x[idx[e],h,:]> by the CSR SDDMM.
Upstream feeds the [N,H,C] grad_out to an SDDMM kernel that indexes it as [N,C]
(src/cpp/src/sddmm_kernel.cu:17), which is wrong for H > 1; the per-head product
is what the chain rule requires and what is computed here.
"""
import torch

import cxgnncomp_backend
from cxgnncomp_backend import _ops


class SpMMValOP(torch.autograd.Function):

    @staticmethod
    def forward(ctx, x, ptr, idx, val, num_center):
        n = _ops.as_int(num_center)
        x = x.contiguous()
        val = val.contiguous()
        ctx.save_for_backward(x, ptr, idx, val)
        ctx.n = n
        return cxgnncomp_backend.spmm_multihead(ptr, idx, val, x, n,
                                                cxgnncomp_backend.SPMM_MULTIHEAD_SCHEDULE.Naive)

    @staticmethod
    def backward(ctx, grad_out):
        x, ptr, idx, val = ctx.saved_tensors
        grad_out = grad_out.contiguous()
        grad_x = grad_val = None
        if ctx.needs_input_grad[0]:
            grad_x = torch.zeros_like(x)
            cxgnncomp_backend.spmm_multihead_bwd(ptr, idx, val, grad_out, grad_x, ctx.n)
        if ctx.needs_input_grad[3]:
            grad_val = _ops.sddmm_csr(ptr, idx, x, grad_out, ctx.n)[:val.shape[0]]
        return grad_x, None, None, grad_val, None
