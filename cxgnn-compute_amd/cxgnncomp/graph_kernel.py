"""``SpMMValOP``: multi-head edge-weighted aggregation with gradients for both the
node features and the edge values (cxgnncomp/graph_kernel.py:5-36).

forward   out[r,h,:] = sum_e val[e,h] * x[idx[e],h,:]
backward  grad_x over the cached transposed CSR (upstream: atomic scatter),
          grad_val[e,h] = <grad_out[row(e),h,:], x[idx[e],h,:]> by the CSR SDDMM, or, for
          rows of 256 floats, by the same pass that computes grad_x.
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
        g = _ops.transposed(ptr, idx, ctx.n, x.shape[0])       # cached with the graph
        if (ctx.needs_input_grad[0] and ctx.needs_input_grad[3] and x.dim() == 3 and val.dim() == 2
                and _ops.spmm_dot_supported(x.shape[1], x.shape[2]) and val.shape[0] == idx.shape[0]):
            # both gradients from one pass over the reversed graph: the rows of grad_out gathered
            # for grad_x are also multiplied with the row of x they are added into
            # the products leave the pass in its own edge order (contiguous stores) and are put into
            # the original order by one 4H-byte row gather: faster than scattering them from the
            # pass (61.9 M edges, 4 x 64: 10.3 against 11.0 ms), the same bits
            grad_x, in_pass_order = _ops.spmm_dot(g.ptr_t, g.idx_t, grad_out, x.shape[0], val, g.perm, x,
                                                  torch.empty_like(val), dot_at_edge=True)
            if g.n_edges == val.shape[0]:
                grad_val = _ops.gather_rows(in_pass_order, _ops.inverse_perm_transposed(g))
            else:
                grad_val = torch.zeros_like(val)
                grad_val[:g.n_edges] = _ops.gather_rows(in_pass_order, _ops.inverse_perm_transposed(g))
            return grad_x, None, None, grad_val, None
        if ctx.needs_input_grad[0]:
            # spmm_multihead_bwd adds into a zeroed tensor; writing the rows of the transposed
            # graph directly saves the fill and the read-back of the accumulation
            grad_x = _ops.spmm(g.ptr_t, g.idx_t, grad_out, x.shape[0], val=val, val_perm=g.perm)
        if ctx.needs_input_grad[3]:
            # the kernel writes the edges of the first ctx.n rows; only a tail past them needs zeros
            grad_val = torch.empty((idx.shape[0], val.shape[1]), dtype=torch.float32, device=x.device)
            if g.n_edges < idx.shape[0]:
                grad_val[g.n_edges:].zero_()
            grad_val = _ops.sddmm_csr(ptr, idx, x, grad_out, ctx.n, out=grad_val)[:val.shape[0]]
        return grad_x, None, None, grad_val, None
