"""The typed_linear family (cxgnncomp/typed_linear.py:10-310) on the MFMA typed
GEMM.  Same names, arguments and return values as upstream.

Upstream defects that are not reproduced (the mathematically intended result is
computed instead):
  * TypedLinearE2EOP.backward takes weight gradients from prefix slices
    ``x[:count[i]]`` (:133); here grad_W[r] = sum_{i: types[i]==r} x_i^T g_i;
  * TypedLinearS2EOP.backward is ``pass`` (:186-188); gradients are implemented;
  * the padded layout loses the last sorted rows (triton_typed_matmul.py:776-777);
    every row is computed.
"""
import torch
import torch.nn.functional as F

import cxgnncomp_backend
from cxgnncomp_backend import _ops, _typed

from .codegen.typed_matmul import typed_matmul


def TypedLinearNaiveS2D(x, weights, types, src, dst, num_center, num_edge):
    """Per-edge gathered weights (memory hungry by construction, :10-21)."""
    assert num_edge != 0
    feat = torch.index_select(x, 0, src[:num_edge])
    w = torch.index_select(weights, 0, types[:num_edge])
    out_e = torch.bmm(feat.unsqueeze(1), w).squeeze(1)
    output = torch.zeros([num_center, out_e.shape[1]], device=x.device, dtype=x.dtype)
    output.index_add_(0, dst[:num_edge], out_e)
    return output


def SelectMMS2EOP(x, weights, idx, types):
    return [torch.mm(x[idx[types == i]], weights[i]) for i in range(weights.shape[0])]


def TypedLinearS2DPushOP(x, weights, types, src, dst, num_type, num_center, num_edge):
    """Transform every distinct (type, source) pair once, then push the rows to their
    destinations (:31-68)."""
    max_src = torch.max(src) + 1
    key = types * max_src + src
    _, order = torch.sort(key, stable=True)
    uniq, inverse = torch.unique(key, return_inverse=True)
    type_unique = torch.div(uniq, max_src, rounding_mode="floor")
    src_unique = uniq % max_src
    transformed = typed_matmul(x, weights, type_unique.contiguous(), uniq.shape[0],
                               src_unique.contiguous(), seq_output=True)
    per_edge = _ops.gather_rows(transformed, inverse.contiguous())
    return cxgnncomp_backend.gather(per_edge, dst[:per_edge.shape[0]].contiguous(), num_center)


def _weight_grad(x_rows, g_rows, perm, seg, shape):
    """grad_W[r] = X_r^T G_r over the rows of relation r (rows given in original order)."""
    return _typed._weight_grad(x_rows, g_rows, perm, perm, seg, shape)


class TypedLinearE2EOP(torch.autograd.Function):
    """out[i] = x[i] @ weights[types[i]] for edge-level x [E, K]."""

    @staticmethod
    def preprocess(weights, types, thres=256):
        """Same four results as upstream (:74-87): padded+sorted relation ids, number of
        real rows, the sorting permutation and the per-relation counts on the CPU."""
        num_rel = weights.shape[0]
        num_item = types.shape[0]
        count = torch.bincount(types, minlength=num_rel)
        new_types = torch.empty([num_item + num_rel * (thres - 1)], device=weights.device,
                                dtype=types.dtype)
        new_types[:num_item] = types
        cxgnncomp_backend.pad_rel(new_types, count, thres, num_rel, num_item)
        indices, _ = _typed.rel_segment(new_types, num_rel + 1)
        sorted_types = new_types[indices]
        return [sorted_types, num_item, indices, count.cpu()]

    @staticmethod
    def forward(ctx, x, weights, types, preprocessed=[], thres=256, count=None):
        if len(preprocessed) == 4:
            sorted_types, num_item, indices, count = preprocessed
        else:
            sorted_types, num_item, indices, count = TypedLinearE2EOP.preprocess(weights, types, thres)
        x = x.contiguous()
        weights = weights.contiguous()
        # padding rows carry indices >= num_item; typed_matmul drops them.  The real rows
        # are a permutation of 0..num_item-1, so every output row is written.
        output = typed_matmul(x, weights, sorted_types, num_item, indices, covers_output=True)
        ctx.save_for_backward(x, weights, types, indices, sorted_types)
        ctx.num_item = num_item
        return output[:num_item]

    @staticmethod
    def backward(ctx, grad_out):
        x, weights, types, indices, sorted_types = ctx.saved_tensors
        grad_out = grad_out.contiguous()
        grad_x = grad_w = None
        if ctx.needs_input_grad[0]:
            wt = torch.transpose(weights, 1, 2).contiguous()
            grad_x = typed_matmul(grad_out, wt, sorted_types, ctx.num_item, indices, covers_output=True)
        if ctx.needs_input_grad[1]:
            perm, seg = _typed.rel_segment(types.contiguous(), weights.shape[0])
            grad_w = _weight_grad(x, grad_out, perm, seg, weights.shape)
        return grad_x, grad_w, None, None, None, None


class TypedLinearS2EOP(torch.autograd.Function):
    """out[e] = x[src_idx[e]] @ weights[types[e]] for node-level x, without
    materialising x[src_idx]."""

    @staticmethod
    def preprocess(weights, types, src_idx, thres):
        num_rel = weights.shape[0]
        num_item = src_idx.shape[0]
        count = torch.bincount(types, minlength=num_rel)
        pad = num_rel * (thres - 1)
        new_types = torch.empty([types.shape[0] + pad], device=weights.device, dtype=types.dtype)
        new_types[:types.shape[0]] = types
        new_src_idx = torch.empty([num_item + pad], device=weights.device, dtype=src_idx.dtype)
        new_src_idx[:num_item] = src_idx
        cxgnncomp_backend.pad_rel_idx(new_types, new_src_idx, count, thres, num_rel, types.shape[0])
        indices, _ = _typed.rel_segment(new_types, num_rel + 1)
        sorted_types = new_types[indices]
        return [sorted_types, num_item, new_src_idx, indices]

    @staticmethod
    def forward(ctx, x, weights, types, src_idx, preprocessed=[], thres=256, count=None):
        if len(preprocessed) == 4:
            sorted_types, num_item, new_src_idx, indices = preprocessed
        else:
            sorted_types, num_item, new_src_idx, indices = TypedLinearS2EOP.preprocess(
                weights, types, src_idx, thres)
        x = x.contiguous()
        weights = weights.contiguous()
        ctx.save_for_backward(x, weights, types, src_idx)
        # every real edge row is written exactly once (indices is a permutation of them)
        output = typed_matmul(x, weights, sorted_types, num_item, new_src_idx[indices].contiguous(),
                              indices, covers_output=True)
        return output[:num_item]

    @staticmethod
    def backward(ctx, grad_out):
        x, weights, types, src_idx = ctx.saved_tensors
        grad_out = grad_out.contiguous()
        n = src_idx.shape[0]
        perm, seg = _typed.rel_segment(types[:n].contiguous(), weights.shape[0])
        grad_x = grad_w = None
        if ctx.needs_input_grad[0]:
            # per-edge rows g[e] @ W[type[e]]^T, then every source sums its own rows (the
            # edge positions grouped by source are kept with src_idx): no atomics
            per_edge = torch.empty((n, x.shape[1]), dtype=torch.float32, device=x.device)
            _typed.typed_gemm(grad_out, torch.transpose(weights, 1, 2).contiguous(), seg, n, src_idx=perm,
                              dst_idx=perm, out=per_edge)
            groups = _ops.dest_groups(src_idx[:n], x.shape[0])
            grad_x = _ops.spmm(groups.ptr, groups.perm, per_edge, x.shape[0])
        if ctx.needs_input_grad[1]:
            grad_w = _typed._weight_grad(x, grad_out, src_idx[perm].contiguous(), perm, seg, weights.shape)
        return grad_x, grad_w, None, None, None, None, None


class TypedLinearS2DMMAggrOP(torch.autograd.Function):
    """RGCN layer as R x (dense transform of all nodes, masked aggregation) (:191-221)."""

    @staticmethod
    def forward(ctx, x, weights, ptr, idx, rel, num_center):
        ctx.save_for_backward(x, weights, ptr, idx, rel)
        output = torch.zeros([num_center, weights.shape[-1]], device=x.device)
        for i in range(weights.shape[0]):
            cxgnncomp_backend.selective_aggr(torch.mm(x, weights[i]), ptr, idx, (rel == i), output,
                                             num_center)
        return output

    @staticmethod
    def backward(ctx, grad_out):
        x, weights, ptr, idx, rel = ctx.saved_tensors
        grad_out = grad_out.contiguous()
        grad_x = torch.zeros_like(x)
        grad_weights = []
        num_center = grad_out.shape[0]
        for i in range(weights.shape[0]):
            g_sel = torch.zeros([x.shape[0], grad_out.shape[-1]], device=x.device)
            cxgnncomp_backend.selective_aggr_bwd(grad_out, ptr, idx, (rel == i), g_sel, num_center)
            grad_x += torch.mm(g_sel, weights[i].t())
            grad_weights.append(torch.mm(x.t(), g_sel))
        return grad_x, torch.stack(grad_weights), None, None, None, None


class TypedLinearS2DAggrMMOP(torch.autograd.Function):
    """RGCN layer as R x (masked aggregation, dense transform of the centers) (:224-258)."""

    @staticmethod
    def forward(ctx, x, weights, ptr, idx, rel, num_center):
        output = torch.zeros([num_center, weights.shape[-1]], device=x.device)
        aggr_outputs = []
        for i in range(weights.shape[0]):
            aggr = torch.zeros([num_center, weights.shape[-2]], device=x.device)
            cxgnncomp_backend.selective_aggr(x, ptr, idx, (rel == i), aggr, num_center)
            output += torch.mm(aggr, weights[i])
            aggr_outputs.append(aggr)
        ctx.save_for_backward(x, weights, ptr, idx, rel, torch.stack(aggr_outputs))
        return output

    @staticmethod
    def backward(ctx, grad_out):
        x, weights, ptr, idx, rel, aggr_outputs = ctx.saved_tensors
        grad_out = grad_out.contiguous()
        grad_x = torch.zeros_like(x)
        grad_weights = []
        num_center = grad_out.shape[0]
        for i in range(weights.shape[0]):
            grad_mm = torch.mm(grad_out, weights[i].t())
            grad_weights.append(torch.mm(aggr_outputs[i].t(), grad_out))
            cxgnncomp_backend.selective_aggr_bwd(grad_mm, ptr, idx, (rel == i), grad_x, num_center)
        return grad_x, torch.stack(grad_weights), None, None, None, None


def TypedLinearS2DSort(x, weights, ptr, idx, rel, num_center, count=None):
    """Pure-torch relation-segmented RGCN (auto-differentiable; runs on CPU tensors too)
    (:262-310)."""
    dst = torch.repeat_interleave(torch.arange(num_center, device=x.device),
                                  ptr[1:num_center + 1] - ptr[:num_center])
    num_rel = weights.shape[0]
    n_edge = dst.shape[0]
    output = torch.zeros([num_center, weights.shape[-1]], device=x.device)
    _, order = torch.sort(rel[:n_edge], stable=True)
    count = torch.bincount(rel[:n_edge], minlength=num_rel).cpu() if count is None else count.cpu()
    src, dst = idx[:n_edge][order], dst[order]
    start = 0
    for i in range(num_rel):
        c = int(count[i])
        output.index_add_(0, dst[start:start + c], F.linear(x[src[start:start + c]], weights[i].T))
        start += c
    return output
