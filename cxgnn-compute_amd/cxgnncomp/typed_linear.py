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


def TypedLinearS2DMMAggrOP_apply(x, weights, ptr, idx, rel, num_center):
    return _typed._RgcnFusedFunction.apply(x, ptr, idx, weights, rel, num_center, False, True)


class TypedLinearS2DMMAggrOP:
    """RGCN layer as "transform every node with every relation's weight, then aggregate"
    (:191-221; upstream: one torch.mm and one masked aggregation per relation).  Here the R
    transforms are one dense typed GEMM against the concatenated weights and the R masked
    aggregations one SpMM over the combined (source, relation) index -- the same values in
    two launches; gradients for x and the weights."""

    apply = staticmethod(TypedLinearS2DMMAggrOP_apply)


class TypedLinearS2DAggrMMOP(torch.autograd.Function):
    """RGCN layer as "aggregate per relation, then transform the centers" (:224-258;
    upstream: one masked aggregation and one torch.mm per relation).  The R masked
    aggregations are one SpMM into one row per (destination, relation) pair that owns an
    edge, the R transforms one typed GEMM over those rows (relation segments), and every
    destination sums the product rows of its pairs; the backward pass mirrors it.  When
    nearly every pair owns an edge the rows are the dense [n, R] table instead and the
    transform one GEMM [n, R*K] x [R*K, N]."""

    @staticmethod
    def forward(ctx, x, weights, ptr, idx, rel, num_center):
        n = int(num_center)
        x = x.contiguous()
        weights = weights.contiguous()
        R, K, N = weights.shape
        pg = _typed._pair_graph(ptr, idx, rel, n, x.shape[0], R)
        ctx.n, ctx.pairs = n, pg.b_dst.shape[0] <= _typed.RGCN_PAIR_FILL_MAX * n * R
        if ctx.pairs:
            out, z = _typed._pairs_aggregate_first(pg, x, weights, idx, n)
            ctx.pg = pg
            ctx.save_for_backward(x, weights, z)
            return out
        ptr_dr, idx_dr = _typed.dst_rel_graph(ptr, idx, rel, n, R)
        z = _ops.spmm(ptr_dr, idx_dr, x, n * R)                     # [n*R, K]
        ctx.save_for_backward(x, weights, ptr_dr, idx_dr, z)
        return torch.mm(z.view(n, R * K), weights.view(R * K, N))

    @staticmethod
    def backward(ctx, grad_out):
        grad_out = grad_out.contiguous()
        n = ctx.n
        grad_x = grad_w = None
        if ctx.pairs:
            x, weights, z = ctx.saved_tensors
            grad_x, grad_w = _typed._pairs_aggregate_first_bwd(ctx.pg, weights, z, grad_out, x.shape[0],
                                                               ctx.needs_input_grad[0], ctx.needs_input_grad[1])
            return grad_x, grad_w, None, None, None, None
        x, weights, ptr_dr, idx_dr, z = ctx.saved_tensors
        R, K, N = weights.shape
        if ctx.needs_input_grad[0]:
            gz = torch.mm(grad_out, weights.view(R * K, N).t())         # [n, R*K]
            g = _ops.transposed(ptr_dr, idx_dr, n * R, x.shape[0])
            grad_x = _ops.spmm(g.ptr_t, g.idx_t, gz.view(n * R, K), x.shape[0])
        if ctx.needs_input_grad[1]:
            grad_w = torch.mm(z.view(n, R * K).t(), grad_out).view(R, K, N)
        return grad_x, grad_w, None, None, None, None


def TypedLinearS2DSort(x, weights, ptr, idx, rel, num_center, count=None):
    """Relation-segmented RGCN (:262-310): upstream sorts the edges by relation and runs one
    gather + F.linear + index_add_ per relation in torch.  GPU tensors take the fused
    relational layer, which segments the edges the same way (stable sort by relation) and
    does the R products in one typed GEMM; CPU tensors run the torch composition."""
    if x.is_cuda:
        return _typed._RgcnFusedFunction.apply(x, ptr, idx, weights, rel, num_center, False, False)
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
