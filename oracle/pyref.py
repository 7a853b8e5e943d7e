"""TEST INFRASTRUCTURE ONLY -- restatements of the reference's pure-Python /
PyTorch functions on the CPU (numpy or CPU torch).  Each function cites the
reference code it follows.  ``torch_scatter`` / PyG / Triton, which the
reference imports, are not available here; their calls are restated with core
torch ops of the same published meaning.
"""
import numpy as np
import torch
import torch.nn.functional as F


def spmm_torch(x, ptr, idx, num_nodes, val=None):
    """cxgnncomp/codegen/torch_spmm.py:4-9 -- the reference's own PyTorch SpMM:
    sparse_csr_tensor(ptr, idx, val or ones) @ x.  ``size`` is passed explicitly
    so that source ids beyond the largest one present keep their columns."""
    if val is None:
        val = torch.ones(idx.shape[0], dtype=torch.float32)
    mat = torch.sparse_csr_tensor(ptr[:num_nodes + 1], idx[:int(ptr[num_nodes])],
                                  val[:int(ptr[num_nodes])], size=(num_nodes, x.shape[0]))
    return torch.sparse.mm(mat, x)


def spmm_opwise(x, ptr, idx, num_nodes, val=None):
    """test/2-benchmark/bench-gcn.py:45-60, test/1-kernels/valid_spmm.py:91-102:
    gather rows, scale, index_add_ by destination."""
    deg = ptr[1:num_nodes + 1] - ptr[:num_nodes]
    dst = torch.repeat_interleave(torch.arange(num_nodes), deg)
    E = int(ptr[num_nodes])
    msg = x[idx[:E]]
    if val is not None:
        msg = msg * val[:E].reshape(E, *([1] * (msg.dim() - 1)))
    out = torch.zeros((num_nodes,) + tuple(x.shape[1:]), dtype=x.dtype)
    out.index_add_(0, dst, msg)
    return out


def gcn_norm(ptr, idx):
    """MyGCNConv.gcn_norm cxgnncomp/graph_conv.py:587-596: 1/in-degree per edge."""
    deg = ptr[1:] - ptr[:-1]
    deg_to = deg.repeat_interleave(deg)
    ev = deg_to.float().pow(-1)
    ev.masked_fill_(ev == float("inf"), 0.0)
    return ev


def _segment_ids(ptr, n):
    return torch.repeat_interleave(torch.arange(n), ptr[1:n + 1] - ptr[:n])


def edge_softmax_opwise(ptr, idx, att_src, att_dst, num_edge, relu_l):
    """MyGATConv.edge_softmax_opwise cxgnncomp/graph_conv.py:437-448.
    gather_csr(v, ptr) repeats v[r] over row r; segment_csr(v, ptr, reduce)
    reduces each row (torch_scatter's documented meaning), restated with
    repeat_interleave / scatter_reduce.  Keeps the reference's +1e-16."""
    n = ptr.shape[0] - 1
    seg = _segment_ids(ptr, n)[:num_edge]
    alpha_src = torch.index_select(att_src, 0, idx[:num_edge])
    alpha_dst = att_dst[seg]
    alpha = F.leaky_relu(alpha_src + alpha_dst, relu_l)
    H = alpha.shape[1]
    segH = seg.unsqueeze(1).expand(-1, H)
    with torch.no_grad():
        amax = torch.full((n, H), -float("inf"), dtype=alpha.dtype)
        amax = amax.scatter_reduce(0, segH, alpha, "amax", include_self=True)
        amax = amax[seg]
    alpha = torch.exp(alpha - amax)
    out_sum = torch.zeros((n, H), dtype=alpha.dtype).index_add_(0, seg, alpha) + 1e-16
    return alpha / out_sum[seg]


def sddmm_einsum(src, dst, src_feat, dst_feat):
    """test/1-kernels/perf-sddmm.py:99-105: per-edge dot products of gathered rows."""
    a = src_feat[src]
    b = dst_feat[dst]
    if b.dim() == 2:
        return torch.einsum("ehc,ec->eh", a, b)
    return torch.einsum("ehc,ehc->eh", a, b)


def typed_linear_s2d_sort(x, weights, ptr, idx, rel, num_center, count=None):
    """TypedLinearS2DSort cxgnncomp/typed_linear.py:262-310 (= RGCNOP_sorted,
    cxgnncomp/graph_conv.py:246-257): sort edges by relation, per relation
    gather -> F.linear(feat, W.T) -> index_add_ by destination.  A stable sort
    is used; the sums do not depend on the order inside a relation."""
    dst = torch.repeat_interleave(torch.arange(num_center), ptr[1:num_center + 1] - ptr[:num_center])
    num_rel = weights.shape[0]
    output = torch.zeros([num_center, weights.shape[-1]], dtype=x.dtype)
    E = dst.shape[0]
    sorted_rel, indices = torch.sort(rel[:E], stable=True)
    if count is None:
        count = torch.bincount(rel[:E], minlength=num_rel)
    src = idx[:E][indices]
    dst = dst[indices]
    cnt = 0
    for i in range(num_rel):
        c = int(count[i])
        s = src[cnt:cnt + c]
        d = dst[cnt:cnt + c]
        cnt += c
        output.index_add_(0, d, F.linear(x[s], weights[i].T))
    return output


def select_mm_s2e(x, weights, idx, types):
    """SelectMMS2EOP cxgnncomp/typed_linear.py:24-28."""
    return [torch.mm(x[idx[types == i]], weights[i]) for i in range(weights.shape[0])]


def typed_linear_naive_s2d(x, weights, types, src, dst, num_center, num_edge):
    """TypedLinearNaiveS2D cxgnncomp/typed_linear.py:10-21 (its torch.mm on a
    3-D gathered weight is read as the batched product it intends)."""
    feat = torch.index_select(x, 0, src[:num_edge])
    w = torch.index_select(weights, 0, types[:num_edge])
    t = torch.bmm(feat.unsqueeze(1), w).squeeze(1)
    out = torch.zeros([num_center, t.shape[1]], dtype=x.dtype)
    out.index_add_(0, dst[:num_edge], t)
    return out


def typed_matmul(a, b, rel, src_idx=None, dst_idx=None):
    """What the Triton typed_matmul kernels compute per valid row
    (cxgnncomp/codegen/triton_typed_matmul.py:146-215, 752-860):
    c[dst_or_i] = a[src_or_i] @ b[rel[i]]."""
    M = rel.shape[0] if src_idx is None else src_idx.shape[0]
    rows = a if src_idx is None else a[src_idx.clamp(min=0)]
    c = torch.bmm(rows[:M].unsqueeze(1), b[rel[:M]]).squeeze(1)
    if dst_idx is None:
        return c
    out = torch.zeros_like(c)
    out[dst_idx] = c
    return out


def e2e_preprocess(num_rel, types, thres=256):
    """TypedLinearE2EOP.preprocess cxgnncomp/typed_linear.py:74-87 with
    bincount(minlength=num_rel) and a stable sort (torch.sort's order inside a
    relation is implementation-defined in the reference).  Uses oracle.pad_rel."""
    from . import pad_rel
    types_np = np.asarray(types, dtype=np.int64)
    num_item = types_np.shape[0]
    count = np.bincount(types_np, minlength=num_rel).astype(np.int64)
    new_types = np.empty(num_item + num_rel * (thres - 1), dtype=np.int64)
    new_types[:num_item] = types_np
    new_types = pad_rel(new_types, count, thres, num_rel, num_item)
    indices = np.argsort(new_types, kind="stable")
    return new_types[indices], num_item, indices, count


def neighbor_grouping_py(ptr, neighbor_thres=32):
    """cxgnncomp/schedule.py:20-35, literal loop (small inputs only)."""
    new_ptr, new_target = [0], []
    for i in range(len(ptr) - 1):
        end, start = int(ptr[i + 1]), int(ptr[i])
        while end - start > neighbor_thres:
            start += neighbor_thres
            new_ptr.append(start)
            new_target.append(i)
        new_ptr.append(end)
        new_target.append(i)
    return np.array(new_ptr, dtype=np.int64), np.array(new_target, dtype=np.int64)


def remove_from_graph(ptr, idx, remove_flag):
    """cxgnncomp/schedule.py:106-121: keep the rows whose flag is false."""
    new_ptr, new_idx = [0], []
    for i in range(len(ptr) - 1):
        if not remove_flag[i]:
            new_ptr.append(new_ptr[-1] + int(ptr[i + 1] - ptr[i]))
            new_idx += [int(v) for v in idx[ptr[i]:ptr[i + 1]]]
    return np.array(new_ptr, dtype=np.int64), np.array(new_idx, dtype=np.int64)


def remove_from_graph_by_edge(ptr, idx, remove_flag):
    """cxgnncomp/schedule.py:124-144: drop flagged edges, then rows left empty."""
    new_ptr, new_idx = [0], []
    for i in range(len(ptr) - 1):
        deg = 0
        for j in range(int(ptr[i]), int(ptr[i + 1])):
            if not remove_flag[j]:
                new_idx.append(int(idx[j]))
                deg += 1
        if deg > 0:
            new_ptr.append(new_ptr[-1] + deg)
    return np.array(new_ptr, dtype=np.int64), np.array(new_idx, dtype=np.int64)


def reorder_by(ptr, idx, metric):
    """cxgnncomp/schedule.py:83-103: rows in the order given by ``metric``."""
    new_ptr, new_idx = [0], []
    for i in range(len(ptr) - 1):
        c = int(metric[i])
        new_ptr.append(new_ptr[-1] + int(ptr[c + 1] - ptr[c]))
        new_idx += [int(v) for v in idx[ptr[c]:ptr[c + 1]]]
    return np.array(new_ptr, dtype=np.int64), np.array(new_idx, dtype=np.int64)


def topo_sort(ptr, idx, degree):
    """src/cpp/src/schedule.cu:71-128 restated with a deque (small inputs only).
    Returns (order list, number emitted)."""
    from collections import deque
    n = len(degree)
    deg = [int(d) for d in degree]
    q = deque(i for i in range(n) if deg[i] == 0)
    out = []
    while len(out) < n:
        while q:
            cur = q.popleft()
            out.append(cur)
            for k in range(int(ptr[cur]), int(ptr[cur + 1])):
                nxt = int(idx[k])
                deg[nxt] -= 1
                if deg[nxt] == 0:
                    q.append(nxt)
        min_deg, pick = n, -1
        for i in range(n):
            if 1 < deg[i] < min_deg:
                min_deg, pick = deg[i], i
            elif deg[i] == 1:
                deg[i] = 0
                q.append(i)
        if pick != -1:
            q.append(pick)
            deg[pick] = 0
        elif not q:
            break
    return out, len(out)


def batchnorm_fwd(x, gamma, beta, eps, relu=False):
    """torch.nn.BatchNorm1d in training mode as the reference's models use it
    (cxgnncomp/model.py:28, :66-67, there followed by F.relu): per column,
    y = (x - mean) / sqrt(biased var + eps) * gamma + beta, in float64.  Returns
    (y, mean, biased var, unbiased var); the running statistics are updated with the mean
    and the unbiased variance."""
    x = np.asarray(x, dtype=np.float64)
    n = x.shape[0]
    mean = x.mean(axis=0)
    var = ((x - mean) ** 2).mean(axis=0)
    y = (x - mean) / np.sqrt(var + eps)
    if gamma is not None:
        y = y * np.asarray(gamma, dtype=np.float64)
    if beta is not None:
        y = y + np.asarray(beta, dtype=np.float64)
    if relu:
        y = np.maximum(y, 0.0)
    return y, mean, var, var * n / max(n - 1, 1)


def batchnorm_bwd(x, dy, gamma, beta, eps, relu=False, active=None):
    """Gradient of batchnorm_fwd (batch statistics are functions of x): with
    xhat = (x - mean) / sqrt(var + eps), dbeta = sum dy, dgamma = sum dy * xhat,
    dx = gamma / sqrt(var + eps) * (dy - mean(dy) - xhat * mean(dy * xhat)); with relu,
    dy is first zeroed where the forward output is not positive (``active``, if given, says
    where it is positive instead of the recomputation: for outputs within rounding of 0).
    float64."""
    x = np.asarray(x, dtype=np.float64)
    dy = np.asarray(dy, dtype=np.float64)
    mean = x.mean(axis=0)
    var = ((x - mean) ** 2).mean(axis=0)
    invstd = 1.0 / np.sqrt(var + eps)
    xhat = (x - mean) * invstd
    g = np.ones(x.shape[1]) if gamma is None else np.asarray(gamma, dtype=np.float64)
    if relu:
        y = xhat * g + (0.0 if beta is None else np.asarray(beta, dtype=np.float64))
        dy = np.where((y > 0) if active is None else active, dy, 0.0)
    dbeta = dy.sum(axis=0)
    dgamma = (dy * xhat).sum(axis=0)
    dx = g * invstd * (dy - dy.mean(axis=0) - xhat * (dy * xhat).mean(axis=0))
    return dx, dgamma, dbeta
