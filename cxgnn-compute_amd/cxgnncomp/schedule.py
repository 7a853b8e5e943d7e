"""Degree bucketing and row filtering of CSR graphs (cxgnncomp/schedule.py:6-144).
Graphs on the GPU go through the library's scan + fill kernels; host tensors are
handled with vectorised index arithmetic instead of upstream's Python loops over
rows.  Results are identical to the upstream loops (bit-exact index work).
"""
import torch

from cxgnncomp_backend import _ops


def _degrees(ptr):
    return ptr[1:] - ptr[:-1]


def _row_of_edge(ptr, n_edges=None):
    n = ptr.shape[0] - 1
    rows = torch.repeat_interleave(torch.arange(n, device=ptr.device), _degrees(ptr))
    return rows if n_edges is None else rows[:n_edges]


def neighbor_grouping(ptr, neighbor_thres=32):
    """Split every row into consecutive chunks of ``neighbor_thres`` edges (the last
    chunk holds the remainder; an empty row gives one empty chunk).  Returns
    (new_ptr, new_target) with new_target[g] = original row of chunk g
    (upstream :20-35)."""
    if not isinstance(ptr, torch.Tensor):
        ptr = torch.as_tensor(ptr)
    ptr = ptr.to(torch.int64)
    if ptr.is_cuda:
        return _ops.neighbor_group(ptr.contiguous(), neighbor_thres)
    n = ptr.shape[0] - 1
    deg = _degrees(ptr)
    groups = torch.clamp((deg + neighbor_thres - 1) // neighbor_thres, min=1)
    new_target = torch.repeat_interleave(torch.arange(n, device=ptr.device), groups)
    first = torch.cumsum(groups, 0) - groups                    # first chunk of each row
    k = torch.arange(new_target.shape[0], device=ptr.device) - first[new_target]
    ends = torch.minimum(ptr[:-1][new_target] + (k + 1) * neighbor_thres, ptr[1:][new_target])
    new_ptr = torch.cat([ptr[:1] * 0, ends])
    return new_ptr, new_target


def neighbor_grouping_gpu(ptr, neighbor_thres=32):
    """new_ptr only (upstream :6-17, whose scatter mis-handles zero-degree rows; this
    follows ``neighbor_grouping``)."""
    return neighbor_grouping(ptr, neighbor_thres)[0]


def remove_from_graph(ptr, idx, remove_flag):
    """Keep the rows whose flag is false (upstream :106-121)."""
    if ptr.is_cuda:
        return _ops.filter_rows(ptr, idx, remove_flag)
    keep = ~remove_flag.to(torch.bool)
    deg = _degrees(ptr)
    new_ptr = torch.cat([ptr[:1] * 0, torch.cumsum(deg[keep], 0)])
    edge_keep = torch.repeat_interleave(keep, deg)
    return new_ptr, idx[:edge_keep.shape[0]][edge_keep]


def remove_from_graph_by_edge(ptr, idx, remove_flag):
    """Drop flagged edges, then drop rows left without edges (upstream :124-144)."""
    assert remove_flag.shape == idx.shape, \
        f"remove_flag.shape != idx.shape {remove_flag.shape} {idx.shape}"
    if ptr.is_cuda:
        return _ops.filter_edges(ptr, idx, remove_flag)[:2]
    keep = ~remove_flag.to(torch.bool)
    n = ptr.shape[0] - 1
    rows = _row_of_edge(ptr)
    e = rows.shape[0]
    new_deg = torch.bincount(rows[keep[:e]], minlength=n)
    new_ptr = torch.cat([ptr[:1] * 0, torch.cumsum(new_deg[new_deg > 0], 0)])
    return new_ptr, idx[:e][keep[:e]]


def reorder_by(ptr, idx, metric):
    """Rows in the order ``metric`` (a permutation of row ids); sources are not
    renumbered (upstream :83-103)."""
    assert metric.shape[0] == ptr.shape[0] - 1
    deg = _degrees(ptr)[metric]
    new_ptr = torch.cat([ptr[:1] * 0, torch.cumsum(deg, 0)])
    e = int(new_ptr[-1])
    start = torch.repeat_interleave(ptr[:-1][metric], deg)
    offset = torch.arange(e, device=ptr.device) - torch.repeat_interleave(new_ptr[:-1], deg)
    return new_ptr, idx[start + offset]


def partition_2d(ptr, idx, num_src, num_dst, num_parts=8):
    """2-D edge partition: for every (destination part i, source part j) the rows of
    part i restricted to sources of part j, rows without such edges dropped; blocks
    are concatenated in (i, j) order (upstream :38-69).  Returns (new_ptr, new_idx)."""
    num_src, num_dst = int(num_src), int(num_dst)
    n = ptr.shape[0] - 1
    src_per, dst_per = num_src // num_parts, num_dst // num_parts
    rows = _row_of_edge(ptr)
    e = rows.shape[0]
    col = idx[:e]
    last = num_parts - 1
    row_part = torch.clamp(torch.div(torch.arange(n, device=ptr.device), max(dst_per, 1),
                                     rounding_mode="floor"), max=last) if dst_per > 0 else \
        torch.full((n,), last, device=ptr.device)
    col_part = torch.clamp(torch.div(col, max(src_per, 1), rounding_mode="floor"), max=last) \
        if src_per > 0 else torch.full_like(col, last)
    degs, idxs = [], []
    for i in range(num_parts):
        for j in range(num_parts):
            m = (row_part[rows] == i) & (col_part == j)
            cnt = torch.bincount(rows[m], minlength=n)
            degs.append(cnt[cnt > 0])
            idxs.append(col[m])
    new_idx = torch.cat(idxs)
    new_ptr = torch.cat([ptr[:1] * 0, torch.cumsum(torch.cat(degs), 0)])
    assert new_idx.shape[0] == e
    return new_ptr, new_idx
