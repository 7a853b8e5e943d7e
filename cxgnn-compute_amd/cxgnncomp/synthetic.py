"""Seeded synthetic graphs in the reference's layout: CSR by destination,
``ptr[num_dst+1]`` / ``idx[num_edge]`` = source ids, int64
(cxgnncomp/data_preparation.py:69-71,97-104 builds the same relation from the
datasets the reference loads through cxgnndl, which is not available here).

Everything is built with torch ops from a ``torch.Generator`` so the same call
runs on the CPU (tests) and on the GPU (benchmark-sized graphs in seconds).
Results are deterministic for a given (seed, device type).
"""
import math

import numpy as np
import torch


def _gen(seed, device):
    g = torch.Generator(device=device)
    g.manual_seed(int(seed))
    return g


def csr_from_coo(src, dst, num_dst):
    """CSR by destination, edges of one destination kept in input order."""
    if src.is_cuda:
        from cxgnncomp_backend import _ops
        return _ops.coo_to_csr(src.contiguous(), dst.contiguous(), num_dst)[:2]
    dst_sorted, order = torch.sort(dst, stable=True)
    idx = src[order].contiguous()
    counts = torch.bincount(dst_sorted, minlength=num_dst)
    ptr = torch.zeros(num_dst + 1, dtype=torch.int64, device=src.device)
    torch.cumsum(counts, 0, out=ptr[1:])
    return ptr, idx


def uniform_graph(num_nodes, num_edges, seed=0, device="cpu"):
    """Config 'GCN layer, CPU-runnable': independent uniform endpoints."""
    g = _gen(seed, device)
    src = torch.randint(0, num_nodes, (num_edges,), generator=g, device=device)
    dst = torch.randint(0, num_nodes, (num_edges,), generator=g, device=device)
    return csr_from_coo(src, dst, num_nodes)


def _clipped_zipf_pmf(alpha, cap):
    """pmf of min(Zipf(alpha), cap) on 1..cap (the tail mass sits on cap)."""
    from scipy.special import zeta
    k = np.arange(1, cap + 1, dtype=np.float64)
    pmf = k ** (-alpha)
    pmf[-1] += zeta(alpha, cap + 1)
    return pmf / pmf.sum()


def _cap_for_max_degree(alpha, n_nodes, endpoint_draws, target_max_degree):
    """Largest weight cap such that the expected degree of a cap-weight node,
    endpoint_draws * cap / (n_nodes * E[w]), equals target_max_degree."""
    lo, hi = 2, 1 << 24
    while lo < hi:
        mid = (lo + hi) // 2
        pmf = _clipped_zipf_pmf(alpha, mid)
        mean_w = float((np.arange(1, mid + 1) * pmf).sum())
        if endpoint_draws * mid / (n_nodes * mean_w) < target_max_degree:
            lo = mid + 1
        else:
            hi = mid
    return lo


def zipf_weights(n, alpha, cap, gen, device):
    pmf = _clipped_zipf_pmf(alpha, cap)
    cdf = torch.from_numpy(np.cumsum(pmf)).to(device)
    u = torch.rand(n, generator=gen, device=device, dtype=torch.float64)
    w = torch.searchsorted(cdf, u).clamp_(max=cap - 1) + 1
    return w.to(torch.float64)


def _draw_weighted(weights, count, gen, device):
    cdf = torch.cumsum(weights, 0)
    cdf = cdf / cdf[-1]
    out = torch.empty(count, dtype=torch.int64, device=device)
    step = 1 << 24
    for s in range(0, count, step):
        n = min(step, count - s)
        u = torch.rand(n, generator=gen, device=device, dtype=torch.float64)
        out[s:s + n] = torch.searchsorted(cdf, u).clamp_(max=weights.shape[0] - 1)
    return out


def powerlaw_symmetric_graph(num_nodes, num_pairs, alpha=2.0, max_degree=17500, seed=0,
                             device="cpu"):
    """Both endpoints of every pair drawn with probability proportional to a
    clipped Zipf(alpha) weight; every pair is stored in both directions
    (duplicates kept), so the edge multiset is symmetric and has exactly
    2 * num_pairs entries.  num_nodes=2,449,029 / num_pairs=30,929,570 gives the
    61,859,140-edge GAT/headline configuration."""
    g = _gen(seed, device)
    cap = _cap_for_max_degree(alpha, num_nodes, 2 * num_pairs, max_degree)
    w = zipf_weights(num_nodes, alpha, cap, g, device)
    a = _draw_weighted(w, num_pairs, g, device)
    b = _draw_weighted(w, num_pairs, g, device)
    src = torch.cat([a, b])
    dst = torch.cat([b, a])
    return csr_from_coo(src, dst, num_nodes)


def powerlaw_directed_symmetrised(num_nodes, num_directed, alpha=2.1, max_degree=13000, seed=0,
                                  device="cpu"):
    """Sources proportional to a clipped Zipf(alpha) weight, destinations
    uniform, then the reverse of every edge appended (duplicates kept):
    num_nodes=169,343 / num_directed=1,166,243 gives the 2,332,486-entry
    3-layer-GCN configuration."""
    g = _gen(seed, device)
    cap = _cap_for_max_degree(alpha, num_nodes, num_directed, max_degree)
    w = zipf_weights(num_nodes, alpha, cap, g, device)
    s = _draw_weighted(w, num_directed, g, device)
    d = torch.randint(0, num_nodes, (num_directed,), generator=g, device=device)
    src = torch.cat([s, d])
    dst = torch.cat([d, s])
    return csr_from_coo(src, dst, num_nodes)


def hetero_graph(num_nodes, num_edges, num_rel=16, rel_alpha=1.2, num_node_types=4, seed=0,
                 device="cpu", min_in_degree_one=True):
    """Uniform endpoints, edge type with probability proportional to
    r^-rel_alpha (r = 1..num_rel), uniform node types: the RGCN configuration.
    With min_in_degree_one the first num_nodes edges go to destinations
    0..num_nodes-1 so that no row is empty (the reference's RGCN layer divides by
    the in-degree without a zero guard, cxgnncomp/graph_conv.py:370-375).
    Returns ptr, idx, etype (int64, CSR order), node_type."""
    g = _gen(seed, device)
    src = torch.randint(0, num_nodes, (num_edges,), generator=g, device=device)
    dst = torch.randint(0, num_nodes, (num_edges,), generator=g, device=device)
    if min_in_degree_one and num_edges >= num_nodes:
        dst[:num_nodes] = torch.arange(num_nodes, device=device)
    p = torch.arange(1, num_rel + 1, dtype=torch.float64, device=device) ** (-rel_alpha)
    et = _draw_weighted(p, num_edges, g, device)
    dst_sorted, order = torch.sort(dst, stable=True)
    idx = src[order].contiguous()
    etype = et[order].contiguous()
    counts = torch.bincount(dst_sorted, minlength=num_nodes)
    ptr = torch.zeros(num_nodes + 1, dtype=torch.int64, device=device)
    torch.cumsum(counts, 0, out=ptr[1:])
    node_type = torch.randint(0, num_node_types, (num_nodes,), generator=g, device=device)
    return ptr, idx, etype, node_type


def sampled_batch(num_seeds=1024, fanouts=(15, 10, 5), id_space=111059956, seed=0, device="cpu"):
    """Layered neighbour sample in the reference's single-CSR layout
    (cxgnncomp/model.py:55-71): nodes are numbered in first-seen order, so the
    destinations of hop h are a prefix of its sources.  Hop h gives every node
    first reached at hop h-1 ``fanouts[h-1]`` neighbour ids drawn uniformly from
    the id space.  Returns ptr, idx, num_node_in_layer, num_edge_in_layer where
    layer l of a model aggregates rows [0, num_node_in_layer[L-1-l]) over
    idx[:num_edge_in_layer[L-1-l]]."""
    g = _gen(seed, device)
    cand = torch.unique(torch.randint(0, id_space, (2 * num_seeds,), generator=g, device=device))
    seeds = cand[torch.randperm(cand.shape[0], generator=g, device=device)[:num_seeds]]
    known = seeds.clone()            # global ids in local-id order
    frontier_lo, frontier_hi = 0, known.shape[0]
    idx_parts, deg_parts = [], []
    num_node_in_layer = [known.shape[0]]
    num_edge_in_layer = []
    total_edges = 0
    for f in fanouts:
        n_front = frontier_hi - frontier_lo
        nbr = torch.randint(0, id_space, (n_front * f,), generator=g, device=device)
        # relabel: ids already known keep their local id, new ids are appended in first-seen order
        allids = torch.cat([known, nbr])
        uniq, inverse = torch.unique(allids, return_inverse=True)
        first_pos = torch.full((uniq.shape[0],), allids.shape[0], dtype=torch.int64, device=device)
        first_pos.scatter_reduce_(0, inverse, torch.arange(allids.shape[0], device=device), "amin")
        order = torch.argsort(first_pos, stable=True)   # unique ids in first-seen order
        local_of_uniq = torch.empty_like(order)
        local_of_uniq[order] = torch.arange(order.shape[0], device=device)
        local = local_of_uniq[inverse]
        known = uniq[order]
        idx_parts.append(local[allids.shape[0] - nbr.shape[0]:])
        deg_parts.append(torch.full((n_front,), f, dtype=torch.int64, device=device))
        total_edges += nbr.shape[0]
        num_edge_in_layer.append(total_edges)
        frontier_lo, frontier_hi = frontier_hi, known.shape[0]
        num_node_in_layer.append(known.shape[0])
    deg = torch.cat(deg_parts)
    ptr = torch.zeros(deg.shape[0] + 1, dtype=torch.int64, device=device)
    torch.cumsum(deg, 0, out=ptr[1:])
    idx = torch.cat(idx_parts).contiguous()
    return ptr, idx, num_node_in_layer, num_edge_in_layer
