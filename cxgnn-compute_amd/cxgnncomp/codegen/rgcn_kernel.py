"""RGCN variants exported by the reference (cxgnncomp/codegen/rgcn_kernel.py:282-461)
by name.  All compute out[r] = sum_e x[idx[e]] @ W[rel[e]] (or its aggregate-only
part); the Triton ones route to the fused relation-segmented MFMA GEMM, the
op-wise ones keep their structure on top of the HIP aggregation kernels."""
import torch

import cxgnncomp_backend


def _rel32(rel):
    # integer ids pass as they are: the relational layer caches its pair tables per (ptr, idx, rel)
    # tensor, and a converted copy per call would rebuild them every time
    return rel if rel.dtype in (torch.int32, torch.int64) else rel.to(torch.int32)


def rgcn_triton(x, ptr, idx, rel, weights, num_nodes):
    assert x.is_cuda and ptr.is_cuda and idx.is_cuda and rel.is_cuda and weights.is_cuda
    with torch.no_grad():
        return cxgnncomp_backend.aggr_rgcn_direct_func(x, ptr, idx, weights, _rel32(rel), int(num_nodes))


def rgcn_triton_opt(x, ptr, idx, rel, weights, num_nodes):
    return rgcn_triton(x, ptr, idx, rel, weights, num_nodes)


def rgcn_scatter(x, ptr, idx, rel, weights, num_nodes):
    """Gather per-edge weights and features, batched product, scatter by destination
    (upstream calls torch.mm on the 3-D gathered weight, :357-358, which cannot run;
    the batched product is what it describes)."""
    num_nodes = int(num_nodes)
    deg = ptr[1:num_nodes + 1] - ptr[:num_nodes]
    target = torch.repeat_interleave(torch.arange(num_nodes, device=x.device), deg)
    e = target.shape[0]
    mid = torch.bmm(x[idx[:e]].unsqueeze(1), weights[rel[:e].long()]).squeeze(1)
    output = torch.zeros((num_nodes, weights.shape[-1]), dtype=torch.float32, device=x.device)
    output.index_add_(0, target, mid)
    return output


def rgcn_just_aggr(x, ptr, idx, rel, weights, num_nodes, num_rel):
    output = torch.zeros((num_nodes, weights.shape[-1]), dtype=torch.float32, device=x.device)
    for i in range(num_rel):
        cxgnncomp_backend.selective_aggr(x, ptr, idx, (rel == i), output, num_nodes)
    return output


def rgcn_just_aggr_prune(x, meta, num_nodes, num_rel):
    output = torch.zeros((num_nodes, x.shape[1]), dtype=torch.float32, device=x.device)
    for i in range(num_rel):
        cxgnncomp_backend.target_aggr(x, meta[3 * i], meta[3 * i + 1], meta[3 * i + 2], output,
                                      meta[3 * i + 2].shape[0])
    return output


def rgcn_full_mm(x, ptr, idx, rel, weights, num_nodes, num_rel):
    output = torch.zeros((num_nodes, weights.shape[-1]), dtype=torch.float32, device=x.device)
    for i in range(num_rel):
        cxgnncomp_backend.selective_aggr(torch.mm(x, weights[i]), ptr, idx, (rel == i), output,
                                         num_nodes)
    return output


def rgcn_full_mm2(x, ptr, idx, rel, weights, num_nodes, num_rel):
    output = torch.zeros((num_nodes, weights.shape[-1]), dtype=torch.float32, device=x.device)
    for i in range(num_rel):
        aggr = torch.zeros((num_nodes, weights.shape[-2]), dtype=torch.float32, device=x.device)
        cxgnncomp_backend.selective_aggr(x, ptr, idx, (rel == i), aggr, num_nodes)
        output += torch.mm(aggr, weights[i])
    return output


def rgcn_prune_mm(x, weights, meta, num_nodes, num_rel):
    output = torch.zeros((num_nodes, weights.shape[-1]), dtype=torch.float32, device=x.device)
    for i in range(num_rel):
        sub = cxgnncomp_backend.sage_sum_forward(x, meta[3 * i], meta[3 * i + 1], 0)
        output.index_add_(0, meta[3 * i + 2], torch.mm(sub, weights[i]))
    return output


def rgcn_full_bmm(x, ptr, idx, rel, weights, comp, num_nodes, num_rel):
    """Basis decomposition: W_rel = sum_b comp[rel, b] * weights[b] (weights [B, in, out])."""
    output = torch.zeros((num_nodes, weights.shape[-1]), dtype=torch.float32, device=x.device)
    basis_out = torch.einsum("ni,bio->nbo", x, weights)
    for i in range(num_rel):
        mm_output = torch.einsum("b,nbo->no", comp[i], basis_out).contiguous()
        cxgnncomp_backend.selective_aggr(mm_output, ptr, idx, (rel == i), output, num_nodes)
    return output
