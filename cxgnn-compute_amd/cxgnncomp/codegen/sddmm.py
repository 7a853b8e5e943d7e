"""``sddmm_dense`` (cxgnncomp/codegen/triton_sddmm.py:173-205) by name:
out[e, h] = sum_k dst_feat[dst_index[e], k] * src_feat[src_index[e], k, h],
with the source features laid out [num_src, feat, head] as upstream."""
import torch

from cxgnncomp_backend import _ops


def sddmm_dense(dst_feat_mat, src_feat_mat, dst_index, src_index, num_edge):
    assert dst_feat_mat.is_cuda and src_feat_mat.is_cuda and dst_index.is_cuda and src_index.is_cuda
    assert dst_feat_mat.is_contiguous(), "matrix A must be contiguous"
    assert src_feat_mat.is_contiguous(), "matrix B must be contiguous"
    assert len(src_feat_mat.shape) == 3  # num_src, feat, head
    assert src_feat_mat.shape[1] == dst_feat_mat.shape[1]
    src_hf = src_feat_mat.transpose(1, 2).contiguous()      # [num_src, head, feat]
    out = torch.empty((int(num_edge), src_hf.shape[1]), device=dst_feat_mat.device,
                      dtype=torch.float32)
    _ops.sddmm_coo(src_index.contiguous(), dst_index.contiguous(), src_hf, dst_feat_mat, out,
                   int(num_edge))
    return out
