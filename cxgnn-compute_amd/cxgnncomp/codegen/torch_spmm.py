"""The reference's PyTorch SpMM (cxgnncomp/codegen/torch_spmm.py:4-9): a CSR
sparse tensor times the feature matrix.  Kept as plain torch -- it is the
cross-check and CPU baseline of the HIP kernels, and runs on CPU tensors too."""
import torch


def spmm_torch(x, ptr, idx, num_nodes, val=None):
    if val is None:
        val = torch.ones(idx.shape[0], dtype=torch.float32, device=idx.device)
    mat = torch.sparse_csr_tensor(ptr, idx, val, size=(ptr.shape[0] - 1, x.shape[0]),
                                  device=ptr.device)
    return torch.sparse.mm(mat, x)
