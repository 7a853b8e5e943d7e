"""``typed_matmul`` with the reference's signature
(cxgnncomp/codegen/triton_typed_matmul.py:752-860), executed by the MFMA typed
GEMM of libcxgnn_hip.so instead of Triton kernels.

Differences from the reference, all on purpose:
  * every row of ``rel`` takes the weight of its own relation id (the Triton
    kernels read one id per 32..256-row tile, which is why the reference pads
    each relation to a multiple of the tile); padded inputs still work because
    rows whose index is negative are skipped and ids equal to the number of
    relations select no weight;
  * all valid rows are computed -- the reference stops after ``num_valid_item``
    *sorted* rows and leaves the rest of ``c`` uninitialised (its FIXME at :776);
  * rows of ``c`` that no input row maps to are zero, not uninitialised memory.
"""
import collections

import torch

from cxgnncomp_backend import _typed

_SEG_CACHE = collections.OrderedDict()
_SEG_CACHE_CAP = 16


def _segments(rel, num_rel):
    """(perm or None, seg_ptr) for a relation-id vector; cached per tensor."""
    key = (rel.data_ptr(), rel.shape[0], rel._version, num_rel, rel.dtype, rel.device.index)
    hit = _SEG_CACHE.get(key)
    if hit is not None:
        _SEG_CACHE.move_to_end(key)
        return hit[0], hit[1]
    perm, seg = _typed.rel_segment(rel, num_rel)
    if rel.shape[0] > 1 and bool((rel[1:] >= rel[:-1]).all().item()):
        perm = None                      # already grouped: a stable sort is the identity
    _SEG_CACHE[key] = (perm, seg, rel)   # keep rel alive so its address is not reused
    while len(_SEG_CACHE) > _SEG_CACHE_CAP:
        _SEG_CACHE.popitem(last=False)
    return perm, seg


def typed_matmul(a, b, rel, num_valid_item=-1, src_idx=None, dst_idx=None, seq_output=False,
                 bf16=False, covers_output=False):
    """c[out_row(i)] = a[in_row(i)] @ b[rel[i]].

    no index:                 in_row = out_row = i
    src_idx only:             in_row = out_row = src_idx[i]      ("single index")
    src_idx, seq_output:      in_row = src_idx[i], out_row = i
    src_idx and dst_idx:      in_row = src_idx[i], out_row = dst_idx[i]
    Rows with a negative (or out-of-range) index are skipped; output rows no input row maps
    to are zero.  ``covers_output=True`` is the caller's promise that every output row is
    written (e.g. the index is a permutation), which saves the zero fill of the output.
    """
    assert a.shape[1] == b.shape[1], "incompatible dimensions"
    assert a.is_contiguous(), "matrix A must be contiguous"
    assert b.is_contiguous(), "matrix B must be contiguous"
    assert rel.is_contiguous(), "matrix rel must be contiguous"
    M, K = a.shape
    R, K, N = b.shape
    if src_idx is not None:
        assert src_idx.is_contiguous(), "matrix idx must be contiguous"
        M = src_idx.shape[0]
    n_rows = min(M, rel.shape[0])        # rows that have a relation id
    n_out = M if num_valid_item == -1 else int(num_valid_item)
    assert K % 32 == 0
    rel_rows = rel if rel.shape[0] == n_rows else rel[:n_rows].contiguous()
    perm, seg = _segments(rel_rows, R)

    def in_order(t):
        if t is None:
            return perm
        t = t[:n_rows]
        return t.contiguous() if perm is None else t[perm]

    if src_idx is None:
        src = dst = perm
    elif dst_idx is not None:
        src, dst = in_order(src_idx), in_order(dst_idx)
    elif seq_output:
        src, dst = in_order(src_idx), perm
    else:
        src = dst = in_order(src_idx)
    if dst is not None:
        # the kernel skips negative rows; rows beyond the output are dropped too
        dst = torch.where(dst < n_out, dst, torch.full_like(dst, -1))
    elif n_out < n_rows:
        n_rows_eff = torch.arange(n_rows, device=a.device)
        dst = torch.where(n_rows_eff < n_out, n_rows_eff, torch.full_like(n_rows_eff, -1))
    if src is not None:
        src = torch.where(src < a.shape[0], src, torch.full_like(src, -1))
    c = (torch.empty if covers_output else torch.zeros)((n_out, N), device=a.device, dtype=torch.float32)
    _typed.typed_gemm(a, b, seg, n_rows, src_idx=src, dst_idx=dst, out=c, bf16=bf16)
    return c
