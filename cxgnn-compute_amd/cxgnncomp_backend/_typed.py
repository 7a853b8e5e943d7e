"""Typed GEMM, relation segmentation and the relational ops built on them
(binding.cpp:45-54): pad_rel*, typed_linear*, aggr_rel_direct,
aggr_rgcn_direct_func, seastar_*."""
import collections
import os

import torch

from . import _lib, _ops
from ._ops import _req, _workspace, as_int

GEMM_ACCUMULATE = 1
GEMM_ATOMIC = 2
GEMM_SPLIT_BF16X6 = 4
GEMM_SPLIT_BF16X3 = 8
GEMM_SPLIT_F16X3 = 16
GEMM_ROUND_BF16 = 32
GEMM_OUT_BF16 = 64
WGRAD_A_BF16 = 128

# How fp32 typed GEMMs multiply: "split_f16" (the default: rows of A and columns of W scaled by
# powers of two and split into two fp16 parts, three fp16 MFMA products per fp32 product, 2^-21
# per product -- fp32-grade -- and HBM bound for K <= 128), "split6" (six bf16 partial products,
# 2^-24), "split3" (three bf16 partial products, relative error below 2^-16 per product), "fp32"
# (v_mfma_f32_32x32x2_f32) or "bf16" (operands rounded to bf16, one bf16 MFMA product, fp32
# accumulation; weight gradients then use "split3").  The weight-gradient kernel has the same
# forms; its "split_f16" scales per 32-column group instead of per row, since its reduction runs
# over the rows.
GEMM_PRECISION = os.environ.get("CXGNN_GEMM_PRECISION", "split_f16")
_PRECISION_FLAGS = {"fp32": 0, "split6": GEMM_SPLIT_BF16X6, "split3": GEMM_SPLIT_BF16X3,
                    "split_f16": GEMM_SPLIT_F16X3}


def rel_segment(types, num_rel):
    """Stable grouping of rows by relation: returns (perm [n] int64, seg_ptr [num_rel+1] int64)."""
    lib = _lib.load()
    if types.dtype not in (torch.int32, torch.int64):
        raise ValueError("types must be int32 or int64, got %s" % types.dtype)
    _req(types, "types", types.dtype, 1)
    n = types.shape[0]
    dev = types.device
    perm = torch.empty(n, dtype=torch.int64, device=dev)
    seg = torch.empty(num_rel + 1, dtype=torch.int64, device=dev)
    nb = 4 if types.dtype == torch.int32 else 8
    ws = _workspace(lib.cxg_rel_segment_workspace_bytes(n, num_rel, nb), dev)
    fn = lib.cxg_rel_segment_i32 if nb == 4 else lib.cxg_rel_segment_i64
    with torch.cuda.device(dev):
        st = fn(_lib.ptr(types), n, num_rel, _lib.ptr(perm), seg.data_ptr(), ws.data_ptr(), ws.numel(),
                _lib.current_stream(dev))
    _lib.check(st)
    return perm, seg


def typed_gemm(a, w, seg_ptr, m_rows, *, src_idx=None, dst_idx=None, out=None, n_out=None,
               accumulate=False, atomic=False, bf16=False, precision=None, out_bf16=False):
    """out[dst(i)] (=|+=) a[src(i)] @ w[r] for rows i of segment r (see cxg_typed_gemm_f32).

    a [*, K] fp32, w [R, K, N] fp32.  precision "split_f16" (the default, see
    GEMM_PRECISION) forms every fp32 product from three fp16 partial products of
    row- / column-scaled operands (2^-21 per product), "split6" from six bf16 partial
    products (2^-24), "split3" from three (relative error per product < 2^-16, the
    reference's tl.dot is TF32); "fp32" forces v_mfma_f32_32x32x2_f32.  With bf16=True or
    precision "bf16" the operands are rounded to bf16 (W transposed to [R, N, K]) and multiplied
    on the bf16 matrix cores with fp32 accumulation."""
    lib = _lib.load()
    bf16 = bf16 or (precision or GEMM_PRECISION) == "bf16"
    _req(a, "a", torch.float32 if not (bf16 and a.dtype == torch.bfloat16) else torch.bfloat16, 2)
    if w.dim() != 3:
        raise ValueError("weights must be [num_rel, K, N]")
    R, K, N = w.shape
    if a.shape[1] != K:
        raise ValueError("incompatible dimensions: a has %d columns, weights K=%d" % (a.shape[1], K))
    _req(seg_ptr, "seg_ptr", torch.int64, 1)
    if seg_ptr.shape[0] < R + 1:
        raise ValueError("seg_ptr needs num_rel+1 entries")
    for t, name in ((src_idx, "src_idx"), (dst_idx, "dst_idx")):
        if t is not None:
            _req(t, name, torch.int64, 1)
            if t.shape[0] < m_rows:
                raise ValueError("%s shorter than the number of rows" % name)
    if src_idx is None and a.shape[0] < m_rows:
        raise ValueError("a has fewer rows than M")
    if out_bf16:
        # bf16 rows of the result (the bf16-operand kernels only: K <= 128, even N, plain stores)
        if out is not None or accumulate or atomic or not bf16 or K > 128 or K % 8 or N % 2:
            raise ValueError("out_bf16 goes with bf16 operands, K <= 128 (a multiple of 8), even N and a fresh output")
        out = torch.empty((m_rows if n_out is None else n_out, N), dtype=torch.bfloat16, device=a.device)
    elif out is None:
        if n_out is None:
            n_out = m_rows
        out = torch.empty((n_out, N), dtype=torch.float32, device=a.device)
    else:
        _req(out, "output", torch.float32, 2)
        if out.shape[1] != N:
            raise ValueError("output has %d columns, weights N=%d" % (out.shape[1], N))
    if dst_idx is None and out.shape[0] < m_rows:
        raise ValueError("output has fewer rows than M")
    flags = (GEMM_ACCUMULATE if accumulate else 0) | (GEMM_ATOMIC if atomic else 0) | (GEMM_OUT_BF16 if out_bf16 else 0)
    precision = precision or GEMM_PRECISION
    if precision == "bf16":
        bf16 = True
    elif precision not in _PRECISION_FLAGS:
        raise ValueError("precision must be one of %s" % sorted(list(_PRECISION_FLAGS) + ["bf16"]))
    else:
        flags |= _PRECISION_FLAGS[precision]
    stream = _lib.current_stream(a.device)
    with torch.cuda.device(a.device):
        if bf16 and a.dtype == torch.float32 and K <= 128 and K % 8 == 0:
            # fp32 operands rounded to bf16 inside the kernel: no conversion pass over a and w
            _req(w, "weights", torch.float32, 3)
            st = lib.cxg_typed_gemm_f32(a.data_ptr(), K, w.data_ptr(), out.data_ptr(), N,
                                        _lib.ptr(src_idx), _lib.ptr(dst_idx), seg_ptr.data_ptr(),
                                        m_rows, K, N, R,
                                        (flags & (GEMM_ACCUMULATE | GEMM_ATOMIC | GEMM_OUT_BF16)) | GEMM_ROUND_BF16, stream)
        elif bf16:
            a16 = a if a.dtype == torch.bfloat16 else a.to(torch.bfloat16)
            wt16 = w.detach().transpose(1, 2).contiguous().to(torch.bfloat16)
            st = lib.cxg_typed_gemm_bf16(a16.data_ptr(), K, wt16.data_ptr(), out.data_ptr(), N,
                                         _lib.ptr(src_idx), _lib.ptr(dst_idx), seg_ptr.data_ptr(),
                                         m_rows, K, N, R, flags, stream)
        elif _takes_wide_form(K, N, flags, src_idx is not None):
            # wide operands: the tiled kernel with both operand tiles in LDS (W split into the workspace)
            _req(w, "weights", torch.float32, 3)
            ws = _workspace(lib.cxg_typed_gemm_wide_workspace_bytes(K, N, R), a.device)
            st = lib.cxg_typed_gemm_wide_f32(a.data_ptr(), K, w.data_ptr(), out.data_ptr(), N,
                                             _lib.ptr(src_idx), _lib.ptr(dst_idx), seg_ptr.data_ptr(),
                                             m_rows, K, N, R, flags, ws.data_ptr(), ws.numel(), stream)
        else:
            _req(w, "weights", torch.float32, 3)
            st = lib.cxg_typed_gemm_f32(a.data_ptr(), K, w.data_ptr(), out.data_ptr(), N,
                                        _lib.ptr(src_idx), _lib.ptr(dst_idx), seg_ptr.data_ptr(),
                                        m_rows, K, N, R, flags, stream)
    _lib.check(st)
    return out


def _takes_wide_form(K, N, flags, gathered=False):
    """The fp16 split arithmetic on the tiled kernel: K above 256 (the register-resident kernel
    holds at most 256 rows of W), and 160 <= K <= 256 where it measures faster -- more than one
    128-column tile (5 M x 256 x 256: 2.8 against 3.9 ms), gathered rows (7.3 M x 256 x 128: 3.0
    against 3.6 ms), or a 256 x 128 register tile that would be mostly empty."""
    if not (flags & GEMM_SPLIT_F16X3) or K % 4 or K < 160:
        return False
    return K > 256 or gathered or N > 128 or not (K >= 176 and N >= 96)


# --------------------------------------------------------------------------- #
# dense x @ W (+ bias) (+ addend) as a typed GEMM with one relation
# --------------------------------------------------------------------------- #
DENSE_MIN_ROWS = 4096        # below this the launch is latency bound either way
DENSE_WIDE_MIN_ROWS = 100000
_one_seg = {}


def _one_segment(m_rows, device):
    key = (int(m_rows), str(device))
    seg = _one_seg.get(key)
    if seg is None:
        if len(_one_seg) > 64:
            _one_seg.clear()
        seg = _one_seg[key] = torch.tensor([0, int(m_rows)], dtype=torch.int64, device=device)
    return seg


def dense_linear(x, w_kn, bias=None, addend=None):
    """x [M, K] @ w_kn [K, N] + bias [N] + addend [M, N] (either may be None) as a typed GEMM over
    one segment, bias and addend added to the accumulator before the rows are stored.  Returns
    None for inputs the split kernels do not take (the caller then uses the library GEMM):
    other dtypes or layouts, few rows, K above 128 (256 when K >= 176, N >= 96 and at least
    10^5 rows; any K without bias and addend from 10^5 rows on: the tiled kernel), K not a multiple
    of 4, a default precision other than the fp16 split form."""
    flags = _PRECISION_FLAGS.get(GEMM_PRECISION, 0)
    if flags != GEMM_SPLIT_F16X3 or not x.is_cuda or x.dim() != 2 or x.dtype != torch.float32 or w_kn.dtype != torch.float32:
        return None
    M, K = x.shape
    N = w_kn.shape[1]
    # the 256-wide form stores from the accumulators (no staged 16-byte stores): it beats the
    # library from about 10^5 rows on (measured on 4 k - 2.4 M rows, with and without addend)
    wide = 176 <= K <= 256 and N >= 96 and M >= DENSE_WIDE_MIN_ROWS
    # the tiled kernel has no epilogue; without one it also takes K above 256 (2.33 M x 512 x 512: 4.0 ms
    # against 8.6 ms in the library)
    tiled = (bias is None and addend is None and K > 256 and K % 4 == 0 and M >= DENSE_WIDE_MIN_ROWS)
    if M < DENSE_MIN_ROWS or K % 4 or not (K <= 128 or wide or tiled) or w_kn.shape[0] != K:
        return None
    if not x.is_contiguous() or x.data_ptr() % 16:
        return None
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() != N or not bias.is_contiguous()):
        return None
    if addend is not None and (addend.dtype != torch.float32 or tuple(addend.shape) != (M, N)
                               or not addend.is_contiguous()):
        return None
    w_kn = w_kn.contiguous()
    if bias is None and addend is None and _takes_wide_form(K, N, flags, False):
        # no epilogue: the tiled kernel for wide operands where it is the faster one (K >= 160 and more
        # than 128 columns; 169,865 x 256 x 256: 0.135 against 0.158 ms)
        return typed_gemm(x, w_kn.unsqueeze(0), _one_segment(M, x.device), M, precision="split_f16")
    lib = _lib.load()
    out = torch.empty((M, N), dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        st = lib.cxg_typed_gemm_epilogue_f32(x.data_ptr(), K, w_kn.data_ptr(), _lib.ptr(bias), _lib.ptr(addend), N,
                                             out.data_ptr(), N, None, None, _one_segment(M, x.device).data_ptr(),
                                             M, K, N, 1, flags, _lib.current_stream(x.device))
    _lib.check(st)
    return out


def dense_linear_heads(x, weight, bias=None):
    """out[:, h*C:(h+1)*C] = x[:, h, :] @ weight[h*C:(h+1)*C, :].T (+ bias) for x [M, H, K] and a
    layer weight [H*C, K]: the per-head products that follow an aggregation of the layer's input
    under H weights.  One launch of the split GEMM per head over strided rows (row stride H*K in,
    H*C out; bias in the epilogue); shapes the kernel does not take go through torch.bmm."""
    M, H, K = x.shape
    C = weight.shape[0] // H
    flags = _PRECISION_FLAGS.get(GEMM_PRECISION, 0)
    ok = (flags == GEMM_SPLIT_F16X3 and x.is_cuda and x.dtype == torch.float32 and weight.dtype == torch.float32
          and x.is_contiguous() and M >= DENSE_MIN_ROWS and K <= 128 and K % 4 == 0 and C % 4 == 0
          and x.data_ptr() % 16 == 0 and (bias is None or (bias.dtype == torch.float32 and bias.is_contiguous()
                                                           and bias.numel() == H * C)))
    if not ok:
        out = torch.bmm(x.transpose(0, 1), weight.view(H, C, K).transpose(1, 2)).transpose(0, 1).reshape(M, H * C)
        return out if bias is None else out.add_(bias)
    lib = _lib.load()
    w_kn = weight.view(H, C, K).transpose(1, 2).contiguous()          # [H, K, C]
    out = torch.empty((M, H * C), dtype=torch.float32, device=x.device)
    seg = _one_segment(M, x.device)
    with torch.cuda.device(x.device):
        for h in range(H):
            st = lib.cxg_typed_gemm_epilogue_f32(x.data_ptr() + 4 * h * K, H * K, w_kn.data_ptr() + 4 * h * K * C,
                                                 None if bias is None else bias.data_ptr() + 4 * h * C, None, 0,
                                                 out.data_ptr() + 4 * h * C, H * C, None, None, seg.data_ptr(),
                                                 M, K, C, 1, flags, _lib.current_stream(x.device))
            _lib.check(st)
    return out


def dense_linear_add_(out, x, w_kn):
    """out [M, N] += x [M, K] @ w_kn [K, N] in place through the typed GEMM (one segment);
    False when the shapes are not taken (nothing is written then)."""
    if (GEMM_PRECISION != "split_f16" or not x.is_cuda or x.dim() != 2 or x.dtype != torch.float32
            or out.dtype != torch.float32 or w_kn.dtype != torch.float32):
        return False
    M, K = x.shape
    N = w_kn.shape[1]
    wide = 176 <= K <= 256 and N >= 96 and M >= DENSE_WIDE_MIN_ROWS
    if (M < DENSE_MIN_ROWS or K % 4 or not (K <= 128 or wide) or tuple(out.shape) != (M, N)
            or not x.is_contiguous() or not out.is_contiguous() or x.data_ptr() % 16):
        return False
    typed_gemm(x, w_kn.contiguous().unsqueeze(0), _one_segment(M, x.device), M, out=out, accumulate=True,
               precision="split_f16")
    return True


# --------------------------------------------------------------------------- #
# pad_rel / pad_rel_idx  (binding.cpp:51-52)
# --------------------------------------------------------------------------- #
def _pad_rel(rel, idx, count, thres, num_rel, base):
    lib = _lib.load()
    thres, num_rel, base = int(thres), int(num_rel), as_int(base)
    _req(rel, "rel", torch.int64, 1)
    _req(count, "count", torch.int64, 1)
    if count.shape[0] < num_rel:
        raise ValueError("count has %d entries, num_rel=%d (use bincount(minlength=num_rel))"
                         % (count.shape[0], num_rel))
    need = base + num_rel * (thres - 1)
    if rel.shape[0] < need:
        raise ValueError("rel has %d entries, %d needed" % (rel.shape[0], need))
    if idx is not None:
        _req(idx, "idx", torch.int64, 1)
        if idx.shape[0] < need:
            raise ValueError("idx has %d entries, %d needed" % (idx.shape[0], need))
    with torch.cuda.device(rel.device):
        st = lib.cxg_pad_rel_i64(rel.data_ptr(), _lib.ptr(idx), count.data_ptr(), thres, num_rel, base,
                                 _lib.current_stream(rel.device))
    _lib.check(st)
    # the library wrote through raw pointers: bump the tensors' version counters, which key
    # the caches of structures derived from index arrays (transposed graphs, pair tables)
    torch.autograd.graph.increment_version(rel)
    if idx is not None:
        torch.autograd.graph.increment_version(idx)


def pad_rel(rel, count, thres, num_rel, base):
    """In place on rel (src/cpp/src/stitch_kernel.cu:23-38,48-53)."""
    _pad_rel(rel, None, count, thres, num_rel, base)


def pad_rel_idx(rel, idx, count, thres, num_rel, base):
    """In place on rel and idx (src/cpp/src/stitch_kernel.cu:3-21,40-46)."""
    _pad_rel(rel, idx, count, thres, num_rel, base)


# --------------------------------------------------------------------------- #
# per-row typed linear  (binding.cpp:48-50)
# --------------------------------------------------------------------------- #
def _typed_rows(vin, weights, output, types, src_id, dst_id, atomic):
    if types.dtype != torch.int32:
        raise ValueError("types must be int32")
    num = types.shape[0] if src_id is None else src_id.shape[0]
    if num == 0:
        return
    if atomic and 4 * num * weights.shape[2] <= RGCN_EDGE_ROWS_MAX_BYTES:
        # several rows share a destination: instead of fp32 atomics, one product row per
        # (source, type) pair that occurs (rows that repeat a pair share it), then every
        # destination sums the product rows of its input rows and adds them.  The pair
        # list and the grouping by destination are built once per index arrays.
        ptr_d, rows_d, pair_src, pair_seg = _scatter_pairs(src_id, types, dst_id, num, vin.shape[0],
                                                           weights.shape[0], output.shape[0])
        products = typed_gemm(vin, weights, pair_seg, pair_src.shape[0], src_idx=pair_src)
        output += _ops.spmm(ptr_d, rows_d, products, output.shape[0])
        return
    perm, seg = rel_segment(types[:num].contiguous(), weights.shape[0])
    src = perm if src_id is None else src_id[perm]
    dst = perm if dst_id is None else dst_id[perm]
    typed_gemm(vin, weights, seg, num, src_idx=src, dst_idx=dst, out=output, accumulate=True,
               atomic=atomic)


_SCATTER_PAIR_CACHE = collections.OrderedDict()


def _scatter_pairs(src_id, types, dst_id, num, n_src, num_rel, n_out):
    """For output[dst[i]] += vin[src[i]] @ W[type[i]], i < num: the (type, source) pairs that
    occur, sorted (pair_src [U], pair_seg [R+1] relation segments), and the CSR over
    destinations whose entries are the pair rows of the destination's input rows
    (ptr_d [n_out+1], rows_d [num]).  Cached per (src_id, types, dst_id) arrays."""
    key = (src_id.data_ptr(), src_id._version, types.data_ptr(), types._version, dst_id.data_ptr(),
           dst_id._version, num, n_src, num_rel, n_out, types.device.index)
    hit = _SCATTER_PAIR_CACHE.get(key)
    if hit is not None:
        _SCATTER_PAIR_CACHE.move_to_end(key)
        return hit[:4]
    types, dst_id = types[:num], dst_id[:num].contiguous()
    if num and (int(types.min()) < 0 or int(types.max()) >= num_rel):
        raise ValueError("type ids must lie in [0, %d)" % num_rel)
    if num and (int(src_id[:num].min()) < 0 or int(src_id[:num].max()) >= n_src):
        raise ValueError("source ids must lie in [0, %d)" % n_src)
    uniq, pair_of_row = torch.unique(types.to(torch.int64) * n_src + src_id[:num], sorted=True, return_inverse=True)
    pair_src = (uniq % n_src).contiguous()
    bounds = torch.arange(num_rel + 1, dtype=torch.int64, device=types.device) * n_src
    pair_seg = torch.searchsorted(uniq, bounds).contiguous()
    groups = _ops.dest_groups(dst_id, n_out)
    rows_d = pair_of_row[groups.perm].contiguous()
    _SCATTER_PAIR_CACHE[key] = (groups.ptr, rows_d, pair_src, pair_seg, (src_id, types, dst_id))
    while len(_SCATTER_PAIR_CACHE) > 4:
        _SCATTER_PAIR_CACHE.popitem(last=False)
    return groups.ptr, rows_d, pair_src, pair_seg


def typed_linear(vin, weights, output, types, in_feat_tile=32):
    """output[i] += vin[i] @ weights[types[i]] (src/cpp/src/rel_spmm.cu:231-269)."""
    _typed_rows(vin, weights, output, types, None, None, False)


def typed_linear_s2e(vin, weights, output, src_id, types, in_feat_tile=32):
    """output[i] += vin[src_id[i]] @ weights[types[i]] (src/cpp/src/rel_spmm.cu:271-312)."""
    _typed_rows(vin, weights, output, types, src_id, None, False)


def typed_linear_s2d(vin, weights, output, src_id, dst_id, types, in_feat_tile=32):
    """output[dst_id[i]] += vin[src_id[i]] @ weights[types[i]], atomically
    (src/cpp/src/rel_spmm.cu:314-358)."""
    _typed_rows(vin, weights, output, types, src_id, dst_id, True)


# --------------------------------------------------------------------------- #
# fused relational aggregate + transform  (binding.cpp:46-47, 53-54)
# --------------------------------------------------------------------------- #
def _edge_segments(ptr, idx, rel, n, num_rel, want_perm=False):
    n_edges = int(ptr[n].item())
    perm, seg = rel_segment(rel[:n_edges].contiguous(), num_rel)
    rows = _ops.csr_row_ids(ptr, n, n_edges)
    if want_perm:
        return n_edges, idx[:n_edges][perm], rows[perm], seg, perm
    return n_edges, idx[:n_edges][perm], rows[perm], seg


_ARANGE_CACHE = {}


def _edge_positions(n, device):
    """arange(n) on the device, kept for the segment sums over per-edge rows."""
    key = (device, )
    t = _ARANGE_CACHE.get(key)
    if t is None or t.shape[0] < n:
        t = _ARANGE_CACHE[key] = torch.arange(n, dtype=torch.int64, device=device)
    return t[:n]


def typed_gemm_wgrad(a, g, seg_ptr, m_rows, num_rel, *, src_idx=None, dst_idx=None, precision=None):
    """gw[r] = sum over the rows i of segment r of a[src(i)]^T (x) g[dst(i)] -> [num_rel, K, N]
    (see cxg_typed_gemm_wgrad_f32).  One launch takes K <= 4096 (a block per 128 x 128 tile of gw and
    row chunk; the tiles of a chunk share its rows through one L2); beyond that, one launch per
    4096 columns of ``a``.  An N that is not a multiple of 4 (a class
    count, say) runs on a copy of g padded with zero columns.  Returns None when K is not a
    multiple of 4, which the kernel does not take."""
    lib = _lib.load()
    a_bf16 = a.dtype == torch.bfloat16                      # rows of a in bf16 (widened exactly as they are staged)
    _req(a, "a", torch.bfloat16 if a_bf16 else torch.float32, 2)
    _req(g, "g", torch.float32, 2)
    K, N = a.shape[1], g.shape[1]
    if K % 4:
        return None
    if N % 4:
        gw = typed_gemm_wgrad(a, torch.nn.functional.pad(g, (0, -N % 4)), seg_ptr, m_rows, num_rel,
                              src_idx=src_idx, dst_idx=dst_idx, precision=precision)
        return gw[:, :, :N].contiguous()
    precision = precision or GEMM_PRECISION
    flags = (GEMM_SPLIT_F16X3 if precision == "split_f16" else
             GEMM_SPLIT_BF16X3 if precision in ("split3", "bf16") else GEMM_SPLIT_BF16X6)
    flags |= WGRAD_A_BF16 if a_bf16 else 0
    esz = 2 if a_bf16 else 4
    gw = torch.empty((num_rel, K, N), dtype=torch.float32, device=a.device)
    k_max = 4096                                            # what one launch takes
    with torch.cuda.device(a.device):
        for k0 in range(0, K, k_max):
            kb = min(k_max, K - k0)
            direct = num_rel == 1 or kb == K
            part = gw if direct else torch.empty((num_rel, kb, N), dtype=torch.float32, device=a.device)
            ws = _workspace(lib.cxg_typed_gemm_wgrad_workspace_bytes(m_rows, kb, N, num_rel), a.device)
            st = lib.cxg_typed_gemm_wgrad_f32(a.data_ptr() + esz * k0, K, g.data_ptr(), N, _lib.ptr(src_idx),
                                              _lib.ptr(dst_idx), seg_ptr.data_ptr(), m_rows, kb, N, num_rel,
                                              part.data_ptr() + (4 * k0 * N if direct else 0), flags, ws.data_ptr(),
                                              ws.numel(), _lib.current_stream(a.device))
            _lib.check(st)
            if not direct:
                gw[:, k0:k0 + kb, :] = part
    return gw


def _weight_grad(x, g, src, dst, seg, shape, precision=None):
    """grad_W[r] = sum over the rows of segment r of x[src]^T g[dst]: one launch of the
    typed weight-gradient kernel; shapes it does not take use a row gather plus one
    library GEMM per relation."""
    x, g = x.contiguous(), g.contiguous()
    gw = typed_gemm_wgrad(x, g, seg, src.shape[0], shape[0], src_idx=src, dst_idx=dst, precision=precision)
    if gw is not None:
        return gw
    gw = torch.zeros(shape, dtype=torch.float32, device=x.device)
    bounds = seg.tolist()
    for r in range(shape[0]):
        b, e = bounds[r], bounds[r + 1]
        if e > b:
            xs = _ops.gather_rows(x, src[b:e].contiguous())
            gs = g[b:e] if dst is None else _ops.gather_rows(g, dst[b:e].contiguous())
            gw[r] = torch.mm(xs.t(), gs)
    return gw


# Transform-first RGCN: out[d] = sum_e Y[idx[e], rel[e]] with Y[s, r] = x[s] @ W[r]
# computed for every (source, relation) pair by one dense GEMM against the
# concatenated weights.  2 * n_src * R * K * N flops instead of 2 * E * K * N, no
# atomics, deterministic; the aggregation is the plain SpMM over a combined index.
# Chosen when the graph has at least half as many edges as (source, relation)
# pairs and Y fits the memory budget -- on the pairs that own an edge only when those
# are a minority (_pair_graph); sparser inputs (sampled blocks with many relations)
# write one GEMM row per edge, or use the fused gather-GEMM-scatter launch.
RGCN_DENSE_MAX_BYTES = 64 << 30
RGCN_EDGE_ROWS_MAX_BYTES = 64 << 30        # per-edge rows of the sparse strategy; above: atomic scatter


class _RelGraph:
    """Index structures of the transform-first path for one (ptr, idx, rel):
    key_fwd[e] = idx[e] * R + rel[e]; the CSR of the reversed graph with one row
    per (source, relation) pair (ptr_key, idx_key = destinations); ptr_src =
    its coarsening to one row per source; key_bwd[k] = idx_key[k] * R + rel."""
    __slots__ = ("key_fwd", "ptr_key", "idx_key", "ptr_src", "key_bwd", "n_edges", "_keep")


_REL_CACHE = collections.OrderedDict()
_REL_CACHE_CAP = 4


def _rel_graph(ptr, idx, rel, n, n_src, R):
    key = (ptr.data_ptr(), idx.data_ptr(), rel.data_ptr(), ptr.shape[0], idx.shape[0], n, n_src, R,
           ptr._version, idx._version, rel._version, ptr.device.index)
    rg = _REL_CACHE.get(key)
    if rg is not None:
        _REL_CACHE.move_to_end(key)
        return rg
    rg = _RelGraph()
    rg.n_edges = int(ptr[n].item())
    rel64 = rel[:rg.n_edges].to(torch.int64)
    if rg.n_edges and (int(rel64.min()) < 0 or int(rel64.max()) >= R):
        raise ValueError("relation ids must lie in [0, %d)" % R)
    rg.key_fwd = idx[:rg.n_edges] * R + rel64
    rg.ptr_key, rg.idx_key, perm, _ = _ops.csr_transpose(ptr, rg.key_fwd, n, n_src * R)
    rg.ptr_src = rg.ptr_key[::R].contiguous()
    rg.key_bwd = rg.idx_key * R + rel64[perm]
    rg._keep = (ptr, idx, rel)
    _REL_CACHE[key] = rg
    while len(_REL_CACHE) > _REL_CACHE_CAP:
        _REL_CACHE.popitem(last=False)
    return rg


class _PairGraph:
    """Index structures of the pair-compacted transform-first path for one (ptr, idx, rel).
    Only the (source, relation) pairs that own an edge get a row of Y = x W, only the
    (destination, relation) pairs that own one a row of Z = g W^T:
      f_src [Uf], f_seg [R+1]  source of every forward pair, pairs sorted by (relation, source);
      f_row [E]                pair row of every edge, in CSR edge order;
      f_ptr [Uf+1], f_dst [E]  CSR over the forward pairs: destinations of a pair's edges;
      b_dst [Ub], b_seg [R+1]  destination of every backward pair, sorted by (relation, destination);
      ptr_src [n_src+1], b_row_rev [E]  reversed graph (rows = sources) and, per reversed edge,
                               its backward pair row.
    For the aggregate-first order (built on first use, _pair_graph_aggregate):
      bp_ptr [Ub+1], bp_src [E]  CSR over the backward pairs: sources of a pair's edges;
      dp_ptr [n+1], dp_rows [Ub] CSR over the destinations: the pair rows of a destination;
      mean_fwd [E], mean_rev [E] 1 / in-degree of every edge's destination in bp and in reversed
                               edge order (the mean layer, _pair_mean_weights)."""
    __slots__ = ("n_edges", "f_src", "f_seg", "f_row", "f_ptr", "f_dst", "b_dst", "b_seg", "ptr_src", "b_row_rev",
                 "b_row", "bp_ptr", "bp_src", "dp_ptr", "dp_rows", "mean_fwd", "mean_rev", "_keep")


_PAIR_CACHE = collections.OrderedDict()


def _pair_graph(ptr, idx, rel, n, n_src, R):
    key = (ptr.data_ptr(), idx.data_ptr(), rel.data_ptr(), ptr.shape[0], idx.shape[0], n, n_src, R,
           ptr._version, idx._version, rel._version, ptr.device.index)
    pg = _PAIR_CACHE.get(key)
    if pg is not None:
        _PAIR_CACHE.move_to_end(key)
        return pg
    pg = _PairGraph()
    e = pg.n_edges = int(ptr[n].item())
    dev = ptr.device
    rel64 = rel[:e].to(torch.int64)
    if e and (int(rel64.min()) < 0 or int(rel64.max()) >= R):
        raise ValueError("relation ids must lie in [0, %d)" % R)
    src = idx[:e]
    dst = _ops.csr_row_ids(ptr, n, e)
    bounds = torch.arange(R + 1, dtype=torch.int64, device=dev)
    uf, pg.f_row = torch.unique(rel64 * n_src + src, sorted=True, return_inverse=True)
    pg.f_src = (uf % n_src).contiguous()
    pg.f_seg = torch.searchsorted(uf, bounds * n_src).contiguous()
    pg.f_row = pg.f_row.contiguous()
    pg.f_ptr, pg.f_dst, _ = _ops.coo_to_csr(dst, pg.f_row, uf.shape[0])
    ub, b_row = torch.unique(rel64 * n + dst, sorted=True, return_inverse=True)
    pg.b_dst = (ub % n).contiguous()
    pg.b_seg = torch.searchsorted(ub, bounds * n).contiguous()
    tg = _ops.transposed(ptr, idx, n, n_src)
    pg.ptr_src = tg.ptr_t
    pg.b_row_rev = b_row[tg.perm].contiguous()
    pg.b_row = b_row.contiguous()
    pg.bp_ptr = pg.bp_src = pg.dp_ptr = pg.dp_rows = pg.mean_fwd = pg.mean_rev = None
    pg._keep = (ptr, idx, rel)
    _PAIR_CACHE[key] = pg
    while len(_PAIR_CACHE) > _REL_CACHE_CAP:
        _PAIR_CACHE.popitem(last=False)
    return pg


def _pair_graph_aggregate(pg, idx, n):
    """The two extra CSRs of the aggregate-first order, kept with the pair graph."""
    if pg.bp_ptr is None:
        n_pairs = pg.b_dst.shape[0]
        pg.bp_ptr, pg.bp_src, _ = _ops.coo_to_csr(idx[:pg.n_edges].contiguous(), pg.b_row, n_pairs)
        rows = torch.arange(n_pairs, dtype=torch.int64, device=idx.device)
        pg.dp_ptr, pg.dp_rows, _ = _ops.coo_to_csr(rows, pg.b_dst, n)
    return pg


def _pair_mean_weights(pg, ptr, n):
    """1 / in-degree of the destination of every edge, in the edge order of the pair rows
    (bp) and of the reversed graph (ptr_src): with these as edge values the two gathers of
    the aggregate-first order apply the division by the degree themselves, so neither the
    output nor its gradient takes a pass of its own.  Kept with the pair graph."""
    if pg.mean_fwd is None:
        per_pair = _inv_degree(ptr, n)[pg.b_dst]
        n_pairs = pg.b_dst.shape[0]
        pg.mean_fwd = per_pair[_ops.csr_row_ids(pg.bp_ptr, n_pairs, pg.bp_src.shape[0])].contiguous()
        pg.mean_rev = per_pair[pg.b_row_rev].contiguous()
    return pg.mean_fwd, pg.mean_rev


def _pairs_aggregate_first(pg, x, weights, idx, n, precision=None, mean_ptr=None):
    """out[d] = sum_r (sum of x over d's edges of relation r) @ W[r] on the (destination,
    relation) pairs that own an edge: one SpMM into the pair rows (gathering rows of x), one
    typed GEMM over the relation segments of pair rows, one SpMM that gives every destination
    the sum of its pairs' product rows.  With ``mean_ptr`` (the row offsets of the graph) the
    first SpMM weights every edge by 1 / in-degree of its destination, which divides out[d] by
    the degree.  Returns (out, z)
    with z the aggregated (and weighted) pair rows."""
    _pair_graph_aggregate(pg, idx, n)
    n_pairs = pg.b_dst.shape[0]
    val = _pair_mean_weights(pg, mean_ptr, n)[0] if mean_ptr is not None else None
    K, N = weights.shape[1], weights.shape[2]
    if _bf16_tables(precision, K, N):
        # the bf16 variant keeps its pair-row tables in bf16: the aggregation into the pair rows
        # rounds as it stores, the typed GEMM reads and writes bf16 rows, the sum per destination
        # gathers bf16 rows and adds in fp32 -- half the bytes on every pass over the tables
        # (x itself is rounded once, 1 M rows, so that the 20 M row gathers move bf16 rows too)
        z = _ops.spmm_bf16_rows(pg.bp_ptr, pg.bp_src, x.to(torch.bfloat16), n_pairs, val=val, out_bf16=True)   # [Ub, K] bf16
        t = typed_gemm(z, weights, pg.b_seg, n_pairs, bf16=True, out_bf16=True)                  # [Ub, N] bf16
        return _ops.spmm_bf16_rows(pg.dp_ptr, pg.dp_rows, t, n), z
    z = _ops.spmm(pg.bp_ptr, pg.bp_src, x, n_pairs, val=val)              # [Ub, K]
    t = typed_gemm(z, weights, pg.b_seg, n_pairs, precision=precision)                         # [Ub, N]
    return _ops.spmm(pg.dp_ptr, pg.dp_rows, t, n), z


def _bf16_tables(precision, K, N):
    return precision == "bf16" and K <= 128 and N <= 128 and K % 8 == 0 and N % 8 == 0


def _pairs_aggregate_first_bwd(pg, weights, z, grad_out, n_src, need_x, need_w, precision=None, mean=False):
    """Gradients of _pairs_aggregate_first for x and the weights (``mean``: the forward pass
    weighted the edges by 1 / degree; z holds the weighted rows, so only the gather of the
    input gradient repeats the weights)."""
    n_pairs = pg.b_dst.shape[0]
    gx = gw = None
    if need_x and z.dtype == torch.bfloat16:
        # bf16 tables (see _pairs_aggregate_first): the per-pair gradient rows are stored and gathered in bf16
        gz = typed_gemm(grad_out.to(torch.bfloat16), weights.transpose(1, 2).contiguous(), pg.b_seg, n_pairs,
                        src_idx=pg.b_dst, bf16=True, out_bf16=True)
        gx = _ops.spmm_bf16_rows(pg.ptr_src, pg.b_row_rev, gz, n_src, val=pg.mean_rev if mean else None)
    elif need_x:
        gz = typed_gemm(grad_out, weights.transpose(1, 2).contiguous(), pg.b_seg, n_pairs, src_idx=pg.b_dst,
                        precision=precision)
        gx = _ops.spmm(pg.ptr_src, pg.b_row_rev, gz, n_src, val=pg.mean_rev if mean else None)
    if need_w:
        gw = _weight_grad(z, grad_out, _edge_positions(n_pairs, z.device), pg.b_dst, pg.b_seg, weights.shape,
                          precision)
    return gx, gw


# The dense table is kept when nearly every (source, relation) pair owns an edge: its GEMM
# reads and writes contiguous rows, the compacted one gathers its input rows.
RGCN_PAIR_FILL_MAX = 0.8


def _dense_seg(n_rows, device):
    return torch.tensor([0, n_rows], dtype=torch.int64, device=device)


def _use_dense(n_edges, n_src, R, N):
    return 2 * n_edges >= n_src * R and 4 * n_src * R * N <= RGCN_DENSE_MAX_BYTES


class _RgcnFusedFunction(torch.autograd.Function):
    """out[r] = sum_e x[idx[e]] @ W[rel[e]] (aggr_rgcn_direct_kernel,
    src/cpp/src/rel_spmm.cu:138-181), optionally divided by the row's edge count.
    The reference's backward returns zeros (rel_spmm.cu:400-432); the true
    gradients are computed here."""

    @staticmethod
    def forward(ctx, x, ptr, idx, weights, rel, num_node, mean=False, force_dense=False, precision=None):
        n = as_int(num_node)
        if n == 0:
            n = ptr.shape[0] - 1
        if x.shape[1] != weights.shape[1]:
            raise ValueError("feat_len weight size %d %d" % (x.shape[1], weights.shape[1]))
        x = x.contiguous()
        weights = weights.contiguous()
        R, K, N = weights.shape
        n_src = x.shape[0]
        ctx.n, ctx.mean = n, mean
        ctx.precision = precision
        n_edges = int(ptr[n].item())
        ctx.dense = force_dense or _use_dense(n_edges, n_src, R, N)
        ctx.pairs = False
        if ctx.dense:
            # transform-first over the pairs that occur: Y and Z hold one row per (node, relation)
            # pair that owns an edge instead of one per pair that could
            pg = _pair_graph(ptr, idx, rel, n, n_src, R)
            ctx.pairs = pg.f_src.shape[0] <= RGCN_PAIR_FILL_MAX * n_src * R
        ctx.aggregate_first = ctx.pairs and K <= N and not force_dense     # gather the narrower rows
        if ctx.aggregate_first:
            out, z = _pairs_aggregate_first(pg, x, weights, idx, n, precision, ptr if mean else None)
            ctx.pg = pg
            ctx.save_for_backward(x, weights, ptr, z)
            return out
        if ctx.pairs:
            y = typed_gemm(x, weights, pg.f_seg, pg.f_src.shape[0], src_idx=pg.f_src, precision=precision)    # [Uf, N]
            out = _ops.spmm(ptr, pg.f_row, y, n, mean=mean)
            ctx.pg = pg
            ctx.save_for_backward(x, weights, ptr)
            return out
        if ctx.dense:
            rg = _rel_graph(ptr, idx, rel, n, n_src, R)
            wcat = weights.permute(1, 0, 2).reshape(1, K, R * N).contiguous()
            y = typed_gemm(x, wcat, _dense_seg(n_src, x.device), n_src, precision=precision)          # [n_src, R*N]
            out = _ops.spmm(ptr, rg.key_fwd, y.view(n_src * R, N), n, mean=mean)
            ctx.rg = rg
            ctx.save_for_backward(x, weights, ptr)
            return out
        n_edges, src, dst, seg, perm = _edge_segments(ptr, idx, rel, n, R, want_perm=True)
        ctx.n_edges = n_edges
        ctx.per_edge = 4 * n_edges * max(K, N) <= RGCN_EDGE_ROWS_MAX_BYTES
        if ctx.per_edge:
            # one output row per edge, written once in CSR order, then the plain sum over
            # each destination's (consecutive) rows: no atomics, reproducible
            tmp = torch.empty((n_edges, N), dtype=torch.float32, device=x.device)
            typed_gemm(x, weights, seg, n_edges, src_idx=src, dst_idx=perm, out=tmp, precision=precision)
            out = _ops.spmm(ptr, _edge_positions(n_edges, x.device), tmp, n, mean=mean)
            ctx.save_for_backward(x, weights, ptr, src, dst, seg, perm, idx)
            return out
        out = torch.zeros((n, N), dtype=torch.float32, device=x.device)
        typed_gemm(x, weights, seg, n_edges, src_idx=src, dst_idx=dst, out=out, atomic=True, precision=precision)
        if mean:
            out *= _inv_degree(ptr, n).unsqueeze(1)
        ctx.save_for_backward(x, weights, ptr, src, dst, seg)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        grad_out = grad_out.contiguous()
        x, weights, ptr = ctx.saved_tensors[:3]
        R, K, N = weights.shape
        n, n_src = ctx.n, x.shape[0]
        precision = ctx.precision
        gx = gw = None
        if ctx.aggregate_first:
            gx, gw = _pairs_aggregate_first_bwd(ctx.pg, weights, ctx.saved_tensors[3], grad_out, n_src,
                                                ctx.needs_input_grad[0], ctx.needs_input_grad[3], precision,
                                                ctx.mean)
            return gx, None, None, gw, None, None, None, None, None
        if ctx.mean:
            grad_out = grad_out * _inv_degree(ptr, n).unsqueeze(1)
        if ctx.pairs:
            pg = ctx.pg
            if ctx.needs_input_grad[0]:
                # Z = g[d] @ W[r]^T for the (destination, relation) pairs that occur, then the
                # plain SpMM over the reversed graph
                z = typed_gemm(grad_out, weights.transpose(1, 2).contiguous(), pg.b_seg, pg.b_dst.shape[0],
                               src_idx=pg.b_dst, precision=precision)
                gx = _ops.spmm(pg.ptr_src, pg.b_row_rev, z, n_src)
            if ctx.needs_input_grad[3]:
                # gY = sum of g over the edges of every (source, relation) pair; gW[r] = x[src]^T gY
                gy = _ops.spmm(pg.f_ptr, pg.f_dst, grad_out, pg.f_src.shape[0])
                gw = _weight_grad(x, gy, pg.f_src, None, pg.f_seg, weights.shape, precision)
            return gx, None, None, gw, None, None, None, None, None
        if ctx.dense:
            rg = ctx.rg
            if ctx.needs_input_grad[0]:
                # Z[d, r] = g[d] @ W[r]^T for every (destination, relation), then the
                # plain SpMM over the reversed graph
                wcat_t = weights.permute(2, 0, 1).reshape(1, N, R * K).contiguous()
                z = typed_gemm(grad_out, wcat_t, _dense_seg(n, x.device), n, precision=precision)      # [n, R*K]
                gx = _ops.spmm(rg.ptr_src, rg.key_bwd, z.view(n * R, K), n_src)
            if ctx.needs_input_grad[3]:
                # gY[s, r] = sum of g over the edges (s -> d) of relation r; gW[r] = x^T gY[:, r]
                gy = _ops.spmm(rg.ptr_key, rg.idx_key, grad_out, n_src * R)      # [n_src*R, N]
                gw = typed_gemm_wgrad(x, gy.view(n_src, R * N), _dense_seg(n_src, x.device), n_src, 1,
                                      precision=precision)
                if gw is None:
                    gw = torch.mm(x.t(), gy.view(n_src, R * N))
                gw = gw.view(K, R, N).permute(1, 0, 2).contiguous()
            return gx, None, None, gw, None, None, None, None, None
        src, dst, seg = ctx.saved_tensors[3:6]
        if ctx.needs_input_grad[0] and ctx.per_edge:
            # per-edge rows g[dst(e)] @ W[rel(e)]^T in CSR order, summed per source over the
            # reversed graph (whose edge permutation says where each source's rows are)
            perm, idx = ctx.saved_tensors[6:8]
            tmp = torch.empty((ctx.n_edges, K), dtype=torch.float32, device=x.device)
            typed_gemm(grad_out, weights.transpose(1, 2).contiguous(), seg, ctx.n_edges, src_idx=dst,
                       dst_idx=perm, out=tmp, precision=precision)
            gt = _ops.transposed(ptr, idx, n, n_src)
            gx = _ops.spmm(gt.ptr_t, gt.perm, tmp, n_src)
        elif ctx.needs_input_grad[0]:
            gx = torch.zeros_like(x)
            typed_gemm(grad_out, weights.transpose(1, 2).contiguous(), seg, ctx.n_edges, src_idx=dst,
                       dst_idx=src, out=gx, atomic=True, precision=precision)
        if ctx.needs_input_grad[3]:
            gw = _weight_grad(x, grad_out, src, dst, seg, weights.shape, precision)
        return gx, None, None, gw, None, None, None, None, None


_DST_REL_CACHE = collections.OrderedDict()


def dst_rel_graph(ptr, idx, rel, n, R):
    """CSR with one row per (destination, relation) pair, row d * R + r holding the sources of
    d's edges of relation r in their original order: (ptr_dr [n*R+1], idx_dr [E]); cached per
    (ptr, idx, rel).  The aggregate-then-transform RGCN sums into these rows."""
    key = (ptr.data_ptr(), idx.data_ptr(), rel.data_ptr(), ptr.shape[0], idx.shape[0], n, R,
           ptr._version, idx._version, rel._version, ptr.device.index)
    hit = _DST_REL_CACHE.get(key)
    if hit is not None:
        _DST_REL_CACHE.move_to_end(key)
        return hit[0], hit[1]
    e = int(ptr[n].item())
    rows = _ops.csr_row_ids(ptr, n, e)
    ptr_dr, idx_dr, _ = _ops.coo_to_csr(idx[:e].contiguous(), rows * R + rel[:e].to(torch.int64), n * R)
    _DST_REL_CACHE[key] = (ptr_dr, idx_dr, (ptr, idx, rel))
    while len(_DST_REL_CACHE) > _REL_CACHE_CAP:
        _DST_REL_CACHE.popitem(last=False)
    return ptr_dr, idx_dr


def _inv_degree(ptr, n):
    deg = (ptr[1:n + 1] - ptr[:n]).to(torch.float32)
    return torch.where(deg > 0, 1.0 / deg, torch.zeros_like(deg))


def aggr_rgcn_direct_func(input, ptr, idx, weights, rel, num_node):
    """src/cpp/src/rel_spmm.cu:442-467 (rel int32)."""
    if weights.dim() != 3:
        raise ValueError("weights must be [num_rel, in, out]")
    return _RgcnFusedFunction.apply(input, ptr, idx, weights, rel, num_node)


def aggr_rgcn_mean(input, ptr, idx, weights, rel, num_node, precision=None):
    """aggr_rgcn_direct_func divided by each row's edge count (rows without edges
    give 0): the whole relational layer of MyRGCNConv
    (cxgnncomp/graph_conv.py:352-378) in one differentiable op.  ``precision`` selects how
    the typed GEMMs multiply (see typed_gemm; None = GEMM_PRECISION)."""
    return _RgcnFusedFunction.apply(input, ptr, idx, weights, rel, num_node, True, False, precision)


def aggr_rel_direct(input, ptr, idx, weights, etype, num_node, num_rel):
    """src/cpp/src/rel_spmm.cu:434-440."""
    if int(num_rel) != weights.shape[0]:
        raise ValueError("num_rel=%d but weights has %d relations" % (int(num_rel), weights.shape[0]))
    return _RgcnFusedFunction.apply(input, ptr, idx, weights, etype, num_node)


def seastar_forward(input, ptr, idx, weights, etype):
    """Seastar RGCN baseline forward (src/cpp/src/rel_spmm.cu:469-521): the same
    sum_e x[idx[e]] @ W[etype[e]] over all rows of ptr."""
    with torch.no_grad():
        return _RgcnFusedFunction.apply(input, ptr, idx, weights, etype, ptr.shape[0] - 1)


def seastar_backward(input, ptr, idx, weights, etype, grad):
    """Returns [grad_input, grad_weights] (src/cpp/src/rel_spmm.cu:523-579).  The gradients of
    seastar_forward's function through the same pair tables and kernels as the fused relational
    layer (no atomics: reproducible, and faster than the scatter form although the forward pass
    is recomputed for the tables it leaves -- 20 M edges, 16 relations, 128 -> 128, forward +
    backward: 15.5 against 17.9 ms)."""
    n = ptr.shape[0] - 1
    with torch.enable_grad():
        xd = input.detach().requires_grad_(True)
        wd = weights.detach().requires_grad_(True)
        out = _RgcnFusedFunction.apply(xd, ptr, idx, wd, etype, n)
    gx, gw = torch.autograd.grad(out, (xd, wd), grad.contiguous())
    return [gx, gw]
