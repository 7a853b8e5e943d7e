/*
 * cxgnn_hip.h -- C ABI of libcxgnn_hip.so, the gfx950 (MI355X) graph-kernel
 * library that stands in for the CUDA extension `cxgnncomp_backend` of
 * xxcclong/CxGNN-Compute (pybind module: src/cpp/python_bindings/binding.cpp:14-130).
 *
 * Conventions
 *   - every pointer is a device pointer unless the name ends in `_host`;
 *   - graphs are CSR by destination: ptr[n_rows+1], idx[...] = source ids,
 *     both int64 (`using Index = int64_t`, src/cpp/include/common.h:15) unless a
 *     function says int32;
 *   - float tensors are fp32, row-major, contiguous (row stride given where a
 *     caller may pass a view);
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); all
 *     work is enqueued on it and nothing synchronises;
 *   - every function returns 0 on success or a negative cxg_status; the message
 *     is available from cxg_last_error() on the calling thread.  Nothing exits or
 *     aborts the process (the reference's ASSERT macros call exit(1),
 *     src/cpp/include/common.h:16-26);
 *   - functions that need scratch memory take `workspace` + `workspace_bytes`;
 *     the matching *_workspace_bytes() query says how much.  The library never
 *     allocates device memory in those functions.
 */
#ifndef CXGNN_HIP_H
#define CXGNN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum cxg_status {
  CXG_OK = 0,
  CXG_ERR_ARG = -1,         /* null pointer, negative size, bad flag */
  CXG_ERR_UNSUPPORTED = -2, /* shape outside what the kernels cover */
  CXG_ERR_WORKSPACE = -3,   /* workspace missing or too small */
  CXG_ERR_HIP = -4          /* a HIP runtime call or kernel launch failed */
} cxg_status;

/* Library version (major*10000 + minor*100 + patch). */
int cxg_version(void);
/* Message of the last failure on this thread ("" if none). */
const char* cxg_last_error(void);

/* ------------------------------------------------------------------------- */
/* SpMM family: out[r, :] = reduce_{e in [ptr[r], ptr[r+1])} w[e] * x[idx[e], :] */
/* ------------------------------------------------------------------------- */

/* flags for cxg_spmm_* */
#define CXG_SPMM_MEAN 1u       /* divide each row by its degree; empty rows stay 0 */
#define CXG_SPMM_ACCUMULATE 2u /* out += result instead of out = result           */
#define CXG_SPMM_HINT_EXACT_EDGES 4u /* n_edges_cap is the real edge count of the rows (tuning hint only) */
#define CXG_SPMM_DOT_AT_EDGE 8u /* cxg_spmm_weighted_dot_f32 only: dot_out rows at the edge's position in idx although val is read through val_perm */

/* Bytes of workspace needed by cxg_spmm_* for a graph whose idx array has
 * n_edges_cap entries and rows of `row_floats` floats (heads*channels). */
size_t cxg_spmm_workspace_bytes(int64_t n_edges_cap, int64_t row_floats);

/*
 * Sum / mean aggregation.  Replaces run_spmm_configurable
 * (src/cpp/src/spmm_host.cu:6-55; the nine launch integers of that function
 * have no meaning here), sage_sum_forward / sage_mean_forward
 * (src/cpp/src/aggr.cu:385-393, kernels src/cpp/src/aggr_kernel.cu:3-53).
 * Rows [0, n_rows) of `out` are written; edges outside [ptr[0], ptr[n_rows])
 * are ignored; n_edges_cap is the length of idx (>= ptr[n_rows]).
 */
int cxg_spmm_sum_f32(const int64_t* ptr, const int64_t* idx, const float* x,
                     int64_t ldx, float* out, int64_t ldo, int64_t n_rows,
                     int64_t n_edges_cap, int feat, unsigned flags,
                     void* workspace, size_t workspace_bytes, void* stream);

/*
 * cxg_spmm_sum_f32 for callers that can neither allocate device memory nor hand over a
 * workspace: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  No counterpart in the reference.  Same kernels and results as
 * cxg_spmm_sum_f32; the carry buffer and span table live in a device array of
 * CXG_SPMM_NOALLOC_SCRATCH_BYTES that is part of the library's code object (every GPU the
 * library runs on holds its own copy until the process ends).  The call allocates and frees
 * nothing.  Shapes whose cxg_spmm_workspace_bytes(n_edges_cap, feat) exceeds that size are
 * rejected with CXG_ERR_WORKSPACE (the limit is 32 million edges at feat = 128, 16 million
 * at feat = 256).  Every call on one GPU uses that GPU's
 * one array: calls that overlap in time on the same GPU (two streams, two threads) race;
 * calls on one stream are ordered and safe.  Nothing in the array needs clearing between
 * calls: each launch writes every slot it later reads.  The first call on a device looks up
 * the array's address (hipGetSymbolAddress) and must therefore happen outside a graph
 * capture; later calls only launch kernels.
 */
#define CXG_SPMM_NOALLOC_SCRATCH_BYTES (64u << 20)
int cxg_spmm_sum_f32_noalloc(const int64_t* ptr, const int64_t* idx, const float* x,
                             int64_t ldx, float* out, int64_t ldo, int64_t n_rows,
                             int64_t n_edges_cap, int feat, unsigned flags, void* stream);

/* Same with int32 ptr/idx.  Replaces run_spmm_configurable_int32
 * (src/cpp/src/spmm_host.cu:99-156). */
int cxg_spmm_sum_f32_i32(const int32_t* ptr, const int32_t* idx, const float* x,
                         int64_t ldx, float* out, int64_t ldo, int64_t n_rows,
                         int64_t n_edges_cap, int feat, unsigned flags,
                         void* workspace, size_t workspace_bytes, void* stream);

/*
 * Edge-weighted aggregation, single- or multi-head:
 *   out[r, h, c] = sum_e val[vrow(e), h] * x[idx[e], h, c],
 *   vrow(e) = val_perm ? val_perm[e] : e.
 * x is [n_src, heads, channels] (row stride ldx floats), val is
 * [n_val_rows, heads].  Replaces sage_sum_forward_edge_value
 * (src/cpp/src/aggr.cu:377-383, kernels aggr_kernel.cu:88-116,155-186) and
 * spmm_multihead(..., Naive) (src/cpp/src/spmm_host.cu:158-196).  With
 * val_perm = the edge permutation of a transposed CSR it also computes the
 * input gradient A^T(val .* g) that the reference obtains with atomics
 * (aggr_kernel.cu:287-319,403-441; spmm_multihead_bwd spmm_host.cu:198-214).
 */
int cxg_spmm_weighted_f32(const int64_t* ptr, const int64_t* idx,
                          const float* val, const int64_t* val_perm,
                          const float* x, int64_t ldx, float* out, int64_t ldo,
                          int64_t n_rows, int64_t n_edges_cap, int heads,
                          int channels, unsigned flags, void* workspace,
                          size_t workspace_bytes, void* stream);

/*
 * Multi-head edge-weighted aggregation summed over the heads inside the kernel:
 *   out[r, c] = sum_h sum_e val[vrow(e), h] * x[idx[e], h, c]     (out is [n_rows, channels]).
 * The wave that gathers a row of heads x channels floats adds its head groups with
 * xor-shuffles when the row ends and stores channels floats: no [n_rows, heads, channels]
 * intermediate is written and read back.  Takes heads * channels in {64, 128, 256} with a
 * power-of-two head count (the whole row in one 64-lane gather), otherwise
 * CXG_ERR_UNSUPPORTED (run cxg_spmm_weighted_f32 and cxg_head_sum_f32 instead).  Workspace
 * as for cxg_spmm_weighted_f32 (cxg_spmm_workspace_bytes(n_edges_cap, heads * channels)).
 * Replaces spmm_multihead(..., PreReduce / Optimal) and run_spmm_multihead_configurable
 * (src/cpp/src/spmm_host.cu:158-256, kernels spmm_multihead_kernel.cu:38-207).
 */
int cxg_spmm_prereduce_f32(const int64_t* ptr, const int64_t* idx, const float* val,
                           const int64_t* val_perm, const float* x, int64_t ldx, float* out,
                           int64_t ldo, int64_t n_rows, int64_t n_edges_cap, int heads,
                           int channels, unsigned flags, void* workspace, size_t workspace_bytes,
                           void* stream);

/*
 * Edge-weighted aggregation of ONE gathered row under several weights:
 *   out[r, h, :] = sum_e val[e, h] * x[idx[e], :]      (x [n_src, feat], out [n_rows, heads, feat]).
 * Where a multi-head layer's features are a linear map of a narrower input, xs[:, h, :] = x W_h^T,
 * its aggregation sum_e val[e, h] xs[idx[e], h, :] equals out[r, h, :] W_h^T: the edges gather
 * feat floats instead of heads * channels, the product follows per destination row (the order
 * "aggregate, then transform" of MyGATConv.forward_1, cxgnncomp/graph_conv.py:523-542, applied to
 * forward_many's aggregation, :481-487).  Takes 2, 4 or 8 heads and 20 <= feat <= 128, a
 * multiple of 4; x, out and val 16-byte aligned, strides multiples of 4; otherwise
 * CXG_ERR_UNSUPPORTED.  Workspace: cxg_spmm_workspace_bytes(n_edges_cap, heads * feat).
 * Deterministic (no atomics), like the other aggregations.
 */
int cxg_spmm_weighted_heads_f32(const int64_t* ptr, const int64_t* idx, const float* val,
                                const float* x, int64_t ldx, float* out, int64_t ldo,
                                int64_t n_rows, int64_t n_edges_cap, int heads, int feat,
                                unsigned flags, void* workspace, size_t workspace_bytes,
                                void* stream);

/*
 * Single-head aggregation (sum, CXG_SPMM_MEAN, or one weight per edge, optionally read through
 * val_perm) of rows of 4 .. 128 values (a multiple of 4) whose rows are bf16 on the gathered
 * side (x_bf16), on the stored side (out_bf16), or both; sums are formed in fp32 and rounded to
 * nearest even when stored.  ldx / ldo count elements of the respective type.  Serves the bf16
 * variant of the relational layer (MyRGCNConv(precision="bf16"), cxgnncomp/graph_conv.py:329-378,
 * where the reference has an fp32 layer only): its pair-row tables are written and gathered at
 * half the bytes.  Workspace: cxg_spmm_workspace_bytes(n_edges_cap, feat).
 */
int cxg_spmm_bf16_rows(const int64_t* ptr, const int64_t* idx, const float* val, const int64_t* val_perm,
                       const void* x, int64_t ldx, int x_bf16, void* out, int64_t ldo, int out_bf16,
                       int64_t n_rows, int64_t n_edges_cap, int feat, unsigned flags, void* workspace,
                       size_t workspace_bytes, void* stream);

/*
 * cxg_spmm_weighted_f32 with bias[heads*channels] added to every output row as it is
 * stored (NULL: none; not with CXG_SPMM_MEAN): the `out + self.bias` that follows the
 * aggregation in MyGATConv.forward_many (cxgnncomp/graph_conv.py:488-494) without a second
 * pass over the output.
 */
int cxg_spmm_weighted_bias_f32(const int64_t* ptr, const int64_t* idx, const float* val,
                               const int64_t* val_perm, const float* x, int64_t ldx,
                               const float* bias, float* out, int64_t ldo, int64_t n_rows,
                               int64_t n_edges_cap, int heads, int channels, unsigned flags,
                               void* workspace, size_t workspace_bytes, void* stream);

/*
 * cxg_spmm_weighted_f32 that also leaves, for every edge e of output row r,
 *   dot_out[vrow(e), h] = sum_c x[idx[e], h, c] * dot_b[r, h, c]
 * from the same gathered rows.  Called on the transposed CSR with x = the gradient of the
 * aggregated features, val / val_perm = the edge values and the transposition's edge
 * permutation, dot_b = the layer's input features, it yields the input gradient AND the
 * edge-value gradient of the multi-head weighted aggregation in one pass: the pair
 * spmm_multihead_bwd + run_sddmm of SpMMValOP.backward (cxgnncomp/graph_kernel.py:20-37,
 * src/cpp/src/spmm_host.cu:198-214, src/cpp/src/sddmm_host.cu:4-14).  dot_b is
 * [n_rows, heads, channels] with row stride ld_dot_b, dot_out [n_val_rows, heads].
 * With CXG_SPMM_DOT_AT_EDGE the row of edge position k (in idx) is dot_out[k] whether or
 * not val is read through val_perm: contiguous stores instead of one scattered 16-byte
 * store per edge (a consumer then reads row e of the original order at the inverse
 * permutation's position, see cxg_edge_softmax_bwd_at_f32).
 * Shapes: heads*channels a multiple of 256, channels in {32, 64, 128, 256}, 16-byte
 * aligned rows; also one head of 16 .. 128 channels (a multiple of 4) when val is read
 * through val_perm and CXG_SPMM_DOT_AT_EDGE is set (the single-head layer's backward pass
 * on narrow rows).  CXG_ERR_UNSUPPORTED otherwise: use the two separate calls.
 */
int cxg_spmm_weighted_dot_f32(const int64_t* ptr, const int64_t* idx, const float* val,
                              const int64_t* val_perm, const float* x, int64_t ldx, float* out,
                              int64_t ldo, const float* dot_b, int64_t ld_dot_b, float* dot_out,
                              int64_t n_rows, int64_t n_edges_cap, int heads, int channels,
                              unsigned flags, void* workspace, size_t workspace_bytes,
                              void* stream);

/*
 * Sum aggregation with optional extras, each enabled by a non-NULL pointer:
 *   mask      [E] bytes: edges whose byte is 0 are skipped; the byte of edge
 *             position e is mask[mask_perm ? mask_perm[e] : e];
 *   rel       [E] int32: the gathered row is x[rel[e]*rel_stride + idx[e]];
 *   src_map   the gathered row is x[src_map[...]];
 *   targets   [n_rows]: row r is added with fp32 atomics into out[targets[r]]
 *             (out must be initialised by the caller) instead of stored.
 * Replaces selective_aggr / selective_aggr_bwd (src/cpp/src/aggr.cu:483-514,
 * kernels aggr_kernel.cu:493-555; use CXG_SPMM_ACCUMULATE, and for the backward
 * the transposed CSR with mask_perm = its edge permutation), target_aggr /
 * target_aggr_backward (aggr.cu:450-481, aggr_kernel.cu:557-607; backward =
 * transposed CSR with src_map = targets and CXG_SPMM_ACCUMULATE) and aggr_rel
 * forward (src/cpp/src/rel_spmm.cu:8-70).
 */
int cxg_spmm_ext_f32(const int64_t* ptr, const int64_t* idx, const float* x,
                     int64_t ldx, float* out, int64_t ldo, int64_t n_rows,
                     int64_t n_edges_cap, int feat, unsigned flags,
                     const uint8_t* mask, const int64_t* mask_perm,
                     const int32_t* rel, int64_t rel_stride,
                     const int64_t* src_map, const int64_t* targets,
                     void* workspace, size_t workspace_bytes, void* stream);

/*
 * Transposed aggregation by atomic scatter into the caller's buffer:
 *   gx[idx[e] (+ rel[e]*rel_stride), :] += (val ? val[e] : 1) * g[row(e), :]
 * for unmasked edges of rows [0, n_rows).  Replaces aggr_rel_bwd
 * (src/cpp/src/rel_spmm.cu:72-136) and is the no-preprocessing form of
 * gen_bwd_sum (src/cpp/src/aggr_kernel.cu:220-249).
 */
int cxg_spmm_scatter_atomic_f32(const int64_t* ptr, const int64_t* idx,
                                const int32_t* rel, int64_t rel_stride,
                                const float* val, const uint8_t* mask,
                                const float* g, float* gx, int64_t n_rows,
                                int64_t n_edges_cap, int feat, void* stream);

/* ------------------------------------------------------------------------- */
/* SDDMM and edge softmax                                                      */
/* ------------------------------------------------------------------------- */

/*
 * out[e, h] = sum_c src_feat[idx[e], h, c] * dst_feat[row(e), (h,) c] for every
 * edge position e in [ptr[0], ptr[n_rows]); out is indexed by edge position and
 * has `heads` floats per edge.  dst_has_heads = 0 means dst_feat is
 * [n_dst, channels] (the layout of the reference kernels), 1 means
 * [n_dst, heads, channels].  Replaces run_sddmm_vertex_centric
 * (src/cpp/src/sddmm_host.cu:16-59) and the edge-value gradient of
 * gen_bwd_sum_edge_value[_multi_head]_edge_grad
 * (src/cpp/src/aggr_kernel.cu:321-361,443-491).
 */
int cxg_sddmm_csr_f32(const int64_t* ptr, const int64_t* idx, const float* src_feat,
                      const float* dst_feat, float* out, int64_t n_rows,
                      int64_t n_edges_cap, int heads, int channels,
                      int dst_has_heads, void* stream);

/* Same product over explicit src[e] / dst[e] arrays.  Replaces run_sddmm
 * (src/cpp/src/sddmm_host.cu:4-14, kernel src/cpp/src/sddmm_kernel.cu:3-25). */
int cxg_sddmm_coo_f32(const int64_t* src, const int64_t* dst, const float* src_feat,
                      const float* dst_feat, float* out, int64_t n_edges, int heads,
                      int channels, int dst_has_heads, void* stream);

/*
 * GAT edge attention: out[e,h] = softmax over the edges of row r of
 * leaky_relu(att_dst[r,h] + att_src[idx[e],h], slope); mask[e,h] = (pre-softmax
 * activation > 0).  att_dst is [n_dst, heads], att_src [n_src, heads], out and
 * mask [n_edges, heads]; rows without edges write nothing.  Replaces
 * edge_softmax_fwd (src/cpp/src/edge_softmax.cu:3-42, host :97-132).
 */
int cxg_edge_softmax_fwd_f32(const int64_t* ptr, const int64_t* idx,
                             const float* att_dst, const float* att_src, float* out,
                             uint8_t* mask, int64_t n_dst, int heads, float slope,
                             void* stream);

/*
 * Backward of the above (edge_softmax_bwd, src/cpp/src/edge_softmax.cu:44-95):
 * s = sum_row out*grad; t = out*(grad - s) * (mask ? 1 : slope);
 * g_dst[r,h] = sum_row t when the row has activations of both signs, else 0;
 * t_edge[e,h] = t.  The source gradient g_src[s,h] = sum over the edges leaving
 * s of t is obtained with cxg_narrow_gather_sum_f32 over the transposed CSR
 * (sel = its edge permutation) where the reference uses atomicAdd (:85).
 */
int cxg_edge_softmax_bwd_f32(const int64_t* ptr, const float* out, const uint8_t* mask,
                             const float* grad, float* g_dst, float* t_edge,
                             int64_t n_dst, int heads, float slope, void* stream);

/*
 * The same backward (src/cpp/src/edge_softmax.cu:44-95) when the incoming gradient was
 * written in another edge order: the row of edge k is grad[grad_pos[k]] (grad_pos NULL:
 * grad[k], i.e. cxg_edge_softmax_bwd_f32).  With grad_pos = the inverse of a transposed
 * CSR's edge permutation it consumes what cxg_spmm_weighted_dot_f32 stored with
 * CXG_SPMM_DOT_AT_EDGE: one 16-byte gather per edge here instead of one scattered store
 * per edge there.  out, mask, t_edge and g_dst are in the order of ptr as before.
 */
int cxg_edge_softmax_bwd_at_f32(const int64_t* ptr, const float* out, const uint8_t* mask,
                                const float* grad, const int64_t* grad_pos, float* g_dst,
                                float* t_edge, int64_t n_dst, int heads, float slope, void* stream);

/* out[r, 0..width) = sum_{k in [ptr[r], ptr[r+1])} in[sel ? sel[k] : k, 0..width)
 * for narrow rows (a few floats).  With width 1 and sel = idx this is spmv
 * (src/cpp/src/edge_softmax.cu:216-244). */
int cxg_narrow_gather_sum_f32(const int64_t* ptr, const int64_t* sel, const float* in,
                              float* out, int64_t n_rows, int width, void* stream);

/*
 * The same row sums, edge-parallel: rows[k] (int32) is the row of edge position
 * ptr[0] + k for k in [0, n_edges), n_edges = ptr[n_rows] - ptr[0] (see
 * cxg_csr_row_ids_i32); every lane owns one edge, the values of 64 edges are
 * summed per row with a segmented scan, rows crossing a span of edges are
 * completed by a fix-up kernel (deterministic, no atomics).  width in
 * {1, 2, 4, 8}; `in` and `out` aligned to one item.  Rows without edges give 0.
 * Same reference code as cxg_narrow_gather_sum_f32 (src/cpp/src/edge_softmax.cu:83-95,
 * 216-232); this form keeps every lane busy on power-law graphs.
 */
size_t cxg_segment_gather_sum_workspace_bytes(int64_t n_edges, int width);
int cxg_segment_gather_sum_f32(const int32_t* rows, const int64_t* ptr, const int64_t* sel,
                               const float* in, float* out, int64_t n_rows, int64_t n_edges,
                               int width, void* workspace, size_t workspace_bytes, void* stream);

/* rows[k] = row containing edge position ptr[0] + k, as int32 (n_rows < 2^31). */
int cxg_csr_row_ids_i32(const int64_t* ptr, int64_t n_rows, int64_t n_edges, int32_t* rows,
                        void* stream);

/* ------------------------------------------------------------------------- */
/* Typed (relation-segmented) GEMM -- the MFMA path                            */
/* ------------------------------------------------------------------------- */

#define CXG_GEMM_ACCUMULATE 1u /* C += A W instead of C = A W (read-add-store: every destination row at most once per call) */
#define CXG_GEMM_ATOMIC 2u     /* add with fp32 atomics (several rows share a dst) */
#define CXG_GEMM_SPLIT_BF16X6 4u /* fp32 products as 6 bf16 partial products (fp32-accurate) */
#define CXG_GEMM_SPLIT_BF16X3 8u /* fp32 products as 3 bf16 partial products (2^-16 / product) */
#define CXG_GEMM_SPLIT_F16X3 16u /* fp32 products as 3 fp16 partial products of row- / column-scaled operands (2^-21 / product) */
#define CXG_GEMM_ROUND_BF16 32u /* fp32 operands rounded to bf16 as they are staged, one bf16 MFMA product, fp32 accumulation */
#define CXG_GEMM_OUT_BF16 64u  /* the rows of C are bf16 (ldc in elements; `c` points to them): bf16-operand forms with K <= 128, even N and ldc, plain stores */

/*
 * C[dst(i), :] = A[src(i), :] @ W[r] for the rows i in [seg_ptr[r], seg_ptr[r+1]),
 * r in [0, R); src(i) = src_idx ? src_idx[i] : i, dst(i) = dst_idx ? dst_idx[i] : i;
 * a negative src or dst skips the row.  A is [*, K] (row stride lda), W is
 * [R, K, N], C is [*, N] (row stride ldc), all fp32; seg_ptr is a device array of
 * R+1 row offsets (see cxg_rel_segment_*).  Computed with
 * v_mfma_f32_32x32x2_f32; with CXG_GEMM_SPLIT_BF16X6 or _X3 (and K <= 128, K and
 * lda multiples of 4, A 16-byte aligned) every operand is split into three (two)
 * bf16 parts and a*b is accumulated in fp32 on v_mfma_f32_32x32x16_bf16 from the
 * six (three) partial products whose magnitude is above 2^-24 (2^-16) of |ab|:
 * X6 is as accurate as an fp32 FMA chain, X3 is off by at most 2^-16 per product
 * (the reference's tl.dot runs in TF32, 2^-11); both are HBM bound instead of
 * matrix-core bound.  With CXG_GEMM_SPLIT_F16X3 (same shape conditions) every row of
 * A and every column of W is scaled by a power of two that brings its largest
 * magnitude into [2^14, 2^15) and split into two fp16 parts (22 significant bits);
 * a*b is accumulated on v_mfma_f32_32x32x16_f16 from three partial products and the
 * scales are undone when the row is stored: 2^-21 per product, half the matrix
 * instructions and two thirds of the LDS traffic of X6; this form also takes
 * 176 <= K <= 256 when N >= 96.  C (and the addend of the epilogue entry point) is
 * written and re-read in 16-byte pieces when c, w and the addend are 16-byte aligned
 * and ldc (ldd) is a multiple of 4, element by element otherwise.  Rows or columns whose largest
 * magnitude is below 2^-112 count as zero; a row holding an infinity or NaN comes out
 * non-finite.  With CXG_GEMM_ROUND_BF16 (K <= 128, K and lda multiples of 8) the fp32
 * operands are rounded to bf16 (nearest even) on their way into the LDS and the
 * registers and multiplied with one bf16 MFMA per k-step: bit for bit the result of
 * cxg_typed_gemm_bf16 on operands rounded beforehand, without the conversion passes.
 * Other shapes ignore these flags.  Replaces
 * typed_matmul
 * (cxgnncomp/codegen/triton_typed_matmul.py:752-860: src_idx only = its
 * "single index" kernel with dst = src, seq_output = dst NULL, both = double
 * index) and, with row maps and CXG_GEMM_ACCUMULATE / CXG_GEMM_ATOMIC, the
 * per-row kernels typed_linear / typed_linear_s2e / typed_linear_s2d
 * (src/cpp/src/rel_spmm.cu:231-358).
 */
int cxg_typed_gemm_f32(const float* a, int64_t lda, const float* w, float* c,
                       int64_t ldc, const int64_t* src_idx, const int64_t* dst_idx,
                       const int64_t* seg_ptr, int64_t M, int K, int N, int R,
                       unsigned flags, void* stream);

/*
 * cxg_typed_gemm_f32 with an epilogue: C[dst(i), :] = A[src(i), :] @ W[r] + bias[r, :] +
 * addend[dst(i), :] (bias [R, N] and addend [*, N] with row stride ldd; either may be
 * NULL), added to the accumulator before the row is stored, so neither costs a pass over
 * C.  Taken by the fp16 split form only (CXG_GEMM_SPLIT_F16X3 and its shapes, no row maps;
 * otherwise CXG_ERR_UNSUPPORTED), not with CXG_GEMM_ACCUMULATE or CXG_GEMM_ATOMIC (the
 * addend may be C itself: a row is read before it is written).  With R = 1 and seg_ptr =
 * {0, M} this is F.linear(x, W^T, bias) (+ addend), which is what the layers of the
 * reference's models call (cxgnncomp/graph_conv.py:132-178 lin_l / lin_r / linear).
 */
int cxg_typed_gemm_epilogue_f32(const float* a, int64_t lda, const float* w, const float* bias,
                                const float* addend, int64_t ldd, float* c, int64_t ldc,
                                const int64_t* src_idx, const int64_t* dst_idx,
                                const int64_t* seg_ptr, int64_t M, int K, int N, int R,
                                unsigned flags, void* stream);

/* Same contraction with bf16 operands on v_mfma_f32_32x32x16_bf16: A is bf16
 * [*, K], w_t is the transposed weight stack W^T as bf16 [R, N, K]; C stays fp32.
 * K and lda must be multiples of 8. */
int cxg_typed_gemm_bf16(const uint16_t* a, int64_t lda, const uint16_t* w_t, float* c,
                        int64_t ldc, const int64_t* src_idx, const int64_t* dst_idx,
                        const int64_t* seg_ptr, int64_t M, int K, int N, int R,
                        unsigned flags, void* stream);

/*
 * The same contraction for wide operands (K >= 160, any N; K and lda multiples of 4, A
 * 16-byte aligned; otherwise CXG_ERR_UNSUPPORTED): a tiled GEMM -- block tile 128 rows x 256
 * columns, K walked in chunks of 32 with both operand tiles in LDS -- in the
 * CXG_GEMM_SPLIT_F16X3 arithmetic (three fp16 partial products of power-of-two-scaled
 * operands, 2^-21 per product, fp32 accumulation; the flag may be passed or left out).  W is
 * split once per call into the workspace (its two fp16 parts per relation, column tile and
 * k-chunk, and the columns' inverse scales).  A row's scale follows the largest magnitude
 * met so far along K with three bits of headroom; when a later value outgrows it the sums so
 * far are multiplied by the power-of-two ratio, so the result does not depend on where along
 * K the large values sit.  flags: CXG_GEMM_ACCUMULATE, CXG_GEMM_ATOMIC as above.  This is
 * the shape class the reference benchmarks its typed_matmul on
 * (cxgnncomp/codegen/triton_typed_matmul.py:752-860 with K = N = 512,
 * test/ae/E3_ablation/test-batch.py:27-52).
 */
size_t cxg_typed_gemm_wide_workspace_bytes(int K, int N, int R);
int cxg_typed_gemm_wide_f32(const float* a, int64_t lda, const float* w, float* c, int64_t ldc,
                            const int64_t* src_idx, const int64_t* dst_idx, const int64_t* seg_ptr,
                            int64_t M, int K, int N, int R, unsigned flags, void* workspace,
                            size_t workspace_bytes, void* stream);

/*
 * Weight gradient of the typed GEMM: gw[r] (K x N, fp32, overwritten) = sum over
 * the rows i of segment r of A[src(i), :]^T (x) G[dst(i), :]; relations without
 * rows give zeros.  A is [*, K] (row stride lda), G is [*, N] (row stride ldg);
 * src / dst / seg_ptr as in cxg_typed_gemm_f32.  fp32 operands multiplied as six
 * (CXG_GEMM_SPLIT_BF16X6 or no flag) or three (CXG_GEMM_SPLIT_BF16X3) bf16 partial
 * products on v_mfma_f32_32x32x16_bf16, or (CXG_GEMM_SPLIT_F16X3) as three fp16
 * partial products of operands scaled by a power of two per group of 32 columns and
 * row chunk (the scale follows the largest magnitude met so far in the chunk; an
 * element keeps 22 significant bits down to 2^-17 of that magnitude); partial sums
 * over row chunks are added in
 * chunk order by a second kernel (deterministic).  A block computes one 128 x 128
 * tile of gw over one row chunk, and the tiles of a chunk run side by side on one die
 * so that its rows of A and G come from memory once.  Needs K <= 4096, K, N, lda, ldg
 * multiples of 4 and 16-byte aligned operands (otherwise CXG_ERR_UNSUPPORTED).
 * Replaces the per-relation torch.mm of TypedLinearE2EOP.backward and
 * TypedLinearS2DMMAggrOP.backward (cxgnncomp/typed_linear.py:114-137,205-221).
 */
#define CXG_WGRAD_A_BF16 128u   /* the rows of A are bf16 (`a` points to them, lda in elements, 8-byte aligned rows) */
size_t cxg_typed_gemm_wgrad_workspace_bytes(int64_t M, int K, int N, int R);
int cxg_typed_gemm_wgrad_f32(const float* a, int64_t lda, const float* g, int64_t ldg,
                             const int64_t* src_idx, const int64_t* dst_idx,
                             const int64_t* seg_ptr, int64_t M, int K, int N, int R, float* gw,
                             unsigned flags, void* workspace, size_t workspace_bytes,
                             void* stream);

/*
 * Relation segmentation: perm[k] = original row of the k-th row in relation
 * order (stable), seg_ptr[r] = number of rows with relation id < r for r in
 * [0, num_rel].  Ids equal to num_rel (the padding sentinel of pad_rel) sort
 * last and are not covered by any segment.  Replaces the bincount + sort of
 * TypedLinearE2EOP.preprocess / TypedLinearS2DSort
 * (cxgnncomp/typed_linear.py:74-87,262-283).  index_bytes is 4 or 8.
 */
size_t cxg_rel_segment_workspace_bytes(int64_t n, int num_rel, int index_bytes);
int cxg_rel_segment_i64(const int64_t* types, int64_t n, int num_rel, int64_t* perm,
                        int64_t* seg_ptr, void* workspace, size_t workspace_bytes,
                        void* stream);
int cxg_rel_segment_i32(const int32_t* types, int64_t n, int num_rel, int64_t* perm,
                        int64_t* seg_ptr, void* workspace, size_t workspace_bytes,
                        void* stream);

/* ------------------------------------------------------------------------- */
/* Row helpers                                                                 */
/* ------------------------------------------------------------------------- */

/* out[dest[e], :] += in[e, :] for e < n_edges (fp32 hardware atomics; the caller
 * zeroes out).  Replaces gather_fwd (src/cpp/src/aggr.cu:42-51, host :395-421). */
int cxg_scatter_add_rows_f32(const float* in, const int64_t* dest, float* out,
                             int64_t n_edges, int feat, void* stream);

/* out[e, :] = in[sel[e], :] for e < n_rows_out.  Replaces gather_bwd
 * (src/cpp/src/aggr.cu:53-62, host :423-443). */
int cxg_gather_rows_f32(const float* in, const int64_t* sel, float* out,
                        int64_t n_rows_out, int feat, void* stream);

/* out[n, c] = sum_h in[n, h, c]: the head reduction of the PreReduce / Optimal
 * schedules of spmm_multihead (src/cpp/src/spmm_multihead_kernel.cu:3-36). */
int cxg_head_sum_f32(const float* in, float* out, int64_t n_rows, int heads,
                     int channels, void* stream);

/* Per-node attention logits of a multi-head GAT layer, both in one pass over x:
 *   out_src[n, h] = sum_c x[n, h, c] * att_src[h, c]   for n < n_src
 *   out_dst[n, h] = sum_c x[n, h, c] * att_dst[h, c]   for n < n_dst (<= n_src)
 * x is [n_src, heads, channels], att_* are [heads, channels].  Replaces the two
 * broadcast-multiply-and-sum expressions of MyGATConv.forward_many
 * (cxgnncomp/graph_conv.py:466-467). */
int cxg_attention_logits_fwd_f32(const float* x, const float* att_src, const float* att_dst,
                                 int64_t n_src, int64_t n_dst, int heads, int channels,
                                 float* out_src, float* out_dst, void* stream);

size_t cxg_attention_logits_workspace_bytes(int64_t n_src, int heads, int channels);

/* Gradients of the logits above for g_src [n_src, heads], g_dst [n_dst, heads]:
 *   grad_x[n, h, c]    = g_src[n, h] * att_src[h, c] + (n < n_dst) g_dst[n, h] * att_dst[h, c]
 *   grad_att_src[h, c] = sum_n g_src[n, h] * x[n, h, c]
 *   grad_att_dst[h, c] = sum_{n < n_dst} g_dst[n, h] * x[n, h, c]
 * grad_att_* are overwritten; grad_x is overwritten, or, with accumulate != 0, added to
 * (the layer's other gradient of x, from the aggregation, is already there: autograd's
 * sum of the two).  The sums run in a fixed order (reproducible).
 * The autograd of the same two expressions (cxgnncomp/graph_conv.py:466-467). */
int cxg_attention_logits_bwd_f32(const float* x, const float* att_src, const float* att_dst,
                                 const float* g_src, const float* g_dst, int64_t n_src,
                                 int64_t n_dst, int heads, int channels, float* grad_x,
                                 int accumulate, float* grad_att_src, float* grad_att_dst,
                                 void* workspace, size_t workspace_bytes, void* stream);

/* The same logits and gradients taken from the layer's input.  With xs = x_in W^T
 * (W [heads*channels, in]) both logits are linear in x_in:
 *   out_src[n, h] = x_in[n, :] . m[h, :],          m[h, :]         = sum_c att_src[h, c] W[h*channels + c, :]
 *   out_dst[n, h] = x_in[n, :] . m[heads + h, :],  m[heads + h, :] = sum_c att_dst[h, c] W[h*channels + c, :]
 * the contraction order upstream's single-head path uses (einsum "mn,nho,ho->mh",
 * cxgnncomp/graph_conv.py:500-511); the several-head path computes the same numbers from
 * xs (cxgnncomp/graph_conv.py:466-467), results agree to fp32 rounding.  The caller forms
 * m [2*heads, in] (a tiny product).  x_in is [n_src, in] with row stride ldx (floats).
 * Shapes: 4 | in <= 256, heads 1, 2, 4 or 8 (cxg_attention_logits_proj_supported);
 * x_in, m, grad_x 16-byte aligned, strides multiples of 4; g_src / g_dst 16-byte aligned
 * when heads is a multiple of 4.
 * Backward, for g_src [n_src, heads], g_dst [n_dst, heads]:
 *   grad_x[n, :]  (+)= sum_h g_src[n, h] m[h, :] + (n < n_dst) g_dst[n, h] m[heads + h, :]
 *                     (grad_x NULL: skipped; accumulate != 0: added to what is there, the
 *                     other gradient of x_in, from the linear map)
 *   grad_m[h, :]         = sum_n g_src[n, h] x_in[n, :]
 *   grad_m[heads + h, :] = sum_{n < n_dst} g_dst[n, h] x_in[n, :]
 * from which the caller takes the logits' share of grad_att_* and grad_W by the chain rule
 * through m.  Sums in a fixed order (reproducible). */
int cxg_attention_logits_proj_supported(int in, int heads);
int cxg_attention_logits_proj_fwd_f32(const float* x, int64_t ldx, const float* m, int64_t n_src,
                                      int64_t n_dst, int in, int heads, float* out_src,
                                      float* out_dst, void* stream);
size_t cxg_attention_logits_proj_workspace_bytes(int in, int heads);
int cxg_attention_logits_proj_bwd_f32(const float* x, int64_t ldx, const float* m,
                                      const float* g_src, const float* g_dst, int64_t n_src,
                                      int64_t n_dst, int in, int heads, float* grad_x, int64_t ldg,
                                      int accumulate, float* grad_m, void* workspace,
                                      size_t workspace_bytes, void* stream);

/* Batch normalisation over the rows of x[n, c] (row stride ldx), the layer the upstream
 * models put between two convolutions (torch.nn.BatchNorm1d, cxgnncomp/model.py:28 and
 * its use followed by F.relu in GNN.forward_cxg, cxgnncomp/model.py:66-67).  Three calls:
 *   stats : mean[c], invstd[c] = 1/sqrt(biased variance + eps), var_unbiased[c] (may be
 *           NULL; the value the running variance is updated with); needs n >= 1;
 *   apply : y = (x - mean) * invstd * gamma + beta, then max(., 0) when relu != 0
 *           (gamma / beta may be NULL: 1 / 0); also serves evaluation mode with the
 *           running statistics;
 *   bwd   : dbeta[c] = sum dy, dgamma[c] = sum dy * xhat, dx = gamma * invstd *
 *           (dy - dbeta/n - xhat * dgamma/n); with relu != 0, dy counts only where the
 *           forward output was positive (recomputed from x, gamma, beta).
 * workspace: cxg_batchnorm_workspace_bytes(n, c) bytes of device memory (per-block
 * partial statistics).  Results do not depend on the run (fixed merge order). */
size_t cxg_batchnorm_workspace_bytes(int64_t n, int c);
int cxg_batchnorm_stats_f32(const float* x, int64_t n, int c, int64_t ldx, float eps, float* mean,
                            float* invstd, float* var_unbiased, void* workspace,
                            size_t workspace_bytes, void* stream);
int cxg_batchnorm_apply_f32(const float* x, int64_t n, int c, int64_t ldx, const float* mean,
                            const float* invstd, const float* gamma, const float* beta, float* y,
                            int64_t ldy, int relu, void* stream);
int cxg_batchnorm_bwd_f32(const float* x, const float* dy, int64_t n, int c, int64_t ldx,
                          int64_t lddy, const float* mean, const float* invstd, const float* gamma,
                          const float* beta, int relu, float* dx, int64_t lddx, float* dgamma,
                          float* dbeta, void* workspace, size_t workspace_bytes, void* stream);

/* out[c] = sum over the n rows of x[n, c] (row stride ldx): the bias gradient of the
 * layers' linear maps (autograd's g.sum(0) for lin_l.bias of MySageConv,
 * cxgnncomp/graph_conv.py:130 and :142-152, and the bias of MyGCNConv, :622-623).  workspace:
 * cxg_batchnorm_workspace_bytes(n, c) bytes.  Fixed summation order. */
int cxg_column_sum_f32(const float* x, int64_t n, int c, int64_t ldx, float* out, void* workspace,
                       size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------- */
/* Index work (bit-exact)                                                     */
/* ------------------------------------------------------------------------- */

/*
 * Transposed CSR of a CSR-by-destination graph with ptr[0] == 0 and
 * n_edges == ptr[n_rows]:  ptr_t[n_cols+1], idx_t[n_edges] = destination row of
 * each edge, perm[n_edges] = position of that edge in the original idx array.
 * Edges of one source keep their original order (stable), so the transposed
 * gather adds contributions in a fixed order.  This is the graph the backward
 * pass runs cxg_spmm_* over; the reference reaches the same sums by atomic
 * scatter (run_spmm_configurable_bwd, src/cpp/src/spmm_host.cu:57-97;
 * gen_bwd_sum, src/cpp/src/aggr_kernel.cu:220-249).
 */
size_t cxg_csr_transpose_workspace_bytes(int64_t n_edges, int64_t n_cols);
int cxg_csr_transpose_i64(const int64_t* ptr, const int64_t* idx, int64_t n_rows,
                          int64_t n_cols, int64_t n_edges, int64_t* ptr_t,
                          int64_t* idx_t, int64_t* perm, void* workspace,
                          size_t workspace_bytes, void* stream);

/*
 * Transposed CSR of the edge prefix [0, edge_limit) of a graph whose whole transposition
 * (ptr_t_all, idx_t_all, perm_all over n_edges_all edges, from cxg_csr_transpose_i64) is at
 * hand: the result equals cxg_csr_transpose_i64 of the first rows of that graph, the rows
 * that own exactly those edges, bit for bit (one scan and one scatter instead of a sort).
 * The layers of a sampled mini-batch aggregate over nested prefixes of one CSR
 * (cxgnncomp/model.py:55-71); their backward passes need the transposed graph of every
 * prefix.  n_cols: sources of the prefix graph (all its edges must have a source below
 * n_cols, and ptr_t_all must hold at least n_cols + 1 entries); ptr_t gets n_cols + 1
 * entries, idx_t and perm edge_limit entries.
 */
size_t cxg_csr_transpose_prefix_workspace_bytes(int64_t n_edges_all);
int cxg_csr_transpose_prefix_i64(const int64_t* ptr_t_all, const int64_t* idx_t_all,
                                 const int64_t* perm_all, int64_t n_edges_all, int64_t edge_limit,
                                 int64_t n_cols, int64_t* ptr_t, int64_t* idx_t, int64_t* perm,
                                 void* workspace, size_t workspace_bytes, void* stream);

/* rows[k] = row that owns edge position ptr[0] + k, k in [0, n_edges): the
 * device form of `repeat_interleave(arange(n), deg)` used by
 * SpMMValOP.backward (cxgnncomp/graph_kernel.py:31-34). */
int cxg_csr_row_ids_i64(const int64_t* ptr, int64_t n_rows, int64_t n_edges,
                        int64_t* rows, void* stream);

/* out[e] = 1 / degree(row of e) for every edge of rows [0, n_rows).  Replaces
 * edge_value_degree (src/cpp/src/edge_softmax.cu:186-214). */
int cxg_edge_value_degree_f32(const int64_t* ptr, int64_t n_rows, float* out,
                              void* stream);

/*
 * Relation padding.  For t in [0, num_rel*(thres-1)): r = t/(thres-1),
 * m = count[r] % thres; rel[base+t] = (m != 0 && t%(thres-1) < thres-m) ? r
 * : num_rel; if idx is not NULL, idx[base+t] = -1.  Replaces pad_rel and
 * pad_rel_idx (src/cpp/src/stitch_kernel.cu:3-53).
 */
int cxg_pad_rel_i64(int64_t* rel, int64_t* idx, const int64_t* count, int thres,
                    int num_rel, int64_t base, void* stream);

/*
 * Generalised CSR SpMM with int32 indices:
 *   out[r, c] = REDUCE_{e in row r} COMPUTE(val[e], b[colind[e], c]),  out [n_rows, feat].
 * reduce_op: 0 sum, 1 max, 2 min, 3 mean; compute_op: 0 val+b, 1 b-val, 2 val*b,
 * 3 b/val (the enum values of src/cpp/include/dgsparse.h:13-14); val == NULL: the
 * operand is b itself and compute_op is ignored.  A non-empty row's accumulator
 * starts at 0 / (float)INT_MIN / (float)INT_MAX / 0, empty rows give 0, mean
 * divides by the row length.  n_edges is the length of colind (at least
 * rowptr[n_rows]); workspace holds cxg_gspmm_workspace_bytes(n_edges, feat) bytes:
 * rows of more than 512 edges are cut at the multiples of 512 in the edge array,
 * one wave per piece leaves a partial row there, and the row's own wave folds
 * them in edge order (results do not depend on the schedule).  Replaces
 * GSpMM_u / GSpMM_u_e (src/cpp/python_bindings/binding.cpp:87-107,
 * src/cpp/src/dgsparse.cu:444-474).
 */
size_t cxg_gspmm_workspace_bytes(int64_t n_edges, int feat);
int cxg_gspmm_i32_f32(const int32_t* rowptr, const int32_t* colind, const float* val,
                      const float* b, float* out, int64_t n_rows, int64_t n_edges, int feat,
                      int reduce_op, int compute_op, void* workspace, size_t workspace_bytes,
                      void* stream);

/* ------------------------------------------------------------------------- */
/* Scheduling helpers as device index work (bit-exact)                          */
/* ------------------------------------------------------------------------- */
/* Output sizes depend on the data: a "plan" call leaves exclusive-scan offsets
 * on the device (n+1 entries; the last one is the output size, which the caller
 * copies back to allocate the outputs), a "fill" call writes the outputs.      */

/* Scratch bytes for the plan calls on arrays of up to n elements. */
size_t cxg_scan_workspace_bytes(int64_t n);

/*
 * Neighbor grouping (degree bucketing): every row is cut into consecutive chunks
 * of `thres` edges, the last chunk holds the remainder, an empty row gives one
 * empty chunk.  plan: group_off[r] = number of chunks of rows < r (n_rows+1
 * entries).  fill: new_ptr[n_groups+1] (new_ptr[0] = 0, then the chunk ends as
 * positions in idx) and new_target[g] = row of chunk g.  Replaces
 * neighbor_grouping / neighbor_grouping_gpu (cxgnncomp/schedule.py:6-35).
 */
int cxg_neighbor_group_plan_i64(const int64_t* ptr, int64_t n_rows, int64_t thres,
                                int64_t* group_off, void* workspace, size_t workspace_bytes,
                                void* stream);
int cxg_neighbor_group_fill_i64(const int64_t* ptr, const int64_t* group_off, int64_t n_rows,
                                int64_t thres, int64_t n_groups, int64_t* new_ptr,
                                int64_t* new_target, void* stream);

/*
 * Row filter: keep the rows r with remove_flag[r] == 0, edges unchanged.
 * plan: row_off / edge_off = kept rows / kept edges before row r (n_rows+1
 * entries each).  fill: new_ptr[row_off[n_rows]+1], new_idx[edge_off[n_rows]].
 * Replaces remove_from_graph (cxgnncomp/schedule.py:106-121).
 */
int cxg_filter_rows_plan_i64(const int64_t* ptr, int64_t n_rows, const uint8_t* remove_flag,
                             int64_t* row_off, int64_t* edge_off, void* workspace,
                             size_t workspace_bytes, void* stream);
int cxg_filter_rows_fill_i64(const int64_t* ptr, const int64_t* idx, int64_t n_rows,
                             const int64_t* row_off, const int64_t* edge_off,
                             int64_t n_edges_out, int64_t* new_ptr, int64_t* new_idx,
                             void* stream);

/*
 * Edge filter: keep edge e if rel ? rel[e] == keep_rel : !remove_flag[e], then
 * drop the rows left without edges; edge order is preserved.  ptr[0] must be 0
 * and ptr[n_rows] == n_edges.  plan: edge_pos (n_edges+1) = kept edges before e,
 * row_off (n_rows+1) = kept rows before r.  fill: new_ptr[row_off[n_rows]+1],
 * new_idx[edge_pos[n_edges]] and, if not NULL, new_target[k] = original id of
 * kept row k.  Replaces remove_from_graph_by_edge (cxgnncomp/schedule.py:124-144)
 * and, called once per relation with rel/keep_rel, the per-relation sub-graphs
 * (ptr_r, idx_r, target_r) of rel_schedule (src/cpp/src/schedule.cu:5-63); the
 * cumulative row counts of its layer table are entries of row_off.
 */
int cxg_filter_edges_plan_i64(const int64_t* ptr, int64_t n_rows, int64_t n_edges,
                              const uint8_t* remove_flag, const int32_t* rel, int32_t keep_rel,
                              int64_t* edge_pos, int64_t* row_off, void* workspace,
                              size_t workspace_bytes, void* stream);
int cxg_filter_edges_fill_i64(const int64_t* ptr, const int64_t* idx, int64_t n_rows,
                              int64_t n_edges, const int64_t* edge_pos, const int64_t* row_off,
                              int64_t* new_ptr, int64_t* new_idx, int64_t* new_target,
                              void* stream);

/*
 * COO -> CSR by destination: edges sorted by dst (stable: edges of one
 * destination keep their input order), ptr[n_rows+1], idx = src in that order,
 * perm[k] = input position of the k-th CSR edge.  The relation the reference
 * builds in cxgnncomp/data_preparation.py:97-104.
 */
size_t cxg_coo_to_csr_workspace_bytes(int64_t n_edges, int64_t n_rows);
int cxg_coo_to_csr_i64(const int64_t* src, const int64_t* dst, int64_t n_edges, int64_t n_rows,
                       int64_t* ptr, int64_t* idx, int64_t* perm, void* workspace,
                       size_t workspace_bytes, void* stream);

/*
 * Host-side (CPU memory, sequential) topological order of a graph given as CSR
 * successor lists: FIFO queue seeded with the nodes whose `degree` counter is 0
 * in id order; when the queue runs dry early, every node with counter 1 and the
 * first node holding the running minimum counter above 1 are released.  Writes
 * the emitted node ids to order[0..ret) and returns their number (< n_nodes for
 * inputs the release rule cannot finish), or a negative status.  Replaces
 * topo_sort (src/cpp/src/schedule.cu:71-128).
 */
int64_t cxg_topo_sort_host_i64(const int64_t* ptr, const int64_t* idx, const int64_t* degree,
                               int64_t n_nodes, int64_t* order);

#ifdef __cplusplus
}
#endif
#endif /* CXGNN_HIP_H */
