/*
 * cxg_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Plain-C, single-threaded CPU restatement of the graph kernels of
 * xxcclong/CxGNN-Compute.  It exists only so that tests, the smoke check and
 * the CPU-baseline leg of the benchmark can compare the HIP kernels against an
 * independent implementation of the same mathematics.  Nothing in the shipped
 * package may call into this file.
 *
 * Each function names the reference code it restates (paths relative to the
 * reference checkout).  Sums are accumulated in double and rounded to float
 * once unless `seq32` asks for the reference's own order (float accumulator,
 * edges in CSR order), so the oracle is the mathematically intended value of
 * each kernel rather than one particular rounding of it.
 *
 * Index type is int64_t everywhere (`using Index = int64_t`,
 * src/cpp/include/common.h:15); relation ids are int32 where the reference
 * reads them with data<int>() (src/cpp/src/rel_spmm.cu:60).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef int64_t Index;

/* ------------------------------------------------------------------------- */
/* SpMM: gen_fwd_sum / gen_fwd_mean / gen_fwd_sum_edge_value[_multi_head]      */
/* src/cpp/src/aggr_kernel.cu:3-53, 88-116, 155-186;                           */
/* run_spmm_sharedmem* src/cpp/src/spmm_kernel.cu:231-512                      */
/*   out[r,h,c] = sum_{e in [ptr[r],ptr[r+1])} val[e,h] * x[idx[e],h,c]        */
/*   val == NULL -> weights 1; mean -> divide by degree, empty rows stay 0     */
/*   (aggr_kernel.cu:26-27).                                                   */
/* ------------------------------------------------------------------------- */
void orc_spmm(const Index* ptr, const Index* idx, const float* val, const float* x, float* out,
              Index n_rows, int heads, int channels, int mean, int seq32) {
  const int F = heads * channels;
  double* acc = (double*)malloc(sizeof(double) * (size_t)F);
  float* accf = (float*)malloc(sizeof(float) * (size_t)F);
  for (Index r = 0; r < n_rows; ++r) {
    for (int c = 0; c < F; ++c) { acc[c] = 0.0; accf[c] = 0.f; }
    const Index b = ptr[r], e = ptr[r + 1];
    for (Index k = b; k < e; ++k) {
      const float* row = x + (size_t)idx[k] * F;
      for (int h = 0; h < heads; ++h) {
        const float w = val ? val[(size_t)k * heads + h] : 1.0f;
        for (int c = 0; c < channels; ++c) {
          const int cc = h * channels + c;
          if (seq32) accf[cc] += row[cc] * w;
          else acc[cc] += (double)row[cc] * (double)w;
        }
      }
    }
    const Index deg = e - b;
    for (int c = 0; c < F; ++c) {
      double v = seq32 ? (double)accf[c] : acc[c];
      if (mean && deg > 0) v = seq32 ? (double)(accf[c] / (float)deg) : v / (double)deg;
      out[(size_t)r * F + c] = (float)v;
    }
  }
  free(acc);
  free(accf);
}

/* ------------------------------------------------------------------------- */
/* Transposed SpMM (input gradient): gen_bwd_sum / gen_bwd_mean /              */
/* gen_bwd_sum_edge_value[_multi_head] src/cpp/src/aggr_kernel.cu:188-319,     */
/* 403-441; run_spmm_sharedmem_bwd src/cpp/src/spmm_kernel.cu:799-851.         */
/*   gx[idx[e],h,c] += val[e,h] * g[r,h,c]   (mean: g[r]/deg(r))               */
/* gx has n_src rows and is zeroed here (the reference allocates zeros_like).  */
/* Accumulation is done in a double shadow buffer.                             */
/* ------------------------------------------------------------------------- */
void orc_spmm_bwd(const Index* ptr, const Index* idx, const float* val, const float* g, float* gx,
                  Index n_rows, Index n_src, int heads, int channels, int mean) {
  const int F = heads * channels;
  double* acc = (double*)calloc((size_t)n_src * F, sizeof(double));
  for (Index r = 0; r < n_rows; ++r) {
    const Index b = ptr[r], e = ptr[r + 1];
    const double scale = (mean && e > b) ? 1.0 / (double)(e - b) : 1.0;
    for (Index k = b; k < e; ++k) {
      double* dst = acc + (size_t)idx[k] * F;
      for (int h = 0; h < heads; ++h) {
        const double w = (val ? (double)val[(size_t)k * heads + h] : 1.0) * scale;
        for (int c = 0; c < channels; ++c)
          dst[h * channels + c] += w * (double)g[(size_t)r * F + h * channels + c];
      }
    }
  }
  for (size_t i = 0; i < (size_t)n_src * F; ++i) gx[i] = (float)acc[i];
  free(acc);
}

/* ------------------------------------------------------------------------- */
/* Edge-value gradient fused in gen_bwd_sum_edge_value[_multi_head]_edge_grad  */
/* src/cpp/src/aggr_kernel.cu:321-361, 443-491:                                */
/*   gval[e,h] = sum_c g[row(e),h,c] * x[idx[e],h,c]                           */
/* ------------------------------------------------------------------------- */
void orc_edge_grad(const Index* ptr, const Index* idx, const float* x, const float* g, float* gval,
                   Index n_rows, int heads, int channels) {
  const int F = heads * channels;
  for (Index r = 0; r < n_rows; ++r) {
    for (Index k = ptr[r]; k < ptr[r + 1]; ++k) {
      for (int h = 0; h < heads; ++h) {
        double s = 0.0;
        for (int c = 0; c < channels; ++c)
          s += (double)g[(size_t)r * F + h * channels + c] *
               (double)x[(size_t)idx[k] * F + h * channels + c];
        gval[(size_t)k * heads + h] = (float)s;
      }
    }
  }
}

/* ------------------------------------------------------------------------- */
/* Head-pre-reduced SpMM: spmm_multihead_pre_reduce                            */
/* src/cpp/src/spmm_multihead_kernel.cu:3-36                                   */
/*   out[r,c] = sum_h sum_e val[e,h] * x[idx[e],h,c]                           */
/* ------------------------------------------------------------------------- */
void orc_spmm_prereduce(const Index* ptr, const Index* idx, const float* val, const float* x,
                        float* out, Index n_rows, int heads, int channels) {
  double* acc = (double*)malloc(sizeof(double) * (size_t)channels);
  for (Index r = 0; r < n_rows; ++r) {
    for (int c = 0; c < channels; ++c) acc[c] = 0.0;
    for (Index k = ptr[r]; k < ptr[r + 1]; ++k)
      for (int h = 0; h < heads; ++h) {
        const double w = val[(size_t)k * heads + h];
        const float* row = x + ((size_t)idx[k] * heads + h) * channels;
        for (int c = 0; c < channels; ++c) acc[c] += w * (double)row[c];
      }
    for (int c = 0; c < channels; ++c) out[(size_t)r * channels + c] = (float)acc[c];
  }
  free(acc);
}

/* ------------------------------------------------------------------------- */
/* SDDMM, edge parallel: sddmm_multihead src/cpp/src/sddmm_kernel.cu:3-25      */
/*   out[e,h] = sum_i src_feat[src[e],h,i] * dst_feat[dst[e],(h,)i]            */
/* dst_has_heads == 0 is the reference's layout (dst operand [Nd, F], :17);    */
/* dst_has_heads == 1 is the per-head form its caller SpMMValOP.backward       */
/* (cxgnncomp/graph_kernel.py:35) mathematically needs.                        */
/* ------------------------------------------------------------------------- */
void orc_sddmm(const Index* src, const Index* dst, const float* src_feat, const float* dst_feat,
               float* out, Index n_edges, int heads, int feat, int dst_has_heads) {
  for (Index e = 0; e < n_edges; ++e)
    for (int h = 0; h < heads; ++h) {
      const float* a = src_feat + ((size_t)src[e] * heads + h) * feat;
      const float* b = dst_has_heads ? dst_feat + ((size_t)dst[e] * heads + h) * feat
                                     : dst_feat + (size_t)dst[e] * feat;
      double s = 0.0;
      for (int i = 0; i < feat; ++i) s += (double)a[i] * (double)b[i];
      out[(size_t)e * heads + h] = (float)s;
    }
}

/* ------------------------------------------------------------------------- */
/* Edge softmax forward: edge_softmax_fwd src/cpp/src/edge_softmax.cu:3-42     */
/*   t = leaky_relu(att_dst[r,h] + att_src[idx[e],h]); mask = t > 0;           */
/*   out = exp(t - max_row) / sum_row; running max starts at -100000.f (:15);  */
/*   no epsilon in the denominator.  Empty rows write nothing.                 */
/* ------------------------------------------------------------------------- */
void orc_edge_softmax_fwd(const Index* ptr, const Index* idx, const float* att_dst,
                          const float* att_src, float* out, uint8_t* mask, Index n_dst, int heads,
                          float slope) {
  for (Index r = 0; r < n_dst; ++r)
    for (int h = 0; h < heads; ++h) {
      const float d = att_dst[(size_t)r * heads + h];
      float mx = -100000.f;
      for (Index k = ptr[r]; k < ptr[r + 1]; ++k) {
        float t = d + att_src[(size_t)idx[k] * heads + h];
        t = fmaxf(t, t * slope);
        out[(size_t)k * heads + h] = t;
        mask[(size_t)k * heads + h] = t > 0.f;
        mx = fmaxf(mx, t);
      }
      double sum = 0.0;
      for (Index k = ptr[r]; k < ptr[r + 1]; ++k)
        sum += exp((double)out[(size_t)k * heads + h] - (double)mx);
      for (Index k = ptr[r]; k < ptr[r + 1]; ++k) {
        const double ev = exp((double)out[(size_t)k * heads + h] - (double)mx);
        out[(size_t)k * heads + h] = (float)(ev / sum);
      }
    }
}

/* ------------------------------------------------------------------------- */
/* Edge softmax backward: edge_softmax_bwd src/cpp/src/edge_softmax.cu:44-95   */
/*   s = sum_row out*g; t = out*(g - s) * (mask ? 1 : slope);                  */
/*   g_src[idx[e],h] += t; g_dst[r,h] = sum_row t, written only when the row   */
/*   has both signs of pre-activation (:91-93), else left 0.                   */
/* ------------------------------------------------------------------------- */
void orc_edge_softmax_bwd(const Index* ptr, const Index* idx, const float* g, const uint8_t* mask,
                          const float* out, float* g_dst, float* g_src, Index n_dst, Index n_src,
                          int heads, float slope) {
  double* acc = (double*)calloc((size_t)n_src * heads, sizeof(double));
  for (size_t i = 0; i < (size_t)n_dst * heads; ++i) g_dst[i] = 0.f;
  for (Index r = 0; r < n_dst; ++r)
    for (int h = 0; h < heads; ++h) {
      double s = 0.0;
      for (Index k = ptr[r]; k < ptr[r + 1]; ++k)
        s += (double)out[(size_t)k * heads + h] * (double)g[(size_t)k * heads + h];
      double dsum = 0.0;
      int pos = 0, neg = 0;
      for (Index k = ptr[r]; k < ptr[r + 1]; ++k) {
        double t = (double)out[(size_t)k * heads + h] * ((double)g[(size_t)k * heads + h] - s);
        if (!mask[(size_t)k * heads + h]) { t *= (double)slope; neg = 1; }
        else pos = 1;
        dsum += t;
        acc[(size_t)idx[k] * heads + h] += t;
      }
      if (pos && neg) g_dst[(size_t)r * heads + h] = (float)dsum;
    }
  for (size_t i = 0; i < (size_t)n_src * heads; ++i) g_src[i] = (float)acc[i];
  free(acc);
}

/* gen_edge_value_degree src/cpp/src/edge_softmax.cu:186-198: val[e] = 1/deg(row) */
void orc_edge_value_degree(const Index* ptr, float* out, Index n_dst) {
  for (Index r = 0; r < n_dst; ++r) {
    const Index b = ptr[r], e = ptr[r + 1];
    if (e <= b) continue;
    const float v = 1.f / (float)(e - b);
    for (Index k = b; k < e; ++k) out[k] = v;
  }
}

/* spmv_csr src/cpp/src/edge_softmax.cu:216-232: out[r] = sum_e in[idx[e]] */
void orc_spmv(const Index* ptr, const Index* idx, const float* in, float* out, Index n_dst) {
  for (Index r = 0; r < n_dst; ++r) {
    double s = 0.0;
    for (Index k = ptr[r]; k < ptr[r + 1]; ++k) s += (double)in[idx[k]];
    out[r] = (float)s;
  }
}

/* ------------------------------------------------------------------------- */
/* GSpMM_u / GSpMM_u_e: generalised CSR SpMM of the dgSPARSE kernels           */
/* src/cpp/include/dgsparse.h:14-131, src/cpp/src/dgsparse.cu:6-125,444-474:   */
/*   out[r,c] = REDUCE_{e in row r} COMPUTE(val[e], b[col[e], c]);             */
/*   REDUCE 0 sum, 1 max, 2 min, 3 mean; COMPUTE 0 val+b, 1 b-val, 2 val*b,    */
/*   3 b/val (dgsparse.h:13-14,53-79); val == NULL: the operand is b itself.   */
/*   The accumulator of a non-empty row starts at init(op): 0, (float)INT_MIN, */
/*   (float)INT_MAX, 0 (dgsparse.h:117-130); empty rows give 0                 */
/*   (dgsparse.cu:23-24); mean divides by the row length.  int32 indices.      */
/* ------------------------------------------------------------------------- */
void orc_gspmm(const int32_t* rowptr, const int32_t* colind, const float* val, const float* b,
               float* out, Index n_rows, int feat, int red, int comp) {
  for (Index r = 0; r < n_rows; ++r) {
    const int lb = rowptr[r], hb = rowptr[r + 1];
    for (int c = 0; c < feat; ++c) {
      if (hb <= lb) { out[r * feat + c] = 0.f; continue; }
      double acc = red == 1 ? (double)(float)INT32_MIN : red == 2 ? (double)(float)INT32_MAX : 0.0;
      for (int k = lb; k < hb; ++k) {
        const float f = b[(Index)colind[k] * feat + c];
        float t = f;
        if (val) {
          const float v = val[k];
          t = comp == 0 ? v + f : comp == 1 ? f - v : comp == 2 ? v * f : f / v;
        }
        if (red == 1) acc = (double)t > acc ? (double)t : acc;
        else if (red == 2) acc = (double)t < acc ? (double)t : acc;
        else acc += (double)t;
      }
      if (red == 3) acc /= (double)(hb - lb);
      out[r * feat + c] = (float)acc;
    }
  }
}

/* ------------------------------------------------------------------------- */
/* gather_fwd / gather_bwd src/cpp/src/aggr.cu:42-62                           */
/*   fwd: out[dest[e]] += in[e] (out zeroed first, aggr.cu:406);               */
/*   bwd: gin[e] = gout[dest[e]]                                               */
/* ------------------------------------------------------------------------- */
void orc_gather_fwd(const float* in, const Index* dest, float* out, Index n_edges, Index n_nodes,
                    int feat) {
  double* acc = (double*)calloc((size_t)n_nodes * feat, sizeof(double));
  for (Index e = 0; e < n_edges; ++e)
    for (int c = 0; c < feat; ++c) acc[(size_t)dest[e] * feat + c] += (double)in[(size_t)e * feat + c];
  for (size_t i = 0; i < (size_t)n_nodes * feat; ++i) out[i] = (float)acc[i];
  free(acc);
}
void orc_gather_bwd(const float* gout, const Index* dest, float* gin, Index n_edges, int feat) {
  for (Index e = 0; e < n_edges; ++e)
    memcpy(gin + (size_t)e * feat, gout + (size_t)dest[e] * feat, sizeof(float) * (size_t)feat);
}

/* ------------------------------------------------------------------------- */
/* selective_aggr_fwd_kernel / _bwd_kernel src/cpp/src/aggr_kernel.cu:493-555  */
/*   fwd: out[r] += sum_{e in row r, mask[e]} x[idx[e]]   (accumulates)        */
/*   bwd: gx[idx[e]] += g[r] for masked edges             (accumulates)        */
/* ------------------------------------------------------------------------- */
void orc_selective_aggr_fwd(const Index* ptr, const Index* idx, const uint8_t* mask, const float* x,
                            float* out, Index n_rows, int feat) {
  double* acc = (double*)malloc(sizeof(double) * (size_t)feat);
  for (Index r = 0; r < n_rows; ++r) {
    for (int c = 0; c < feat; ++c) acc[c] = 0.0;
    for (Index k = ptr[r]; k < ptr[r + 1]; ++k)
      if (mask[k])
        for (int c = 0; c < feat; ++c) acc[c] += (double)x[(size_t)idx[k] * feat + c];
    for (int c = 0; c < feat; ++c)
      out[(size_t)r * feat + c] = (float)((double)out[(size_t)r * feat + c] + acc[c]);
  }
  free(acc);
}
void orc_selective_aggr_bwd(const Index* ptr, const Index* idx, const uint8_t* mask, const float* g,
                            float* gx, Index n_rows, Index n_src, int feat) {
  double* acc = (double*)calloc((size_t)n_src * feat, sizeof(double));
  for (Index r = 0; r < n_rows; ++r)
    for (Index k = ptr[r]; k < ptr[r + 1]; ++k)
      if (mask[k])
        for (int c = 0; c < feat; ++c)
          acc[(size_t)idx[k] * feat + c] += (double)g[(size_t)r * feat + c];
  for (size_t i = 0; i < (size_t)n_src * feat; ++i) gx[i] = (float)((double)gx[i] + acc[i]);
  free(acc);
}

/* ------------------------------------------------------------------------- */
/* target_aggr / target_aggr_backward src/cpp/src/aggr_kernel.cu:557-607       */
/*   fwd: out[targets[r]] += sum_{e in row r} x[idx[e]]                        */
/*   bwd: gx[idx[e]] += g[targets[r]]                                          */
/* ------------------------------------------------------------------------- */
void orc_target_aggr_fwd(const Index* ptr, const Index* idx, const Index* targets, const float* x,
                         float* out, Index n_rows, Index n_out, int feat) {
  double* acc = (double*)calloc((size_t)n_out * feat, sizeof(double));
  for (Index r = 0; r < n_rows; ++r)
    for (Index k = ptr[r]; k < ptr[r + 1]; ++k)
      for (int c = 0; c < feat; ++c)
        acc[(size_t)targets[r] * feat + c] += (double)x[(size_t)idx[k] * feat + c];
  for (size_t i = 0; i < (size_t)n_out * feat; ++i) out[i] = (float)((double)out[i] + acc[i]);
  free(acc);
}
void orc_target_aggr_bwd(const Index* ptr, const Index* idx, const Index* targets, const float* g,
                         float* gx, Index n_rows, Index n_src, int feat) {
  double* acc = (double*)calloc((size_t)n_src * feat, sizeof(double));
  for (Index r = 0; r < n_rows; ++r)
    for (Index k = ptr[r]; k < ptr[r + 1]; ++k)
      for (int c = 0; c < feat; ++c)
        acc[(size_t)idx[k] * feat + c] += (double)g[(size_t)targets[r] * feat + c];
  for (size_t i = 0; i < (size_t)n_src * feat; ++i) gx[i] = (float)((double)gx[i] + acc[i]);
  free(acc);
}

/* ------------------------------------------------------------------------- */
/* aggr_rel_fwd / aggr_rel_bwd src/cpp/src/rel_spmm.cu:8-35, 72-104            */
/*   x is [num_rel * n_per_rel, feat]; out[r] = sum_e x[rel[e]*n_per_rel+idx[e]]*/
/*   bwd: gx[rel[e]*n_per_rel + idx[e]] += g[r]                                */
/* ------------------------------------------------------------------------- */
void orc_aggr_rel_fwd(const Index* ptr, const Index* idx, const int32_t* rel, const float* x,
                      float* out, Index n_rows, Index n_per_rel, int feat) {
  double* acc = (double*)malloc(sizeof(double) * (size_t)feat);
  for (Index r = 0; r < n_rows; ++r) {
    for (int c = 0; c < feat; ++c) acc[c] = 0.0;
    for (Index k = ptr[r]; k < ptr[r + 1]; ++k) {
      const float* row = x + ((size_t)rel[k] * n_per_rel + idx[k]) * feat;
      for (int c = 0; c < feat; ++c) acc[c] += (double)row[c];
    }
    for (int c = 0; c < feat; ++c) out[(size_t)r * feat + c] = (float)acc[c];
  }
  free(acc);
}
void orc_aggr_rel_bwd(const Index* ptr, const Index* idx, const int32_t* rel, const float* g,
                      float* gx, Index n_rows, Index n_per_rel, int num_rel, int feat) {
  const size_t total = (size_t)num_rel * n_per_rel * feat;
  double* acc = (double*)calloc(total, sizeof(double));
  for (Index r = 0; r < n_rows; ++r)
    for (Index k = ptr[r]; k < ptr[r + 1]; ++k)
      for (int c = 0; c < feat; ++c)
        acc[((size_t)rel[k] * n_per_rel + idx[k]) * feat + c] += (double)g[(size_t)r * feat + c];
  for (size_t i = 0; i < total; ++i) gx[i] = (float)acc[i];
  free(acc);
}

/* ------------------------------------------------------------------------- */
/* Fused RGCN aggregate+transform: aggr_rgcn_direct_kernel                     */
/* src/cpp/src/rel_spmm.cu:138-181 (without its read past the row end, :162)   */
/*   out[r,:] = sum_e x[idx[e],:] @ W[rel[e]],  W is [R, K, N]                 */
/* ------------------------------------------------------------------------- */
void orc_rgcn_fused(const Index* ptr, const Index* idx, const int32_t* rel, const float* x,
                    const float* w, float* out, Index n_rows, int K, int N) {
  double* acc = (double*)malloc(sizeof(double) * (size_t)N);
  for (Index r = 0; r < n_rows; ++r) {
    for (int j = 0; j < N; ++j) acc[j] = 0.0;
    for (Index k = ptr[r]; k < ptr[r + 1]; ++k) {
      const float* row = x + (size_t)idx[k] * K;
      const float* W = w + (size_t)rel[k] * K * N;
      for (int i = 0; i < K; ++i) {
        const double xi = row[i];
        for (int j = 0; j < N; ++j) acc[j] += xi * (double)W[(size_t)i * N + j];
      }
    }
    for (int j = 0; j < N; ++j) out[(size_t)r * N + j] = (float)acc[j];
  }
  free(acc);
}

/* ------------------------------------------------------------------------- */
/* Per-row typed linear: typed_linear_kernel / _s2e / _s2d                     */
/* src/cpp/src/rel_spmm.cu:231-342                                             */
/*   out[dst_i] += x[src_i] @ W[types[i]]; src == NULL -> src_i = i,           */
/*   dst == NULL -> dst_i = i.  Accumulates onto the existing output.          */
/* The Triton typed_matmul (cxgnncomp/codegen/triton_typed_matmul.py:752-860)  */
/* computes the same product, overwriting instead of accumulating.             */
/* ------------------------------------------------------------------------- */
void orc_typed_linear(const float* x, const float* w, float* out, const Index* src, const Index* dst,
                      const int32_t* types, Index n, Index n_out, int K, int N) {
  double* acc = (double*)calloc((size_t)n_out * N, sizeof(double));
  for (Index i = 0; i < n; ++i) {
    const Index s = src ? src[i] : i;
    const Index d = dst ? dst[i] : i;
    const float* row = x + (size_t)s * K;
    const float* W = w + (size_t)types[i] * K * N;
    for (int k = 0; k < K; ++k) {
      const double xk = row[k];
      for (int j = 0; j < N; ++j) acc[(size_t)d * N + j] += xk * (double)W[(size_t)k * N + j];
    }
  }
  for (size_t i = 0; i < (size_t)n_out * N; ++i) out[i] = (float)((double)out[i] + acc[i]);
  free(acc);
}

/* ------------------------------------------------------------------------- */
/* pad_rel / pad_rel_idx src/cpp/src/stitch_kernel.cu:3-38 (bit-exact)         */
/* ------------------------------------------------------------------------- */
void orc_pad_rel(Index* rel, Index* idx, const Index* count, int thres, int num_rel, Index base) {
  const Index slots = (Index)num_rel * (thres - 1);
  for (Index tid = 0; tid < slots; ++tid) {
    const int which = (int)(tid / (thres - 1));
    const int rel_count = (int)count[which];
    const int mod = rel_count % thres;
    const Index pos = base + tid;
    if ((tid % (thres - 1)) < (thres - mod) && (mod != 0)) rel[pos] = which;
    else rel[pos] = num_rel;
    if (idx) idx[pos] = -1;
  }
}

/* ------------------------------------------------------------------------- */
/* neighbor_grouping cxgnncomp/schedule.py:20-35 (bit-exact)                   */
/* Returns the number of groups; new_ptr needs n_groups+1 slots, new_target    */
/* n_groups.  Call with new_ptr == NULL to count only.                         */
/* ------------------------------------------------------------------------- */
Index orc_neighbor_grouping(const Index* ptr, Index n_rows, Index thres, Index* new_ptr,
                            Index* new_target) {
  Index n = 0;
  if (new_ptr) new_ptr[0] = 0;
  for (Index i = 0; i < n_rows; ++i) {
    const Index end = ptr[i + 1];
    Index start = ptr[i];
    while (end - start > thres) {
      start += thres;
      if (new_ptr) { new_ptr[n + 1] = start; new_target[n] = i; }
      ++n;
    }
    if (new_ptr) { new_ptr[n + 1] = end; new_target[n] = i; }
    ++n;
  }
  return n;
}

/* ------------------------------------------------------------------------- */
/* rel_schedule src/cpp/src/schedule.cu:5-63 (bit-exact), one relation at a    */
/* time: sub-CSR of the edges with rel == which.  Returns the number of kept   */
/* rows; sub_idx receives the kept edges in order; layer_counts[l] = number of */
/* kept rows among the first num_node_in_layer[l] rows.  Pass sub_ptr == NULL  */
/* to count: *n_sub_edges receives the edge count.                             */
/* ------------------------------------------------------------------------- */
Index orc_rel_schedule_one(const Index* ptr, const Index* idx, const int32_t* rel, Index n_rows,
                           int which, const Index* num_node_in_layer, int num_layer, Index* sub_ptr,
                           Index* sub_idx, Index* sub_target, Index* layer_counts,
                           Index* n_sub_edges) {
  Index rows = 0, edges = 0;
  int layer_id = 0;
  if (sub_ptr) sub_ptr[0] = 0;
  for (Index i = 0; i < n_rows; ++i) {
    Index cnt = 0;
    for (Index j = ptr[i]; j < ptr[i + 1]; ++j)
      if (rel[j] == which) {
        if (sub_idx) sub_idx[edges] = idx[j];
        ++edges;
        ++cnt;
      }
    if (cnt > 0) {
      if (sub_ptr) { sub_target[rows] = i; sub_ptr[rows + 1] = sub_ptr[rows] + cnt; }
      ++rows;
    }
    if (layer_id < num_layer && i == num_node_in_layer[layer_id] - 1) {
      if (layer_counts) layer_counts[layer_id] = rows;
      ++layer_id;
    }
  }
  if (n_sub_edges) *n_sub_edges = edges;
  return rows;
}

/* ------------------------------------------------------------------------- */
/* CSR transposition (the graph of the backward pass).  No single reference    */
/* function: it is the index relation behind the atomic scatter kernels        */
/* (src/cpp/src/aggr_kernel.cu:220-249).  Stable counting sort by source.      */
/* ------------------------------------------------------------------------- */
void orc_csr_transpose(const Index* ptr, const Index* idx, Index n_rows, Index n_cols, Index* ptr_t,
                       Index* idx_t, Index* perm) {
  const Index E = ptr[n_rows];
  for (Index c = 0; c <= n_cols; ++c) ptr_t[c] = 0;
  for (Index k = 0; k < E; ++k) ptr_t[idx[k] + 1]++;
  for (Index c = 0; c < n_cols; ++c) ptr_t[c + 1] += ptr_t[c];
  Index* cur = (Index*)malloc(sizeof(Index) * (size_t)(n_cols > 0 ? n_cols : 1));
  for (Index c = 0; c < n_cols; ++c) cur[c] = ptr_t[c];
  for (Index r = 0; r < n_rows; ++r)
    for (Index k = ptr[r]; k < ptr[r + 1]; ++k) {
      const Index p = cur[idx[k]]++;
      idx_t[p] = r;
      perm[p] = k;
    }
  free(cur);
}

/* CSR by destination from an edge list, stable in edge order
 * (cxgnncomp/data_preparation.py:97-104 builds the inverse relation). */
void orc_coo_to_csr(const Index* src, const Index* dst, Index n_edges, Index n_dst, Index* ptr,
                    Index* idx) {
  for (Index r = 0; r <= n_dst; ++r) ptr[r] = 0;
  for (Index e = 0; e < n_edges; ++e) ptr[dst[e] + 1]++;
  for (Index r = 0; r < n_dst; ++r) ptr[r + 1] += ptr[r];
  Index* cur = (Index*)malloc(sizeof(Index) * (size_t)(n_dst > 0 ? n_dst : 1));
  for (Index r = 0; r < n_dst; ++r) cur[r] = ptr[r];
  for (Index e = 0; e < n_edges; ++e) idx[cur[dst[e]]++] = src[e];
  free(cur);
}
