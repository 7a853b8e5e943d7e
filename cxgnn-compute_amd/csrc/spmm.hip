// CSR-by-destination SpMM for gfx950: sum / mean / edge-weighted (single and
// multi-head), forward and -- on a transposed CSR -- backward.
//
// Work decomposition ("edge spans").  The edge array [ptr[0], ptr[n_rows]) is
// cut into spans of T consecutive edges and every wavefront owns one span, so
// the load per wave is the same for a degree-4 row and for a 17k-degree hub.
// A wave locates the first row of its span with a 64-ary search over ptr, then
// streams the span: 64 source ids are fetched with one coalesced load, each id
// is broadcast to a scalar register and the whole wave gathers that source row
// (64 lanes x V floats), U gathers in flight at a time.  Row boundaries are
// wave-uniform, so a finished row is stored directly by the wave.  Rows that
// cross a span boundary leave partial sums in a carry buffer; a second small
// kernel adds the partials of each such row in span order.  No atomics: the
// result is deterministic run to run.
//
// Semantics follow the reference kernels gen_fwd_sum / gen_fwd_mean /
// gen_fwd_sum_edge_value[_multi_head] (src/cpp/src/aggr_kernel.cu:3-186) and
// run_spmm_sharedmem* (src/cpp/src/spmm_kernel.cu:231-512).
#include "cxg_common.hpp"

#include <atomic>

// Carry buffer and span table of cxg_spmm_sum_f32_noalloc: one copy per GPU, part of the
// code object, held until the process ends.  In host code this name is only a handle for
// hipGetSymbolAddress; the device address is looked up once per device (static_scratch()).
static __device__ __align__(256) unsigned char scratch[CXG_SPMM_NOALLOC_SCRATCH_BYTES];

namespace cxg {
namespace {

#ifndef CXG_SPMM_SPAN_DIV
#define CXG_SPMM_SPAN_DIV 16384   // target number of spans for graphs too small for 512-edge spans
#endif
#ifndef CXG_SPMM_GROUP_UF
#define CXG_SPMM_GROUP_UF 4
#endif
#ifndef CXG_SPMM_U
#define CXG_SPMM_U 1
#endif
#ifndef CXG_SPMM_U_V4
#define CXG_SPMM_U_V4 8
#endif
#ifndef CXG_SPMM_U_DOT
#define CXG_SPMM_U_DOT 4
#endif

constexpr int kWavesPerBlock = 4;
constexpr int kBlock = kWavesPerBlock * CXG_WAVE;
// Windows of 64 rows without edges after which the end of a run of them is found with a search
// and the run left to the fix-up kernel (for a shorter run the search costs more than a look
// at the next windows: with the search from the first window on, an RGCN layer whose pair
// tables hold many runs of 64-200 such rows lost 2 %).
constexpr int kRunWindows = 4;

template <int V> struct Vec;
template <> struct Vec<1> { using type = float; };
template <> struct Vec<2> { using type = float2; };
template <> struct Vec<4> { using type = float4; };
struct float8 { float4 lo, hi; };            // eight values per lane: a 16-byte piece of a bf16 row, widened
template <> struct Vec<8> { using type = float8; };

template <int V> __device__ __forceinline__ typename Vec<V>::type vzero();
template <> __device__ __forceinline__ float vzero<1>() { return 0.f; }
template <> __device__ __forceinline__ float2 vzero<2>() { return make_float2(0.f, 0.f); }
template <> __device__ __forceinline__ float4 vzero<4>() { return make_float4(0.f, 0.f, 0.f, 0.f); }
template <> __device__ __forceinline__ float8 vzero<8>() { return float8{make_float4(0.f, 0.f, 0.f, 0.f), make_float4(0.f, 0.f, 0.f, 0.f)}; }

// (explicit fused multiply-adds: left to the compiler, one instantiation of a kernel fused `a += v * w`
// and another, whose weight came out of a select, did not -- the same sums, last bits apart)
__device__ __forceinline__ void vfma(float& a, float v, float w) { a = __builtin_fmaf(v, w, a); }
__device__ __forceinline__ void vfma(float2& a, float2 v, float w) { a.x = __builtin_fmaf(v.x, w, a.x); a.y = __builtin_fmaf(v.y, w, a.y); }
__device__ __forceinline__ void vfma(float4& a, float4 v, float w) {
  a.x = __builtin_fmaf(v.x, w, a.x); a.y = __builtin_fmaf(v.y, w, a.y);
  a.z = __builtin_fmaf(v.z, w, a.z); a.w = __builtin_fmaf(v.w, w, a.w);
}
__device__ __forceinline__ void vadd(float& a, float v) { a += v; }
__device__ __forceinline__ void vadd(float2& a, float2 v) { a.x += v.x; a.y += v.y; }
__device__ __forceinline__ void vadd(float4& a, float4 v) { a.x += v.x; a.y += v.y; a.z += v.z; a.w += v.w; }
__device__ __forceinline__ void vscale(float& a, float s) { a *= s; }
__device__ __forceinline__ void vscale(float2& a, float s) { a.x *= s; a.y *= s; }
__device__ __forceinline__ void vscale(float4& a, float s) { a.x *= s; a.y *= s; a.z *= s; a.w *= s; }
__device__ __forceinline__ void vfma(float8& a, float8 v, float w) { vfma(a.lo, v.lo, w); vfma(a.hi, v.hi, w); }
__device__ __forceinline__ void vadd(float8& a, float8 v) { vadd(a.lo, v.lo); vadd(a.hi, v.hi); }
__device__ __forceinline__ void vscale(float8& a, float s) { vscale(a.lo, s); vscale(a.hi, s); }

template <typename IdxT>
struct SpmmArgs {
  const IdxT* ptr;
  const IdxT* idx;
  const float* x;
  float* out;
  const float* val;        // [*, heads] or null
  const int64_t* perm;     // val row of edge position, or null
  int64_t ldx, ldo;
  int64_t n_rows;
  int F;                   // floats per row (heads * channels)
  int heads, channels;
  int T;                   // edges per span (multiple of 64)
  int64_t exact_edges;     // > 0: the caller vouches for this edge count (span-length hint)
  int mean, accumulate;
  float* carry;            // [n_spans_cap][2][F]: head partial, tail partial
  int64_t* tail_row;       // [n_spans_cap][3]: row whose tail partial the span holds, or -1; then the
                           // run [begin, end) of rows without edges the span leaves to the fix-up kernel
  // extended gather (EXT kernels only); every pointer may be null
  const uint8_t* mask;     // skip edges whose mask byte is 0
  const int64_t* mask_perm;// mask index of edge position (null: the position itself)
  const int32_t* rel;      // source row += rel[e] * rel_stride
  int64_t rel_stride;
  const int64_t* src_map;  // source row = src_map[source row]
  const int64_t* targets;  // row r is added (atomically) into out[targets[r]]
  // per-edge dot products beside the aggregation (DOTG kernels only):
  // dot_out[vrow(e), h] = <x[idx[e], h, :], dot_b[r, h, :]> for every edge e of row r
  const float* dot_b;
  int64_t ld_dot_b;
  float* dot_out;
  int dot_at_edge;         // dot_out rows at the edge's own position although val is read through perm
  const float* bias;       // [F] added to every output row, or null
  int out_bf16;            // the rows of `out` are bf16 (grouped-lane kernel with IO & 2, and its fix-up launch)
};

__device__ __forceinline__ void atomic_add_vec(float* p, float v) { unsafeAtomicAdd(p, v); }
__device__ __forceinline__ void atomic_add_vec(float* p, float2 v) {
  unsafeAtomicAdd(p, v.x); unsafeAtomicAdd(p + 1, v.y);
}
__device__ __forceinline__ void atomic_add_vec(float* p, float4 v) {
  unsafeAtomicAdd(p, v.x); unsafeAtomicAdd(p + 1, v.y);
  unsafeAtomicAdd(p + 2, v.z); unsafeAtomicAdd(p + 3, v.w);
}

// WMODE: 0 = unweighted, 1 = one weight per edge (heads == 1), 2 = one weight
// per edge and head (each lane's V columns lie in one head).
// a[i] + a[i + M] for the lanes whose partner exists in this sense, without a trip through the LDS
// crossbar (which is what a shuffle costs: 5,800 of them were this file's share): inside a row of 16
// lanes a data-parallel move that shifts the row left by M (lanes past the row's end read 0), across
// rows the half-swap instructions of this chip -- v_permlane16_swap exchanges the odd rows of its
// first operand with the even rows of its second, v_permlane32_swap the upper half with the lower
// half, so with both operands equal the two results are the two partners side by side in every lane.
// Only lanes i with (i & M) == 0 hold a meaningful sum; every user below reads such a lane.
template <int M> __device__ __forceinline__ float shift_add(float a) {
  typedef unsigned v2u __attribute__((ext_vector_type(2)));
  if constexpr (M == 32) {
    const v2u r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(a), false, false);
    return __uint_as_float(r.x) + __uint_as_float(r.y);
  } else if constexpr (M == 16) {
    const v2u r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(a), false, false);
    return __uint_as_float(r.x) + __uint_as_float(r.y);
  } else {
    static_assert(M >= 1 && M < 16, "shift inside a row of 16 lanes");
    return a + __uint_as_float((unsigned)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(a), 0x100 + M, 0xf, 0xf, true));
  }
}
template <int M> __device__ __forceinline__ void vshift_add(float& a) { a = shift_add<M>(a); }
template <int M> __device__ __forceinline__ void vshift_add(float2& a) { a.x = shift_add<M>(a.x); a.y = shift_add<M>(a.y); }
template <int M> __device__ __forceinline__ void vshift_add(float4& a) {
  a.x = shift_add<M>(a.x); a.y = shift_add<M>(a.y); a.z = shift_add<M>(a.z); a.w = shift_add<M>(a.w);
}
// Sum over `G` consecutive lanes (power of two, aligned); the group's first lane holds it.
template <int G> __device__ __forceinline__ float lane_group_sum(float v) {
  if constexpr (G >= 64) v = shift_add<32>(v);
  if constexpr (G >= 32) v = shift_add<16>(v);
  if constexpr (G >= 16) v = shift_add<8>(v);
  if constexpr (G >= 8) v = shift_add<4>(v);
  if constexpr (G >= 4) v = shift_add<2>(v);
  if constexpr (G >= 2) v = shift_add<1>(v);
  return v;
}
__device__ __forceinline__ void vxor_add(float& a, int m) { a += __shfl_xor(a, m, CXG_WAVE); }
__device__ __forceinline__ void vxor_add(float2& a, int m) {
  a.x += __shfl_xor(a.x, m, CXG_WAVE); a.y += __shfl_xor(a.y, m, CXG_WAVE);
}
__device__ __forceinline__ void vxor_add(float4& a, int m) {
  a.x += __shfl_xor(a.x, m, CXG_WAVE); a.y += __shfl_xor(a.y, m, CXG_WAVE);
  a.z += __shfl_xor(a.z, m, CXG_WAVE); a.w += __shfl_xor(a.w, m, CXG_WAVE);
}
__device__ __forceinline__ void vxor_add(float8& a, int m) { vxor_add(a.lo, m); vxor_add(a.hi, m); }
template <int M> __device__ __forceinline__ void vshift_add(float8& a) { vshift_add<M>(a.lo); vshift_add<M>(a.hi); }
using cxg::stream_store;   // (an overload declared here would otherwise hide the ones of the enclosing namespace)
__device__ __forceinline__ void stream_store(float* p, float8 v) { stream_store(p, v.lo); stream_store(p + 4, v.hi); }

__device__ __forceinline__ float vdot4(float4 a, float4 b) { return a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w; }

// DOTG > 0 (V == 4, whole column tiles, DOTG = channels / 4 lanes per head): the wave also
// multiplies every gathered row with the row of `dot_b` that belongs to the output row and
// stores the per-head sums at the edge's weight row -- the edge-value gradient of the
// attention layer from the gathers of its input gradient.  The rows of dot_b are loaded
// one output row ahead (a deeper ring measured the same).
// PRE (WMODE 2, the whole row of heads x channels = 64 * V floats in one column tile): the
// heads are summed before a row -- or a partial row on its way to the carry buffer -- is
// stored: out[r, :] = sum_h sum_e val[e, h] x[idx[e], h, :].  A head occupies channels / V
// consecutive lanes, so the sum over heads is a butterfly over the lane bits above that, and
// the lanes of the first head store the channels floats of the row (out, bias, the carry rows
// and the fix-up kernel then all work on rows of `channels` floats).
template <typename IdxT, int V, bool GUARD, int WMODE, bool PERM, bool EXT, int U, int DOTG = 0, bool PRE = false>
__global__ __launch_bounds__(kBlock) void spmm_span_kernel(SpmmArgs<IdxT> a) {
  static_assert(!PRE || (WMODE == 2 && !GUARD && !EXT && DOTG == 0), "head pre-reduction: plain per-head weights only");
  using vec_t = typename Vec<V>::type;
  constexpr int kDotHeads = DOTG > 0 ? CXG_WAVE / DOTG : 1;       // heads of one 256-float column tile
  __shared__ __attribute__((aligned(16))) float s_dot[DOTG > 0 ? kWavesPerBlock : 1][DOTG > 0 ? CXG_WAVE * kDotHeads : 1];
  const int lane = lane_id();
  const int wave = uniform_i32(threadIdx.x >> 6);
  const int64_t s = (int64_t)blockIdx.x * kWavesPerBlock + wave;
  const int64_t n_rows = a.n_rows;
  const int64_t e_begin = (int64_t)a.ptr[0];
  const int64_t e_end = (int64_t)a.ptr[n_rows];
  const int64_t total = e_end - e_begin;
  const int T = a.T;
  const int64_t n_spans = total > 0 ? (total + T - 1) / T : 1;
  if (s >= n_spans) return;
  const bool last = (s == n_spans - 1);
  const int64_t e0 = e_begin + s * T;
  const int n = (int)((e_end - e0) < (int64_t)T ? (e_end - e0) : (int64_t)T);

  // column tile of this block (grid.y tiles rows wider than 64*V floats)
  const int col = blockIdx.y * (CXG_WAVE * V) + lane * V;
  const bool col_ok = GUARD ? (col < a.F) : true;
  const int F = PRE ? a.channels : a.F;      // floats of a stored row
  const int lanes_per_head = PRE ? a.channels / V : CXG_WAVE;
  const bool st_ok = PRE ? lane < lanes_per_head : col_ok;   // this lane stores (its column of the stored row is `col`)

  const int64_t r_lo = wave_lower_bound(a.ptr, n_rows, e0);
  bool is_head = (r_lo == n_rows) || ((int64_t)a.ptr[r_lo] > e0);
  int64_t r = is_head ? r_lo - 1 : r_lo;

  // Row ends of rows [rbase, rbase + 64) relative to e0, clamped to n + 1.
  int64_t rbase = r;
  auto load_row_ends = [&](int64_t rb) -> int {
    int64_t q = rb + 1 + lane;
    if (q > n_rows) q = n_rows;
    const int64_t d = (int64_t)a.ptr[q] - e0;
    return (int)(d < (int64_t)n + 1 ? d : (int64_t)n + 1);
  };
  int row_ends = load_row_ends(rbase);
  int cur_start = is_head ? -1 : 0;
  int cur_end = (r < n_rows) ? bcast_i32(row_ends, 0) : 0x7fffffff;

  vec_t acc = vzero<V>();
  float* const carry_head = a.carry + (size_t)(2 * s) * F;
  float* const carry_tail = carry_head + F;

  int head_of_lane = 0;
  if (WMODE == 2) head_of_lane = col / a.channels;

  vec_t xr0 = vzero<V>(), xr1 = vzero<V>();   // rows r and r + 1 of dot_b
  auto load_dot_row = [&](int64_t row) -> vec_t {
    const int64_t rc = row < n_rows ? row : n_rows - 1;
    return *reinterpret_cast<const vec_t*>(a.dot_b + rc * a.ld_dot_b + col);
  };
  if (DOTG > 0) {
    xr0 = load_dot_row(r); xr1 = load_dot_row(r + 1);
  }

  auto store_vec = [&](float* dst, vec_t v) {
    if (st_ok) stream_store(dst + col, v);
  };
  // PRE: sum over the heads, left in every lane (the lanes of head 0 store it)
  auto head_reduce = [&](vec_t& v) {
    if constexpr (PRE) {
      for (int m = lanes_per_head; m < CXG_WAVE; m <<= 1) vxor_add(v, m);
    }
  };
  // What finish_row leaves in a row without edges.
  auto store_empty_row = [&](int64_t row) {
    if ((EXT && a.targets) || (a.accumulate && !a.bias) || !st_ok) return;
    float* dst = a.out + row * a.ldo;
    vec_t z = vzero<V>();
    if (a.bias) vadd(z, *reinterpret_cast<const vec_t*>(a.bias + col));
    if (a.accumulate) vadd(z, *reinterpret_cast<const vec_t*>(dst + col));
    *reinterpret_cast<vec_t*>(dst + col) = z;
  };
  // (not in the per-head kernels: there the extra live registers cost a wave of occupancy, and
  // the fused dot-product form prefetches rows of dot_b in step with the walk)
  constexpr bool kSkipRuns = DOTG == 0 && WMODE != 2;
  bool run_left = false;                       // this span's slot holds a run
  if (lane == 0 && blockIdx.y == 0) { a.tail_row[3 * s + 1] = 0; a.tail_row[3 * s + 2] = 0; }
  // A long run of rows without edges (the seed rows of a sampled batch in the reversed graph):
  // walked row by row, every 64 rows cost a load of the next row ends that first waits for the
  // 64 stores before it (1024 such rows: 125 us), and one wave keeps at most 64 stores in
  // flight.  Called with rbase == r and a window whose rows all end at `end_rel`, i.e. have no
  // edges: looks on window by window, and after kRunWindows of them finds the end of the run
  // with one search.  A run of kRunWindows windows or more is left to the fix-up kernel, where
  // sixteen waves share it (the first one of a span; its workspace slot holds one run), a
  // shorter one is stored here, now without loads between the stores.
  auto skip_rows_without_edges = [&](int end_rel) {
    const int64_t first = r;
    int64_t q = r;
    for (int hop = 1;; ++hop) {
      q += CXG_WAVE;
      if (q >= n_rows) { q = rbase = n_rows; break; }
      if (hop == kRunWindows) {
        q += wave_lower_bound(a.ptr + q + 1, n_rows - q, e0 + end_rel + 1);
        rbase = q;
        if (q < n_rows) row_ends = load_row_ends(rbase);
        break;
      }
      const int w = load_row_ends(q);
      const unsigned long long busy = __ballot(w != end_rel);
      if (busy) {
        rbase = q;
        row_ends = w;
        q += __ffsll((long long)busy) - 1;
        break;
      }
    }
    r = q;
    if (r - first >= kRunWindows * CXG_WAVE && !run_left) {
      run_left = true;
      if (lane == 0 && blockIdx.y == 0) { a.tail_row[3 * s + 1] = first; a.tail_row[3 * s + 2] = r; }
    } else {
      for (int64_t row = first; row < r; ++row) store_empty_row(row);
    }
  };
  // `own`: the rows without edges that follow the finished row belong to this span.
  auto next_row = [&](bool own) {
    ++r;
    if (DOTG > 0) { xr0 = xr1; xr1 = load_dot_row(r + 1); }
    if (r - rbase == CXG_WAVE) {
      rbase = r;
      row_ends = load_row_ends(rbase);
      if constexpr (kSkipRuns) {
        if (own && r < n_rows && __ballot(row_ends != cur_end) == 0) skip_rows_without_edges(cur_end);
      }
    }
    cur_start = cur_end;
    cur_end = (r < n_rows) ? bcast_i32(row_ends, (int)(r - rbase)) : 0x7fffffff;
    is_head = false;
  };
  if constexpr (kSkipRuns) {
    // the same for a span that starts with a window of rows without edges
    if (!is_head && r < n_rows && __ballot(row_ends != 0) == 0) {
      skip_rows_without_edges(0);
      cur_end = (r < n_rows) ? bcast_i32(row_ends, (int)(r - rbase)) : 0x7fffffff;
    }
  }
  // Row r is complete inside this span: write it (or its head partial).
  auto finish_row = [&]() {
    head_reduce(acc);
    if (is_head) {
      store_vec(carry_head, acc);
    } else if (EXT && a.targets) {
      if (col_ok && cur_end > cur_start) atomic_add_vec(a.out + a.targets[r] * a.ldo + col, acc);
    } else {
      float* dst = a.out + r * a.ldo;
      if (a.mean) {
        const int deg = cur_end - cur_start;
        if (deg > 0) vscale(acc, 1.0f / (float)deg);
      }
      if (a.bias) {
        if (st_ok) vadd(acc, *reinterpret_cast<const vec_t*>(a.bias + col));
      }
      if (a.accumulate) {
        if (st_ok) vadd(acc, *reinterpret_cast<const vec_t*>(dst + col));
      }
      store_vec(dst, acc);
    }
    acc = vzero<V>();
  };

  for (int c0 = 0; c0 < n; c0 += CXG_WAVE) {
    const int cn = (n - c0) < CXG_WAVE ? (n - c0) : CXG_WAVE;
    int64_t my_src = 0;
    int64_t my_vrow = 0;
    float my_w = 0.f;
    if (lane < cn) {
      const int64_t pos = e0 + c0 + lane;
      my_src = (int64_t)stream_load(a.idx + pos);
      if (EXT) {
        if (a.rel) my_src += (int64_t)a.rel[pos] * a.rel_stride;
        if (a.src_map) my_src = a.src_map[my_src];
        if (a.mask && !a.mask[a.mask_perm ? a.mask_perm[pos] : pos]) my_src = -1;
      }
      if (PERM) my_vrow = stream_load(a.perm + pos);
      if (WMODE == 1 && !PERM) my_w = stream_load(a.val + pos);
    }
    // (The loads of a group sit under a condition each, and the compiler, whose count of requests in
    // flight is a guess at every join, waits for each gather before it issues the next.  Written without
    // the conditions the gathers of a group do stay in flight together -- and every kernel built on this
    // loop is slower for it, at any group size: multi-head forward 7.77 -> 8.03 ms, single head F = 256
    // on the 2.3 M-entry graph 0.325 -> 0.350 ms.  With eight waves per SIMD one gather per wave already
    // fills the fabric's queues; more only lengthens them.)
    for (int b = 0; b < cn; b += U) {
      vec_t v[U];
      float w[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int jj = b + u;
        if (jj < cn) {
          const int64_t src = bcast_i64(my_src, jj);
          const float* row = a.x + src * a.ldx;
          if (EXT && src < 0) v[u] = vzero<V>();
          else v[u] = col_ok ? *reinterpret_cast<const vec_t*>(row + col) : vzero<V>();
          if (WMODE == 1) {
            if (PERM) w[u] = a.val[bcast_i64(my_vrow, jj)];
            else w[u] = bcast_f32(my_w, jj);
          } else if (WMODE == 2) {
            const int64_t vrow = PERM ? bcast_i64(my_vrow, jj) : (e0 + c0 + jj);
            w[u] = col_ok ? a.val[vrow * a.heads + head_of_lane] : 0.f;
          }
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int jj = b + u;
        if (jj < cn) {
          const int j = c0 + jj;
          while (j >= cur_end) {
            finish_row();
            next_row(true);
          }
          if (WMODE == 0) vadd(acc, v[u]);
          else vfma(acc, v[u], w[u]);
          if constexpr (DOTG > 0) {
            const float p = lane_group_sum<DOTG>(vdot4(v[u], xr0));
            if ((lane & (DOTG - 1)) == 0) s_dot[wave][jj * kDotHeads + lane / DOTG] = p;
          }
        }
      }
    }
    if constexpr (DOTG > 0) {
      // the chunk's products leave through LDS: one vector store per edge and chunk instead of
      // one 4-byte store per (edge, head) between the gathers (stores and loads of a wave
      // complete in order, so every scattered store held up the next gathers)
      __builtin_amdgcn_wave_barrier();
      if (lane < cn) {
        const int64_t vrow = (PERM && !a.dot_at_edge) ? my_vrow : (e0 + c0 + lane);
        float* dst = a.dot_out + vrow * a.heads + blockIdx.y * kDotHeads;
        const float* src = &s_dot[wave][lane * kDotHeads];
        if constexpr (kDotHeads == 8) {
          *reinterpret_cast<float4*>(dst) = *reinterpret_cast<const float4*>(src);
          *reinterpret_cast<float4*>(dst + 4) = *reinterpret_cast<const float4*>(src + 4);
        } else if constexpr (kDotHeads == 4) {
          *reinterpret_cast<float4*>(dst) = *reinterpret_cast<const float4*>(src);
        } else if constexpr (kDotHeads == 2) {
          *reinterpret_cast<float2*>(dst) = *reinterpret_cast<const float2*>(src);
        } else {
          dst[0] = src[0];
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
  }

  // Rows that end at or before the span end, then the row (if any) that runs on.
  int64_t tail = -1;
  while (r < n_rows) {
    if (cur_end > n) {
      head_reduce(acc);
      if (is_head) {
        store_vec(carry_head, acc);
      } else if (cur_start < n) {
        store_vec(carry_tail, acc);
        tail = r;
      }
      break;
    }
    if (!(is_head || cur_start < n || last)) break;
    const bool own = last || cur_end < n;
    finish_row();
    next_row(own);
  }
  if (lane == 0 && blockIdx.y == 0) a.tail_row[3 * s] = tail;
}

// ----------------------------------------------------------------------------
// Narrow rows: several edges per gather instruction
// ----------------------------------------------------------------------------
// For rows of at most 32 * V floats a whole wave per edge leaves most lanes idle
// and the kernel is bound by one gather instruction per edge (F <= 64 took the
// same ~3.5 ms as F = 128 on the 61.9M-edge graph).  Here the wave is cut into
// G = 64 / L groups of L lanes (L * V >= F): one step gathers G consecutive edges
// of the current row, one per group, each group keeping its own partial sum; when
// the row ends the partials are added across groups with xor-shuffles and group 0
// writes the row.  Same spans, row walk, carry buffer and fix-up kernel as
// spmm_span_kernel.  WMODE 0 (sum / mean), 1 (one weight per edge) and 2 (one weight
// per edge and head; a lane's V columns lie in one head), weights optionally read
// through `perm`.
__device__ __forceinline__ int64_t shfl_i64(int64_t v, int src_lane) {
  const int lo = __shfl((int)(v & 0xffffffffll), src_lane, CXG_WAVE);
  const int hi = __shfl((int)(v >> 32), src_lane, CXG_WAVE);
  return ((int64_t)hi << 32) | (uint32_t)lo;
}
// bf16 rows: four values are 8 bytes; widened by a shift, narrowed with round-to-nearest-even
__device__ __forceinline__ float4 load_bf16x4(const uint16_t* p) {
  const uint2 u = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                     __uint_as_float(u.y & 0xffff0000u));
}
__device__ __forceinline__ unsigned pack_bf16x2(float lo, float hi) {
  typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
  v2bf t = {(__bf16)lo, (__bf16)hi};
  return __builtin_bit_cast(unsigned, t);
}
__device__ __forceinline__ void store_bf16x4(uint16_t* p, float4 v) {
  *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16x2(v.x, v.y), pack_bf16x2(v.z, v.w));
}
// The bits of a gathered piece as they come from memory: widening bf16 values belongs where the
// piece is used, not where it is requested -- a conversion next to the load makes the wave wait
// for that load before it requests the next one.
typedef unsigned raw2u __attribute__((ext_vector_type(2)));
typedef unsigned raw4u __attribute__((ext_vector_type(4)));
template <int V, int IO> struct RawPiece { using type = typename Vec<V>::type; };
template <> struct RawPiece<4, 1> { using type = raw2u; };
template <> struct RawPiece<4, 3> { using type = raw2u; };
template <> struct RawPiece<8, 1> { using type = raw4u; };
template <> struct RawPiece<8, 3> { using type = raw4u; };
__device__ __forceinline__ float widen_piece(float q) { return q; }
__device__ __forceinline__ float2 widen_piece(float2 q) { return q; }
__device__ __forceinline__ float4 widen_piece(float4 q) { return q; }
__device__ __forceinline__ float4 widen_piece(raw2u u) {
  return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                     __uint_as_float(u.y & 0xffff0000u));
}
__device__ __forceinline__ float8 widen_piece(raw4u u) {
  return float8{make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                            __uint_as_float(u.y & 0xffff0000u)),
                make_float4(__uint_as_float(u.z << 16), __uint_as_float(u.z & 0xffff0000u), __uint_as_float(u.w << 16),
                            __uint_as_float(u.w & 0xffff0000u))};
}
template <typename T> __device__ __forceinline__ T zero_piece();
template <> __device__ __forceinline__ float zero_piece<float>() { return 0.f; }
template <> __device__ __forceinline__ float2 zero_piece<float2>() { return make_float2(0.f, 0.f); }
template <> __device__ __forceinline__ float4 zero_piece<float4>() { return make_float4(0.f, 0.f, 0.f, 0.f); }
template <> __device__ __forceinline__ raw2u zero_piece<raw2u>() { return raw2u{0u, 0u}; }
template <> __device__ __forceinline__ raw4u zero_piece<raw4u>() { return raw4u{0u, 0u, 0u, 0u}; }
// eight values, 16 bytes
__device__ __forceinline__ float8 load_bf16x8(const uint16_t* p) {
  typedef unsigned v4u __attribute__((ext_vector_type(4)));
  const v4u u = *reinterpret_cast<const v4u*>(p);
  return float8{make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                            __uint_as_float(u.y & 0xffff0000u)),
                make_float4(__uint_as_float(u.z << 16), __uint_as_float(u.z & 0xffff0000u), __uint_as_float(u.w << 16),
                            __uint_as_float(u.w & 0xffff0000u))};
}
__device__ __forceinline__ void store_bf16x8(uint16_t* p, float8 v) {
  typedef unsigned v4u __attribute__((ext_vector_type(4)));
  const v4u u = {pack_bf16x2(v.lo.x, v.lo.y), pack_bf16x2(v.lo.z, v.lo.w), pack_bf16x2(v.hi.x, v.hi.y), pack_bf16x2(v.hi.z, v.hi.w)};
  *reinterpret_cast<v4u*>(p) = u;
}

// IO & 1: the rows of x are bf16 (ldx in elements); IO & 2: the rows of out are bf16 (ldo in
// elements) -- sums and carried partial rows stay fp32.  V == 4, or V == 8 with bf16 rows of x:
// a lane then gathers 16 bytes of a bf16 row like it does of an fp32 row, a 256-byte row takes 16
// lanes and a step gathers four edges instead of two (a pair row of the relational layer has
// three edges on average).
// HM > 1 (WMODE == 3): every edge carries HM weights and the gathered row is added HM times, once per
// weight, into HM output blocks of F floats: out[r, h, :] = sum_e val[e, h] * x[idx[e], :] (out rows
// and carried partial rows of HM * F floats).  One gather of F floats serves HM heads.
// DOT: beside the aggregation, dot_out[p] = <x[idx[p], :], dot_b[r, :]> for every edge position p of row r
// (the product of the gathered row with the row the sums go to).  A group forms its edge's product when
// the gathered row arrives; the products of a 64-edge chunk are collected lane by lane in one register
// (a scalar read of the group's first lane and a select, no memory) and leave with one contiguous store per chunk.  The row of dot_b for the
// next output row is requested one row ahead.
template <typename IdxT, int V, int L, int WMODE, bool PERM, int IO = 0, int HM = 1, bool DOT = false>
__global__ __launch_bounds__(kBlock) void spmm_group_kernel(SpmmArgs<IdxT> a) {
  static_assert(!DOT || (HM == 1 && IO == 0 && V == 4), "edge products: fp32 rows of 16-byte pieces, one weight per edge");
  static_assert(IO == 0 || V == 4 || (V == 8 && (IO & 1)), "bf16 rows are handled four or eight values at a time");
  static_assert(V != 8 || (IO & 1), "eight values per lane: bf16 rows of x only");
  static_assert((HM == 1) == (WMODE != 3), "several weights per edge are WMODE 3");
  static_assert(HM == 1 || (IO == 0 && !PERM), "several weights per edge: fp32 rows, weights in edge order");
  using vec_t = typename Vec<V>::type;
  using raw_t = typename RawPiece<V, IO>::type;
  constexpr int G = CXG_WAVE / L;
  // steps requested together inside long rows (eight values per lane: half as many -- the same edges in
  // flight, and registers for eight waves per SIMD)
  constexpr int UF = (V == 8 || HM > 1) ? (CXG_SPMM_GROUP_UF + 1) / 2 : CXG_SPMM_GROUP_UF;
  const int lane = lane_id();
  const int wave = uniform_i32(threadIdx.x >> 6);
  const int64_t s = (int64_t)blockIdx.x * kWavesPerBlock + wave;
  const int64_t n_rows = a.n_rows;
  const int64_t e_begin = (int64_t)a.ptr[0];
  const int64_t e_end = (int64_t)a.ptr[n_rows];
  const int64_t total = e_end - e_begin;
  const int T = a.T;
  const int64_t n_spans = total > 0 ? (total + T - 1) / T : 1;
  if (s >= n_spans) return;
  const bool last = (s == n_spans - 1);
  const int64_t e0 = e_begin + s * T;
  const int n = (int)((e_end - e0) < (int64_t)T ? (e_end - e0) : (int64_t)T);
  const int F = a.F;
  const int g = lane / L;
  const int col = (lane % L) * V;
  const bool col_ok = col < F;
  const bool writer = (g == 0) && col_ok;

  const int64_t r_lo = wave_lower_bound(a.ptr, n_rows, e0);
  bool is_head = (r_lo == n_rows) || ((int64_t)a.ptr[r_lo] > e0);
  int64_t r = is_head ? r_lo - 1 : r_lo;
  int64_t rbase = r;
  auto load_row_ends = [&](int64_t rb) -> int {
    int64_t q = rb + 1 + lane;
    if (q > n_rows) q = n_rows;
    const int64_t d = (int64_t)a.ptr[q] - e0;
    return (int)(d < (int64_t)n + 1 ? d : (int64_t)n + 1);
  };
  int row_ends = load_row_ends(rbase);
  int cur_start = is_head ? -1 : 0;
  int cur_end = (r < n_rows) ? bcast_i32(row_ends, 0) : 0x7fffffff;

  int head_of_lane = 0;
  if (WMODE == 2) head_of_lane = col_ok ? col / a.channels : 0;
  vec_t acc[HM];
#pragma unroll
  for (int h = 0; h < HM; ++h) acc[h] = vzero<V>();
  int row_take = 0;                          // most groups used by a step of the current row
  // DOT: the row of dot_b that belongs to output row r, and the one after it (requested a row ahead)
  vec_t brow = vzero<V>(), brow_next = vzero<V>();
  int64_t brow_next_row = -1;
  auto load_brow_row = [&](int64_t row) -> vec_t {
    return (row >= 0 && row < n_rows && col_ok) ? *reinterpret_cast<const vec_t*>(a.dot_b + row * a.ld_dot_b + col) : vzero<V>();
  };
  auto enter_row = [&]() {                    // r has changed
    if constexpr (DOT) {
      brow = (r == brow_next_row) ? brow_next : load_brow_row(r);
      brow_next_row = r + 1;
      brow_next = load_brow_row(brow_next_row);
    }
  };
  float* const carry_head = a.carry + (size_t)(2 * s) * F * HM;
  float* const carry_tail = carry_head + F * HM;

  // What finish_row leaves in a row without edges.
  auto store_empty_row = [&](int64_t row) {
    if ((a.accumulate && !a.bias) || !col_ok) return;
    if constexpr (HM > 1) {
#pragma unroll
      for (int h = 0; h < HM; ++h) *reinterpret_cast<vec_t*>(a.out + row * a.ldo + h * F + col) = vzero<V>();
      return;
    }
    if constexpr ((IO & 2) != 0) {
      uint16_t* d16 = reinterpret_cast<uint16_t*>(a.out) + row * a.ldo + col;
      *reinterpret_cast<uint2*>(d16) = make_uint2(0u, 0u);
      if constexpr (V == 8) *reinterpret_cast<uint2*>(d16 + 4) = make_uint2(0u, 0u);
      return;
    }
    float* dst = a.out + row * a.ldo;
    vec_t z = vzero<V>();
    if (a.bias) vadd(z, *reinterpret_cast<const vec_t*>(a.bias + col));
    if (a.accumulate) vadd(z, *reinterpret_cast<const vec_t*>(dst + col));
    *reinterpret_cast<vec_t*>(dst + col) = z;
  };
  // `own`: the rows without edges that follow the finished row belong to this span.  A whole
  // window of them is not walked row by row (see spmm_span_kernel): one search finds the end of
  // the run; the first run of a span is left to the fix-up kernel, later ones the groups store,
  // G rows at a time.
  bool run_left = false;                       // this span's slot holds a run
  if (lane == 0) { a.tail_row[3 * s + 1] = 0; a.tail_row[3 * s + 2] = 0; }
  auto skip_rows_without_edges = [&](int end_rel) {     // see spmm_span_kernel
    const int64_t first = r;
    int64_t q = r;
    for (int hop = 1;; ++hop) {
      q += CXG_WAVE;
      if (q >= n_rows) { q = rbase = n_rows; break; }
      if (hop == kRunWindows) {
        q += wave_lower_bound(a.ptr + q + 1, n_rows - q, e0 + end_rel + 1);
        rbase = q;
        if (q < n_rows) row_ends = load_row_ends(rbase);
        break;
      }
      const int w = load_row_ends(q);
      const unsigned long long busy = __ballot(w != end_rel);
      if (busy) {
        rbase = q;
        row_ends = w;
        q += __ffsll((long long)busy) - 1;
        break;
      }
    }
    r = q;
    if (r - first >= kRunWindows * CXG_WAVE && !run_left) {
      run_left = true;
      if (lane == 0) { a.tail_row[3 * s + 1] = first; a.tail_row[3 * s + 2] = r; }
    } else {
      for (int64_t row = first + g; row < r; row += G) store_empty_row(row);
    }
  };
  auto next_row = [&](bool own) {
    ++r;
    if (r - rbase == CXG_WAVE) {
      rbase = r;
      row_ends = load_row_ends(rbase);
      if (own && r < n_rows && __ballot(row_ends != cur_end) == 0) skip_rows_without_edges(cur_end);
    }
    cur_start = cur_end;
    cur_end = (r < n_rows) ? bcast_i32(row_ends, (int)(r - rbase)) : 0x7fffffff;
    is_head = false;
  };
  // the same for a span that starts with a window of rows without edges
  if (!is_head && r < n_rows && __ballot(row_ends != 0) == 0) {
    skip_rows_without_edges(0);
    cur_end = (r < n_rows) ? bcast_i32(row_ends, (int)(r - rbase)) : 0x7fffffff;
  }
  enter_row();
  // sum of the groups' partials, valid in group 0 afterwards
  auto reduce_groups = [&]() {
#pragma unroll
    for (int h = 0; h < HM; ++h) {
      if constexpr (L <= 1) { if (row_take > 1 / L) vshift_add<1>(acc[h]); }
      if constexpr (L <= 2) { if (row_take > 2 / L) vshift_add<2>(acc[h]); }
      if constexpr (L <= 4) { if (row_take > 4 / L) vshift_add<4>(acc[h]); }
      if constexpr (L <= 8) { if (row_take > 8 / L) vshift_add<8>(acc[h]); }
      if constexpr (L <= 16) { if (row_take > 16 / L) vshift_add<16>(acc[h]); }
      if constexpr (L <= 32) { if (row_take > 32 / L) vshift_add<32>(acc[h]); }
    }
  };
  auto store_vec = [&](float* dst, const vec_t (&v)[HM]) {
#pragma unroll
    for (int h = 0; h < HM; ++h) {
      if (writer) stream_store(dst + h * F + col, v[h]);
    }
  };
  auto finish_row = [&]() {
    reduce_groups();
    if (is_head) {
      store_vec(carry_head, acc);
    } else if constexpr (HM > 1) {
      store_vec(a.out + r * a.ldo, acc);
    } else if constexpr ((IO & 2) != 0) {
      if (a.mean) {
        const int deg = cur_end - cur_start;
        if (deg > 0) vscale(acc[0], 1.0f / (float)deg);
      }
      if constexpr (V == 4) {
        if (writer) store_bf16x4(reinterpret_cast<uint16_t*>(a.out) + r * a.ldo + col, acc[0]);
      } else if constexpr (V == 8) {
        if (writer) store_bf16x8(reinterpret_cast<uint16_t*>(a.out) + r * a.ldo + col, acc[0]);
      }
    } else {
      float* dst = a.out + r * a.ldo;
      if (a.mean) {
        const int deg = cur_end - cur_start;
        if (deg > 0) vscale(acc[0], 1.0f / (float)deg);
      }
      if (a.bias) {
        if (writer) vadd(acc[0], *reinterpret_cast<const vec_t*>(a.bias + col));
      }
      if (a.accumulate) {
        if (writer) vadd(acc[0], *reinterpret_cast<const vec_t*>(dst + col));
      }
      store_vec(dst, acc);
    }
#pragma unroll
    for (int h = 0; h < HM; ++h) acc[h] = vzero<V>();
    row_take = 0;
  };

  for (int c0 = 0; c0 < n; c0 += CXG_WAVE) {
    const int cn = (n - c0) < CXG_WAVE ? (n - c0) : CXG_WAVE;
    int64_t my_src = 0, my_vrow = 0;
    float my_w = 0.f;
    if (lane < cn) {
      const int64_t pos = e0 + c0 + lane;
      my_src = (int64_t)stream_load(a.idx + pos);
      if (PERM) my_vrow = stream_load(a.perm + pos);
      if (WMODE == 1 && !PERM) my_w = stream_load(a.val + pos);
    }
    // The chunk's ids and weights are complete from here on, and the compiler is made to know it: it
    // counts a wave's requests in flight statically, and inside the loops below it cannot tell how many
    // requests are younger than these loads, so every later look at one of these registers would wait
    // for everything in flight -- the previous row's store included, once per row on short rows.
    asm volatile("" : "+v"(my_src), "+v"(my_vrow), "+v"(my_w));
    // (the weight first: it comes out of a register that a load filled at the start of the chunk, and a
    // look at such a register behind a row request that may or may not have been issued -- the request
    // sits under a condition -- makes the compiler wait for everything in flight)
    auto gather = [&](int e_idx, bool act, raw_t& v, float (&w)[HM]) {
      if (WMODE == 1 && !PERM) w[0] = __shfl(my_w, e_idx & 63, CXG_WAVE);
      const int64_t src = shfl_i64(my_src, e_idx & 63);
      int64_t vrow = 0;
      if (WMODE != 0 && PERM) vrow = shfl_i64(my_vrow, e_idx & 63);
      if constexpr ((IO & 1) != 0) {
        v = (act && col_ok) ? *reinterpret_cast<const raw_t*>(reinterpret_cast<const uint16_t*>(a.x) + src * a.ldx + col)
                            : zero_piece<raw_t>();
      } else {
        v = (act && col_ok) ? *reinterpret_cast<const raw_t*>(a.x + src * a.ldx + col) : zero_piece<raw_t>();
      }
      if (WMODE == 1) {
        if (PERM) w[0] = act ? a.val[vrow] : 0.f;
      } else if (WMODE == 2) {
        if (!PERM) vrow = e0 + c0 + e_idx;
        w[0] = (act && col_ok) ? a.val[vrow * a.heads + head_of_lane] : 0.f;
      } else if (WMODE == 3) {
        // the HM weights of the edge: one address for all lanes of the group
        const float* wp = a.val + (e0 + c0 + e_idx) * HM;
        if constexpr (HM % 4 == 0) {
#pragma unroll
          for (int h = 0; h < HM; h += 4) {
            const float4 q = act ? *reinterpret_cast<const float4*>(wp + h) : make_float4(0.f, 0.f, 0.f, 0.f);
            w[h] = q.x; w[h + 1] = q.y; w[h + 2] = q.z; w[h + 3] = q.w;
          }
        } else {
#pragma unroll
          for (int h = 0; h < HM; ++h) w[h] = act ? wp[h] : 0.f;
        }
      }
    };
    auto add_edge = [&](const raw_t& v, const float (&w)[HM]) {
      if (WMODE == 0) {
        vadd(acc[0], widen_piece(v));
      } else {
#pragma unroll
        for (int h = 0; h < HM; ++h) vfma(acc[h], widen_piece(v), w[h]);
      }
    };
    // DOT: the product of chunk edge i ends up in lane i of my_dot
    float my_dot = 0.f;
    auto note_products = [&](const raw_t& v, int first_edge, int n_groups) {
      if constexpr (DOT) {
        const float total = lane_group_sum<L>(vdot4(widen_piece(v), brow));     // in the group's first lane
#pragma unroll
        for (int gi = 0; gi < G; ++gi) {
          if (gi < n_groups) {
            const int sv = __builtin_amdgcn_readlane((int)__float_as_uint(total), gi * L);
            if (lane == ((first_edge + gi) & 63)) my_dot = __uint_as_float((unsigned)sv);
          }
        }
      }
    };
    int j = 0;
    while (j < cn) {
      if (c0 + j >= cur_end) {
        do {
          finish_row();
          next_row(true);
        } while (c0 + j >= cur_end);
        enter_row();
      }
      const int left = (cur_end - (c0 + j)) < (cn - j) ? (cur_end - (c0 + j)) : (cn - j);
      if (left >= UF * G) {                   // long row: UF steps of G edges, loads first
        raw_t v[UF];
        float w[UF][HM];
#pragma unroll
        for (int u = 0; u < UF; ++u) gather(j + u * G + g, true, v[u], w[u]);
#pragma unroll
        for (int u = 0; u < UF; ++u) {
          add_edge(v[u], w[u]);
          note_products(v[u], j + u * G, G);
        }
        row_take = G;
        j += UF * G;
      } else {
        const int take = left < G ? left : G;
        raw_t v;
        float w[HM] = {};
        gather(j + g, g < take, v, w);
        add_edge(v, w);
        note_products(v, j, take);
        if (take > row_take) row_take = take;
        j += take;
      }
    }
    if constexpr (DOT) {
      if (lane < cn) stream_store(a.dot_out + (e0 + c0 + lane), my_dot);
    }
  }

  int64_t tail = -1;
  while (r < n_rows) {
    if (cur_end > n) {
      reduce_groups();
      if (is_head) {
        store_vec(carry_head, acc);
      } else if (cur_start < n) {
        store_vec(carry_tail, acc);
        tail = r;
      }
      break;
    }
    if (!(is_head || cur_start < n || last)) break;
    const bool own = last || cur_end < n;
    finish_row();
    next_row(own);
  }
  if (lane == 0) a.tail_row[3 * s] = tail;
}

constexpr int kRunHelpers = 16;   // fix-up waves that share one span's run of rows without edges

// One wave per span: if the span holds the tail partial of row t, add the head
// partials of the following spans that row t runs through, in span order.
template <typename IdxT, int V, bool GUARD>
__global__ __launch_bounds__(kBlock) void spmm_fixup_kernel(SpmmArgs<IdxT> a) {
  using vec_t = typename Vec<V>::type;
  const int lane = lane_id();
  const int wave = uniform_i32(threadIdx.x >> 6);
  const int64_t s = (int64_t)blockIdx.x * kWavesPerBlock + wave;
  const int64_t e_begin = (int64_t)a.ptr[0];
  const int64_t e_end = (int64_t)a.ptr[a.n_rows];
  const int64_t total = e_end - e_begin;
  const int T = a.T;
  const int64_t n_spans = total > 0 ? (total + T - 1) / T : 1;
  if (s >= n_spans) return;
  const int col = blockIdx.y * (CXG_WAVE * V) + lane * V;
  const bool col_ok = GUARD ? (col < a.F) : true;
  // Runs of rows without edges that the spans left behind: the run of span q is shared by the
  // waves q, q + 1, ..., q + J - 1 (modulo the span count), row by row in turn.  (Sixteen
  // helpers: with 64 the slot reads alone cost the headline launch 13 us.)
  const int64_t t_slot = a.tail_row[3 * s];       // issued with the slot reads below: one wait for both
  if (!a.targets && !(a.accumulate && !a.bias)) {
    const int64_t J = n_spans < kRunHelpers ? n_spans : kRunHelpers;
    int64_t rb = 0, re = 0;
    if (lane < J) {
      const int64_t q = (s - lane + n_spans) % n_spans;
      rb = a.tail_row[3 * q + 1];
      re = a.tail_row[3 * q + 2];
    }
    unsigned long long pending = __ballot(re > rb);
    while (pending) {
      const int j = __ffsll((long long)pending) - 1;
      pending &= pending - 1;
      const int64_t row_b = shfl_i64(rb, j), row_e = shfl_i64(re, j);
      for (int64_t row = row_b + j; row < row_e; row += J) {
        if (!col_ok) continue;
        if (a.out_bf16) {
          uint16_t* d16 = reinterpret_cast<uint16_t*>(a.out) + row * a.ldo + col;
          for (int k = 0; k < V; ++k) d16[k] = 0;
          continue;
        }
        float* dst = a.out + row * a.ldo;
        vec_t z = vzero<V>();
        if (a.bias) vadd(z, *reinterpret_cast<const vec_t*>(a.bias + col));
        if (a.accumulate) vadd(z, *reinterpret_cast<const vec_t*>(dst + col));
        *reinterpret_cast<vec_t*>(dst + col) = z;
      }
    }
  }
  const int64_t t = uniform_i64(t_slot);
  if (t < 0) return;
  if (!col_ok) return;
  const int F = a.F;
  const int64_t row_begin = (int64_t)a.ptr[t];
  const int64_t row_end = (int64_t)a.ptr[t + 1];
  const int64_t s_last = (row_end - 1 - e_begin) / T;
  // Head partials of the following spans, 16 independent loads at a time (a row that
  // covers thousands of spans would otherwise be one long chain of dependent loads);
  // the 16 running sums are combined in a fixed order, so the result is deterministic.
  constexpr int kChain = 16;
  vec_t part[kChain];
#pragma unroll
  for (int u = 0; u < kChain; ++u) part[u] = vzero<V>();
  int64_t q = s + 1;
  for (; q + kChain - 1 <= s_last; q += kChain) {      // whole groups: no guards, loads cluster
    vec_t got[kChain];
#pragma unroll
    for (int u = 0; u < kChain; ++u)
      got[u] = *reinterpret_cast<const vec_t*>(a.carry + (size_t)(2 * (q + u)) * F + col);
#pragma unroll
    for (int u = 0; u < kChain; ++u) vadd(part[u], got[u]);
  }
  for (; q <= s_last; ++q)
    vadd(part[0], *reinterpret_cast<const vec_t*>(a.carry + (size_t)(2 * q) * F + col));
  vec_t acc = *reinterpret_cast<const vec_t*>(a.carry + (size_t)(2 * s + 1) * F + col);
#pragma unroll
  for (int u = 0; u < kChain; ++u) vadd(acc, part[u]);
  if (a.targets) {
    atomic_add_vec(a.out + a.targets[t] * a.ldo + col, acc);
    return;
  }
  if (a.mean) vscale(acc, 1.0f / (float)(row_end - row_begin));
  if (a.out_bf16) {
    uint16_t* d16 = reinterpret_cast<uint16_t*>(a.out) + t * a.ldo + col;
    const float* av = reinterpret_cast<const float*>(&acc);
    for (int k = 0; k < V; ++k) d16[k] = (uint16_t)(pack_bf16x2(av[k], 0.f) & 0xffffu);
    return;
  }
  float* dst = a.out + t * a.ldo;
  if (a.bias) vadd(acc, *reinterpret_cast<const vec_t*>(a.bias + col));
  if (a.accumulate) vadd(acc, *reinterpret_cast<const vec_t*>(dst + col));
  *reinterpret_cast<vec_t*>(dst + col) = acc;
}

// Span length: 512 edges for large graphs, shorter for small ones so that the
// launch still has a few thousand waves.
int choose_span(int64_t n_edges_cap) {
  int64_t t = n_edges_cap / CXG_SPMM_SPAN_DIV;
  t = (t + 63) / 64 * 64;
  if (t < 64) t = 64;
  if (t > 512) t = 512;
  return (int)t;
}

struct Plan {
  int T;
  int64_t n_spans_cap;
  size_t tail_bytes;   // aligned
  size_t carry_bytes;
};

Plan make_plan(int64_t n_edges_cap, int64_t row_floats) {
  Plan p;
  p.T = choose_span(n_edges_cap);
  p.n_spans_cap = n_edges_cap > 0 ? ceil_div(n_edges_cap, p.T) : 1;
  p.tail_bytes = (size_t)((p.n_spans_cap * 3 * sizeof(int64_t) + 255) / 256 * 256);
  p.carry_bytes = (size_t)p.n_spans_cap * 2 * (size_t)row_floats * sizeof(float);
  return p;
}

template <typename IdxT, int V, bool GUARD, int WMODE, bool PERM, bool EXT, int DOTG = 0, bool PRE = false>
int launch_spmm(const SpmmArgs<IdxT>& a_in, int64_t n_spans_cap, hipStream_t stream) {
  // Gathers in flight per wave.  Measured on MI355X (61.9M-edge power-law graph):
  // with 32 waves per CU the memory system is already saturated, and issuing more
  // than one row gather per wave at a time only lengthens the queues and lowers
  // the L2 hit rate (F=128: 16 in flight 5.56 ms, 8: 4.94, 4: 4.51, 1: 4.31 ms).
  // 16-byte-per-lane gathers (V == 4) are flat from 1 to 8 and best at 8.
  // With the per-edge dot products four in flight are best: 62 registers instead of 80 keep eight
  // waves per SIMD resident (12.7 -> 11.5 ms on the GAT graph; 16 in flight: 14.5 ms).
  // (More gathers in flight for the narrow kernels on launches too small to fill the chip were
  // measured too: 15 k - 936 k edges of 47 floats, no gain or a loss.)
  constexpr int U = DOTG > 0 ? CXG_SPMM_U_DOT : ((V == 4) ? CXG_SPMM_U_V4 : CXG_SPMM_U);
  const int tile = CXG_WAVE * V;
  const int64_t n_ct = ceil_div(a_in.F, tile);
  SpmmArgs<IdxT> a = a_in;
  if (a.exact_edges > 0 && V <= 2) {
    // The edge count is known: lengthen the spans (never shorten: the workspace was sized for
    // the default) until all waves -- spans x column tiles -- are resident at once instead of
    // one full round and a partly filled second one.  The number of resident waves is what the
    // occupancy of THIS kernel allows on the chip.  Measured on the 2.33M-edge graph: F=128
    // 0.195 -> 0.161 ms; the 16-byte-per-lane kernels (V == 4, 8 gathers in flight) do not gain
    // from it (F=256: 0.337 -> 0.405 ms) and keep the default span length.
    static const int64_t resident_waves = [] {
      int blocks = 0, cus = 256;
      int dev = 0, n_cu = 0;
      if (hipGetDevice(&dev) == hipSuccess &&
          hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n_cu > 0)
        cus = n_cu;
      if (hipOccupancyMaxActiveBlocksPerMultiprocessor(
              &blocks, spmm_span_kernel<IdxT, V, GUARD, WMODE, PERM, EXT, U, DOTG, PRE>, kBlock, 0) != hipSuccess || blocks < 1)
        blocks = 4;
      return (int64_t)blocks * kWavesPerBlock * cus;
    }();
    int64_t t = ceil_div(ceil_div(a.exact_edges * n_ct, resident_waves), 64) * 64;
    if (t > 512) t = 512;
    if (t > a.T) {
      a.T = (int)t;
      n_spans_cap = ceil_div(a.exact_edges, a.T);
    }
  }
  dim3 grid((unsigned)ceil_div(n_spans_cap, kWavesPerBlock), (unsigned)n_ct, 1);
  dim3 block(kBlock, 1, 1);
  hipLaunchKernelGGL((spmm_span_kernel<IdxT, V, GUARD, WMODE, PERM, EXT, U, DOTG, PRE>), grid, block, 0, stream, a);
  CXG_LAUNCH_CHECK("spmm_span_kernel");
  if constexpr (PRE) {
    // the stored rows (and the carry rows) hold `channels` floats
    SpmmArgs<IdxT> f = a;
    f.F = a.channels;
    if (f.F % 128 == 0) {
      hipLaunchKernelGGL((spmm_fixup_kernel<IdxT, 2, false>), dim3(grid.x, (unsigned)(f.F / 128), 1), block, 0, stream, f);
    } else {
      hipLaunchKernelGGL((spmm_fixup_kernel<IdxT, 1, true>), dim3(grid.x, (unsigned)ceil_div(f.F, CXG_WAVE), 1), block, 0,
                         stream, f);
    }
  } else {
    hipLaunchKernelGGL((spmm_fixup_kernel<IdxT, V, GUARD>), grid, block, 0, stream, a);
  }
  CXG_LAUNCH_CHECK("spmm_fixup_kernel");
  return CXG_OK;
}

// Narrow rows (at most 32 lanes of the widest aligned vector): grouped-lane kernel.
// Returns 1 if it launched, 0 if the shape is not narrow, < 0 on a launch error.
template <typename IdxT, int WMODE, bool PERM>
int launch_group(const SpmmArgs<IdxT>& a, int64_t n_spans_cap, hipStream_t stream) {
  const uintptr_t align_bits = (uintptr_t)a.x | (uintptr_t)a.out | (uintptr_t)a.carry | (uintptr_t)a.bias |
                               (uintptr_t)(a.ldx * 4) | (uintptr_t)(a.ldo * 4) | (uintptr_t)(a.F * 4);
  const int unit = (WMODE == 2) ? a.channels : a.F;
  int v = 1;
  for (int t = 2; t <= 4; t *= 2) {
    if (unit % t != 0 || a.F % t != 0 || (align_bits & (uintptr_t)(4 * t - 1)) != 0) break;
    v = t;
  }
  const int lanes = (int)ceil_div(a.F, v);
  if (lanes > 32) return 0;
  int L = 4;
  while (L < lanes) L <<= 1;
  const dim3 grid((unsigned)ceil_div(n_spans_cap, kWavesPerBlock), 1, 1), block(kBlock, 1, 1);
  bool done = false;
#define CXG_GROUP(VV, LL)                                                                        \
  if (!done && v == VV && L == LL) {                                                             \
    hipLaunchKernelGGL((spmm_group_kernel<IdxT, VV, LL, WMODE, PERM>), grid, block, 0, stream, a); \
    done = true;                                                                                 \
  }
  CXG_GROUP(4, 4) CXG_GROUP(4, 8) CXG_GROUP(4, 16) CXG_GROUP(4, 32)
  CXG_GROUP(2, 4) CXG_GROUP(2, 8) CXG_GROUP(2, 16) CXG_GROUP(2, 32)
  CXG_GROUP(1, 4) CXG_GROUP(1, 8) CXG_GROUP(1, 16) CXG_GROUP(1, 32)
#undef CXG_GROUP
  if (!done) return 0;
  CXG_LAUNCH_CHECK("spmm_group_kernel");
  if (a.F % 128 == 0 && v >= 2) {
    hipLaunchKernelGGL((spmm_fixup_kernel<IdxT, 2, false>), dim3(grid.x, (unsigned)(a.F / 128), 1), block, 0, stream, a);
  } else {
    const dim3 fgrid(grid.x, (unsigned)ceil_div(a.F, CXG_WAVE), 1);
    hipLaunchKernelGGL((spmm_fixup_kernel<IdxT, 1, true>), fgrid, block, 0, stream, a);
  }
  CXG_LAUNCH_CHECK("spmm_fixup_kernel");
  return 1;
}

template <typename IdxT, int WMODE, bool PERM, bool EXT = false>
int dispatch_shape(const SpmmArgs<IdxT>& a, int64_t n_spans_cap, hipStream_t stream) {
  if constexpr (!EXT) {
    const int rc = launch_group<IdxT, WMODE, PERM>(a, n_spans_cap, stream);
    if (rc != 0) return rc < 0 ? rc : CXG_OK;
  }
  // widest vector that divides the row (and the head, for per-head weights) and
  // keeps every access aligned; among those the one needing the fewest column
  // tiles, ties to the narrower vector (more lanes busy).
  const uintptr_t align_bits = (uintptr_t)a.x | (uintptr_t)a.out | (uintptr_t)a.carry | (uintptr_t)a.bias |
                               (uintptr_t)(a.ldx * 4) | (uintptr_t)(a.ldo * 4) | (uintptr_t)(a.F * 4);
  int unit = (WMODE == 2) ? a.channels : a.F;
  int best_v = 1;
  int64_t best_tiles = ceil_div(a.F, CXG_WAVE);
  for (int v = 2; v <= 4; v *= 2) {
    if (unit % v != 0 || (align_bits & (uintptr_t)(4 * v - 1)) != 0) break;
    const int64_t tiles = ceil_div(a.F, CXG_WAVE * v);
    if (tiles < best_tiles) { best_tiles = tiles; best_v = v; }
  }
  const bool guard = (best_tiles * CXG_WAVE * best_v != a.F);
#define CXG_CASE(VV)                                                                  \
  if (best_v == VV) {                                                                  \
    return guard ? launch_spmm<IdxT, VV, true, WMODE, PERM, EXT>(a, n_spans_cap, stream)   \
                 : launch_spmm<IdxT, VV, false, WMODE, PERM, EXT>(a, n_spans_cap, stream); \
  }
  CXG_CASE(1) CXG_CASE(2) CXG_CASE(4)
#undef CXG_CASE
  return set_error(CXG_ERR_UNSUPPORTED, "no kernel for vector width %d", best_v);
}

struct SpmmExt {
  const uint8_t* mask = nullptr;
  const int64_t* mask_perm = nullptr;
  const int32_t* rel = nullptr;
  int64_t rel_stride = 0;
  const int64_t* src_map = nullptr;
  const int64_t* targets = nullptr;
};

struct SpmmDot {
  const float* b = nullptr;     // [n_rows, heads, channels], row stride ld_b
  int64_t ld_b = 0;
  float* out = nullptr;         // [n_val_rows, heads]
  bool at_edge = false;         // rows of `out` at the edge's position in idx, not at perm[position]
};

template <typename IdxT>
int spmm_common(const IdxT* ptr, const IdxT* idx, const float* val, const int64_t* perm,
                const float* x, int64_t ldx, float* out, int64_t ldo, int64_t n_rows,
                int64_t n_edges_cap, int heads, int channels, unsigned flags, void* workspace,
                size_t workspace_bytes, void* stream, const SpmmExt* ext = nullptr,
                const SpmmDot* dot = nullptr, const float* bias = nullptr, bool prereduce = false) {
  CXG_REQUIRE(n_rows >= 0 && n_edges_cap >= 0, CXG_ERR_ARG, "negative size");
  CXG_REQUIRE(heads >= 1 && channels >= 1, CXG_ERR_ARG, "heads/channels must be >= 1");
  CXG_REQUIRE((int64_t)heads * channels <= (1 << 20), CXG_ERR_UNSUPPORTED, "row too wide");
  CXG_REQUIRE((flags & ~(CXG_SPMM_MEAN | CXG_SPMM_ACCUMULATE | CXG_SPMM_HINT_EXACT_EDGES)) == 0, CXG_ERR_ARG,
              "unknown flag");
  if (n_rows == 0) return CXG_OK;
  CXG_REQUIRE(ptr && out, CXG_ERR_ARG, "null ptr/out");
  CXG_REQUIRE(n_edges_cap == 0 || (idx && x), CXG_ERR_ARG, "null idx/x");
  const int F = heads * channels;
  CXG_REQUIRE(ldx >= F && ldo >= (prereduce ? channels : F), CXG_ERR_ARG, "row stride smaller than row");
  CXG_REQUIRE(!perm || val, CXG_ERR_ARG, "val_perm without val");
  const Plan plan = make_plan(n_edges_cap, F);
  CXG_REQUIRE(workspace && workspace_bytes >= plan.tail_bytes + plan.carry_bytes, CXG_ERR_WORKSPACE,
              "workspace of %zu bytes needed, %zu given", plan.tail_bytes + plan.carry_bytes,
              workspace_bytes);
  CXG_REQUIRE(((uintptr_t)workspace & 255) == 0, CXG_ERR_WORKSPACE, "workspace must be 256-byte aligned");

  SpmmArgs<IdxT> a;
  a.ptr = ptr; a.idx = idx; a.x = x; a.out = out; a.val = val; a.perm = perm;
  a.ldx = ldx; a.ldo = ldo; a.n_rows = n_rows; a.F = F; a.heads = heads; a.channels = channels;
  a.T = plan.T;
  a.exact_edges = (flags & CXG_SPMM_HINT_EXACT_EDGES) ? n_edges_cap : 0;
  a.mean = (flags & CXG_SPMM_MEAN) ? 1 : 0;
  a.accumulate = (flags & CXG_SPMM_ACCUMULATE) ? 1 : 0;
  a.tail_row = reinterpret_cast<int64_t*>(workspace);
  a.carry = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + plan.tail_bytes);
  a.mask = nullptr; a.mask_perm = nullptr; a.rel = nullptr; a.rel_stride = 0;
  a.src_map = nullptr; a.targets = nullptr;
  a.dot_b = nullptr; a.ld_dot_b = 0; a.dot_out = nullptr; a.dot_at_edge = 0;
  a.bias = bias;
  a.out_bf16 = 0;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (ext) {
    CXG_REQUIRE(!val, CXG_ERR_UNSUPPORTED, "extended gather takes no edge weights");
    CXG_REQUIRE(!(ext->targets && a.mean), CXG_ERR_ARG, "targets cannot be combined with mean");
    a.mask = ext->mask; a.mask_perm = ext->mask_perm; a.rel = ext->rel; a.rel_stride = ext->rel_stride;
    a.src_map = ext->src_map; a.targets = ext->targets;
    if constexpr (sizeof(IdxT) == 8) return dispatch_shape<IdxT, 0, false, true>(a, plan.n_spans_cap, st);
    return set_error(CXG_ERR_UNSUPPORTED, "extended gather needs int64 indices");
  }
  if (dot) {
    if constexpr (sizeof(IdxT) == 8) {
      CXG_REQUIRE(val && dot->b && dot->out, CXG_ERR_ARG, "null val/dot_b/dot_out");
      CXG_REQUIRE(dot->ld_b >= F, CXG_ERR_ARG, "row stride of dot_b smaller than row");
      const uintptr_t align_bits = (uintptr_t)x | (uintptr_t)out | (uintptr_t)a.carry | (uintptr_t)dot->b |
                                   (uintptr_t)a.bias |
                                   (uintptr_t)(ldx * 4) | (uintptr_t)(ldo * 4) | (uintptr_t)(dot->ld_b * 4);
      if (heads == 1 && F <= 128 && F % 4 == 0 && F >= 16 && (align_bits & 15) == 0 && perm && dot->at_edge && !a.mean &&
          !a.accumulate && !a.bias) {
        // narrow single-head rows: the grouped-lane kernel forms the products (weights through perm,
        // products at the edge's own position)
        a.dot_b = dot->b; a.ld_dot_b = dot->ld_b; a.dot_out = dot->out; a.dot_at_edge = 1;
        // the lane groups of the plain weighted aggregation of this width: the sums agree bit for bit
        const int L = F > 64 ? 32 : (F > 32 ? 16 : (F > 16 ? 8 : 4));
        const dim3 grid((unsigned)ceil_div(plan.n_spans_cap, kWavesPerBlock), 1, 1), block(kBlock, 1, 1);
        if (L == 32) hipLaunchKernelGGL((spmm_group_kernel<IdxT, 4, 32, 1, true, 0, 1, true>), grid, block, 0, st, a);
        else if (L == 16) hipLaunchKernelGGL((spmm_group_kernel<IdxT, 4, 16, 1, true, 0, 1, true>), grid, block, 0, st, a);
        else if (L == 8) hipLaunchKernelGGL((spmm_group_kernel<IdxT, 4, 8, 1, true, 0, 1, true>), grid, block, 0, st, a);
        else hipLaunchKernelGGL((spmm_group_kernel<IdxT, 4, 4, 1, true, 0, 1, true>), grid, block, 0, st, a);
        CXG_LAUNCH_CHECK("spmm_group_kernel");
        if (F % 128 == 0) {
          hipLaunchKernelGGL((spmm_fixup_kernel<IdxT, 2, false>), dim3(grid.x, (unsigned)(F / 128), 1), block, 0, st, a);
        } else {
          hipLaunchKernelGGL((spmm_fixup_kernel<IdxT, 1, true>), dim3(grid.x, (unsigned)ceil_div(F, CXG_WAVE), 1), block, 0, st, a);
        }
        CXG_LAUNCH_CHECK("spmm_fixup_kernel");
        return CXG_OK;
      }
      CXG_REQUIRE(F % 256 == 0 && (align_bits & 15) == 0 &&
                      (channels == 32 || channels == 64 || channels == 128 || channels == 256),
                  CXG_ERR_UNSUPPORTED, "spmm with dot products needs heads*channels %% 256 == 0, channels in "
                  "{32, 64, 128, 256} and 16-byte aligned rows");
      a.dot_b = dot->b; a.ld_dot_b = dot->ld_b; a.dot_out = dot->out; a.dot_at_edge = dot->at_edge ? 1 : 0;
#define CXG_DOT(WM, GG)                                                                          \
  return perm ? launch_spmm<IdxT, 4, false, WM, true, false, GG>(a, plan.n_spans_cap, st)          \
              : launch_spmm<IdxT, 4, false, WM, false, false, GG>(a, plan.n_spans_cap, st)
      if (heads == 1) { CXG_DOT(1, 64); }
      if (channels == 32) { CXG_DOT(2, 8); }
      if (channels == 64) { CXG_DOT(2, 16); }
      if (channels == 128) { CXG_DOT(2, 32); }
      CXG_DOT(2, 64);
#undef CXG_DOT
    }
    return set_error(CXG_ERR_UNSUPPORTED, "spmm with dot products needs int64 indices");
  }
  if (prereduce) {
    if constexpr (sizeof(IdxT) == 8) {
      CXG_REQUIRE(val && heads > 1, CXG_ERR_ARG, "head pre-reduction needs per-head weights and more than one head");
      CXG_REQUIRE(!a.mean, CXG_ERR_ARG, "head pre-reduction cannot be combined with mean");
      // the row of heads x channels floats must be exactly one column tile of 64 lanes x V floats
      int v = 0;
      for (int t = 4; t >= 1; t /= 2)
        if (F == CXG_WAVE * t && channels % t == 0) { v = t; break; }
      const uintptr_t align_bits = (uintptr_t)x | (uintptr_t)out | (uintptr_t)a.carry | (uintptr_t)a.bias |
                                   (uintptr_t)(ldx * 4) | (uintptr_t)(ldo * 4) | (uintptr_t)(channels * 4);
      CXG_REQUIRE(v > 0 && (align_bits & (uintptr_t)(4 * v - 1)) == 0 && (heads & (heads - 1)) == 0, CXG_ERR_UNSUPPORTED,
                  "head pre-reduction in the kernel needs heads * channels in {64, 128, 256}, a power-of-two head "
                  "count and aligned rows");
#define CXG_PRE(VV)                                                                                       \
  if (v == VV)                                                                                            \
    return perm ? launch_spmm<IdxT, VV, false, 2, true, false, 0, true>(a, plan.n_spans_cap, st)           \
                : launch_spmm<IdxT, VV, false, 2, false, false, 0, true>(a, plan.n_spans_cap, st)
      CXG_PRE(4); CXG_PRE(2); CXG_PRE(1);
#undef CXG_PRE
    }
    return set_error(CXG_ERR_UNSUPPORTED, "head pre-reduction needs int64 indices");
  }
  if (!val) return dispatch_shape<IdxT, 0, false>(a, plan.n_spans_cap, st);
  if constexpr (sizeof(IdxT) == 8) {
    if (heads == 1) {
      return perm ? dispatch_shape<IdxT, 1, true>(a, plan.n_spans_cap, st)
                  : dispatch_shape<IdxT, 1, false>(a, plan.n_spans_cap, st);
    }
    return perm ? dispatch_shape<IdxT, 2, true>(a, plan.n_spans_cap, st)
                : dispatch_shape<IdxT, 2, false>(a, plan.n_spans_cap, st);
  }
  return set_error(CXG_ERR_UNSUPPORTED, "weighted SpMM needs int64 indices");
}

// Device address of `scratch` on the current device, looked up on the first call there.
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

int static_scratch(void** out) {
  int dev = -1;
  CXG_HIP_CHECK(hipGetDevice(&dev));
  CXG_REQUIRE(dev >= 0 && dev < kMaxDevices, CXG_ERR_UNSUPPORTED, "device ordinal %d out of range", dev);
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    CXG_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    CXG_REQUIRE(p != nullptr, CXG_ERR_HIP, "hipGetSymbolAddress returned a null address");
    g_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return CXG_OK;
}

}  // namespace
}  // namespace cxg

extern "C" {

size_t cxg_spmm_workspace_bytes(int64_t n_edges_cap, int64_t row_floats) {
  if (n_edges_cap < 0 || row_floats < 1) return 0;
  const cxg::Plan p = cxg::make_plan(n_edges_cap, row_floats);
  return p.tail_bytes + p.carry_bytes;
}

int cxg_spmm_sum_f32(const int64_t* ptr, const int64_t* idx, const float* x, int64_t ldx,
                     float* out, int64_t ldo, int64_t n_rows, int64_t n_edges_cap, int feat,
                     unsigned flags, void* workspace, size_t workspace_bytes, void* stream) {
  return cxg::spmm_common<int64_t>(ptr, idx, nullptr, nullptr, x, ldx, out, ldo, n_rows,
                                   n_edges_cap, 1, feat, flags, workspace, workspace_bytes, stream);
}

int cxg_spmm_sum_f32_noalloc(const int64_t* ptr, const int64_t* idx, const float* x, int64_t ldx,
                             float* out, int64_t ldo, int64_t n_rows, int64_t n_edges_cap, int feat,
                             unsigned flags, void* stream) {
  CXG_REQUIRE(n_edges_cap >= 0 && feat >= 1, CXG_ERR_ARG, "negative size");
  const cxg::Plan p = cxg::make_plan(n_edges_cap, feat);
  const size_t need = p.tail_bytes + p.carry_bytes;
  CXG_REQUIRE(need <= (size_t)CXG_SPMM_NOALLOC_SCRATCH_BYTES, CXG_ERR_WORKSPACE,
              "cxg_spmm_sum_f32_noalloc: %lld edges of %d floats need %zu bytes of scratch, the built-in "
              "buffer holds %zu; use cxg_spmm_sum_f32 with a workspace",
              (long long)n_edges_cap, feat, need, (size_t)CXG_SPMM_NOALLOC_SCRATCH_BYTES);
  void* ws = nullptr;
  const int rc = cxg::static_scratch(&ws);
  if (rc != CXG_OK) return rc;
  return cxg::spmm_common<int64_t>(ptr, idx, nullptr, nullptr, x, ldx, out, ldo, n_rows, n_edges_cap,
                                   1, feat, flags, ws, (size_t)CXG_SPMM_NOALLOC_SCRATCH_BYTES, stream);
}

int cxg_spmm_sum_f32_i32(const int32_t* ptr, const int32_t* idx, const float* x, int64_t ldx,
                         float* out, int64_t ldo, int64_t n_rows, int64_t n_edges_cap, int feat,
                         unsigned flags, void* workspace, size_t workspace_bytes, void* stream) {
  return cxg::spmm_common<int32_t>(ptr, idx, nullptr, nullptr, x, ldx, out, ldo, n_rows,
                                   n_edges_cap, 1, feat, flags, workspace, workspace_bytes, stream);
}

int cxg_spmm_weighted_f32(const int64_t* ptr, const int64_t* idx, const float* val,
                          const int64_t* val_perm, const float* x, int64_t ldx, float* out,
                          int64_t ldo, int64_t n_rows, int64_t n_edges_cap, int heads, int channels,
                          unsigned flags, void* workspace, size_t workspace_bytes, void* stream) {
  if (!val) return cxg::set_error(CXG_ERR_ARG, "val is null");
  return cxg::spmm_common<int64_t>(ptr, idx, val, val_perm, x, ldx, out, ldo, n_rows, n_edges_cap,
                                   heads, channels, flags, workspace, workspace_bytes, stream);
}

int cxg_spmm_prereduce_f32(const int64_t* ptr, const int64_t* idx, const float* val, const int64_t* val_perm,
                           const float* x, int64_t ldx, float* out, int64_t ldo, int64_t n_rows, int64_t n_edges_cap,
                           int heads, int channels, unsigned flags, void* workspace, size_t workspace_bytes,
                           void* stream) {
  if (!val) return cxg::set_error(CXG_ERR_ARG, "val is null");
  return cxg::spmm_common<int64_t>(ptr, idx, val, val_perm, x, ldx, out, ldo, n_rows, n_edges_cap, heads, channels,
                                   flags, workspace, workspace_bytes, stream, nullptr, nullptr, nullptr, true);
}

// single-head aggregation of rows of at most 128 values with bf16 rows on either side
int cxg_spmm_bf16_rows(const int64_t* ptr, const int64_t* idx, const float* val, const int64_t* val_perm, const void* x,
                       int64_t ldx, int x_bf16, void* out, int64_t ldo, int out_bf16, int64_t n_rows, int64_t n_edges_cap,
                       int feat, unsigned flags, void* workspace, size_t workspace_bytes, void* stream) {
  using namespace cxg;
  CXG_REQUIRE(n_rows >= 0 && n_edges_cap >= 0, CXG_ERR_ARG, "negative size");
  CXG_REQUIRE((flags & ~(CXG_SPMM_MEAN | CXG_SPMM_HINT_EXACT_EDGES)) == 0, CXG_ERR_ARG, "unknown flag");
  CXG_REQUIRE(x_bf16 || out_bf16, CXG_ERR_ARG, "fp32 rows on both sides: use cxg_spmm_sum_f32 / cxg_spmm_weighted_f32");
  CXG_REQUIRE(feat >= 4 && feat <= 128 && feat % 4 == 0, CXG_ERR_UNSUPPORTED, "bf16 rows: 4 <= feat <= 128, a multiple of 4");
  if (n_rows == 0) return CXG_OK;
  CXG_REQUIRE(ptr && out && (n_edges_cap == 0 || (idx && x)), CXG_ERR_ARG, "null pointer");
  CXG_REQUIRE(ldx >= feat && ldo >= feat && ldx % 4 == 0 && ldo % 4 == 0, CXG_ERR_ARG, "row strides: at least feat, multiples of 4");
  CXG_REQUIRE((((uintptr_t)x | (uintptr_t)out) & 15) == 0, CXG_ERR_ARG, "rows must be 16-byte aligned");
  CXG_REQUIRE(!val_perm || val, CXG_ERR_ARG, "val_perm without val");
  const Plan plan = make_plan(n_edges_cap, feat);
  CXG_REQUIRE(workspace && workspace_bytes >= plan.tail_bytes + plan.carry_bytes && ((uintptr_t)workspace & 255) == 0,
              CXG_ERR_WORKSPACE, "workspace of %zu bytes (256-byte aligned) needed", plan.tail_bytes + plan.carry_bytes);
  SpmmArgs<int64_t> a;
  a.ptr = ptr; a.idx = idx; a.x = reinterpret_cast<const float*>(x); a.out = reinterpret_cast<float*>(out);
  a.val = val; a.perm = val_perm; a.ldx = ldx; a.ldo = ldo; a.n_rows = n_rows; a.F = feat; a.heads = 1; a.channels = feat;
  a.T = plan.T; a.exact_edges = 0; a.mean = (flags & CXG_SPMM_MEAN) ? 1 : 0; a.accumulate = 0;
  a.tail_row = reinterpret_cast<int64_t*>(workspace);
  a.carry = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + plan.tail_bytes);
  a.mask = nullptr; a.mask_perm = nullptr; a.rel = nullptr; a.rel_stride = 0; a.src_map = nullptr; a.targets = nullptr;
  a.dot_b = nullptr; a.ld_dot_b = 0; a.dot_out = nullptr; a.dot_at_edge = 0; a.bias = nullptr; a.out_bf16 = out_bf16 ? 1 : 0;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  // 16 bytes of a bf16 row per lane where the rows allow it (eight values: feat and the strides multiples
  // of 8) and the output rows have four edges or more on average: with shorter rows the wider lanes'
  // longer reduction and store at every row end cost more than the halved gather steps save (8.2 M pair
  // rows of 2.4 edges: 2.13 against 1.88 ms; 1 M rows of 8 edges: 0.63 against 0.76 ms)
  const bool v8 = x_bf16 && feat % 8 == 0 && feat >= 32 && ldx % 8 == 0 && (!out_bf16 || ldo % 8 == 0) &&
                  n_edges_cap >= 4 * n_rows;
  const int lanes = v8 ? feat / 8 : feat / 4;
  int L = 4;
  while (L < lanes) L <<= 1;
  const dim3 grid((unsigned)ceil_div(plan.n_spans_cap, kWavesPerBlock), 1, 1), block(kBlock, 1, 1);
  const int io = (x_bf16 ? 1 : 0) | (out_bf16 ? 2 : 0);
  const int wmode = val ? 1 : 0;
  bool done = false;
#define CXG_IO8(LL, WM, PM, IOV)                                                                             \
  if (!done && v8 && L == LL && wmode == WM && (val_perm != nullptr) == PM && io == IOV) {                    \
    hipLaunchKernelGGL((spmm_group_kernel<int64_t, 8, LL, WM, PM, IOV>), grid, block, 0, st, a);               \
    done = true;                                                                                             \
  }
#define CXG_IO8_L(LL)                                                                                         \
  CXG_IO8(LL, 0, false, 1) CXG_IO8(LL, 0, false, 3) CXG_IO8(LL, 1, false, 1) CXG_IO8(LL, 1, false, 3)           \
  CXG_IO8(LL, 1, true, 1) CXG_IO8(LL, 1, true, 3)
  CXG_IO8_L(4) CXG_IO8_L(8) CXG_IO8_L(16)
#undef CXG_IO8_L
#undef CXG_IO8
#define CXG_IO(LL, WM, PM, IOV)                                                                              \
  if (!done && L == LL && wmode == WM && (val_perm != nullptr) == PM && io == IOV) {                          \
    hipLaunchKernelGGL((spmm_group_kernel<int64_t, 4, LL, WM, PM, IOV>), grid, block, 0, st, a);               \
    done = true;                                                                                             \
  }
#define CXG_IO_L(LL)                                                                                          \
  CXG_IO(LL, 0, false, 1) CXG_IO(LL, 0, false, 2) CXG_IO(LL, 0, false, 3)                                       \
  CXG_IO(LL, 1, false, 1) CXG_IO(LL, 1, false, 2) CXG_IO(LL, 1, false, 3)                                       \
  CXG_IO(LL, 1, true, 1) CXG_IO(LL, 1, true, 2) CXG_IO(LL, 1, true, 3)
  CXG_IO_L(4) CXG_IO_L(8) CXG_IO_L(16) CXG_IO_L(32)
#undef CXG_IO_L
#undef CXG_IO
  CXG_REQUIRE(done, CXG_ERR_UNSUPPORTED, "no kernel for this combination");
  CXG_LAUNCH_CHECK("spmm_group_kernel");
  if (feat % 128 == 0) {
    hipLaunchKernelGGL((spmm_fixup_kernel<int64_t, 2, false>), dim3(grid.x, (unsigned)(feat / 128), 1), block, 0, st, a);
  } else {
    hipLaunchKernelGGL((spmm_fixup_kernel<int64_t, 1, true>), dim3(grid.x, (unsigned)ceil_div(feat, CXG_WAVE), 1), block, 0, st, a);
  }
  CXG_LAUNCH_CHECK("spmm_fixup_kernel");
  return CXG_OK;
}

// out[r, h, :] = sum_e val[e, h] * x[idx[e], :]: one gathered row of `feat` floats per edge, `heads` weights
int cxg_spmm_weighted_heads_f32(const int64_t* ptr, const int64_t* idx, const float* val, const float* x, int64_t ldx,
                                float* out, int64_t ldo, int64_t n_rows, int64_t n_edges_cap, int heads, int feat,
                                unsigned flags, void* workspace, size_t workspace_bytes, void* stream) {
  using namespace cxg;
  CXG_REQUIRE(n_rows >= 0 && n_edges_cap >= 0, CXG_ERR_ARG, "negative size");
  CXG_REQUIRE((flags & ~CXG_SPMM_HINT_EXACT_EDGES) == 0, CXG_ERR_ARG, "unknown flag");
  CXG_REQUIRE((heads == 2 || heads == 4 || heads == 8) && feat >= 20 && feat <= 128 && feat % 4 == 0, CXG_ERR_UNSUPPORTED,
              "heads = %d, feat = %d: takes 2, 4 or 8 heads and 20 <= feat <= 128, a multiple of 4", heads, feat);
  if (n_rows == 0) return CXG_OK;
  CXG_REQUIRE(ptr && out && (n_edges_cap == 0 || (idx && x && val)), CXG_ERR_ARG, "null pointer");
  CXG_REQUIRE(ldx >= feat && ldo >= (int64_t)heads * feat && ldx % 4 == 0 && ldo % 4 == 0, CXG_ERR_ARG,
              "row strides: at least feat / heads * feat, multiples of 4");
  CXG_REQUIRE((((uintptr_t)x | (uintptr_t)out | (uintptr_t)val) & 15) == 0, CXG_ERR_ARG, "x, out and val must be 16-byte aligned");
  const Plan plan = make_plan(n_edges_cap, (int64_t)heads * feat);
  CXG_REQUIRE(workspace && workspace_bytes >= plan.tail_bytes + plan.carry_bytes && ((uintptr_t)workspace & 255) == 0,
              CXG_ERR_WORKSPACE, "workspace of %zu bytes (256-byte aligned) needed", plan.tail_bytes + plan.carry_bytes);
  SpmmArgs<int64_t> a;
  a.ptr = ptr; a.idx = idx; a.x = x; a.out = out; a.val = val; a.perm = nullptr; a.ldx = ldx; a.ldo = ldo;
  a.n_rows = n_rows; a.F = feat; a.heads = heads; a.channels = feat;
  a.T = plan.T; a.exact_edges = 0; a.mean = 0; a.accumulate = 0;
  a.tail_row = reinterpret_cast<int64_t*>(workspace);
  a.carry = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + plan.tail_bytes);
  a.mask = nullptr; a.mask_perm = nullptr; a.rel = nullptr; a.rel_stride = 0; a.src_map = nullptr; a.targets = nullptr;
  a.dot_b = nullptr; a.ld_dot_b = 0; a.dot_out = nullptr; a.dot_at_edge = 0; a.bias = nullptr; a.out_bf16 = 0;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const int L = feat > 64 ? 32 : (feat > 32 ? 16 : 8);
  const dim3 grid((unsigned)ceil_div(plan.n_spans_cap, kWavesPerBlock), 1, 1), block(kBlock, 1, 1);
  bool done = false;
#define CXG_HM(LL, HH)                                                                                 \
  if (!done && L == LL && heads == HH) {                                                               \
    hipLaunchKernelGGL((spmm_group_kernel<int64_t, 4, LL, 3, false, 0, HH>), grid, block, 0, st, a);     \
    done = true;                                                                                       \
  }
  CXG_HM(8, 2) CXG_HM(8, 4) CXG_HM(8, 8) CXG_HM(16, 2) CXG_HM(16, 4) CXG_HM(16, 8) CXG_HM(32, 2) CXG_HM(32, 4) CXG_HM(32, 8)
#undef CXG_HM
  CXG_REQUIRE(done, CXG_ERR_UNSUPPORTED, "no kernel for this combination");
  CXG_LAUNCH_CHECK("spmm_group_kernel");
  // the carried partial rows and the output rows are heads * feat floats to the fix-up kernel
  SpmmArgs<int64_t> f = a;
  f.F = heads * feat;
  if (f.F % 128 == 0) {
    hipLaunchKernelGGL((spmm_fixup_kernel<int64_t, 2, false>), dim3(grid.x, (unsigned)(f.F / 128), 1), block, 0, st, f);
  } else {
    hipLaunchKernelGGL((spmm_fixup_kernel<int64_t, 1, true>), dim3(grid.x, (unsigned)ceil_div(f.F, CXG_WAVE), 1), block, 0, st, f);
  }
  CXG_LAUNCH_CHECK("spmm_fixup_kernel");
  return CXG_OK;
}

int cxg_spmm_weighted_bias_f32(const int64_t* ptr, const int64_t* idx, const float* val,
                               const int64_t* val_perm, const float* x, int64_t ldx, const float* bias,
                               float* out, int64_t ldo, int64_t n_rows, int64_t n_edges_cap, int heads,
                               int channels, unsigned flags, void* workspace, size_t workspace_bytes,
                               void* stream) {
  if (!val) return cxg::set_error(CXG_ERR_ARG, "val is null");
  CXG_REQUIRE(!(bias && (flags & CXG_SPMM_MEAN)), CXG_ERR_ARG, "bias cannot be combined with mean");
  return cxg::spmm_common<int64_t>(ptr, idx, val, val_perm, x, ldx, out, ldo, n_rows, n_edges_cap,
                                   heads, channels, flags, workspace, workspace_bytes, stream, nullptr, nullptr,
                                   bias);
}

int cxg_spmm_weighted_dot_f32(const int64_t* ptr, const int64_t* idx, const float* val,
                              const int64_t* val_perm, const float* x, int64_t ldx, float* out,
                              int64_t ldo, const float* dot_b, int64_t ld_dot_b, float* dot_out,
                              int64_t n_rows, int64_t n_edges_cap, int heads, int channels,
                              unsigned flags, void* workspace, size_t workspace_bytes, void* stream) {
  if (!val) return cxg::set_error(CXG_ERR_ARG, "val is null");
  cxg::SpmmDot dot;
  dot.b = dot_b; dot.ld_b = ld_dot_b; dot.out = dot_out;
  dot.at_edge = (flags & CXG_SPMM_DOT_AT_EDGE) != 0;
  return cxg::spmm_common<int64_t>(ptr, idx, val, val_perm, x, ldx, out, ldo, n_rows, n_edges_cap,
                                   heads, channels, flags & ~CXG_SPMM_DOT_AT_EDGE, workspace, workspace_bytes, stream, nullptr, &dot);
}

int cxg_spmm_ext_f32(const int64_t* ptr, const int64_t* idx, const float* x, int64_t ldx, float* out,
                     int64_t ldo, int64_t n_rows, int64_t n_edges_cap, int feat, unsigned flags,
                     const uint8_t* mask, const int64_t* mask_perm, const int32_t* rel,
                     int64_t rel_stride, const int64_t* src_map, const int64_t* targets,
                     void* workspace, size_t workspace_bytes, void* stream) {
  cxg::SpmmExt ext;
  ext.mask = mask; ext.mask_perm = mask_perm; ext.rel = rel; ext.rel_stride = rel_stride;
  ext.src_map = src_map; ext.targets = targets;
  if (mask_perm && !mask) return cxg::set_error(CXG_ERR_ARG, "mask_perm without mask");
  if (rel && rel_stride <= 0) return cxg::set_error(CXG_ERR_ARG, "rel needs a positive rel_stride");
  return cxg::spmm_common<int64_t>(ptr, idx, nullptr, nullptr, x, ldx, out, ldo, n_rows, n_edges_cap,
                                   1, feat, flags, workspace, workspace_bytes, stream, &ext);
}

}  // extern "C"
