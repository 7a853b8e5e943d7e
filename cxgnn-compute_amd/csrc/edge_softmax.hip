// Per-destination edge softmax (GAT attention) and other row reductions over
// narrow per-edge data (a few floats per edge) for gfx950.
//
// Two work decompositions.
// "Three-tier row blocks" (narrow_gather_sum, and the softmax with a head count that is
// not 1, 2, 4 or 8).  A block of 4 wavefronts owns 256 consecutive rows, 64 per wave.
//   * rows of at most kShortDeg edges: one row per lane;
//   * rows of at most kWaveDeg edges: one row at a time by a whole wave, lanes
//     striding over the row's edges, wave reduction at the end;
//   * longer rows: one row at a time by the whole block (256 threads) with an LDS
//     reduction, so that a 17k-edge hub is a chain of ~70 steps instead of ~270.
// Power-law graphs have millions of degree-1..8 rows and a few hundred rows with
// more than 10k edges; each tier keeps its lanes busy on its share.
// "Edge-parallel walk" (the softmax with 1, 2, 4 or 8 heads): rows of at most kWaveDeg
// edges are visited one EDGE per lane, 64 consecutive edges at a time, with segmented
// scans for the per-row reductions (see SegmentWalk); longer rows as above.  Every
// per-edge array is then read and written in whole contiguous lines.
//
//   forward  (edge_softmax_fwd, src/cpp/src/edge_softmax.cu:3-42):
//     t = leaky_relu(att_dst[r,h] + att_src[idx[e],h]);  out = softmax_row(t);
//     mask = t > 0.  First sweep: gather, online max/sum, t parked in `out`;
//     second sweep: the same lane normalises its own t in place.  One 16-byte
//     gather per edge in total -- every gather is a whole cache line over the
//     fabric, the re-read of `out` is a coalesced stream (the reference makes
//     three read-modify-write sweeps over out).
//   backward (edge_softmax_bwd, src/cpp/src/edge_softmax.cu:44-95):
//     s = sum_row out*g;  t = out*(g-s)*(mask ? 1 : slope);
//     g_dst[r,h] = sum_row t (left 0 unless the row has both signs, :91-93);
//     t is stored per edge and the source gradient is the row sum of t over the
//     transposed CSR (narrow_gather_sum below) instead of fp32 atomics.
//   spmv (spmv_csr, src/cpp/src/edge_softmax.cu:216-232) is narrow_gather_sum
//     with one float per edge.
#include "cxg_common.hpp"

namespace cxg {
namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kBlock = kWavesPerBlock * CXG_WAVE;
#ifndef CXG_SOFTMAX_SHORT_DEG
#define CXG_SOFTMAX_SHORT_DEG 16
#endif
#ifndef CXG_SOFTMAX_WAVE_DEG
#define CXG_SOFTMAX_WAVE_DEG 512
#endif
#ifndef CXG_SOFTMAX_TIERS
#define CXG_SOFTMAX_TIERS 7   // bit 0 lane tier, bit 1 wave tier, bit 2 block tier (timing experiments)
#endif
constexpr int kShortDeg = CXG_SOFTMAX_SHORT_DEG;
constexpr int kWaveDeg = CXG_SOFTMAX_WAVE_DEG;
constexpr int kTiers = CXG_SOFTMAX_TIERS;

__device__ __forceinline__ float wave_max(float v) {
  for (int m = 32; m > 0; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, CXG_WAVE));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
  for (int m = 32; m > 0; m >>= 1) v += __shfl_xor(v, m, CXG_WAVE);
  return v;
}

// Cooperative scopes: the same row code runs with 64 lanes (one wave) or with the
// 256 threads of the block; `li`/`nl` enumerate the participants.  Reductions take
// all N per-head values at once so that the block scope needs one LDS exchange
// (two barriers) per reduction, not one per head.
constexpr int kMaxRed = 8;    // most values reduced together (heads handled at once)

__device__ __forceinline__ float wave_or_bits(float v) {   // small non-negative integers as floats
  int b = (int)v;
  for (int m = 32; m > 0; m >>= 1) b |= __shfl_xor(b, m, CXG_WAVE);
  return (float)b;
}
// (m, s) pairs of an online softmax: s = sum of exp(t - m) over the values seen.
__device__ __forceinline__ void merge_max_sum(float& m, float& s, float m2, float s2) {
  const float mn = fmaxf(m, m2);
  s = s * __expf(m - mn) + s2 * __expf(m2 - mn);
  m = mn;
}

struct WaveScope {
  int li;
  static constexpr int nl = CXG_WAVE;
  template <int N> __device__ __forceinline__ void sum_n(float (&v)[N]) const {
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] = wave_sum(v[i]);
  }
  template <int N> __device__ __forceinline__ void or_n(float (&v)[N]) const {
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] = wave_or_bits(v[i]);
  }
  template <int N> __device__ __forceinline__ void combine_max_sum(float (&m)[N], float (&s)[N]) const {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const float mw = wave_max(m[i]);
      s[i] = wave_sum(s[i] * __expf(m[i] - mw));
      m[i] = mw;
    }
  }
  __device__ __forceinline__ float sum(float v) const { return wave_sum(v); }
  __device__ __forceinline__ bool leader() const { return li == 0; }
};
struct BlockScope {
  int li;
  float* red;   // kWavesPerBlock * 2 * kMaxRed floats of LDS
  static constexpr int nl = kBlock;
  // every wave leaves K values, every thread reads all of them back
  template <int K> __device__ __forceinline__ void exchange(const float (&mine)[K], float (&all)[kWavesPerBlock][K]) const {
    __syncthreads();                      // previous use of `red` is over
    if ((li & 63) == 0) {
#pragma unroll
      for (int i = 0; i < K; ++i) red[(li >> 6) * K + i] = mine[i];
    }
    __syncthreads();
#pragma unroll
    for (int w = 0; w < kWavesPerBlock; ++w)
#pragma unroll
      for (int i = 0; i < K; ++i) all[w][i] = red[w * K + i];
  }
  template <int N> __device__ __forceinline__ void sum_n(float (&v)[N]) const {
    float all[kWavesPerBlock][N];
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] = wave_sum(v[i]);
    exchange<N>(v, all);
#pragma unroll
    for (int i = 0; i < N; ++i) {
      v[i] = all[0][i];
#pragma unroll
      for (int w = 1; w < kWavesPerBlock; ++w) v[i] += all[w][i];
    }
  }
  template <int N> __device__ __forceinline__ void or_n(float (&v)[N]) const {
    float all[kWavesPerBlock][N];
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] = wave_or_bits(v[i]);
    exchange<N>(v, all);
#pragma unroll
    for (int i = 0; i < N; ++i) {
      int b = (int)all[0][i];
#pragma unroll
      for (int w = 1; w < kWavesPerBlock; ++w) b |= (int)all[w][i];
      v[i] = (float)b;
    }
  }
  template <int N> __device__ __forceinline__ void combine_max_sum(float (&m)[N], float (&s)[N]) const {
    float mine[2 * N], all[kWavesPerBlock][2 * N];
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const float mw = wave_max(m[i]);
      mine[2 * i] = mw;
      mine[2 * i + 1] = wave_sum(s[i] * __expf(m[i] - mw));
    }
    exchange<2 * N>(mine, all);
#pragma unroll
    for (int i = 0; i < N; ++i) {
      m[i] = all[0][2 * i];
      s[i] = all[0][2 * i + 1];
#pragma unroll
      for (int w = 1; w < kWavesPerBlock; ++w) merge_max_sum(m[i], s[i], all[w][2 * i], all[w][2 * i + 1]);
    }
  }
  __device__ __forceinline__ float sum(float v) const {
    float a[1] = {v};
    sum_n<1>(a);
    return a[0];
  }
  __device__ __forceinline__ bool leader() const { return li == 0; }
};

// short_fn(r, begin, end): one lane per short row.  coop_fn(scope, r, begin, end):
// wave-uniform (WaveScope) or block-uniform (BlockScope) arguments.
template <int TIERS = kTiers, class ShortFn, class CoopFn>
__device__ __forceinline__ void tiered_rows(const int64_t* __restrict__ ptr, int64_t n_rows,
                                            ShortFn short_fn, CoopFn coop_fn) {
  __shared__ unsigned long long s_very_long[kWavesPerBlock];
  __shared__ float s_red[kWavesPerBlock * 2 * kMaxRed];
  const int lane = lane_id();
  const int wave = uniform_i32(threadIdx.x >> 6);
  const int64_t row0 = (int64_t)blockIdx.x * kBlock;
  const int64_t r = row0 + wave * CXG_WAVE + lane;
  const bool valid = r < n_rows;
  int64_t b = 0, e = 0;
  if (valid) { b = ptr[r]; e = ptr[r + 1]; }
  const int64_t deg = e - b;
  if ((TIERS & 1) && valid && deg <= kShortDeg) short_fn(r, b, e);
  uint64_t todo = __ballot((TIERS & 2) && valid && deg > kShortDeg && deg <= kWaveDeg);
  const uint64_t very_long = __ballot((TIERS & 4) && valid && deg > kWaveDeg);
  WaveScope ws{lane};
  while (todo) {
    const int l = __ffsll((unsigned long long)todo) - 1;
    todo &= todo - 1;
    coop_fn(ws, bcast_i64(r, l), bcast_i64(b, l), bcast_i64(e, l));
  }
  if (lane == 0) s_very_long[wave] = very_long;
  __syncthreads();
  BlockScope bs{(int)threadIdx.x, s_red};
  for (int w = 0; w < kWavesPerBlock; ++w) {
    unsigned long long m = s_very_long[w];
    while (m) {
      const int l = __ffsll(m) - 1;
      m &= m - 1;
      const int64_t rr = row0 + w * CXG_WAVE + l;
      coop_fn(bs, rr, (int64_t)ptr[rr], (int64_t)ptr[rr + 1]);
    }
  }
  __syncthreads();   // s_very_long / s_red are reused by the next call
}

__device__ __forceinline__ float leaky(float t, float slope) { return fmaxf(t, t * slope); }

// N consecutive floats / bytes starting at p, as one vector access where N allows
// (p is N*4-byte / N-byte aligned: the arrays are [*, N] with an aligned base).
template <int N> __device__ __forceinline__ void load_f(const float* __restrict__ p, float (&v)[N]) {
  if constexpr (N == 4) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  } else if constexpr (N == 2) {
    const float2 t = *reinterpret_cast<const float2*>(p);
    v[0] = t.x; v[1] = t.y;
  } else if constexpr (N == 8) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    const float4 u = *reinterpret_cast<const float4*>(p + 4);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w; v[4] = u.x; v[5] = u.y; v[6] = u.z; v[7] = u.w;
  } else {
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] = p[i];
  }
}
template <int N> __device__ __forceinline__ void store_f(float* __restrict__ p, const float (&v)[N]) {
  if constexpr (N == 4) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  } else if constexpr (N == 2) {
    *reinterpret_cast<float2*>(p) = make_float2(v[0], v[1]);
  } else if constexpr (N == 8) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
  } else {
#pragma unroll
    for (int i = 0; i < N; ++i) p[i] = v[i];
  }
}
// The same for data that is written once and not read again by this launch (non-temporal:
// it should not displace the gathered logits from the L2).
template <int N> __device__ __forceinline__ void store_f_stream(float* __restrict__ p, const float (&v)[N]) {
  if constexpr (N == 4) {
    stream_store(p, make_float4(v[0], v[1], v[2], v[3]));
  } else if constexpr (N == 2) {
    stream_store(p, make_float2(v[0], v[1]));
  } else if constexpr (N == 8) {
    stream_store(p, make_float4(v[0], v[1], v[2], v[3]));
    stream_store(p + 4, make_float4(v[4], v[5], v[6], v[7]));
  } else {
#pragma unroll
    for (int i = 0; i < N; ++i) stream_store(p + i, v[i]);
  }
}
template <int N> __device__ __forceinline__ void load_b(const uint8_t* __restrict__ p, bool (&v)[N]) {
  if constexpr (N == 4 || N == 8) {
#pragma unroll
    for (int w = 0; w < N / 4; ++w) {
      const uint32_t t = reinterpret_cast<const uint32_t*>(p)[w];
#pragma unroll
      for (int i = 0; i < 4; ++i) v[4 * w + i] = ((t >> (8 * i)) & 0xffu) != 0;
    }
  } else {
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] = p[i] != 0;
  }
}
template <int N> __device__ __forceinline__ void store_b(uint8_t* __restrict__ p, const bool (&v)[N]) {
  if constexpr (N == 4 || N == 8) {
#pragma unroll
    for (int w = 0; w < N / 4; ++w) {
      uint32_t t = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) t |= (v[4 * w + i] ? 1u : 0u) << (8 * i);
      __builtin_nontemporal_store(t, reinterpret_cast<uint32_t*>(p) + w);
    }
  } else {
#pragma unroll
    for (int i = 0; i < N; ++i) p[i] = v[i] ? 1 : 0;
  }
}

// Online softmax state update: (m, s) <- combine with one value t.
__device__ __forceinline__ void online_add(float& m, float& s, float t) {
  const float mn = fmaxf(m, t);
  s = s * __expf(m - mn) + __expf(t - mn);
  m = mn;
}

constexpr float kMaxInit = -100000.f;  // running-max start of the reference kernel

// Edges are visited kU at a time: the kU index loads, then the kU gathers, are
// issued back to back (addresses past the row end are clamped to its last edge
// and their results dropped), so a lane has kU independent memory round trips
// in flight instead of one.  The row loops are latency chains; this is what
// shortens them.
constexpr int kU = 4;

template <int H>
__global__ __launch_bounds__(kBlock) void edge_softmax_fwd_kernel(
    const int64_t* __restrict__ ptr, const int64_t* __restrict__ idx,
    const float* __restrict__ att_dst, const float* __restrict__ att_src, float* __restrict__ out,
    uint8_t* __restrict__ mask, int64_t n_rows, int heads, float slope) {
  // H > 0: compile-time head count; H == 0: runtime `heads`, one head at a time.
  const int nh = H > 0 ? H : heads;
  constexpr int HB = H > 0 ? H : 1;     // heads processed together
  for (int h0 = 0; h0 < nh; h0 += HB) {
    // rows of row r visited by this participant: first, first + stride, ... < e
    auto sweep_rows = [&](int64_t r, int64_t first, int64_t stride, int64_t e, float (&m)[HB], float (&s)[HB]) {
      float d[HB];
      load_f<HB>(att_dst + r * nh + h0, d);
#pragma unroll
      for (int h = 0; h < HB; ++h) { m[h] = kMaxInit; s[h] = 0.f; }
      for (int64_t k = first; k < e; k += kU * stride) {
        int64_t kk[kU], src[kU];
        float as[kU][HB];
#pragma unroll
        for (int u = 0; u < kU; ++u) {
          kk[u] = k + u * stride;
          src[u] = idx[kk[u] < e ? kk[u] : e - 1];
        }
#pragma unroll
        for (int u = 0; u < kU; ++u) load_f<HB>(att_src + src[u] * nh + h0, as[u]);
#pragma unroll
        for (int u = 0; u < kU; ++u) {
          if (kk[u] < e) {
            float t[HB];
#pragma unroll
            for (int h = 0; h < HB; ++h) {
              t[h] = leaky(d[h] + as[u][h], slope);
              online_add(m[h], s[h], t[h]);
            }
            store_f<HB>(out + kk[u] * nh + h0, t);   // parked in `out` until the row's max / sum are known
          }
        }
      }
    };
    auto write_rows = [&](int64_t first, int64_t stride, int64_t e, const float (&m)[HB], const float (&s)[HB]) {
      for (int64_t k = first; k < e; k += kU * stride) {
        int64_t kk[kU];
        float t[kU][HB];
#pragma unroll
        for (int u = 0; u < kU; ++u) {
          kk[u] = k + u * stride;
          load_f<HB>(out + (kk[u] < e ? kk[u] : first) * nh + h0, t[u]);   // written by this lane above
        }
#pragma unroll
        for (int u = 0; u < kU; ++u) {
          if (kk[u] < e) {
            float o[HB];
            bool mk[HB];
#pragma unroll
            for (int h = 0; h < HB; ++h) {
              o[h] = __expf(t[u][h] - m[h]) * s[h];
              mk[h] = t[u][h] > 0.f;
            }
            store_f<HB>(out + kk[u] * nh + h0, o);
            store_b<HB>(mask + kk[u] * nh + h0, mk);
          }
        }
      }
    };
    auto short_fn = [&](int64_t r, int64_t b, int64_t e) {
      float m[HB], s[HB];
      sweep_rows(r, b, 1, e, m, s);
#pragma unroll
      for (int h = 0; h < HB; ++h) s[h] = 1.0f / s[h];
      write_rows(b, 1, e, m, s);
    };
    auto coop_fn = [&](auto sc, int64_t r, int64_t b, int64_t e) {
      float m[HB], s[HB];
      sweep_rows(r, b + sc.li, sc.nl, e, m, s);
      sc.template combine_max_sum<HB>(m, s);           // row-wide max and sum of exp(t - max)
#pragma unroll
      for (int h = 0; h < HB; ++h) s[h] = 1.0f / s[h];
      write_rows(b + sc.li, sc.nl, e, m, s);             // the same lane revisits the same edges
    };
    tiered_rows(ptr, n_rows, short_fn, coop_fn);
  }
}

// ----------------------------------------------------------------------------
// Edge-parallel walk.  A wave owns 64 consecutive rows and visits their edges 64 at a
// time, one edge per lane, so that idx, out and mask are read and written as whole
// contiguous lines whatever the degrees are.  Lane l also keeps the running state of
// row l.  Per chunk of 64 positions:
//   * the row of a lane's edge = the number of row ends at or before its position, by a
//     six-step search through lane shuffles of the 64 ends;
//   * a lane's segment = the lanes of the chunk that hold edges of the same row, known
//     from that row's begin and end; a reduction over a segment is a scan bounded by the
//     segment's first lane, its last lane then holds the total;
//   * the lane that owns a row pulls the total from the last lane of the row's segment.
// The order of every floating-point sum is fixed by the positions alone.  Rows of more
// than kWaveDeg edges are stepped over (the walk jumps to their end) and left to the
// whole block.
struct SegmentWalk {
  int64_t eb;                   // first edge of the wave
  int total;                    // number of edges of its 64 rows
  int begin_rel, end_rel;       // of the lane's own row, relative to eb
  uint64_t long_mask;           // rows left to the block
  int lane;

  __device__ __forceinline__ void init(const int64_t* __restrict__ ptr, int64_t n_rows, int64_t first_row) {
    lane = lane_id();
    const int64_t r = first_row + lane;
    const int64_t b = ptr[r < n_rows ? r : n_rows], e = ptr[r + 1 < n_rows ? r + 1 : n_rows];
    eb = bcast_i64(b, 0);
    const int64_t all = bcast_i64(e, CXG_WAVE - 1) - eb;
    long_mask = __ballot(e - b > kWaveDeg);
    if (all >= (int64_t)1 << 30) {           // positions are kept in 32 bits: leave such a wave to the block
      long_mask = __ballot(e > b);
      total = 0;
      begin_rel = end_rel = 0;
    } else {
      total = (int)all;
      begin_rel = (int)(b - eb);
      end_rel = (int)(e - eb);
    }
  }
  // One chunk at wave-uniform position `pos`.  Returns false (and moves pos to the end of
  // the row) when the chunk starts inside a stepped-over row.  Otherwise: `row` = the
  // lane's row (0..63), `act` = the lane holds an edge of a row handled here, `lo` / `hi`
  // = the first / last lane of its segment; pos moves on by 64.
  __device__ __forceinline__ bool chunk(int& pos, int& row, bool& act, int& lo, int& hi) const {
    const int rel = pos + lane;
    int cnt = 0;
#pragma unroll
    for (int step = 32; step >= 1; step >>= 1)
      if (__shfl(end_rel, cnt + step - 1, CXG_WAVE) <= rel) cnt += step;
    row = cnt;
    const int rb = __shfl(begin_rel, row, CXG_WAVE), re = __shfl(end_rel, row, CXG_WAVE);
    const int row_first = uniform_i32(row);
    if ((long_mask >> row_first) & 1) {
      pos = uniform_i32(re);
      return false;
    }
    act = rel < total && !((long_mask >> row) & 1);
    const int l = rb - pos, h = re - pos;
    lo = l > 0 ? l : 0;
    hi = (h < CXG_WAVE ? h : CXG_WAVE) - 1;
    pos += CXG_WAVE;
    return true;
  }
  // first / last lane of the chunk at `at` holding the lane's OWN row; last = -1: none
  __device__ __forceinline__ void own_segment(int at, int& first, int& last) const {
    const int l = begin_rel - at, h = end_rel - at;
    first = l > 0 ? l : 0;
    last = (h < CXG_WAVE ? h : CXG_WAVE) - 1;
    if (((long_mask >> lane) & 1) || h <= 0 || l >= CXG_WAVE || end_rel == begin_rel) last = -1;
  }
};

// Inclusive scans over the lanes [lo, lane] of a segment, by data-parallel primitives:
// four shifts inside each row of 16 lanes, then the last lane of row 0 / 2 to rows 1 / 3
// and the last lane of row 1 to rows 2 and 3.  A lane takes a contribution only when
// the lanes it stands for belong to its segment.
template <int CTRL> __device__ __forceinline__ float dpp_f32(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), CTRL, 0xf, 0xf, false));
}
template <class Op, int N> __device__ __forceinline__ void segment_scan(float (&v)[N], int lane, int lo, Op op) {
  const int in_row = lane & 15, row_start = lane & ~15;
  const int lo_row = lo > row_start ? lo - row_start : 0;   // first lane of the segment inside this row of 16
#pragma unroll
  for (int i = 0; i < N; ++i) {
    float o;
    o = dpp_f32<0x111>(v[i]); if (in_row - 1 >= lo_row) v[i] = op(v[i], o);   // row_shr:1
    o = dpp_f32<0x112>(v[i]); if (in_row - 2 >= lo_row) v[i] = op(v[i], o);   // row_shr:2
    o = dpp_f32<0x114>(v[i]); if (in_row - 4 >= lo_row) v[i] = op(v[i], o);   // row_shr:4
    o = dpp_f32<0x118>(v[i]); if (in_row - 8 >= lo_row) v[i] = op(v[i], o);   // row_shr:8
    o = dpp_f32<0x142>(v[i]); if ((lane & 16) && lo < row_start) v[i] = op(v[i], o);          // row_bcast:15
    o = dpp_f32<0x143>(v[i]); if (lane >= 32 && lo < 32) v[i] = op(v[i], o);                 // row_bcast:31
  }
}
struct OpMax { __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); } };
struct OpSum { __device__ __forceinline__ float operator()(float a, float b) const { return a + b; } };

// Rows left to the whole block: every wave announces its mask, then the block takes the
// rows one at a time.  `rows_per_wave` consecutive rows per wave from `block_row0`.
template <class CoopFn>
__device__ __forceinline__ void block_rows(const int64_t* __restrict__ ptr, int64_t block_row0, int rows_per_wave,
                                           uint64_t wave_mask, CoopFn coop_fn) {
  __shared__ unsigned long long s_mask[kWavesPerBlock];
  __shared__ float s_red[kWavesPerBlock * 2 * kMaxRed];
  if (lane_id() == 0) s_mask[threadIdx.x >> 6] = wave_mask;
  __syncthreads();
  BlockScope bs{(int)threadIdx.x, s_red};
  for (int w = 0; w < kWavesPerBlock; ++w) {
    unsigned long long m = s_mask[w];
    while (m) {
      const int l = __ffsll(m) - 1;
      m &= m - 1;
      const int64_t rr = block_row0 + (int64_t)w * rows_per_wave + l;
      coop_fn(bs, rr, (int64_t)ptr[rr], (int64_t)ptr[rr + 1]);
    }
  }
}

template <int H>
__global__ __launch_bounds__(kBlock) void edge_softmax_fwd_walk_kernel(
    const int64_t* __restrict__ ptr, const int64_t* __restrict__ idx,
    const float* __restrict__ att_dst, const float* __restrict__ att_src, float* __restrict__ out,
    uint8_t* __restrict__ mask, int64_t n_rows, float slope) {
  const int lane = lane_id();
  const int64_t block_row0 = (int64_t)blockIdx.x * kBlock;
  const int64_t first_row = block_row0 + (int64_t)uniform_i32(threadIdx.x >> 6) * CXG_WAVE;
  SegmentWalk w;
  w.init(ptr, n_rows, first_row < n_rows ? first_row : n_rows);
  float m[H], s[H];                          // of row first_row + lane
#pragma unroll
  for (int h = 0; h < H; ++h) { m[h] = kMaxInit; s[h] = 0.f; }
  // sweep 1: logits parked in `out`, the rows' max and sum of exp
  for (int pos = 0; pos < w.total;) {
    int row, lo, hi, first, last;
    bool act;
    const int at = pos;
    if (!w.chunk(pos, row, act, lo, hi)) continue;
    const int rel = at + lane;
    const int64_t k = w.eb + (rel < w.total ? rel : w.total - 1);
    const int64_t r = first_row + row;
    float a[H], d[H], t[H], mx[H], p[H];
    load_f<H>(att_src + stream_load(idx + k) * H, a);
    load_f<H>(att_dst + (r < n_rows ? r : n_rows - 1) * H, d);
#pragma unroll
    for (int h = 0; h < H; ++h) mx[h] = t[h] = leaky(d[h] + a[h], slope);
    if (act) store_f<H>(out + k * H, t);
    segment_scan(mx, lane, lo, OpMax());
#pragma unroll
    for (int h = 0; h < H; ++h) {
      mx[h] = __shfl(mx[h], hi, CXG_WAVE);               // the segment's max on all its lanes
      p[h] = __expf(t[h] - mx[h]);
    }
    segment_scan(p, lane, lo, OpSum());
    w.own_segment(at, first, last);
#pragma unroll
    for (int h = 0; h < H; ++h) {
      const float m2 = __shfl(mx[h], last < 0 ? 0 : last, CXG_WAVE);
      const float s2 = __shfl(p[h], last < 0 ? 0 : last, CXG_WAVE);
      if (last >= 0) merge_max_sum(m[h], s[h], m2, s2);
    }
  }
#pragma unroll
  for (int h = 0; h < H; ++h) s[h] = 1.0f / s[h];
  // sweep 2: the same lane revisits the same edges
  for (int pos = 0; pos < w.total;) {
    int row, lo, hi;
    bool act;
    const int at = pos;
    if (!w.chunk(pos, row, act, lo, hi)) continue;
    const int rel = at + lane;
    const int64_t k = w.eb + (rel < w.total ? rel : w.total - 1);
    float t[H], o[H];
    bool mk[H];
    load_f<H>(out + k * H, t);
#pragma unroll
    for (int h = 0; h < H; ++h) {
      const float mr = __shfl(m[h], row, CXG_WAVE), sr = __shfl(s[h], row, CXG_WAVE);
      o[h] = __expf(t[h] - mr) * sr;
      mk[h] = t[h] > 0.f;
    }
    if (act) {
      store_f_stream<H>(out + k * H, o);
      store_b<H>(mask + k * H, mk);
    }
  }

  // rows of more than kWaveDeg edges: one at a time by the whole block
  auto coop_fn = [&](auto sc, int64_t r, int64_t b, int64_t e) {
    float d[H], bm[H], bsum[H];
    load_f<H>(att_dst + r * H, d);
#pragma unroll
    for (int h = 0; h < H; ++h) { bm[h] = kMaxInit; bsum[h] = 0.f; }
    for (int64_t k = b + sc.li; k < e; k += kU * sc.nl) {
      int64_t kk[kU], src[kU];
      float a[kU][H];
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        kk[u] = k + u * sc.nl;
        src[u] = stream_load(idx + (kk[u] < e ? kk[u] : e - 1));
      }
#pragma unroll
      for (int u = 0; u < kU; ++u) load_f<H>(att_src + src[u] * H, a[u]);
#pragma unroll
      for (int u = 0; u < kU; ++u)
        if (kk[u] < e) {
          float t[H];
#pragma unroll
          for (int h = 0; h < H; ++h) {
            t[h] = leaky(d[h] + a[u][h], slope);
            online_add(bm[h], bsum[h], t[h]);
          }
          store_f<H>(out + kk[u] * H, t);
        }
    }
    sc.template combine_max_sum<H>(bm, bsum);
#pragma unroll
    for (int h = 0; h < H; ++h) bsum[h] = 1.0f / bsum[h];
    for (int64_t k = b + sc.li; k < e; k += kU * sc.nl) {
      int64_t kk[kU];
      float t[kU][H];
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        kk[u] = k + u * sc.nl;
        load_f<H>(out + (kk[u] < e ? kk[u] : b + sc.li) * H, t[u]);   // written by this thread above
      }
#pragma unroll
      for (int u = 0; u < kU; ++u)
        if (kk[u] < e) {
          float o[H];
          bool mk[H];
#pragma unroll
          for (int h = 0; h < H; ++h) {
            o[h] = __expf(t[u][h] - bm[h]) * bsum[h];
            mk[h] = t[u][h] > 0.f;
          }
          store_f_stream<H>(out + kk[u] * H, o);
          store_b<H>(mask + kk[u] * H, mk);
        }
    }
  };
  block_rows(ptr, block_row0, CXG_WAVE, w.long_mask, coop_fn);
}

template <int H>
__global__ __launch_bounds__(kBlock) void edge_softmax_bwd_kernel(
    const int64_t* __restrict__ ptr, const float* __restrict__ out, const uint8_t* __restrict__ mask,
    const float* __restrict__ grad, const int64_t* __restrict__ gpos, float* __restrict__ g_dst,
    float* __restrict__ t_edge, int64_t n_rows, int heads, float slope) {
  const int nh = H > 0 ? H : heads;
  constexpr int HB = H > 0 ? H : 1;
  for (int h0 = 0; h0 < nh; h0 += HB) {
    auto dot_rows = [&](int64_t first, int64_t stride, int64_t e, float (&s)[HB]) {
#pragma unroll
      for (int h = 0; h < HB; ++h) s[h] = 0.f;
      for (int64_t k = first; k < e; k += kU * stride) {
        int64_t kk[kU];
        float o[kU][HB], g[kU][HB];
#pragma unroll
        for (int u = 0; u < kU; ++u) {
          kk[u] = k + u * stride;
          const int64_t c = kk[u] < e ? kk[u] : first;
          load_f<HB>(out + c * nh + h0, o[u]);
          load_f<HB>(grad + (gpos ? gpos[c] : c) * nh + h0, g[u]);
        }
#pragma unroll
        for (int u = 0; u < kU; ++u)
          if (kk[u] < e)
#pragma unroll
            for (int h = 0; h < HB; ++h) s[h] += o[u][h] * g[u][h];
      }
    };
    auto edge_rows = [&](int64_t first, int64_t stride, int64_t e, const float (&s)[HB], float (&dsum)[HB],
                         int (&pos)[HB], int (&neg)[HB]) {
#pragma unroll
      for (int h = 0; h < HB; ++h) { dsum[h] = 0.f; pos[h] = 0; neg[h] = 0; }
      for (int64_t k = first; k < e; k += kU * stride) {
        int64_t kk[kU];
        float o[kU][HB], g[kU][HB];
        bool mk[kU][HB];
#pragma unroll
        for (int u = 0; u < kU; ++u) {
          kk[u] = k + u * stride;
          const int64_t c = kk[u] < e ? kk[u] : first;
          load_f<HB>(out + c * nh + h0, o[u]);
          load_f<HB>(grad + (gpos ? gpos[c] : c) * nh + h0, g[u]);
          load_b<HB>(mask + c * nh + h0, mk[u]);
        }
#pragma unroll
        for (int u = 0; u < kU; ++u) {
          if (kk[u] < e) {
            float tv[HB];
#pragma unroll
            for (int h = 0; h < HB; ++h) {
              float t = o[u][h] * (g[u][h] - s[h]);
              if (!mk[u][h]) { t *= slope; neg[h] = 1; } else { pos[h] = 1; }
              dsum[h] += t;
              tv[h] = t;
            }
            store_f<HB>(t_edge + kk[u] * nh + h0, tv);
          }
        }
      }
    };
    auto short_fn = [&](int64_t r, int64_t b, int64_t e) {
      float s[HB], dsum[HB];
      int pos[HB], neg[HB];
      dot_rows(b, 1, e, s);
      edge_rows(b, 1, e, s, dsum, pos, neg);
#pragma unroll
      for (int h = 0; h < HB; ++h) g_dst[r * nh + h0 + h] = (pos[h] && neg[h]) ? dsum[h] : 0.f;
    };
    auto coop_fn = [&](auto sc, int64_t r, int64_t b, int64_t e) {
      float s[HB], dsum[HB];
      int pos[HB], neg[HB];
      dot_rows(b + sc.li, sc.nl, e, s);
      sc.template sum_n<HB>(s);
      edge_rows(b + sc.li, sc.nl, e, s, dsum, pos, neg);
      float flags[HB];                                   // 1: positive seen, 2: negative seen
#pragma unroll
      for (int h = 0; h < HB; ++h) flags[h] = (float)(pos[h] + 2 * neg[h]);
      sc.template sum_n<HB>(dsum);
      sc.template or_n<HB>(flags);
      if (sc.leader()) {
#pragma unroll
        for (int h = 0; h < HB; ++h) g_dst[r * nh + h0 + h] = ((int)flags[h] == 3) ? dsum[h] : 0.f;
      }
    };
    tiered_rows(ptr, n_rows, short_fn, coop_fn);
  }
}

// Backward as an edge-parallel walk (see SegmentWalk): s = sum_row out*g, then
// t = out*(g-s)*(mask ? 1 : slope) per edge and g_dst = sum_row t where the row has both
// signs.
// AT: the gradient row of edge k sits at grad[gpos[k]] (the producer wrote it in another edge order).
template <int H, bool AT>
__global__ __launch_bounds__(kBlock) void edge_softmax_bwd_walk_kernel(
    const int64_t* __restrict__ ptr, const float* __restrict__ out, const uint8_t* __restrict__ mask,
    const float* __restrict__ grad, const int64_t* __restrict__ gpos, float* __restrict__ g_dst,
    float* __restrict__ t_edge, int64_t n_rows, float slope) {
  const int lane = lane_id();
  const int64_t block_row0 = (int64_t)blockIdx.x * kBlock;
  const int64_t first_row = block_row0 + (int64_t)uniform_i32(threadIdx.x >> 6) * CXG_WAVE;
  SegmentWalk w;
  w.init(ptr, n_rows, first_row < n_rows ? first_row : n_rows);
  float s[H], dsum[H];                       // of row first_row + lane
  unsigned seen = 0;                         // bit h: a positive logit seen, bit H + h: a negative one
#pragma unroll
  for (int h = 0; h < H; ++h) { s[h] = 0.f; dsum[h] = 0.f; }
  // sweep 1: s = sum out*g
  for (int pos = 0; pos < w.total;) {
    int row, lo, hi, first, last;
    bool act;
    const int at = pos;
    if (!w.chunk(pos, row, act, lo, hi)) continue;
    const int rel = at + lane;
    const int64_t k = w.eb + (rel < w.total ? rel : w.total - 1);
    float o[H], g[H], v[H];
    load_f<H>(out + k * H, o);
    load_f<H>(grad + (AT ? gpos[k] : k) * H, g);
    // AT: one gather per edge -- the row is left at the edge's own place in t_edge, where the
    // same lane finds it in sweep 2 before it overwrites it
    if (AT && rel < w.total) store_f<H>(t_edge + k * H, g);
#pragma unroll
    for (int h = 0; h < H; ++h) v[h] = o[h] * g[h];
    segment_scan(v, lane, lo, OpSum());
    w.own_segment(at, first, last);
#pragma unroll
    for (int h = 0; h < H; ++h) {
      const float x = __shfl(v[h], last < 0 ? 0 : last, CXG_WAVE);
      if (last >= 0) s[h] += x;
    }
  }
  // sweep 2: per-edge values, their row sums, the signs seen in each row
  for (int pos = 0; pos < w.total;) {
    int row, lo, hi, first, last;
    bool act;
    const int at = pos;
    if (!w.chunk(pos, row, act, lo, hi)) continue;
    const int rel = at + lane;
    const int64_t k = w.eb + (rel < w.total ? rel : w.total - 1);
    float o[H], g[H], t[H];
    bool mk[H];
    load_f<H>(out + k * H, o);
    load_f<H>((AT ? t_edge : grad) + k * H, g);
    load_b<H>(mask + k * H, mk);
    w.own_segment(at, first, last);
    const uint64_t own = last < 0 ? 0ull : ((~0ull >> (CXG_WAVE - 1 - last)) & (~0ull << first));
#pragma unroll
    for (int h = 0; h < H; ++h) {
      const float sr = __shfl(s[h], row, CXG_WAVE);
      t[h] = o[h] * (g[h] - sr) * (mk[h] ? 1.0f : slope);
      const uint64_t pos_m = __ballot(act && mk[h]), neg_m = __ballot(act && !mk[h]);
      if (pos_m & own) seen |= 1u << h;
      if (neg_m & own) seen |= 1u << (H + h);
    }
    if (act) store_f<H>(t_edge + k * H, t);
    segment_scan(t, lane, lo, OpSum());
#pragma unroll
    for (int h = 0; h < H; ++h) {
      const float x = __shfl(t[h], last < 0 ? 0 : last, CXG_WAVE);
      if (last >= 0) dsum[h] += x;
    }
  }
  if (first_row + lane < n_rows && !((w.long_mask >> lane) & 1)) {
    float gd[H];
#pragma unroll
    for (int h = 0; h < H; ++h) gd[h] = ((seen >> h) & (seen >> (H + h)) & 1u) ? dsum[h] : 0.f;
    store_f<H>(g_dst + (first_row + lane) * H, gd);
  }

  // rows of more than kWaveDeg edges: one at a time by the whole block
  auto coop_fn = [&](auto sc, int64_t r, int64_t b, int64_t e) {
    float bs[H], bd[H], flags[H];
    int pos[H], neg[H];
#pragma unroll
    for (int h = 0; h < H; ++h) { bs[h] = 0.f; bd[h] = 0.f; pos[h] = 0; neg[h] = 0; }
    for (int64_t k = b + sc.li; k < e; k += kU * sc.nl) {
      int64_t kk[kU];
      float o[kU][H], g[kU][H];
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        kk[u] = k + u * sc.nl;
        const int64_t c = kk[u] < e ? kk[u] : b + sc.li;
        load_f<H>(out + c * H, o[u]);
        load_f<H>(grad + (AT ? gpos[c] : c) * H, g[u]);
      }
#pragma unroll
      for (int u = 0; u < kU; ++u)
        if (kk[u] < e) {
          if (AT) store_f<H>(t_edge + kk[u] * H, g[u]);
#pragma unroll
          for (int h = 0; h < H; ++h) bs[h] += o[u][h] * g[u][h];
        }
    }
    sc.template sum_n<H>(bs);
    for (int64_t k = b + sc.li; k < e; k += kU * sc.nl) {
      int64_t kk[kU];
      float o[kU][H], g[kU][H];
      bool mk[kU][H];
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        kk[u] = k + u * sc.nl;
        const int64_t c = kk[u] < e ? kk[u] : b + sc.li;
        load_f<H>(out + c * H, o[u]);
        load_f<H>((AT ? t_edge : grad) + c * H, g[u]);
        load_b<H>(mask + c * H, mk[u]);
      }
#pragma unroll
      for (int u = 0; u < kU; ++u)
        if (kk[u] < e) {
          float t[H];
#pragma unroll
          for (int h = 0; h < H; ++h) {
            t[h] = o[u][h] * (g[u][h] - bs[h]);
            if (!mk[u][h]) { t[h] *= slope; neg[h] = 1; } else { pos[h] = 1; }
            bd[h] += t[h];
          }
          store_f<H>(t_edge + kk[u] * H, t);
        }
    }
#pragma unroll
    for (int h = 0; h < H; ++h) flags[h] = (float)(pos[h] + 2 * neg[h]);   // 1: positive seen, 2: negative seen
    sc.template sum_n<H>(bd);
    sc.template or_n<H>(flags);
    if (sc.leader()) {
#pragma unroll
      for (int h = 0; h < H; ++h) g_dst[r * H + h] = ((int)flags[h] == 3) ? bd[h] : 0.f;
    }
  };
  block_rows(ptr, block_row0, CXG_WAVE, w.long_mask, coop_fn);
}

// out[r, 0..W) = sum_{k in row r} in[sel[k], 0..W)   (sel == nullptr: in[k]).
template <int W>
__global__ __launch_bounds__(kBlock) void narrow_gather_sum_kernel(
    const int64_t* __restrict__ ptr, const int64_t* __restrict__ sel, const float* __restrict__ in,
    float* __restrict__ out, int64_t n_rows, int width) {
  const int nw = W > 0 ? W : width;
  constexpr int WB = W > 0 ? W : 1;
  for (int w0 = 0; w0 < nw; w0 += WB) {
    auto short_fn = [&](int64_t r, int64_t b, int64_t e) {
      float acc[WB];
#pragma unroll
      for (int w = 0; w < WB; ++w) acc[w] = 0.f;
      for (int64_t k = b; k < e; ++k) {
        float p[WB];
        load_f<WB>(in + (sel ? sel[k] : k) * nw + w0, p);
#pragma unroll
        for (int w = 0; w < WB; ++w) acc[w] += p[w];
      }
#pragma unroll
      for (int w = 0; w < WB; ++w) out[r * nw + w0 + w] = acc[w];
    };
    auto coop_fn = [&](auto sc, int64_t r, int64_t b, int64_t e) {
      float acc[WB];
#pragma unroll
      for (int w = 0; w < WB; ++w) acc[w] = 0.f;
      for (int64_t k = b + sc.li; k < e; k += sc.nl) {
        float p[WB];
        load_f<WB>(in + (sel ? sel[k] : k) * nw + w0, p);
#pragma unroll
        for (int w = 0; w < WB; ++w) acc[w] += p[w];
      }
#pragma unroll
      for (int w = 0; w < WB; ++w) {
        const float total = sc.sum(acc[w]);
        if (sc.leader()) out[r * nw + w0 + w] = total;
      }
    };
    tiered_rows(ptr, n_rows, short_fn, coop_fn);
  }
}

dim3 row_grid(int64_t n_rows) { return dim3((unsigned)ceil_div(n_rows, kBlock)); }

}  // namespace
}  // namespace cxg

extern "C" {

int cxg_edge_softmax_fwd_f32(const int64_t* ptr, const int64_t* idx, const float* att_dst,
                             const float* att_src, float* out, uint8_t* mask, int64_t n_dst,
                             int heads, float slope, void* stream) {
  CXG_REQUIRE(n_dst >= 0 && heads >= 1, CXG_ERR_ARG, "bad n_dst/heads");
  if (n_dst == 0) return CXG_OK;
  CXG_REQUIRE(ptr && att_dst, CXG_ERR_ARG, "null ptr/att_dst");
  CXG_REQUIRE(idx && att_src && out && mask, CXG_ERR_ARG, "null idx/att_src/out/mask");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  dim3 grid = cxg::row_grid(n_dst), block(cxg::kBlock);
#define CXG_FWD(HH)                                                                              \
  hipLaunchKernelGGL(cxg::edge_softmax_fwd_walk_kernel<HH>, grid, block, 0, st, ptr, idx, att_dst, \
                     att_src, out, mask, n_dst, slope)
  if (heads == 1) CXG_FWD(1);
  else if (heads == 2) CXG_FWD(2);
  else if (heads == 4) CXG_FWD(4);
  else if (heads == 8) CXG_FWD(8);
  else
    hipLaunchKernelGGL(cxg::edge_softmax_fwd_kernel<0>, grid, block, 0, st, ptr, idx, att_dst, att_src,
                       out, mask, n_dst, heads, slope);
#undef CXG_FWD
  CXG_LAUNCH_CHECK("edge_softmax_fwd_kernel");
  return CXG_OK;
}

int cxg_edge_softmax_bwd_at_f32(const int64_t* ptr, const float* out, const uint8_t* mask,
                                const float* grad, const int64_t* grad_pos, float* g_dst, float* t_edge,
                                int64_t n_dst, int heads, float slope, void* stream) {
  CXG_REQUIRE(n_dst >= 0 && heads >= 1, CXG_ERR_ARG, "bad n_dst/heads");
  if (n_dst == 0) return CXG_OK;
  CXG_REQUIRE(ptr && g_dst, CXG_ERR_ARG, "null ptr/g_dst");
  CXG_REQUIRE(out && mask && grad && t_edge, CXG_ERR_ARG, "null out/mask/grad/t_edge");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  dim3 grid = cxg::row_grid(n_dst), block(cxg::kBlock);
#define CXG_BWD(HH)                                                                                  \
  do {                                                                                               \
    if (grad_pos)                                                                                    \
      hipLaunchKernelGGL((cxg::edge_softmax_bwd_walk_kernel<HH, true>), grid, block, 0, st, ptr, out, mask, \
                         grad, grad_pos, g_dst, t_edge, n_dst, slope);                               \
    else                                                                                             \
      hipLaunchKernelGGL((cxg::edge_softmax_bwd_walk_kernel<HH, false>), grid, block, 0, st, ptr, out, mask, \
                         grad, grad_pos, g_dst, t_edge, n_dst, slope);                               \
  } while (0)
  if (heads == 1) CXG_BWD(1);
  else if (heads == 2) CXG_BWD(2);
  else if (heads == 4) CXG_BWD(4);
  else if (heads == 8) CXG_BWD(8);
  else
    hipLaunchKernelGGL(cxg::edge_softmax_bwd_kernel<0>, grid, block, 0, st, ptr, out, mask, grad, grad_pos,
                       g_dst, t_edge, n_dst, heads, slope);
#undef CXG_BWD
  CXG_LAUNCH_CHECK("edge_softmax_bwd_kernel");
  return CXG_OK;
}

int cxg_edge_softmax_bwd_f32(const int64_t* ptr, const float* out, const uint8_t* mask,
                             const float* grad, float* g_dst, float* t_edge, int64_t n_dst, int heads,
                             float slope, void* stream) {
  return cxg_edge_softmax_bwd_at_f32(ptr, out, mask, grad, nullptr, g_dst, t_edge, n_dst, heads, slope, stream);
}

int cxg_narrow_gather_sum_f32(const int64_t* ptr, const int64_t* sel, const float* in, float* out,
                              int64_t n_rows, int width, void* stream) {
  CXG_REQUIRE(n_rows >= 0 && width >= 1, CXG_ERR_ARG, "bad n_rows/width");
  if (n_rows == 0) return CXG_OK;
  CXG_REQUIRE(ptr && out, CXG_ERR_ARG, "null ptr/out");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  dim3 grid = cxg::row_grid(n_rows), block(cxg::kBlock);
#define CXG_NGS(WW)                                                                          \
  hipLaunchKernelGGL(cxg::narrow_gather_sum_kernel<WW>, grid, block, 0, st, ptr, sel, in, out, \
                     n_rows, width)
  if (width == 1) CXG_NGS(1);
  else if (width == 2) CXG_NGS(2);
  else if (width == 4) CXG_NGS(4);
  else if (width == 8) CXG_NGS(8);
  else CXG_NGS(0);
#undef CXG_NGS
  CXG_LAUNCH_CHECK("narrow_gather_sum_kernel");
  return CXG_OK;
}

}  // extern "C"
