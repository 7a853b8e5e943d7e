// Weight gradient of the typed GEMM on the gfx950 matrix cores:
//
//   gW[r] (K x N)  =  sum over the rows i of segment r of  A[src(i), :]^T  (x)  G[dst(i), :]
//
// i.e. a GEMM whose reduction runs over the (gathered) rows.  fp32 operands are
// split into NS bf16 parts and multiplied as partial products on
// v_mfma_f32_32x32x16_bf16 exactly as in the forward kernel (NS = 3: six products,
// fp32-accurate; NS = 2: three products).
//
// The MFMA wants eight consecutive reduction indices per lane, and the reduction
// index is the row index of both operands in memory, so both tiles are transposed
// on their way into LDS: a thread fetches one float4 from each of 4 consecutive
// rows (coalesced along the row), and writes, for each of its 4 columns, the 4
// row-consecutive bf16 values as one 8-byte LDS store into [column][row] order.
//
// Split over the rows: a block owns `rows_per_chunk` rows of one relation and one
// 128-column tile of G, keeps the 128 x 128 partial in the registers of its four
// consumer waves (wave w: output rows 32w .. 32w+31) and writes it to a partial buffer;
// a second kernel adds the partials of each relation in chunk order -- no atomics,
// deterministic.
//
// Replaces the weight-gradient half of TypedLinearE2EOP.backward /
// TypedLinearS2DMMAggrOP.backward (cxgnncomp/typed_linear.py:114-137,205-221),
// which the reference computes with one torch.mm per relation.
#include <type_traits>

#include "cxg_common.hpp"
#include "split_f16.hpp"

namespace cxg {
namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef __bf16 v4bf __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kXcds = 8;                 // accelerator dies of an MI355X, one L2 each
constexpr int kMT = 32;                  // rows per step
constexpr int kMP = kMT + 8;             // padded row extent in LDS (bf16 elements): 80-byte pitch

struct WgradArgs {
  const float* a;
  int64_t lda;
  const float* g;
  int64_t ldg;
  const int64_t* src;
  const int64_t* dst;
  const int64_t* seg;
  float* partial;
  int64_t M;
  int K, N, R;
  int64_t rows_per_chunk;
  int a_bf16;              // the rows of A are bf16 (lda in elements)
};

template <int NS>
__device__ __forceinline__ void split_parts(float x, __bf16 (&p)[NS]) {
#pragma unroll
  for (int i = 0; i < NS; ++i) {
    p[i] = (__bf16)x;
    x -= (float)p[i];
  }
}

// Chunk number -> (relation, first row, end of the relation's rows); block-uniform.
__device__ __forceinline__ bool locate_chunk(const int64_t* __restrict__ seg, int R, int64_t span,
                                             int64_t chunk, int& rel, int64_t& row0, int64_t& row_end) {
  int64_t t = chunk;
  for (int r = 0; r < R; ++r) {
    const int64_t b = seg[r], e = seg[r + 1];
    const int64_t nt = (e - b + span - 1) / span;
    if (t < nt) { rel = r; row0 = b + t * span; row_end = e; return true; }
    t -= nt;
  }
  return false;
}

// 768 threads in three groups of four waves, so that the conversion work (vector ALU, LDS
// stores) of the next tile runs beside the matrix instructions of the current one on
// every SIMD:
//   waves 4-7 load 32 rows of A two tiles ahead, split them into bf16 parts and stage
//     tile t+1 into one half of the double-buffered LDS; waves 8-11 do the same for G;
//   waves 0-3 (consumers) multiply tile t from the other half, 32 output rows each.
// One barrier per tile.  Each role has its own loop: the register needs differ (staging
// registers against accumulators) and a common loop would hold the union.
//
// Row maps (MAPPED): the maps of ALL the chunk's rows are fetched into LDS before the first
// tile, so a chunk has at most kMappedRows rows then.  The loads of a wave complete in order:
// a map load inside the tile loop would make its wave wait for the row loads issued before
// it, the loads that are meant to stay in flight while two tiles are staged.
//
// Scaled fp16 parts (F16): two fp16 parts per operand and three products instead of three bf16
// parts and six products.  fp16's exponent range is narrow, so the values are scaled by a power
// of two first -- and since the reduction runs over the rows, a scale may depend on the column
// only.  A producer wave owns the same 32 columns of its operand through all tiles of the chunk
// and scales them by 2^(14 - e), e the exponent of the largest magnitude it has met in those
// columns SO FAR in the chunk (it only grows); the consumer keeps each accumulator block in
// the units of the current scales, multiplies it by the (rare) power-of-two step when a scale
// grows, and undoes the final scales when it stores.  The matrix instruction keeps fp16
// subnormals, so an element keeps 22 significant bits down to 2^-17 of its column group's
// largest magnitude and is off by at most 2^-39 of that magnitude below.
constexpr int kWgThreads = 768;
constexpr int kMappedRows = 2048;
constexpr int kExpBytes = 64;            // F16: biased exponents [operand][tile buffer][column group] as int

template <int NS>
constexpr size_t wgrad_lds_bytes(bool mapped) {
  return (size_t)2 * 2 * NS * 128 * kMP * sizeof(uint16_t) + kExpBytes +
         (mapped ? (size_t)2 * kMappedRows * sizeof(int64_t) : 0);
}

template <int CTRL>
__device__ __forceinline__ unsigned dpp_max_u32(unsigned m) {
  const unsigned o = (unsigned)__builtin_amdgcn_update_dpp(0, (int)m, CTRL, 0xf, 0xf, false);
  return o > m ? o : m;
}
// largest value over the wave, wave-uniform
__device__ __forceinline__ unsigned wave_max_u32(unsigned m) {
  m = dpp_max_u32<0xB1>(m);                  // quad_perm [1,0,3,2]
  m = dpp_max_u32<0x4E>(m);                  // quad_perm [2,3,0,1]
  m = dpp_max_u32<0x141>(m);                 // row_half_mirror
  m = dpp_max_u32<0x140>(m);                 // row_mirror
  const unsigned a = (unsigned)__builtin_amdgcn_readlane((int)m, 0), b = (unsigned)__builtin_amdgcn_readlane((int)m, 16);
  const unsigned c = (unsigned)__builtin_amdgcn_readlane((int)m, 32), d = (unsigned)__builtin_amdgcn_readlane((int)m, 48);
  const unsigned ab = a > b ? a : b, cd = c > d ? c : d;
  return ab > cd ? ab : cd;
}

// ABF16: the rows of A are bf16 in memory (a compile-time choice: a run-time branch around the
// two kinds of load made the compiler wait for every load in flight, 1.6 -> 2.6 ms on the pair
// rows of the relational layer).
template <int NS, bool MAPPED, bool F16, bool ABF16 = false>
__global__ __launch_bounds__(kWgThreads) __attribute__((amdgpu_waves_per_eu(3)))
void typed_wgrad_split_kernel(WgradArgs g) {
  static_assert(!F16 || NS == 2, "the fp16 form has two parts");
  extern __shared__ __attribute__((aligned(16))) uint16_t s_tiles[];
  typedef uint16_t (*tile_t)[128][kMP];                       // [part][column][row]
  // s_tiles: At[2][NS][128][kMP], then Gt[2][NS][128][kMP], then s_exp[2][2][4], then (MAPPED)
  // s_map[2][kMappedRows]
  auto tile_buf = [&](int operand, int b) -> tile_t {
    return reinterpret_cast<tile_t>(s_tiles + (size_t)(2 * operand + b) * NS * 128 * kMP);
  };
  int (*s_exp)[2][4] = reinterpret_cast<int (*)[2][4]>(s_tiles + (size_t)4 * NS * 128 * kMP);   // [operand][buffer][column group]
  int64_t* const s_map = reinterpret_cast<int64_t*>(reinterpret_cast<unsigned char*>(s_exp) + kExpBytes);   // [operand][row of the chunk]
  // A block owns one 128 x 128 tile of gw: columns n0 .. n0+127 of G against columns k0 .. k0+127 of
  // A.  All tiles of one row chunk get consecutive slots of one XCD (blocks go to the 8 XCDs
  // round-robin by index), so the chunk's A and G rows are fetched from memory into one L2 once and
  // the other tiles of the chunk find them there (K = N = 512: sixteen tiles per chunk; one launch
  // per 128 columns of A read G four times from memory and A once per column tile).
  const int n_ct = (g.N + 127) / 128, n_kt = (g.K + 127) / 128;
  const int n_tile = n_ct * n_kt;
  const int64_t slot = blockIdx.x / kXcds;
  const int64_t chunk = (slot / n_tile) * kXcds + (blockIdx.x % kXcds);
  const int n0 = (int)((slot % n_tile) % n_ct) * 128;
  const int k0 = (int)((slot % n_tile) / n_ct) * 128;
  int rel = 0;
  int64_t row0 = 0, row_end = 0;
  const bool have = locate_chunk(g.seg, g.R, g.rows_per_chunk, chunk, rel, row0, row_end);
  const int tid = threadIdx.x, lane = tid & 63, wave = uniform_i32(tid >> 6);
  const int K = g.K, N = g.N;
  const int64_t rows_here = !have ? 0 : ((row_end - row0) < g.rows_per_chunk ? (row_end - row0) : g.rows_per_chunk);
  const int n_tiles = (int)((rows_here + kMT - 1) / kMT);

  if (wave >= 4) {
    // ---- producers: operand 0 = A (waves 4-7), operand 1 = G (waves 8-11) ---------------
    if (n_tiles == 0) return;
    const int operand = (wave - 4) >> 2, pwave = (wave - 4) & 3, ptid = tid - 256 - operand * 256;
    // float4 column and group of 4 rows of this thread.  The low lane bits select the row
    // group and the high ones the column: the 16 lanes the LDS serves together then
    // write 8 row groups of 2 columns, 32 different banks with the 80-byte pitch (with
    // the bits the other way round four lanes met in every bank), while a global load
    // still covers 8 rows with 128 contiguous bytes each.
    const int c4 = pwave * 8 + (lane >> 3), mg = lane & 7;
    const bool col_ok = operand ? (n0 + 4 * c4 < N) : (k0 + 4 * c4 < K);      // K % 4 == 0 and N % 4 == 0 are required
    const float* const base = operand ? g.g + (col_ok ? n0 + 4 * c4 : 0) : g.a + (col_ok ? k0 + 4 * c4 : 0);
    const int64_t ld = operand ? g.ldg : g.lda;
    const uint16_t* const base16 = reinterpret_cast<const uint16_t*>(g.a) + (col_ok ? k0 + 4 * c4 : 0);
    // row of this operand behind row r of tile t (-1: no such row)
    auto row_index = [&](int t, int r) -> int64_t {
      if constexpr (MAPPED) {
        return s_map[operand * kMappedRows + t * kMT + r];
      } else {
        const int64_t gr = row0 + (int64_t)t * kMT + r;
        return gr < row_end ? gr : -1;
      }
    };
    if constexpr (MAPPED) {
      for (int i = tid - 256; i < n_tiles * kMT; i += 512) {     // n_tiles * kMT <= kMappedRows (the launch sees to it)
        const int64_t gr = row0 + i;
        int64_t sidx = -1, didx = -1;
        if (gr < row_end) {
          sidx = g.src ? g.src[gr] : gr;
          didx = g.dst ? g.dst[gr] : gr;
          if (sidx < 0 || didx < 0) sidx = didx = -1;            // a negative entry in either map drops the row
        }
        s_map[i] = sidx;
        s_map[kMappedRows + i] = didx;
      }
    }
    // (a generic lambda: with bf16 rows of A the A producers run their own copy of the loop, whose
    // loads are all of one kind -- the compiler counts the loads in flight statically)
    auto produce = [&](auto a16_tag) {
    constexpr bool A16 = decltype(a16_tag)::value;
    // Loads are issued unconditionally: rows and columns that do not exist are redirected
    // to an address that does and zeroed when the tile is staged (a select between a
    // loaded vector and a zero vector made the compiler route the load through scratch).
    // (which rows exist is noted as a bit mask that travels with the register set, so that
    // the staging code needs no table look-up between its conversions)
    auto gload = [&](float4 (&r4)[4], unsigned& live_mask, int t) {
      const int tc = t < n_tiles ? t : n_tiles - 1;
      unsigned mask = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int64_t ridx = row_index(tc, mg * 4 + i);
        mask |= (ridx >= 0 ? 1u : 0u) << i;
        if constexpr (A16) {
          // four bf16 values in two registers of the set, widened when the tile is staged
          const uint2 u = *reinterpret_cast<const uint2*>(base16 + (ridx >= 0 ? ridx : 0) * ld);
          r4[i] = make_float4(__uint_as_float(u.x), __uint_as_float(u.y), 0.f, 0.f);
        } else {
          r4[i] = *reinterpret_cast<const float4*>(base + (ridx >= 0 ? ridx : 0) * ld);
        }
      }
      live_mask = mask;
    };
    // registers (4 rows x 4 columns) -> LDS [column][4 consecutive rows], split into parts
    int e_run = 0;                                     // F16: largest biased exponent met in this wave's columns
    auto stage_tile = [&](const float4 (&r4)[4], unsigned live_mask, int t) {
      if (t >= n_tiles) return;
      const tile_t dst = tile_buf(operand, t & 1);
      float v[4][4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bool live = col_ok && ((live_mask >> i) & 1u) != 0;
        float4 w4 = r4[i];
        if constexpr (A16) {                           // two registers of four bf16 values (exact)
          const unsigned lo = __float_as_uint(r4[i].x), hi = __float_as_uint(r4[i].y);
          w4 = make_float4(__uint_as_float(lo << 16), __uint_as_float(lo & 0xffff0000u), __uint_as_float(hi << 16),
                           __uint_as_float(hi & 0xffff0000u));
        }
        v[i][0] = live ? w4.x : 0.f;
        v[i][1] = live ? w4.y : 0.f;
        v[i][2] = live ? w4.z : 0.f;
        v[i][3] = live ? w4.w : 0.f;
      }
      if constexpr (F16) {
        unsigned m = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const unsigned b = abs_max4_bits(v[i][0], v[i][1], v[i][2], v[i][3]);
          m = b > m ? b : m;
        }
        int eb = (int)(wave_max_u32(m) >> 23);
        eb = eb > 254 ? 254 : eb;                      // an infinity or NaN still comes out non-finite
        e_run = eb > e_run ? eb : e_run;
        const float scale = e_run >= 15 ? __uint_as_float((unsigned)(268 - e_run) << 23) : 0.f;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          typedef unsigned v2u __attribute__((ext_vector_type(2)));
          unsigned h01, l01, h23, l23;
          split_f16_pair(v[0][c], v[1][c], scale, h01, l01);
          split_f16_pair(v[2][c], v[3][c], scale, h23, l23);
          const v2u out[2] = {{h01, h23}, {l01, l23}};     // [high / low parts][rows 0-1, rows 2-3 of the group]
#pragma unroll
          for (int q = 0; q < 2; ++q) *reinterpret_cast<v2u*>(&dst[q][4 * c4 + c][mg * 4]) = out[q];
        }
        if (lane == 0) s_exp[operand][t & 1][pwave] = e_run;
        return;
      }
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        v4bf out[NS];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          __bf16 p[NS];
          split_parts<NS>(v[i][c], p);
#pragma unroll
          for (int q = 0; q < NS; ++q) out[q][i] = p[q];
        }
#pragma unroll
        for (int q = 0; q < NS; ++q) *reinterpret_cast<v4bf*>(&dst[q][4 * c4 + c][mg * 4]) = out[q];
      }
    };
    float4 r0[4], r1[4];                               // rows of two tiles in flight
    unsigned live0 = 0, live1 = 0;
    __syncthreads();                                   // #1: the row maps are there
    gload(r0, live0, 0);
    gload(r1, live1, 1);
    stage_tile(r0, live0, 0);
    gload(r0, live0, 2);
    __syncthreads();                                   // #2: tile 0 is staged
    // iteration t: stage tile t+1, barrier, load tile t+3.  Two iterations per trip, so that
    // both register sets keep their place in the order of the loads, and no path other than
    // the second iteration's leads back to the loop head (the compiler counts the loads in
    // flight statically and would otherwise wait for all of them there).  (Rows of four
    // tiles in flight instead of two were measured: slower, 2.30 against 2.12 ms.)
    for (int t = 0;; t += 2) {
      stage_tile(r1, live1, t + 1);
      __syncthreads();
      gload(r1, live1, t + 3);
      if (t + 1 >= n_tiles) return;
      stage_tile(r0, live0, t + 2);
      __syncthreads();
      gload(r0, live0, t + 4);
      if (t + 2 >= n_tiles) return;
    }
      };
    if (ABF16 && operand == 0) produce(std::true_type{});
    else produce(std::false_type{});
    return;
  }

  // ---- consumers --------------------------------------------------------------------
  if (k0 + wave * 32 >= K) {
    // this wave's 32 rows of gw lie past K: nothing to multiply or store, only the barriers
    if (n_tiles > 0) {
      __syncthreads();                                 // #1
      __syncthreads();                                 // #2
      for (int t = 0; t < n_tiles; ++t) __syncthreads();
    }
    return;
  }
  float* const part = g.partial + ((size_t)chunk * K) * (size_t)N;
  v16f acc[4];
#pragma unroll
  for (int nb = 0; nb < 4; ++nb)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[nb][i] = 0.f;
  int e_a = 0, e_g[4] = {0, 0, 0, 0};                  // F16: the exponents the accumulator blocks are scaled by
  if (n_tiles > 0) {
    __syncthreads();                                   // #1
    __syncthreads();                                   // #2
    for (int t = 0; t < n_tiles; ++t) {
      const tile_t At = tile_buf(0, t & 1), Gt = tile_buf(1, t & 1);
      if constexpr (F16) {
        // a scale that grew since the last tile: bring the accumulator block to the new units
        const int na = s_exp[0][t & 1][wave];
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) {
          const int ng = s_exp[1][t & 1][nb];
          const int d = (na - e_a) + (ng - e_g[nb]);   // >= 0: the exponents only grow
          if (d != 0) {
            const float f = d >= 126 ? 0.f : __uint_as_float((unsigned)(127 - d) << 23);
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[nb][i] *= f;
          }
          e_g[nb] = ng;
        }
        e_a = na;
      }
#pragma unroll
      for (int ms = 0; ms < kMT / 16; ++ms) {
        const int m = ms * 16 + (lane >> 5) * 8;
        v8bf af[NS];
#pragma unroll
        for (int q = 0; q < NS; ++q) af[q] = *reinterpret_cast<const v8bf*>(&At[q][wave * 32 + (lane & 31)][m]);
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) {
          v8bf bf[NS];
#pragma unroll
          for (int q = 0; q < NS; ++q) bf[q] = *reinterpret_cast<const v8bf*>(&Gt[q][nb * 32 + (lane & 31)][m]);
#pragma unroll
          for (int order = NS - 1; order >= 0; --order)
#pragma unroll
            for (int i = 0; i <= order; ++i) {
              if constexpr (F16)
                acc[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, af[i]),
                                                                 __builtin_bit_cast(v8h, bf[order - i]), acc[nb], 0, 0, 0);
              else
                acc[nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bf[order - i], acc[nb], 0, 0, 0);
            }
        }
      }
      __syncthreads();   // tile t+1 is staged, and every wave is done with tile t
    }
  }
  if constexpr (F16) {
    // undo the scales 2^(14 - (e - 127)) of the two operands, the smaller factor first
    const float fa = e_a >= 15 ? __uint_as_float((unsigned)(e_a - 14) << 23) : 0.f;
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
      const float fg = e_g[nb] >= 15 ? __uint_as_float((unsigned)(e_g[nb] - 14) << 23) : 0.f;
      const float f1 = fa < fg ? fa : fg, f2 = fa < fg ? fg : fa;
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[nb][i] = acc[nb][i] * f1 * f2;
    }
  }
  // partial[chunk][k][n] (zeros for chunk numbers past the last relation)
#pragma unroll
  for (int nb = 0; nb < 4; ++nb) {
    const int col = n0 + nb * 32 + (lane & 31);
    if (col >= N) continue;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int k = k0 + wave * 32 + (i >> 2) * 8 + (lane >> 5) * 4 + (i & 3);
      if (k < K) part[(size_t)k * N + col] = acc[nb][i];
    }
  }
}

// Dynamic LDS above the default 64 KB limit has to be enabled per kernel.
template <typename KernelT>
hipError_t allow_lds(KernelT kernel, size_t bytes) {
  if (bytes <= 64 * 1024) return hipSuccess;
  return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                             (int)bytes);
}

// gw[r][k][n] = sum of the partials of relation r's chunks, in a fixed order: the chunks
// are cut into kReduceSlices contiguous runs, each run is summed by one thread (four
// interleaved chains, so the loads overlap) and the runs are added in run order.
constexpr int kReduceSlices = 4;

__global__ __launch_bounds__(64 * kReduceSlices) void wgrad_reduce_kernel(
    const int64_t* __restrict__ seg, int R, int64_t rows_per_chunk, const float* __restrict__ partial,
    float* __restrict__ gw, int64_t kn) {
  __shared__ float s_run[kReduceSlices][64];
  const int el = threadIdx.x & 63, sl = threadIdx.x >> 6;
  const int64_t e = (int64_t)blockIdx.x * 64 + el;
  const int r = blockIdx.y;
  int64_t first = 0;
  for (int q = 0; q < r; ++q) first += (seg[q + 1] - seg[q] + rows_per_chunk - 1) / rows_per_chunk;
  const int64_t cnt = (seg[r + 1] - seg[r] + rows_per_chunk - 1) / rows_per_chunk;
  const int64_t per = (cnt + kReduceSlices - 1) / kReduceSlices;
  const int64_t c0 = sl * per, c1 = (c0 + per) < cnt ? (c0 + per) : cnt;
  float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
  if (e < kn) {
    const float* p = partial + (size_t)first * kn + e;
    int64_t c = c0;
    for (; c + 4 <= c1; c += 4) {
      a0 += p[(size_t)(c + 0) * kn];
      a1 += p[(size_t)(c + 1) * kn];
      a2 += p[(size_t)(c + 2) * kn];
      a3 += p[(size_t)(c + 3) * kn];
    }
    for (; c < c1; ++c) a0 += p[(size_t)c * kn];
  }
  s_run[sl][el] = (a0 + a1) + (a2 + a3);
  __syncthreads();
  if (sl == 0 && e < kn) {
    float acc = s_run[0][el];
#pragma unroll
    for (int q = 1; q < kReduceSlices; ++q) acc += s_run[q][el];
    gw[(size_t)r * kn + e] = acc;
  }
}

// Rows per chunk.  A CU runs one block (chunk x column tile) at a time and every block ends
// with a K x 128 partial that the reduction reads again, so few long chunks beat many short
// ones: the number of rounds of one block per CU that the longest chunks would need, then
// the chunk length that fills those rounds evenly.
int64_t chunk_rows(int64_t M, int K, int N, bool mapped) {
  const int64_t g_max = (mapped ? kMappedRows : 256 * kMT) / kMT;
  const int64_t tiles = ceil_div(M, (int64_t)kMT) * ceil_div(N, 128) * ceil_div(K, 128);
  int64_t rounds = ceil_div(tiles, 256 * g_max);
  if (rounds < 1) rounds = 1;
  int64_t g = ceil_div(tiles, 256 * rounds);
  if (g < 8) g = 8;
  if (g > g_max) g = g_max;
  return g * kMT;
}

}  // namespace
}  // namespace cxg

extern "C" {

size_t cxg_typed_gemm_wgrad_workspace_bytes(int64_t M, int K, int N, int R) {
  if (M < 0 || K < 1 || N < 1 || R < 1) return 0;
  // the chunks of a launch with row maps are the shorter ones: their count bounds both cases
  const int64_t chunks = cxg::ceil_div(cxg::ceil_div(M, cxg::chunk_rows(M, K, N, true)) + R, cxg::kXcds) * cxg::kXcds;
  return (size_t)chunks * (size_t)K * (size_t)N * sizeof(float) + 256;
}

int cxg_typed_gemm_wgrad_f32(const float* a, int64_t lda, const float* g, int64_t ldg,
                             const int64_t* src_idx, const int64_t* dst_idx, const int64_t* seg_ptr,
                             int64_t M, int K, int N, int R, float* gw, unsigned flags, void* workspace,
                             size_t workspace_bytes, void* stream) {
  CXG_REQUIRE(M >= 0 && K >= 1 && N >= 1 && R >= 1, CXG_ERR_ARG, "bad M/K/N/R");
  CXG_REQUIRE((flags & ~(CXG_GEMM_SPLIT_BF16X6 | CXG_GEMM_SPLIT_BF16X3 | CXG_GEMM_SPLIT_F16X3 | CXG_WGRAD_A_BF16)) == 0,
              CXG_ERR_ARG, "unknown flag");
  CXG_REQUIRE(gw && seg_ptr, CXG_ERR_ARG, "null gw/seg_ptr");
  CXG_REQUIRE(M == 0 || (a && g), CXG_ERR_ARG, "null a/g");
  CXG_REQUIRE(K <= 4096 && (K & 3) == 0 && (N & 3) == 0 && (lda & 3) == 0 && (ldg & 3) == 0 &&
                  ((uintptr_t)a & 15) == 0 && ((uintptr_t)g & 15) == 0,
              CXG_ERR_UNSUPPORTED, "wgrad needs K <= 4096, K, N, lda, ldg multiples of 4 and 16-byte aligned operands");
  CXG_REQUIRE(lda >= K && ldg >= N, CXG_ERR_ARG, "row stride smaller than row");
  const size_t need = cxg_typed_gemm_wgrad_workspace_bytes(M, K, N, R);
  CXG_REQUIRE(workspace && workspace_bytes >= need, CXG_ERR_WORKSPACE,
              "workspace of %zu bytes needed, %zu given", need, workspace_bytes);
  CXG_REQUIRE(((uintptr_t)workspace & 255) == 0, CXG_ERR_WORKSPACE, "workspace must be 256-byte aligned");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const bool mapped = src_idx || dst_idx;
  const int64_t rows = cxg::chunk_rows(M, K, N, mapped);
  const int64_t chunks = cxg::ceil_div(cxg::ceil_div(M, rows) + R, cxg::kXcds) * cxg::kXcds;
  const int n_ct = (int)(cxg::ceil_div(N, 128) * cxg::ceil_div(K, 128));     // 128 x 128 tiles of gw
  CXG_REQUIRE(chunks * n_ct < ((int64_t)1 << 31), CXG_ERR_UNSUPPORTED, "too many chunks for one launch");
  cxg::WgradArgs wa{a, lda, g, ldg, src_idx, dst_idx, seg_ptr, reinterpret_cast<float*>(workspace),
                    M, K, N, R, rows, (int)((flags & CXG_WGRAD_A_BF16) != 0)};
  const dim3 grid((unsigned)(chunks * n_ct)), block(cxg::kWgThreads);
#define CXG_WGRAD_LAUNCH_T(NSV, MAP, HALF, AH)                                                             \
  do {                                                                                                    \
    CXG_HIP_CHECK(cxg::allow_lds(cxg::typed_wgrad_split_kernel<NSV, MAP, HALF, AH>, cxg::wgrad_lds_bytes<NSV>(MAP))); \
    hipLaunchKernelGGL((cxg::typed_wgrad_split_kernel<NSV, MAP, HALF, AH>), grid, block, cxg::wgrad_lds_bytes<NSV>(MAP), st, wa); \
  } while (0)
#define CXG_WGRAD_LAUNCH(NSV, MAP, HALF)                                                                  \
  do {                                                                                                    \
    if (wa.a_bf16) CXG_WGRAD_LAUNCH_T(NSV, MAP, HALF, true);                                              \
    else CXG_WGRAD_LAUNCH_T(NSV, MAP, HALF, false);                                                       \
  } while (0)
  if (flags & CXG_GEMM_SPLIT_F16X3) {
    if (mapped) CXG_WGRAD_LAUNCH(2, true, true);
    else CXG_WGRAD_LAUNCH(2, false, true);
  } else if (flags & CXG_GEMM_SPLIT_BF16X3) {
    if (mapped) CXG_WGRAD_LAUNCH(2, true, false);
    else CXG_WGRAD_LAUNCH(2, false, false);
  } else {
    if (mapped) CXG_WGRAD_LAUNCH(3, true, false);
    else CXG_WGRAD_LAUNCH(3, false, false);
  }
#undef CXG_WGRAD_LAUNCH
#undef CXG_WGRAD_LAUNCH_T
  CXG_LAUNCH_CHECK("typed_wgrad_split_kernel");
  const int64_t kn = (int64_t)K * N;
  hipLaunchKernelGGL(cxg::wgrad_reduce_kernel, dim3((unsigned)cxg::ceil_div(kn, 64), (unsigned)R),
                     dim3(64 * cxg::kReduceSlices), 0,
                     st, seg_ptr, R, rows, reinterpret_cast<const float*>(workspace), gw, kn);
  CXG_LAUNCH_CHECK("wgrad_reduce_kernel");
  return CXG_OK;
}

}  // extern "C"
