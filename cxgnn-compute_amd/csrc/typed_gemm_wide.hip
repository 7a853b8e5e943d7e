// Typed GEMM for wide operands (K above what a wave can keep of W in registers):
//
//   C[dst(i), :] (=, +=, atomic +=)  A[src(i), :] @ W[rel(i)],   K >= 160, any N
//
// fp32 operands, every product formed on the fp16 matrix cores from three partial products
// of scaled fp16 parts (the CXG_GEMM_SPLIT_F16X3 arithmetic of typed_gemm.hip: x s = h0 + h1,
// 22 significant bits, a b ~ a0 b1 + a1 b0 + a0 b0 on v_mfma_f32_32x32x16_f16).  At K = N = 512
// the product is matrix-core bound (128 flop per byte moved), so unlike the narrow forms this
// is a classical tiled GEMM: block tile 128 rows x 256 columns, K walked in chunks of 32 with
// both operand tiles in LDS.
//
//   * W is split once per call by a small kernel (wide_split_w_kernel) into the caller's
//     workspace: per relation, column tile and k-chunk the two fp16 parts of a 256 x 32 block,
//     k fastest, zero padded, each column scaled by the power of two that brings its largest
//     magnitude into [2^14, 2^15); the inverse scales go next to it.
//   * Four producer waves fetch the A rows of a chunk (128 bytes per row), two chunks ahead in
//     two register sets, scale and split the values and write the parts into one half of a
//     double-buffered LDS area.  The matching 32 KB block of split W needs no arithmetic: it
//     goes from memory straight into LDS (global_load_lds_dwordx4, 1 KB per instruction, lane l
//     lands at base + 16 l), two chunks ahead into one of three W areas; the workspace holds
//     each block in LDS order, with the 16-byte pieces of a column swizzled ((k / 8) ^ (column /
//     4 mod 4)) so that the unpadded 64-byte columns are read without bank conflicts.
//   * Four consumer waves (2 x 2, each 64 rows x 128 columns = eight 32 x 32 accumulators)
//     multiply a chunk out of the other half.  The block barrier of a chunk sits between the
//     chunk's two k-steps: the operands of the second step are read before it and those of the
//     next chunk's first step right after it, so the matrix pipe never waits for an LDS round
//     trip at a chunk boundary.
//   * Row scales.  A row's largest magnitude is only known once all of K has been seen, and a
//     512-wide row tile does not fit the LDS, so the scale of a row follows the largest
//     magnitude met so far: it starts at 2^127 and is lowered, so that the magnitude lands in
//     [2^12, 2^13), whenever a value would otherwise reach 2^15 -- three bits of headroom, so
//     for rows of comparable entries it moves once, in the first chunk that holds a value.  When it does move, the producers leave the power-of-two ratio per row in
//     LDS and raise a per-chunk flag, and the consumers multiply their accumulators by the
//     ratios before they add that chunk (exact: powers of two).  An element keeps its 22 bits
//     down to 2^-15 of the magnitude that set the scale and is off by at most 2^-37 of it below.
//
// Replaces the Triton typed_matmul launcher for the wide shapes its benchmarks use
// (cxgnncomp/codegen/triton_typed_matmul.py:752-860; test/ae/E3_ablation/test-batch.py:27-52
// runs K = N = 512).
#include "cxg_common.hpp"
#include "split_f16.hpp"

namespace cxg {
namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));   // native vectors for values kept in flight: a struct
typedef float v4f __attribute__((ext_vector_type(4)));      // copy from global memory is a memcpy into a stack slot

constexpr int kWM = 128;                   // rows of a block tile
constexpr int kWN = 256;                   // columns of a block tile
constexpr int kWK = 32;                    // k per chunk
constexpr int kWP = 40;                    // LDS row pitch in fp16 elements (80 bytes: 16 rows cover all banks)
constexpr int kWThreads = 512;             // waves 0-3 consume, waves 4-7 produce
constexpr int kWXcds = 8;
constexpr int kWBlockHalfs = 2 * kWN * kWK;   // fp16 elements of one (relation, column tile, chunk) block of split W
constexpr int kWMaxTiles = 8;              // row tiles per block
constexpr int kWBlockBytes = kWBlockHalfs * 2;                       // 32 KB
constexpr int kWAsBytes = 2 * 2 * kWM * kWP * 2;                     // both stages, both parts of the A tile
// Requests per producer wave and chunk: 16-byte A loads per lane, 1 KB memory -> LDS requests of the W
// block.  The producers wait with hand-written counts -- vmcnt(12) before a set of A registers is
// used, vmcnt(16) before the barrier that publishes a W block -- which hold for exactly these numbers.
constexpr int kWReqA = 4;
constexpr int kWReqW = 8;
static_assert(kWReqA + kWReqW == 12 && 2 * kWReqA + kWReqW == 16, "the s_waitcnt vmcnt(12) / vmcnt(16) of the producers");
static_assert(kWReqW * 1024 * 4 == kWBlockBytes, "four producer waves fetch one W block");
static_assert(kWReqA * 16 * 64 * 4 == kWM * kWK * 4, "four producer waves fetch one A chunk");
constexpr int kWCP = 136;                  // floats per row of a consumer wave's store staging area

struct WideArgs {
  const float* a;
  int64_t lda;
  const uint16_t* wt;                      // [R][n_ct][n_kc][2][256][32] fp16
  const float* inv_w;                      // [R][n_ct * 256]
  float* c;
  int64_t ldc;
  const int64_t* src;
  const int64_t* dst;
  const int64_t* seg;
  int64_t M;
  int K, N, R;
  int accumulate, atomic;
  int n_ct, n_kc;
};

// scale 2^(target - e) and its inverse for a magnitude with biased exponent eb (e = eb - 127)
__device__ __forceinline__ void col_scales(unsigned max_bits, float& scale, float& inv) {
  const int eb = (int)(max_bits >> 23);
  scale = 0.f;
  inv = 0.f;
  if (eb == 255) {
    scale = 1.f;
    inv = 1.f;
  } else if (eb >= 15) {
    scale = __uint_as_float((unsigned)(268 - eb) << 23);    // magnitude -> [2^14, 2^15)
    inv = __uint_as_float((unsigned)(eb - 14) << 23);
  }
}

// One block per (relation, column tile): 1024 threads = 256 columns x 4 quarters of the chunks.
__global__ __launch_bounds__(1024) void wide_split_w_kernel(const float* __restrict__ w, uint16_t* __restrict__ wt,
                                                            float* __restrict__ inv_w, int K, int N, int n_ct,
                                                            int n_kc) {
  __shared__ unsigned s_max[4][256];
  const int r = blockIdx.x / n_ct, ct = blockIdx.x % n_ct;
  const int cl = threadIdx.x & 255, kq = threadIdx.x >> 8;
  const int col = ct * kWN + cl;
  const float* W = w + (int64_t)r * K * N;
  const int per = (n_kc + 3) / 4;
  const int c_lo = kq * per, c_hi = (c_lo + per) < n_kc ? (c_lo + per) : n_kc;
  unsigned m = 0;
  if (col < N) {
    const int k_hi = c_hi * kWK < K ? c_hi * kWK : K;
    for (int k = c_lo * kWK; k < k_hi; ++k) {
      const unsigned b = __float_as_uint(W[(int64_t)k * N + col]) & 0x7fffffffu;
      m = b > m ? b : m;
    }
  }
  s_max[kq][cl] = m;
  __syncthreads();
#pragma unroll
  for (int q = 0; q < 4; ++q) m = s_max[q][cl] > m ? s_max[q][cl] : m;
  float scale, inv;
  col_scales(m, scale, inv);
  if (kq == 0) inv_w[((int64_t)r * n_ct + ct) * kWN + cl] = inv;
  for (int c = c_lo; c < c_hi; ++c) {
    uint16_t* base = wt + ((int64_t)(r * n_ct + ct) * n_kc + c) * kWBlockHalfs;
#pragma unroll
    for (int k8 = 0; k8 < kWK / 8; ++k8) {
      v8h h0, h1;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int k = c * kWK + k8 * 8 + j;
        const float x = (k < K && col < N) ? W[(int64_t)k * N + col] * scale : 0.f;
        h0[j] = (_Float16)x;
        h1[j] = (_Float16)(x - (float)h0[j]);
      }
      const int slot = cl * 4 + (k8 ^ ((cl >> 2) & 3));       // LDS order: see wide_w_offset
      *reinterpret_cast<v8h*>(base + (0 * kWN * 4 + slot) * 8) = h0;
      *reinterpret_cast<v8h*>(base + (1 * kWN * 4 + slot) * 8) = h1;
    }
  }
}

template <int CTRL>
__device__ __forceinline__ unsigned wide_dpp_max(unsigned m) {
  const unsigned o = (unsigned)__builtin_amdgcn_update_dpp(0, (int)m, CTRL, 0xf, 0xf, false);
  return o > m ? o : m;
}

__global__ __launch_bounds__(kWThreads) __attribute__((amdgpu_waves_per_eu(2)))
void typed_gemm_wide_kernel(WideArgs g, int G) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  // As[2 stages][2 parts][128][40] fp16, Ws[3 areas][2 parts][256 columns x 64 bytes]; then the per-row tables
  uint16_t (*As)[2][kWM][kWP] = reinterpret_cast<uint16_t (*)[2][kWM][kWP]>(smem);
  unsigned char* const Ws = smem + kWAsBytes;
  unsigned char* tail = smem + kWAsBytes + 3 * kWBlockBytes;
  float (*s_ratio)[kWM] = reinterpret_cast<float (*)[kWM]>(tail);                    // per stage
  float (*s_inv)[kWM] = reinterpret_cast<float (*)[kWM]>(tail + 2 * kWM * 4);         // per tile parity
  int64_t (*s_src)[kWM] = reinterpret_cast<int64_t (*)[kWM]>(tail + 4 * kWM * 4);     // per tile parity
  int64_t (*s_dst)[kWM] = s_src + 2;
  int* s_flag = reinterpret_cast<int*>(s_dst + 2);                                   // per stage

  const int64_t span = (int64_t)kWM * G;
  int rel = -1;
  int64_t row0 = 0, row_end = 0;
  // the column tiles of one row chunk take consecutive slots of ONE accelerator die, whose L2
  // then serves the chunk's A rows to all of them (blocks go to the dies round-robin)
  const int n_ct = g.n_ct;
  const int64_t slot = blockIdx.x / kWXcds;
  const int64_t chunk = (slot / n_ct) * kWXcds + (blockIdx.x % kWXcds);
  {
    int64_t t = chunk;
    for (int r = 0; r < g.R; ++r) {
      const int64_t b = g.seg[r], e = g.seg[r + 1];
      const int64_t nt = (e - b + span - 1) / span;
      if (t < nt) { rel = r; row0 = b + t * span; row_end = e; break; }
      t -= nt;
    }
  }
  if (rel < 0) return;                       // whole block, before any barrier
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = uniform_i32(tid >> 6);
  const int ct = (int)(slot % n_ct);
  const int n0 = ct * kWN;
  const int K = g.K, N = g.N, NC = g.n_kc;
  const int64_t rows_here = (row_end - row0) < span ? (row_end - row0) : span;
  const int n_tiles = (int)((rows_here + kWM - 1) / kWM);
  const int total = n_tiles * NC;            // chunks of this block
  if (tid < 2) s_flag[tid] = 0;

  if (wave < 4) {
    // ---------------------------------------------------------------- consumers
    const int wm = wave >> 1, wn = wave & 1;
    __syncthreads();                         // T: row tables of tile 0
    __syncthreads();                         // P: chunk 0 staged
    if (n0 + wn * 128 >= N) {                // all of this wave's columns lie past N
      for (int gc = 0; gc < total; ++gc) __syncthreads();
      return;
    }
    // this wave's staging area for stores, 8 rows x (128 + 8) floats (rows 4 apart land 32 banks apart)
    float (*Cw)[kWCP] = reinterpret_cast<float (*)[kWCP]>(reinterpret_cast<unsigned char*>(s_flag) + 16) + (size_t)wave * 8;
    const bool wide_store = !g.atomic && n0 + wn * 128 + 128 <= N && (g.ldc & 3) == 0 && ((uintptr_t)g.c & 15) == 0;
    float invw[4];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
      invw[nt] = g.inv_w[((int64_t)rel * n_ct + ct) * kWN + wn * 128 + nt * 32 + (lane & 31)];
    v16f acc[4][2];
    v8h xa[2][2], xb[4][2], ya[2][2], yb[4][2];
    // byte offset of this lane's W operand inside a part of a W area, k-step s: column
    // (lane & 31) of its 32, piece 2 s + (lane >> 5) of the column's four, swizzled
    const int wsw = (lane >> 2) & 3;
    const int woff[2] = {(wn * 128 + (lane & 31)) * 64 + (((lane >> 5)) ^ wsw) * 16,
                         (wn * 128 + (lane & 31)) * 64 + ((2 + (lane >> 5)) ^ wsw) * 16};
    auto read_ops = [&](v8h (&a)[2][2], v8h (&b)[4][2], int st, int wst, int s) __attribute__((always_inline)) {
      const int k = s * 16 + (lane >> 5) * 8;
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int p = 0; p < 2; ++p)
          a[mt][p] = *reinterpret_cast<const v8h*>(&As[st][p][wm * 64 + mt * 32 + (lane & 31)][k]);
      const unsigned char* wb = Ws + wst * kWBlockBytes + woff[s];
#pragma unroll
      for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int p = 0; p < 2; ++p)
          b[nt][p] = *reinterpret_cast<const v8h*>(wb + p * (kWBlockBytes / 2) + nt * 32 * 64);
    };
    // smallest products first; the eight accumulators take turns, so consecutive matrix
    // instructions never depend on each other
    auto mfmas = [&](const v8h (&a)[2][2], const v8h (&b)[4][2]) __attribute__((always_inline)) {
#pragma unroll
      for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
          acc[nt][mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[mt][0], b[nt][1], acc[nt][mt], 0, 0, 0);
#pragma unroll
      for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
          acc[nt][mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[mt][1], b[nt][0], acc[nt][mt], 0, 0, 0);
#pragma unroll
      for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
          acc[nt][mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[mt][0], b[nt][0], acc[nt][mt], 0, 0, 0);
    };
    read_ops(xa, xb, 0, 0, 0);
    int gc = 0;
    int wst = 0;                             // W area of chunk gc: gc mod 3
    int flag = 0;                            // s_flag of the chunk about to start, read a k-step ahead
    for (int t = 0; t < n_tiles; ++t) {
#pragma unroll
      for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[nt][mt][i] = 0.f;
      for (int c = 0; c < NC; ++c, ++gc) {
        const int st = gc & 1;
        if (c > 0 && uniform_i32(flag) == gc + 1) {
          // a row scale was lowered for this chunk: bring the sums so far to the new unit
#pragma unroll
          for (int mt = 0; mt < 2; ++mt)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const float4 rr = *reinterpret_cast<const float4*>(&s_ratio[st][wm * 64 + mt * 32 + q * 8 + (lane >> 5) * 4]);
#pragma unroll
              for (int nt = 0; nt < 4; ++nt) {
                acc[nt][mt][q * 4 + 0] *= rr.x;
                acc[nt][mt][q * 4 + 1] *= rr.y;
                acc[nt][mt][q * 4 + 2] *= rr.z;
                acc[nt][mt][q * 4 + 3] *= rr.w;
              }
            }
        }
        // (the scheduling groups put the LDS reads of the next k-step between the first matrix
        // instructions of this step; left alone, the compiler sinks each read to just before its
        // first use and the matrix pipe waits for an LDS round trip per operand)
        read_ops(ya, yb, st, wst, 1);
        mfmas(xa, xb);
#pragma unroll
        for (int i = 0; i < 12; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one matrix instruction
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 12, 0);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();                     // chunk gc + 1 is staged; chunk gc has been read
        flag = s_flag[st ^ 1];
        wst = wst == 2 ? 0 : wst + 1;
        read_ops(xa, xb, st ^ 1, wst, 0);
        mfmas(ya, yb);
#pragma unroll
        for (int i = 0; i < 13; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 11, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
      // undo the scales and store: accumulator element i of (nt, mt) is row
      // wm*64 + mt*32 + (i>>2)*8 + (lane>>5)*4 + (i&3), column n0 + wn*128 + nt*32 + (lane&31)
      const int64_t* drow = s_dst[t & 1];
      float4 pv[4];                          // the group of rows read back last, not yet stored
      int64_t pd[4];
      auto store_group = [&](const float4 (&v)[4], const int64_t (&d)[4]) __attribute__((always_inline)) {
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          if (d[it] < 0) continue;
          float4* const p = reinterpret_cast<float4*>(g.c + d[it] * g.ldc + n0 + wn * 128 + (lane & 31) * 4);
          if (g.accumulate) {
            const float4 o = *p;
            *p = make_float4(o.x + v[it].x, o.y + v[it].y, o.z + v[it].z, o.w + v[it].w);
          } else {
            stream_store(reinterpret_cast<float*>(p), v[it]);   // written once: not kept in the L2, where W and the A rows live
          }
        }
      };
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int rl0 = wm * 64 + mt * 32 + q * 8 + (lane >> 5) * 4;
          const float4 ri = *reinterpret_cast<const float4*>(&s_inv[t & 1][rl0]);
          const float rinv[4] = {ri.x, ri.y, ri.z, ri.w};
          if (wide_store) {
            // Eight rows x this wave's 128 columns go through the wave's own LDS area and leave
            // as 16 bytes per lane, 512 contiguous bytes per row: a quarter of the store
            // instructions of 4-byte stores from the accumulators (128 per tile and wave, which
            // cost the K = N = 512 product 1.5 of its 5.1 ms).  LDS operations of one wave
            // execute in order, so the area needs no barrier, and the rows of a group are stored
            // only after the next group has been written and read back: its LDS round trip runs
            // while the stores are issued (a group at a time, every store behind two LDS round
            // trips of its own, took 1,200 cycles per group).
#pragma unroll
            for (int nt = 0; nt < 4; ++nt)
#pragma unroll
              for (int j = 0; j < 4; ++j)
                Cw[(lane >> 5) * 4 + j][nt * 32 + (lane & 31)] = acc[nt][mt][q * 4 + j] * (rinv[j] * invw[nt]);
            float4 cv[4];
            int64_t cd[4];
#pragma unroll
            for (int it = 0; it < 4; ++it) {
              const int rl = it * 2 + (lane >> 5);
              cv[it] = *reinterpret_cast<const float4*>(&Cw[rl][(lane & 31) * 4]);
              cd[it] = drow[wm * 64 + mt * 32 + q * 8 + rl];
            }
            if (mt + q > 0) store_group(pv, pd);
#pragma unroll
            for (int it = 0; it < 4; ++it) { pv[it] = cv[it]; pd[it] = cd[it]; }
            if (mt == 1 && q == 3) store_group(pv, pd);
            continue;
          }
          int64_t d[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) d[j] = drow[rl0 + j];
#pragma unroll
          for (int nt = 0; nt < 4; ++nt) {
            const int col = n0 + wn * 128 + nt * 32 + (lane & 31);
            if (col >= N) continue;
            float v[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = acc[nt][mt][q * 4 + j] * (rinv[j] * invw[nt]);
            if (g.atomic) {
#pragma unroll
              for (int j = 0; j < 4; ++j)
                if (d[j] >= 0) unsafeAtomicAdd(g.c + d[j] * g.ldc + col, v[j]);
            } else if (g.accumulate) {
              float o[4];
#pragma unroll
              for (int j = 0; j < 4; ++j) o[j] = d[j] >= 0 ? g.c[d[j] * g.ldc + col] : 0.f;
#pragma unroll
              for (int j = 0; j < 4; ++j)
                if (d[j] >= 0) g.c[d[j] * g.ldc + col] = o[j] + v[j];
            } else {
#pragma unroll
              for (int j = 0; j < 4; ++j)
                if (d[j] >= 0) g.c[d[j] * g.ldc + col] = v[j];
            }
          }
        }
    }
    return;
  }

  // ------------------------------------------------------------------ producers
  const int ptid = tid & 255;
  const int c4 = ptid & 7, rsub = ptid >> 3;           // a row chunk is 8 lanes x 16 bytes; 32 rows per instruction
  const float* const A = g.a;
  const uint16_t* const Wb = g.wt + (int64_t)(rel * n_ct + ct) * NC * kWBlockHalfs;
  auto fill_tables = [&](int t) __attribute__((always_inline)) {
    if (ptid < kWM && t < n_tiles) {
      const int64_t gr = row0 + (int64_t)t * kWM + ptid;
      int64_t s = -1, d = -1;
      if (gr < row_end) {
        s = g.src ? g.src[gr] : gr;
        d = g.dst ? g.dst[gr] : gr;
        if (s < 0 || d < 0) s = d = -1;                // a negative entry in either map drops the row
      }
      s_src[t & 1][ptid] = s;
      s_dst[t & 1][ptid] = d;
    }
  };
  // load side: chunk (ld_t, ld_c) is the next one to request
  int ld_t = 0, ld_c = 0;
  int64_t rowoff[4];
  auto gload = [&](v4f (&ar)[4]) __attribute__((always_inline)) {
    const int tc = ld_t < n_tiles ? ld_t : n_tiles - 1;   // past the end: the last tile again (never staged)
    if (ld_c == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int64_t s = s_src[tc & 1][rsub + 32 * i];
        rowoff[i] = (s >= 0 ? s : 0) * g.lda;
      }
    }
    const int kcol = ld_c * kWK + 4 * c4;
    const int koff = kcol < K ? kcol : 0;
    // (inline assembly, like the W requests below and for the same reason: the waits are placed
    // by hand, see a_wait)
#pragma unroll
    for (int i = 0; i < kWReqA; ++i) {
      const float* p = A + rowoff[i] + koff;
      asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(ar[i]) : "v"(p) : "memory");
    }
    if (++ld_c == NC) { ld_c = 0; ++ld_t; }
  };
  // The A registers of a set may be used once at most 12 younger requests (a W block and the
  // other set) are outstanding: a wave's memory requests complete in order.
  auto a_wait = [&](v4f (&ar)[4]) __attribute__((always_inline)) {
    asm volatile("s_waitcnt vmcnt(12)" : "+v"(ar[0]), "+v"(ar[1]), "+v"(ar[2]), "+v"(ar[3]) : : "memory");
  };
  // W side: the block of chunk dm_c goes straight into W area dm_a, 8 KB per producer wave
  int dm_c = 0, dm_a = 0;
  const int pw = wave - 4;
  // (Written as inline assembly: for a load into LDS that the compiler knows of, it waits for
  // every outstanding load of the wave before each later LDS access of the wave and before
  // every barrier -- the A rows two chunks ahead included -- and requests it does not know of
  // would be missing from its count of loads in flight.  So every request of the producers'
  // loop is issued and waited for by hand: the order is A, W, A, W, ...)
  const unsigned lane16 = (unsigned)lane * 16u;
  auto dma_w = [&]() __attribute__((always_inline)) {
    const unsigned char* src = reinterpret_cast<const unsigned char*>(Wb) + (int64_t)dm_c * kWBlockBytes + pw * 8192;
    const unsigned dst = (unsigned)(uintptr_t)(__attribute__((address_space(3))) void*)(Ws + dm_a * kWBlockBytes + pw * 8192);
#pragma unroll
    for (int j = 0; j < kWReqW; ++j) {
      const unsigned char* sj = src + j * 1024;
      const unsigned dj = dst + j * 1024;
      asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(lane16), "s"(sj), "s"(dj) : "memory", "m0");
    }
    if (++dm_c == NC) dm_c = 0;
    dm_a = dm_a == 2 ? 0 : dm_a + 1;
  };
  // staging side: chunk (st_t, st_c), global number st_g
  int st_t = 0, st_c = 0, st_g = 0;
  unsigned rmax[4] = {0u, 0u, 0u, 0u};
  int sb[4] = {254, 254, 254, 254};                      // biased exponent of the row scale
  auto stage = [&](const v4f (&ar)[4]) __attribute__((always_inline)) {
    if (st_g >= total) return;
    const int st = st_g & 1;
    if (st_c == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) { rmax[i] = 0u; sb[i] = 254; }
    }
    v4f v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = ar[i];
    if ((st_c + 1) * kWK > K) {                            // the chunk that holds the end of K (K not a multiple of 32)
      const bool k_ok = st_c * kWK + 4 * c4 < K;
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) v[i][j] = k_ok ? v[i][j] : 0.f;
    }
    // The scale of a row is 2^(sb - 127).  It starts at 2^127 (rows that never exceed 2^-113
    // are multiplied by it and come out as zeros: their inverse scale is 0) and is lowered, to
    // put the largest magnitude met so far into [2^12, 2^13), whenever that magnitude times
    // the scale would reach 2^15.  A row with an infinity gets 2^-116 and comes out non-finite.
    float ratio[4];
    int lowered = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      unsigned m = abs_max4_bits(v[i][0], v[i][1], v[i][2], v[i][3]);
      m = wide_dpp_max<0xB1>(m);                         // lane ^ 1
      m = wide_dpp_max<0x4E>(m);                         // lane ^ 2
      m = wide_dpp_max<0x141>(m);                        // mirror of the 8 lanes that hold the row chunk
      rmax[i] = m > rmax[i] ? m : rmax[i];
      const int eb = (int)(rmax[i] >> 23);
      const int lower = eb + sb[i] >= 269;               // unbiased exponent of (maximum x scale) >= 15
      const int nsb = lower ? 266 - eb : sb[i];
      const int re = 127 + nsb - sb[i];                  // <= 127; below 1 the old sums vanish next to the new values
      ratio[i] = __uint_as_float((unsigned)(re > 0 ? re : 0) << 23);
      lowered |= lower;
      sb[i] = nsb;
      const float scale = __uint_as_float((unsigned)nsb << 23);
      unsigned hi2[2], lo2[2];
#pragma unroll
      for (int jp = 0; jp < 2; ++jp) split_f16_pair(v[i][2 * jp], v[i][2 * jp + 1], scale, hi2[jp], lo2[jp]);
      typedef unsigned v2u __attribute__((ext_vector_type(2)));
      const v2u part0 = {hi2[0], hi2[1]}, part1 = {lo2[0], lo2[1]};
      const int row = rsub + 32 * i;
      *reinterpret_cast<v2u*>(&As[st][0][row][4 * c4]) = part0;
      *reinterpret_cast<v2u*>(&As[st][1][row][4 * c4]) = part1;
    }
    if (c4 == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) s_ratio[st][rsub + 32 * i] = ratio[i];
      if (st_c == NC - 1) {
#pragma unroll
        for (int i = 0; i < 4; ++i) s_inv[st_t & 1][rsub + 32 * i] = __uint_as_float((unsigned)(254 - sb[i]) << 23);
      }
      if (lowered) s_flag[st] = st_g + 1;
    }
    ++st_g;
    if (++st_c == NC) { st_c = 0; ++st_t; }
  };

  v4f a0[4], a1[4];
  fill_tables(0);
  __syncthreads();                           // T
  gload(a0);                                 // chunk 0
  dma_w();                                   // W of chunk 0
  gload(a1);                                 // chunk 1
  a_wait(a0);
  stage(a0);
  dma_w();                                   // W of chunk 1
  gload(a0);                                 // chunk 2
  // the W block of chunk 0 has arrived when at most the 4 + 8 + 4 requests issued after it are
  // outstanding.  vmcnt(16), no wait on the other counters:
  __builtin_amdgcn_s_waitcnt(0x4F70);
  __syncthreads();                           // P
  // Iteration gc (between the barriers of chunks gc-1 and gc): split chunk gc+1 of A into its
  // LDS half, send chunk gc+2 of W on its way into the W area that chunk gc-1 has left, and
  // request chunk gc+3 of A.  (With the W block requested first it would have half an iteration
  // more to arrive; measured, that order is slower, 4.43 against 4.22 ms at K = N = 512.)  Two
  // iterations per trip so that each register set keeps its role.  The row tables of tile t+1
  // are written during chunk 1 of tile t: the consumers are then done with the tables of tile
  // t-1 (same slots), and the loads of tile t+1 start at the earliest in chunk NC-3 >= 2.
  int it_c = 0, it_t = 0;                    // (tile, chunk) of iteration gc
  auto tables_due = [&]() __attribute__((always_inline)) {
    if (it_c == 1) fill_tables(it_t + 1);
    if (++it_c == NC) { it_c = 0; ++it_t; }
  };
  for (int gc = 0;; gc += 2) {
    if (gc >= total) break;
    tables_due();
    a_wait(a1);
    stage(a1);
    dma_w();
    gload(a1);
    __builtin_amdgcn_s_waitcnt(0x4F70);      // W of chunk gc+1 is in LDS: 4 + 8 + 4 requests were issued after it
    __syncthreads();
    if (gc + 1 >= total) break;
    tables_due();
    a_wait(a0);
    stage(a0);
    dma_w();
    gload(a0);
    __builtin_amdgcn_s_waitcnt(0x4F70);
    __syncthreads();
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);        // nothing of this wave is on its way into LDS when it ends
}

constexpr size_t kWideLds = kWAsBytes + 3 * kWBlockBytes + 4 * kWM * 4 + 4 * kWM * 8 + 16 + 4 * 8 * kWCP * 4;
static_assert(kWideLds <= 160 * 1024, "LDS of a CU");

}  // namespace
}  // namespace cxg

extern "C" {

size_t cxg_typed_gemm_wide_workspace_bytes(int K, int N, int R) {
  if (K < 1 || N < 1 || R < 1) return 0;
  const int64_t n_ct = cxg::ceil_div(N, cxg::kWN), n_kc = cxg::ceil_div(K, cxg::kWK);
  return (size_t)(R * n_ct * n_kc * cxg::kWBlockHalfs * 2 + R * n_ct * cxg::kWN * 4);
}

int cxg_typed_gemm_wide_f32(const float* a, int64_t lda, const float* w, float* c, int64_t ldc,
                            const int64_t* src_idx, const int64_t* dst_idx, const int64_t* seg_ptr, int64_t M, int K,
                            int N, int R, unsigned flags, void* workspace, size_t workspace_bytes, void* stream) {
  CXG_REQUIRE(M >= 0 && K >= 1 && N >= 1 && R >= 1, CXG_ERR_ARG, "bad M/K/N/R");
  CXG_REQUIRE((flags & ~(CXG_GEMM_ACCUMULATE | CXG_GEMM_ATOMIC | CXG_GEMM_SPLIT_F16X3)) == 0, CXG_ERR_ARG,
              "the wide form takes CXG_GEMM_ACCUMULATE, CXG_GEMM_ATOMIC and CXG_GEMM_SPLIT_F16X3 only");
  if (M == 0) return CXG_OK;
  CXG_REQUIRE(a && w && c && seg_ptr, CXG_ERR_ARG, "null pointer");
  CXG_REQUIRE(lda >= K && ldc >= N, CXG_ERR_ARG, "row stride smaller than row");
  CXG_REQUIRE(K >= 160 && (K & 3) == 0 && (lda & 3) == 0 && ((uintptr_t)a & 15) == 0, CXG_ERR_UNSUPPORTED,
              "the wide form needs K >= 160, K and lda multiples of 4 and A 16-byte aligned");
  const size_t need = cxg_typed_gemm_wide_workspace_bytes(K, N, R);
  CXG_REQUIRE(workspace && workspace_bytes >= need && ((uintptr_t)workspace & 15) == 0, CXG_ERR_WORKSPACE,
              "workspace too small or misaligned: need %zu bytes", need);
  const int n_ct = (int)cxg::ceil_div(N, cxg::kWN), n_kc = (int)cxg::ceil_div(K, cxg::kWK);
  uint16_t* wt = reinterpret_cast<uint16_t*>(workspace);
  float* inv_w = reinterpret_cast<float*>(wt + (size_t)R * n_ct * n_kc * cxg::kWBlockHalfs);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(cxg::wide_split_w_kernel, dim3((unsigned)(R * n_ct)), dim3(1024), 0, st, w, wt, inv_w, K, N, n_ct,
                     n_kc);
  CXG_LAUNCH_CHECK("wide_split_w_kernel");
  cxg::WideArgs g{a, lda, wt, inv_w, c, ldc, src_idx, dst_idx, seg_ptr, M, K, N, R,
                  (int)(flags & CXG_GEMM_ACCUMULATE), (int)((flags & CXG_GEMM_ATOMIC) != 0), n_ct, n_kc};
  // row tiles per block: the rounds of one block per CU that the largest blocks would need,
  // then the size that fills those rounds evenly
  const int64_t tiles = cxg::ceil_div(M, cxg::kWM) * n_ct;
  const int64_t rounds = cxg::ceil_div(tiles, (int64_t)256 * cxg::kWMaxTiles);
  int G = (int)cxg::ceil_div(tiles, 256 * (rounds < 1 ? 1 : rounds));
  G = G < 1 ? 1 : (G > cxg::kWMaxTiles ? cxg::kWMaxTiles : G);
  const int64_t n_chunks = cxg::ceil_div(cxg::ceil_div(M, (int64_t)cxg::kWM * G) + R, cxg::kWXcds) * cxg::kWXcds;
  const int64_t n_blocks = n_chunks * n_ct;
  CXG_REQUIRE(n_blocks < (int64_t)1 << 31, CXG_ERR_UNSUPPORTED, "too many tiles for one launch");
  CXG_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(cxg::typed_gemm_wide_kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)cxg::kWideLds));
  hipLaunchKernelGGL(cxg::typed_gemm_wide_kernel, dim3((unsigned)n_blocks), dim3(cxg::kWThreads), cxg::kWideLds, st, g,
                     G);
  CXG_LAUNCH_CHECK("typed_gemm_wide_kernel");
  return CXG_OK;
}

}  // extern "C"
