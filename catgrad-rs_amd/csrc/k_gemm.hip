// k_gemm.hip — batched matmul for gfx950: MFMA GEMM (LDS-tiled), row-dot and column GEMV.
//
// Backend::matmul (mod.rs:41; ndarray.rs:549-615): (N.., A, B) x (N.., B, C) -> (N.., A, C).
// Operands arrive as strided views, never copies: a `linear` weight W[out, in] reaches matmul
// as transpose(0,1) + reshape([1, in, out]) (stdlib/nn/mod.rs:182-192), i.e. B[k, n] with
// stride 1 along k — the "NT" layout both MFMA operands want.  K^T of attention has the same
// layout; V and rank-2 user matmuls have stride 1 along n.
//
//  * gemm_kernel: 128x128 output tile per 256-thread workgroup, four wavefronts in a 2x2 grid,
//    each owning 64x64 = 2x2 MFMA 32x32 accumulators (64 VGPRs).  Tiles are staged through LDS
//    k-contiguous for both operands; global loads for step i+1 are issued before the MFMAs of
//    step i.  bf16 mode: operands rounded to bf16 on the way into LDS, v_mfma_f32_32x32x16_bf16.
//    f32 mode: v_mfma_f32_32x32x2_f32 (gfx950 has no xf32).  MFMA-bound for M >= 64.
//  * gemv_rowdot_kernel (M <= 8, B k-contiguous): the decode path.  HBM-bound on the weight
//    matrix: every lane streams 16 bytes per load, a group of lanes owns one output column,
//    partial dots meet in a DPP/shuffle reduction; x stays in L2/registers.
//  * gemv_col_kernel (M <= 8, B n-contiguous): lanes across n, k split over the workgroup.
#include <hip/hip_runtime.h>
#include <cstring>
#include "launch.hpp"
#include "dev_common.hpp"

namespace cgk {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

__device__ __forceinline__ uint32_t bf16_rne(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (u >> 16) | 0x40u;
  return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}
__device__ __forceinline__ float widen(float v) { return v; }
__device__ __forceinline__ float widen(uint16_t v) { return __uint_as_float((uint32_t)v << 16); }

// element offset of batch (b0, b1)'s B matrix
__device__ __forceinline__ int64_t b_batch_offset(const GemmDesc &g, uint32_t bz, uint32_t b0, uint32_t b1) {
  if (g.b_index) {
    uint32_t ix = g.b_index[(int64_t)bz * g.b_index_stride];
    if (ix >= g.b_index_limit) {  // the reference's select() panics; flag it and stay in bounds
      atomicOr(g.err, ERRF_INDEX_OOB);
      ix = g.b_index_limit - 1;
    }
    return (int64_t)ix * g.sb_index;
  }
  return b0 * g.sb_b0 + b1 * g.sb_b1;
}

// ---- tile loading -------------------------------------------------------------------------
// Eight consecutive elements of a [rows, K] operand tile, either along k (KC) or along the row
// axis (!KC), zero-filled out of bounds, widened to f32.
template <typename T, bool KC>
__device__ __forceinline__ void load8(const T *base, int64_t s_row, int64_t s_k, uint32_t row,
                                      uint32_t k, uint32_t n_rows, uint32_t K, bool vec,
                                      float (&v)[8]) {
  if (KC) {
    const T *p = base + (int64_t)row * s_row + k;
    if (row < n_rows && k + 8 <= K && vec) {
      if (sizeof(T) == 4) {
        float4 q0 = *(const float4 *)p, q1 = *(const float4 *)(p + 4);
        v[0] = q0.x; v[1] = q0.y; v[2] = q0.z; v[3] = q0.w;
        v[4] = q1.x; v[5] = q1.y; v[6] = q1.z; v[7] = q1.w;
      } else {
        uint4 q = *(const uint4 *)p;
        v[0] = __uint_as_float(q.x << 16); v[1] = __uint_as_float(q.x & 0xFFFF0000u);
        v[2] = __uint_as_float(q.y << 16); v[3] = __uint_as_float(q.y & 0xFFFF0000u);
        v[4] = __uint_as_float(q.z << 16); v[5] = __uint_as_float(q.z & 0xFFFF0000u);
        v[6] = __uint_as_float(q.w << 16); v[7] = __uint_as_float(q.w & 0xFFFF0000u);
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = (row < n_rows && k + j < K) ? widen(p[j]) : 0.f;
    }
  } else {
    const T *p = base + (int64_t)k * s_k + row;
    if (k < K && row + 8 <= n_rows && vec) {
      if (sizeof(T) == 4) {
        float4 q0 = *(const float4 *)p, q1 = *(const float4 *)(p + 4);
        v[0] = q0.x; v[1] = q0.y; v[2] = q0.z; v[3] = q0.w;
        v[4] = q1.x; v[5] = q1.y; v[6] = q1.z; v[7] = q1.w;
      } else {
        uint4 q = *(const uint4 *)p;
        v[0] = __uint_as_float(q.x << 16); v[1] = __uint_as_float(q.x & 0xFFFF0000u);
        v[2] = __uint_as_float(q.y << 16); v[3] = __uint_as_float(q.y & 0xFFFF0000u);
        v[4] = __uint_as_float(q.z << 16); v[5] = __uint_as_float(q.z & 0xFFFF0000u);
        v[6] = __uint_as_float(q.w << 16); v[7] = __uint_as_float(q.w & 0xFFFF0000u);
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = (k < K && row + j < n_rows) ? widen(p[j]) : 0.f;
    }
  }
}

template <bool BF16> struct Tile;
template <> struct Tile<true> {
  enum { BK = 32, LD = 40 };  // row pitch 80 bytes: 16-byte aligned, spreads banks
  typedef uint16_t LT;
};
template <> struct Tile<false> {
  // row pitch 136 bytes: the 32 rows a wave reads for one k land on the 32 even banks, the rows of k + 1 (the upper
  // half of the wave) on the odd ones; rows are 8-byte aligned
  enum { BK = 32, LD = 34 };
  typedef float LT;
};

enum { BM = 128, BN = 128 };

template <typename TA, typename TB, bool A_KC, bool B_KC, bool BF16>
__global__ void __launch_bounds__(256) gemm_kernel(GemmDesc g, int a_vec, int b_vec) {
  typedef Tile<BF16> TL;
  typedef typename TL::LT LT;
  constexpr int BK = TL::BK, LD = TL::LD;
  constexpr int CPT = BM * BK / 8 / 256;  // 8-element chunks per thread per operand tile
  // two stages: the tile of step s + 1 is written while the MFMAs of step s read the other one
  __shared__ __attribute__((aligned(16))) LT As2[2][BM * LD];
  __shared__ __attribute__((aligned(16))) LT Bs2[2][BN * LD];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const uint32_t m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  // split-K: slice `split` of k goes to workspace[split] and a second pass sums the slices
  const uint32_t batch = g.nb0 * g.nb1, split = blockIdx.z / batch, bz = blockIdx.z - split * batch;
  const uint32_t b0 = bz / g.nb1, b1 = bz - b0 * g.nb1;
  const TA *A = (const TA *)g.a + b0 * g.sa_b0 + b1 * g.sa_b1;
  const TB *B = (const TB *)g.b + b0 * g.sb_b0 + b1 * g.sb_b1;
  float *C = (g.splits > 1 ? g.workspace + (uint64_t)split * batch * g.M * g.N : g.c) + (uint64_t)bz * g.M * g.N;
  const uint32_t k_begin = g.splits > 1 ? min(g.K, split * g.k_per_split) : 0;
  const uint32_t k_end = g.splits > 1 ? min(g.K, k_begin + g.k_per_split) : g.K;

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  float ra[CPT][8], rb[CPT][8];

  auto fetch = [&](uint32_t k0) {
#pragma unroll
    for (int c = 0; c < CPT; ++c) {
      const int chunk = tid + c * 256;
      if (A_KC) {
        const int row = chunk / (BK / 8), kc = (chunk % (BK / 8)) * 8;
        load8<TA, true>(A, g.sam, g.sak, m0 + row, k0 + kc, g.M, k_end, a_vec, ra[c]);
      } else {
        const int kk = chunk / (BM / 8), rc = (chunk % (BM / 8)) * 8;
        load8<TA, false>(A, g.sam, g.sak, m0 + rc, k0 + kk, g.M, k_end, a_vec, ra[c]);
      }
      if (B_KC) {
        const int row = chunk / (BK / 8), kc = (chunk % (BK / 8)) * 8;
        load8<TB, true>(B, g.sbn, g.sbk, n0 + row, k0 + kc, g.N, k_end, b_vec, rb[c]);
      } else {
        const int kk = chunk / (BN / 8), rc = (chunk % (BN / 8)) * 8;
        load8<TB, false>(B, g.sbn, g.sbk, n0 + rc, k0 + kk, g.N, k_end, b_vec, rb[c]);
      }
    }
  };

  auto put = [&](LT *S, const float (&v)[8], int chunk, bool kc_layout, int rows_total) {
    if (kc_layout) {
      const int row = chunk / (BK / 8), kc = (chunk % (BK / 8)) * 8;
      LT *d = S + row * LD + kc;
      if (BF16) {
        uint4 q;
        q.x = bf16_rne(v[0]) | (bf16_rne(v[1]) << 16);
        q.y = bf16_rne(v[2]) | (bf16_rne(v[3]) << 16);
        q.z = bf16_rne(v[4]) | (bf16_rne(v[5]) << 16);
        q.w = bf16_rne(v[6]) | (bf16_rne(v[7]) << 16);
        *(uint4 *)d = q;
      } else {
        *(float2 *)d = make_float2(v[0], v[1]);
        *(float2 *)(d + 2) = make_float2(v[2], v[3]);
        *(float2 *)(d + 4) = make_float2(v[4], v[5]);
        *(float2 *)(d + 6) = make_float2(v[6], v[7]);
      }
    } else {
      const int kk = chunk / (rows_total / 8), rc = (chunk % (rows_total / 8)) * 8;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if (BF16) S[(rc + j) * LD + kk] = (LT)bf16_rne(v[j]);
        else S[(rc + j) * LD + kk] = (LT)v[j];
      }
    }
  };

  auto stash = [&](int buf) {
#pragma unroll
    for (int c = 0; c < CPT; ++c) {
      put(As2[buf], ra[c], tid + c * 256, A_KC, BM);
      put(Bs2[buf], rb[c], tid + c * 256, B_KC, BN);
    }
  };

  // Step s: the registers hold tile s + 1 (asked for a whole step ago); it goes into the stage that step s - 1
  // read - every wave is past that step's barrier -, tile s + 2 is asked for, and the MFMAs of step s run on the
  // other stage with those loads and LDS writes under them.  One barrier per step.
  const uint32_t n_steps = (k_end - k_begin + BK - 1) / BK;
  if (n_steps) {
    fetch(k_begin);
    stash(0);
    if (n_steps > 1) fetch(k_begin + BK);
  }
  __syncthreads();
  for (uint32_t s = 0; s < n_steps; ++s) {
    if (s + 1 < n_steps) {
      stash((s + 1) & 1);
      if (s + 2 < n_steps) fetch(k_begin + (s + 2) * BK);
    }
    const LT *As = As2[s & 1], *Bs = Bs2[s & 1];
    if (BF16) {
#pragma unroll
      for (int kk = 0; kk < BK; kk += 16) {
        bf16x8 af[2], bfr[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          af[i] = *(const bf16x8 *)(&As[(wm * 64 + i * 32 + (lane & 31)) * LD + kk + (lane >> 5) * 8]);
          bfr[i] = *(const bf16x8 *)(&Bs[(wn * 64 + i * 32 + (lane & 31)) * LD + kk + (lane >> 5) * 8]);
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
      }
    } else {
#pragma unroll
      for (int kk = 0; kk < BK; kk += 2) {
        float af[2], bfr[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          af[i] = (float)As[(wm * 64 + i * 32 + (lane & 31)) * LD + kk + (lane >> 5)];
          bfr[i] = (float)Bs[(wn * 64 + i * 32 + (lane & 31)) * LD + kk + (lane >> 5)];
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i], bfr[j], acc[i][j], 0, 0, 0);
      }
    }
    __syncthreads();  // stage (s + 1) & 1 is complete, and every wave is done reading stage s & 1
  }

  // 32x32 accumulator layout: element e of a lane sits at
  //   row = (e / 4) * 8 + (lane / 32) * 4 + e % 4,  col = lane % 32
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const uint32_t col = n0 + wn * 64 + j * 32 + (lane & 31);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const uint32_t row = m0 + wm * 64 + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
        if (row < g.M && col < g.N) C[(uint64_t)row * g.N + col] = acc[i][j][e];
      }
    }
}

// ---- small f32 products ----------------------------------------------------------------------------
// A product with a handful of 128 x 128 tiles (the 64 x 256 and 64 x 10 layers of a small MLP) leaves
// the kernel above with one or two workgroups walking K sixteen columns at a time, every step a full
// memory round trip.  Here a workgroup owns a 32 x 32 tile of C and its four wavefronts each take a
// quarter of K: every lane fetches its own MFMA operands straight from memory, 32 values of k per
// round trip and the next round trip already in flight, and the four partial tiles meet in LDS.
// Lane (r, h) = (lane % 32, lane / 32) supplies A[m0 + r][k] and B[k][n0 + r] for
// k = chunk * 32 + q * 8 + h * 4 + j; MFMA (q, j) pairs element j of both.
template <bool KC>
__device__ __forceinline__ float4 load4(const float *base, int64_t s_k, uint32_t k, uint32_t K, bool ok, int vec) {
  float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
  if (!ok) return v;
  if (KC && vec && k + 4 <= K) return *(const float4 *)(base + k);
  const float *p = base + (int64_t)k * s_k;
  if (k < K) v.x = p[0];
  if (k + 1 < K) v.y = p[s_k];
  if (k + 2 < K) v.z = p[2 * s_k];
  if (k + 3 < K) v.w = p[3 * s_k];
  return v;
}

template <bool A_KC, bool B_KC>
__global__ void __launch_bounds__(256) gemm_small_f32_kernel(GemmDesc g, int a_vec, int b_vec) {
  __shared__ float part[4][16 * 64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, h = lane >> 5;
  const uint32_t m0 = blockIdx.y * 32, n0 = blockIdx.x * 32;
  // split-K as in gemm_kernel: slice `split` of k goes to workspace[split], summed by a second pass
  const uint32_t batch = g.nb0 * g.nb1, split = blockIdx.z / batch, bz = blockIdx.z - split * batch;
  const uint32_t b0 = bz / g.nb1, b1 = bz - b0 * g.nb1;
  const float *A = (const float *)g.a + b0 * g.sa_b0 + b1 * g.sa_b1;
  const float *B = (const float *)g.b + b0 * g.sb_b0 + b1 * g.sb_b1;
  float *C = (g.splits > 1 ? g.workspace + (uint64_t)split * batch * g.M * g.N : g.c) + (uint64_t)bz * g.M * g.N;
  const uint32_t k_begin = g.splits > 1 ? min(g.K, split * g.k_per_split) : 0;  // a multiple of 32
  const uint32_t k_end = g.splits > 1 ? min(g.K, k_begin + g.k_per_split) : g.K;
  const uint32_t chunks = (k_end - k_begin + 31) / 32, per = (chunks + 3) / 4;
  const uint32_t c_begin = min(chunks, wave * per), c_end = min(chunks, c_begin + per);
  const bool row_ok = m0 + r < g.M, col_ok = n0 + r < g.N;
  const float *Ar = A + (int64_t)(m0 + r) * g.sam, *Bc = B + (int64_t)(n0 + r) * g.sbn;
  const int64_t sak = A_KC ? 1 : g.sak, sbk = B_KC ? 1 : g.sbk;
  f32x16 acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0.f;
  float4 ra[2][4], rb[2][4];
  auto fetch = [&](int buf, uint32_t c) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const uint32_t k = k_begin + c * 32 + q * 8 + h * 4;
      ra[buf][q] = load4<A_KC>(Ar, sak, k, k_end, row_ok, a_vec);
      rb[buf][q] = load4<B_KC>(Bc, sbk, k, k_end, col_ok, b_vec);
    }
  };
  auto multiply = [&](int buf) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ra[buf][q].x, rb[buf][q].x, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ra[buf][q].y, rb[buf][q].y, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ra[buf][q].z, rb[buf][q].z, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ra[buf][q].w, rb[buf][q].w, acc, 0, 0, 0);
    }
  };
  if (c_begin < c_end) fetch(0, c_begin);
  for (uint32_t c = c_begin; c < c_end; c += 2) {
    if (c + 1 < c_end) fetch(1, c + 1);
    multiply(0);
    if (c + 1 < c_end) {
      if (c + 2 < c_end) fetch(0, c + 2);
      multiply(1);
    }
  }
#pragma unroll
  for (int e = 0; e < 16; ++e) part[wave][e * 64 + lane] = acc[e];
  __syncthreads();
  // element e of lane l: row (e / 4) * 8 + (l / 32) * 4 + e % 4, column l % 32
  for (int i = tid; i < 1024; i += 256) {
    const int e = i >> 6, l = i & 63;
    const uint32_t row = m0 + (e >> 2) * 8 + (l >> 5) * 4 + (e & 3), col = n0 + (l & 31);
    if (row < g.M && col < g.N)
      C[(uint64_t)row * g.N + col] = (part[0][i] + part[1][i]) + (part[2][i] + part[3][i]);
  }
}

// few enough 32 x 32 tiles that the kernel above has the machine to itself
static bool gemm_small_ok(const LaunchCtx &lc, const GemmDesc &g) {
  if (g.bf16_math || g.a_stype != ST_F32 || g.b_stype != ST_F32 || g.M <= 8 || g.b_index || !g.K) return false;
  const uint64_t t32 = (uint64_t)((g.M + 31) / 32) * ((g.N + 31) / 32) * g.nb0 * g.nb1;
  return t32 <= 2 * (uint64_t)lc.n_cus;
}

// ---- bf16 x bf16 "NT" GEMM: the prefill fast path --------------------------------------------------
// A[M, K] and B[N, K] both bf16 with unit stride along k (activations are narrowed once by
// cast_bf16_kernel and the copy is shared by every GEMM that reads them; weights are stored
// bf16).  BM x BN tile per 256-thread workgroup, 2 x 2 waves, BK = 64.  LDS is double buffered:
// the global loads of step s+1 are issued before the MFMAs of step s and land in the other
// buffer after them, one barrier per step.  16-byte global loads, 16-byte LDS reads feeding
// v_mfma_f32_32x32x16_bf16 directly.
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(2))) float f32x2_t;

template <int BM_, int BN_, bool B_KC>
__global__ void __launch_bounds__(256) gemm_bf16_nt_kernel(GemmDesc g) {
  constexpr int BK = 64, LD = BK + 8;          // row pitch 144 bytes
  constexpr int WM = BM_ / 2, WN = BN_ / 2;    // wave tile
  constexpr int TM = WM / 32, TN = WN / 32;    // MFMA tiles per wave
  constexpr int ACH = BM_ * BK / 8 / 256, BCH = BN_ * BK / 8 / 256;  // 16-byte chunks per thread
  __shared__ __attribute__((aligned(16))) uint16_t As[2][BM_ * LD];
  __shared__ __attribute__((aligned(16))) uint16_t Bs[2][BN_ * LD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const uint32_t m0 = blockIdx.y * BM_, n0 = blockIdx.x * BN_;
  // blockIdx.z = split * batch + batch index; split s covers k in [s * k_per, (s + 1) * k_per)
  const uint32_t batch = g.nb0 * g.nb1;
  const uint32_t split = blockIdx.z / batch, bz = blockIdx.z - split * batch;
  const uint32_t b0 = bz / g.nb1, b1 = bz - b0 * g.nb1;
  const uint16_t *A = (const uint16_t *)g.a + b0 * g.sa_b0 + b1 * g.sa_b1;
  const uint16_t *B = (const uint16_t *)g.b + b0 * g.sb_b0 + b1 * g.sb_b1;
  float *C = (g.splits > 1 ? g.workspace + (uint64_t)split * batch * g.M * g.N : g.c) +
             (uint64_t)bz * g.M * g.N;
  const uint32_t k_begin = split * g.k_per_split;
  const uint32_t k_end = min(g.K, k_begin + g.k_per_split);

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  uint4 ra[ACH], rb[BCH];
  auto fetch = [&](uint32_t k0) {
#pragma unroll
    for (int c = 0; c < ACH; ++c) {
      const int chunk = tid + c * 256, row = chunk >> 3, kc = (chunk & 7) * 8;
      ra[c] = (m0 + row < g.M && k0 + kc < k_end)
                  ? *(const uint4 *)(A + (int64_t)(m0 + row) * g.sam + k0 + kc)
                  : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int c = 0; c < BCH; ++c) {
      const int chunk = tid + c * 256;
      if (B_KC) {
        const int row = chunk >> 3, kc = (chunk & 7) * 8;
        rb[c] = (n0 + row < g.N && k0 + kc < k_end)
                    ? *(const uint4 *)(B + (int64_t)(n0 + row) * g.sbn + k0 + kc)
                    : make_uint4(0, 0, 0, 0);
      } else {  // B[k, n] with unit stride along n: 8 columns of one k row
        const int kk = chunk / (BN_ / 8), nc = (chunk % (BN_ / 8)) * 8;
        rb[c] = (k0 + kk < k_end && n0 + nc < g.N)
                    ? *(const uint4 *)(B + (int64_t)(k0 + kk) * g.sbk + n0 + nc)
                    : make_uint4(0, 0, 0, 0);
      }
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int c = 0; c < ACH; ++c) {
      const int chunk = tid + c * 256, row = chunk >> 3, kc = (chunk & 7) * 8;
      *(uint4 *)(&As[buf][row * LD + kc]) = ra[c];
    }
#pragma unroll
    for (int c = 0; c < BCH; ++c) {
      const int chunk = tid + c * 256;
      if (B_KC) {
        const int row = chunk >> 3, kc = (chunk & 7) * 8;
        *(uint4 *)(&Bs[buf][row * LD + kc]) = rb[c];
      } else {  // transpose on the way into LDS
        const int kk = chunk / (BN_ / 8), nc = (chunk % (BN_ / 8)) * 8;
        const uint32_t w[4] = {rb[c].x, rb[c].y, rb[c].z, rb[c].w};
#pragma unroll
        for (int j = 0; j < 8; ++j)
          Bs[buf][(nc + j) * LD + kk] = (uint16_t)(w[j >> 1] >> ((j & 1) * 16));
      }
    }
  };

  const uint32_t n_steps = k_end > k_begin ? (k_end - k_begin + BK - 1) / BK : 0;
  if (n_steps) {
    fetch(k_begin);
    stash(0);
  }
  __syncthreads();
  for (uint32_t s = 0; s < n_steps; ++s) {
    const int buf = s & 1;
    if (s + 1 < n_steps) fetch(k_begin + (s + 1) * BK);
#pragma unroll
    for (int kk = 0; kk < BK; kk += 16) {
      bf16x8 af[TM], bfr[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        af[i] = *(const bf16x8 *)(&As[buf][(wm * WM + i * 32 + (lane & 31)) * LD + kk + (lane >> 5) * 8]);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        bfr[j] = *(const bf16x8 *)(&Bs[buf][(wn * WN + j * 32 + (lane & 31)) * LD + kk + (lane >> 5) * 8]);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
    }
    if (s + 1 < n_steps) stash(buf ^ 1);
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const uint32_t col = n0 + wn * WN + j * 32 + (lane & 31);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const uint32_t row = m0 + wm * WM + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
        if (row < g.M && col < g.N) C[(uint64_t)row * g.N + col] = acc[i][j][e];
      }
    }
}

// ---- bf16 NT GEMM with direct-to-LDS loads: the large-problem path --------------------------------
// Same operands as above with K a multiple of 64 (per split).  Tiles travel HBM/L2 -> LDS with
// global_load_lds_dwordx4 (16 bytes per lane, no VGPR staging, no ds_write): a wave's load lands
// as 1 KB contiguous in LDS, so a tile row is 128 bytes unpadded and bank conflicts are avoided
// by an XOR swizzle applied on the global side (the lane that fills physical 16-byte slot p of
// row r fetches logical chunk p ^ ((r >> 1) & 7), which spreads any 16 consecutive rows over
// all 64 banks).  Two stages: the loads of step s+1 are issued right after the barrier of step
// s and complete under its MFMAs; the compiler does not know the asm writes LDS, so the waits
// are explicit (s_waitcnt vmcnt + barrier before the stage is read).  Rows past M / N are
// clamped on the load side and masked at the store.  Fragment reads of k-slice ks+1 are issued
// among the MFMAs of slice ks, one read behind each of the first MFMAs (sched_group_barrier).
__device__ __forceinline__ void lds_dma16(const void *gptr, uint32_t lds_byte_off) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_byte_off), "v"(gptr)
               : "memory", "m0");
}
// the same for data read once (an expert's weight rows): streamed past the L2 lines worth keeping
__device__ __forceinline__ void lds_dma16_stream(const void *gptr, uint32_t lds_byte_off) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt" ::"s"(lds_byte_off), "v"(gptr)
               : "memory", "m0");
}
template <int N> __device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

// EPI: the MFMA operands change places, so that a lane holds four consecutive columns of a row of C: the optional
// gate (C = act(gate) * product) is read, and C and its bf16 copy are written, 16 / 8 bytes per lane along rows,
// straight from the accumulators.
// NS stages of operand tiles in LDS: two when several workgroups share a CU (large problems, bound by
// the L2 -> LDS rate), four when a CU holds one workgroup and every k-step would otherwise wait out a
// full trip to HBM (few tiles, cold weights: the prefill-sized products).
// DUAL (with EPI): the B tile stacks 128 rows of g.b (gate_proj) on 128 rows of g.dual_b (up_proj), a
// wavefront holds the same columns of both products, and the tile that leaves is act(gate) * up,
// 128 columns wide (BN_ = 256 counts the stacked rows): the gated MLP's two products and its
// activation in one pass over the activations, neither product ever stored.
// BKM: B is k-major - [K, N] with unit stride along n, rows g.sbk apart (the right operand of a product of two
// activations, ndarray.rs:549-615) - and is used where it lies: its tile travels as 64 k-rows of BN_ columns
// (16-byte pieces of a row swizzled by (k & 3) << 2, so that the four rows a fragment read touches fall on
// different banks), and the MFMA operand - eight consecutive k of one column per lane - comes out of LDS through
// the transposing read (ds_read_b64_tr_b16: the 16 lanes of a group hand in four rows of 16 columns, lane c
// receives column c of the four rows), two reads per fragment.
template <int BM_, int BN_, int WR, int WC, bool EPI, int NS, bool DUAL = false, bool BKM = false, bool ROPE = false>
__global__ void __launch_bounds__(WR *WC * 64) gemm_bf16_dma_kernel(GemmDesc g) {
  constexpr int NW = WR * WC, BK = 64;
  static_assert(!ROPE || (BN_ % 64 == 0 && !EPI && !DUAL && !BKM && (BM_ * BN_ / 4) % (WR * WC * 64) == 0),
                "rotated heads: whole heads of 64 columns per tile");
  static_assert(!BKM || (!EPI && !DUAL && (BM_ / 8) % ((BM_ + BN_) / 8 / (WR * WC)) == 0), "k-major B: the plain product");
  constexpr int WM = BM_ / WR, WN = BN_ / WC, TM = WM / 32, TN = WN / 32;
  constexpr int BNO = DUAL ? BN_ / 2 : BN_;    // output columns of a tile
  constexpr int OC = BNO / WC, TNH = OC / 32;  // DUAL: output columns per wave, fragments per product
  static_assert(!DUAL || (EPI && BN_ == 256 && TN == 2 * TNH), "stacked gate / up tile");
  constexpr int LPW = (BM_ + BN_) / 8 / NW;   // 1 KB loads per wave per stage
  constexpr int STAGE = (BM_ + BN_) * BK * 2;  // bytes
  extern __shared__ __attribute__((aligned(16))) uint16_t dma_smem[];
  warm_kernel_arguments<sizeof(GemmDesc)>();
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WC, wn = wave % WC;
  const uint32_t tiles_m = (g.M + BM_ - 1) / BM_, tiles_n = (g.N + BNO - 1) / BNO;
  const uint32_t per_batch = tiles_m * tiles_n, batch = g.nb0 * g.nb1;
  // Workgroups are dealt round-robin to the 8 XCDs (one L2 each): give every XCD a contiguous
  // range of logical tiles, and walk tiles in groups of 4 tile rows so that the ~32 tiles an
  // XCD works on at once share their A and B panels in that L2.
  uint32_t id = blockIdx.x;
  if (gridDim.x % 8 == 0) id = (id % 8) * (gridDim.x / 8) + id / 8;
  const uint32_t zz = id / per_batch;  // split * batch + batch index
  const uint32_t t = id - zz * per_batch;
  const uint32_t split = zz / batch, bz = zz - split * batch;
  const uint32_t b0 = bz / g.nb1, b1 = bz - b0 * g.nb1;
  constexpr uint32_t GM = 4;
  const uint32_t first_m = t / (GM * tiles_n) * GM, gsz = min(tiles_m - first_m, GM);
  const uint32_t tg = t % (GM * tiles_n);
  const uint32_t m0 = (first_m + tg % gsz) * BM_, n0_all = tg / gsz * BNO;
  const uint16_t *A = (const uint16_t *)g.a + b0 * g.sa_b0 + b1 * g.sa_b1;
  const uint16_t *B = (const uint16_t *)g.b + b0 * g.sb_b0 + b1 * g.sb_b1;
  const uint16_t *B2 = DUAL ? (const uint16_t *)g.dual_b + b0 * g.sb_b0 + b1 * g.sb_b1 : nullptr;
  float *C = (g.splits > 1 ? g.workspace + (uint64_t)split * batch * g.M * g.N : g.c) +
             (uint64_t)bz * g.M * g.N;
  // grouped products: this tile's columns belong to one of them (tiles never straddle two)
  uint32_t n0 = n0_all, Nl = g.N, grp = 0;
  if (g.n_group) {
    uint32_t p = 0;
    while (p + 1 < g.n_group && n0 >= g.grp_n[p]) {
      n0 -= g.grp_n[p];
      ++p;
    }
    B = (const uint16_t *)g.grp_b[p];
    C = g.grp_c[p];
    Nl = g.grp_n[p];
    grp = p;
  }
  const float *Bias = g.n_group ? g.grp_bias[grp] : nullptr;
  const float *Gate = g.glu_gate ? g.glu_gate + (uint64_t)bz * g.M * g.N : nullptr;  // only without split-K
  uint16_t *C16 = g.c16 ? g.c16 + (uint64_t)bz * g.M * g.N : nullptr;
  const uint32_t k_begin = split * g.k_per_split;
  const uint32_t k_end = min(g.K, k_begin + g.k_per_split);

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint16_t *)dma_smem;
  const uint16_t *gp[LPW];  // per-lane source of each of this wave's loads; advances by BK per stage
#pragma unroll
  for (int i = 0; i < LPW; ++i) {
    const int q = wave * LPW + i;  // 8-row block of the stacked [A; B] tile
    const int R = q * 8 + (lane >> 3);
    const int c = (lane & 7) ^ ((R >> 1) & 7);
    if (q * 8 < BM_) {
      gp[i] = A + (int64_t)min(m0 + R, g.M - 1) * g.sam + k_begin + c * 8;
    } else if (BKM) {
      // 1 KB of the B tile = 1024 / (2 BN_) k-rows; this lane's 16 bytes: row kr, physical piece pc
      const int qb = q - BM_ / 8, kr = qb * (512 / BN_) + lane / (BN_ / 8), pc = lane % (BN_ / 8);
      const uint32_t n = n0 + (uint32_t)((pc ^ ((kr & 3) << 2)) * 8);
      gp[i] = B + (int64_t)(k_begin + kr) * g.sbk + min(n, Nl - 8);
    } else if (DUAL) gp[i] = (R - BM_ < BNO ? B : B2) + (int64_t)min(n0 + (uint32_t)((R - BM_) % BNO), Nl - 1) * g.sbn + k_begin + c * 8;
    else gp[i] = B + (int64_t)min(n0 + (R - BM_), Nl - 1) * g.sbn + k_begin + c * 8;
  }
  // (k-major B: a wave's loads are all A's or all B's, and B's step down 64 rows per stage)
  const int64_t gp_step = BKM && wave * LPW * 8 >= BM_ ? (int64_t)BK * g.sbk : (int64_t)BK;
  auto issue = [&](int buf) {
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
      lds_dma16(gp[i], lds0 + buf * STAGE + (wave * LPW + i) * 1024);
      gp[i] += gp_step;
    }
  };
  const int sw = (lane >> 1) & 7, half = lane >> 5;
  auto compute = [&](int buf) {
    const uint16_t *As = dma_smem + buf * (STAGE / 2), *Bs = As + BM_ * BK;
    bf16x8 af[2][TM], bfr[2][TN];
    auto frags = [&](int ks, int set) {
      const int p = ((ks * 2 + half) ^ sw) * 8;
#pragma unroll
      for (int i = 0; i < TM; ++i)
        af[set][i] = *(const bf16x8 *)(&As[(wm * WM + i * 32 + (lane & 31)) * BK + p]);
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        if constexpr (BKM) {
          typedef short v4s __attribute__((ext_vector_type(4)));
          const int r = (lane & 15) >> 2, col = wn * WN + j * 32 + ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
          const int at = (ks * 16 + half * 8 + r) * BN_ + (((col >> 3) ^ (r << 2)) << 3) + (col & 7);
          union {
            v4s q[2];
            bf16x8 f;
          } u;
          u.q[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s *)(Bs + at));
          u.q[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s *)(Bs + at + 4 * BN_));
          bfr[set][j] = u.f;
        } else {
          // DUAL: fragments [0, TNH) are this wave's gate columns, [TNH, TN) the same columns of up
          const int brow = DUAL ? (j / TNH) * BNO + wn * OC + (j % TNH) * 32 : wn * WN + j * 32;
          bfr[set][j] = *(const bf16x8 *)(&Bs[(brow + (lane & 31)) * BK + p]);
        }
      }
    };
    frags(0, 0);
    // the wave that is in its MFMA phase goes first when both waves of a SIMD have something to issue
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      if (ks + 1 < BK / 16) frags(ks + 1, (ks + 1) & 1);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          // (EPI: the product transposed - a lane then holds four consecutive columns of one row of C, which
          // is what the epilogue stores, 16 bytes at a time, without a trip through LDS)
          acc[i][j] = EPI ? __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[ks & 1][j], af[ks & 1][i], acc[i][j], 0, 0, 0)
                          : __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[ks & 1][i], bfr[ks & 1][j], acc[i][j], 0, 0, 0);
      // Issue order within the slice: one LDS read behind each of the first MFMAs, so that the reads of
      // the next slice go out while the matrix pipe is busy instead of in a block during which it drains
      // (measured on 4096^3: 0.93 -> 1.06 PFLOP/s).
      if (ks + 1 < BK / 16) {
        constexpr int READS = TM + TN < TM * TN ? TM + TN : TM * TN;
#pragma unroll
        for (int q = 0; q < READS; ++q) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
        }
        if (TM * TN > READS) __builtin_amdgcn_sched_group_barrier(0x008, TM * TN - READS, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    __builtin_amdgcn_s_setprio(0);
  };
  const int n_steps = k_end > k_begin ? (int)((k_end - k_begin) / BK) : 0;
  // (clock probe only) s_memtime ticks with the shader clock, s_memrealtime with a constant 100 MHz: their ratio
  // over the main loop is the clock this kernel really ran at
  unsigned long long tick0 = 0, real0 = 0;
  if (g.clock_ticks) {
    tick0 = __builtin_amdgcn_s_memtime();
    real0 = __builtin_amdgcn_s_memrealtime();
  }
#pragma unroll
  for (int s0 = 0; s0 < NS - 1; ++s0)
    if (s0 < n_steps) issue(s0);
  for (int step = 0; step < n_steps; ++step) {
    // stage `step` has landed (this wave's part): at most the NS - 2 younger stages are still in
    // flight; in the tail, where fewer were issued, wait for everything
    if (step + NS - 1 <= n_steps) wait_vmcnt<(NS - 2) * LPW>();
    else wait_vmcnt<0>();
    __syncthreads();   // ... and everyone's; all waves are done reading the buffer refilled next
    if (step + NS - 1 < n_steps) issue((step + NS - 1) % NS);
    compute(step % NS);
  }
  if (g.clock_ticks && tid == 0) {
    atomicAdd(g.clock_ticks, __builtin_amdgcn_s_memtime() - tick0);
    atomicAdd(g.clock_ticks + 1, __builtin_amdgcn_s_memrealtime() - real0);
  }
  if constexpr (EPI) {
    // acc[i][j][e] = C[m0 + wm * WM + i * 32 + (lane & 31)][n0 + (this fragment's columns) + (e >> 2) * 8 + half * 4 + (e & 3)]:
    // pieces of four columns (N % 4 == 0: a piece is inside or outside), the optional gate read the same way
    constexpr int TJ = DUAL ? TNH : TN;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const uint32_t row = m0 + wm * WM + i * 32 + (lane & 31);
#pragma unroll
      for (int j = 0; j < TJ; ++j) {
        float4 gt[4];
        uint64_t at[4];
        bool live[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const uint32_t col = n0 + (DUAL ? wn * OC : wn * WN) + j * 32 + q * 8 + half * 4;
          live[q] = row < g.M && col < Nl;
          at[q] = (uint64_t)row * Nl + col;
          if (!DUAL && Gate && live[q]) gt[q] = *(const float4 *)(Gate + at[q]);
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          if (!live[q]) continue;
          float4 v = make_float4(acc[i][j][q * 4], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]);
          if constexpr (DUAL) {
            const float u0 = acc[i][TNH + j][q * 4], u1 = acc[i][TNH + j][q * 4 + 1], u2 = acc[i][TNH + j][q * 4 + 2],
                        u3 = acc[i][TNH + j][q * 4 + 3];
            if (g.c) {  // (the activation as the stdlib defines it when the f32 tile is stored too)
              if (g.glu_kind) v = make_float4(gelu_ref(v.x) * u0, gelu_ref(v.y) * u1, gelu_ref(v.z) * u2, gelu_ref(v.w) * u3);
              else v = make_float4(v.x * sigmoid_ref(v.x) * u0, v.y * sigmoid_ref(v.y) * u1, v.z * sigmoid_ref(v.z) * u2, v.w * sigmoid_ref(v.w) * u3);
            } else {
              if (g.glu_kind) v = make_float4(gelu_fast(v.x) * u0, gelu_fast(v.y) * u1, gelu_fast(v.z) * u2, gelu_fast(v.w) * u3);
              else v = make_float4(silu_fast(v.x) * u0, silu_fast(v.y) * u1, silu_fast(v.z) * u2, silu_fast(v.w) * u3);
            }
          } else if (Gate) {
            if (g.glu_kind) {
              v.x *= gelu_ref(gt[q].x); v.y *= gelu_ref(gt[q].y); v.z *= gelu_ref(gt[q].z); v.w *= gelu_ref(gt[q].w);
            } else {
              v.x *= gt[q].x * sigmoid_ref(gt[q].x); v.y *= gt[q].y * sigmoid_ref(gt[q].y);
              v.z *= gt[q].z * sigmoid_ref(gt[q].z); v.w *= gt[q].w * sigmoid_ref(gt[q].w);
            }
          }
          if (!DUAL || g.c) *(float4 *)(C + at[q]) = v;
          if (C16) *(uint2 *)(C16 + at[q]) = bf16_pack4(v);
        }
      }
    }
    return;
  }
  if constexpr (ROPE) {
    // The tile holds whole heads of hd = 64 or 128 columns (BN_ is a multiple of hd).
    const uint32_t role = g.rope_s ? g.rope_role[grp] : 0;
    const uint32_t hd = g.rope_hd, S = g.rope_s, heads = Nl / hd;
    if (role == 1) {
      // apply_rope_embedding (catgrad-llm/src/helpers.rs:195-221) on the tile while it is still on the chip, the
      // arithmetic of rope_kernel: out = cos * x + sin * rot, rot = -x[j + hd / 2] in the lower half of a head,
      // x[j - hd / 2] in the upper.  The tile goes through LDS once, so that a thread holds four consecutive
      // columns of a row and their partners, the tables come in 16 bytes at a time, and the rows of a head
      // (contiguous in the result) leave as whole lines.
      constexpr int P = BN_ + 8;  // floats per tile row: rows four apart, which a wave writes together, fall on different banks
      constexpr int F4 = BN_ / 4, ITERS = BM_ * F4 / (NW * 64), CH = ITERS < 4 ? ITERS : 4;
      static_assert(ITERS % CH == 0, "table rows are requested a chunk of iterations ahead");
      const float *cs = g.rope_cos[grp], *sn = g.rope_sin[grp];
      const int64_t ss = g.rope_cs_ss[grp];
      auto table = [&](const float *tb, int it) {
        const int idx = it * NW * 64 + tid, r = idx / F4, c4 = (idx % F4) * 4;
        return *(const float4 *)(tb + (int64_t)(min(m0 + r, g.M - 1) % S) * ss + (c4 & (hd - 1)));
      };
      // Table rows are requested a chunk of iterations ahead of their use (the first chunk before the tile is
      // exchanged): behind the stores of the iteration before, each would cost a trip to L2 of its own.
      float4 cv[2][CH], sv[2][CH];
#pragma unroll
      for (int u = 0; u < CH; ++u) {
        cv[0][u] = table(cs, u);
        sv[0][u] = table(sn, u);
      }
      float *tile = (float *)dma_smem;
      __syncthreads();  // every wave is done with the last stage
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const int cl = wn * WN + j * 32 + (lane & 31);
          const float bv = Bias ? Bias[min(n0 + cl, Nl - 1)] : 0.f;
#pragma unroll
          for (int e = 0; e < 16; ++e)
            tile[(wm * WM + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3)) * P + cl] = acc[i][j][e] + bv;
        }
      __syncthreads();
      const int half = (int)hd / 2;
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        if (it % CH == 0 && it + CH < ITERS) {
#pragma unroll
          for (int u = 0; u < CH; ++u) {
            cv[(it / CH + 1) & 1][u] = table(cs, it + CH + u);
            sv[(it / CH + 1) & 1][u] = table(sn, it + CH + u);
          }
        }
        const int idx = it * NW * 64 + tid, r = idx / F4, c4 = (idx % F4) * 4;
        const uint32_t row = m0 + r;
        const float4 c = cv[(it / CH) & 1][it % CH], sn4 = sv[(it / CH) & 1][it % CH];
        const float4 xv = *(const float4 *)(tile + r * P + c4);
        float4 pv = *(const float4 *)(tile + r * P + (c4 ^ half));
        if (!(c4 & half)) { pv.x = -pv.x; pv.y = -pv.y; pv.z = -pv.z; pv.w = -pv.w; }
        float4 o;
        o.x = c.x * xv.x + sn4.x * pv.x; o.y = c.y * xv.y + sn4.y * pv.y;
        o.z = c.z * xv.z + sn4.z * pv.z; o.w = c.w * xv.w + sn4.w * pv.w;
        if (row < g.M) {
          const uint32_t sq = row / S, pos = row - sq * S, head = (n0 + c4) / hd;
          const uint64_t at = (((uint64_t)sq * heads + head) * S + pos) * hd + (c4 & (hd - 1));
          *(float4 *)(g.rope_out[grp] + at) = o;
          if (g.rope_out16[grp]) *(uint2 *)(g.rope_out16[grp] + at) = bf16_pack4(o);
        }
      }
      return;
    }
    if (role == 2) {  // the values: also as bf16 [sequence][head][hd][position], four consecutive positions per store
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const uint32_t col = n0 + wn * WN + j * 32 + (lane & 31);  // = head * hd + column of the head
          const float bv = Bias ? Bias[min(col, Nl - 1)] : 0.f;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const uint32_t r0 = m0 + wm * WM + i * 32 + q * 8 + (lane >> 5) * 4;  // S % 4 == 0: the four share a sequence
            if (r0 < g.M && col < Nl) {
              const uint32_t sq = r0 / S, pos = r0 - sq * S;
              *(uint2 *)(g.rope_out16[grp] + ((uint64_t)sq * Nl + col) * S + pos) =
                  bf16_pack4(make_float4(acc[i][j][q * 4] + bv, acc[i][j][q * 4 + 1] + bv, acc[i][j][q * 4 + 2] + bv, acc[i][j][q * 4 + 3] + bv));
            }
          }
        }
    }
  }
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const uint32_t col = n0 + wn * WN + j * 32 + (lane & 31);
      if (Bias) {
        const float bv = Bias[min(col, Nl - 1)];
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const uint32_t row = m0 + wm * WM + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
          if (row < g.M && col < Nl) C[(uint64_t)row * Nl + col] = acc[i][j][e] + bv;
        }
        continue;
      }
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const uint32_t row = m0 + wm * WM + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
        if (row < g.M && col < Nl) C[(uint64_t)row * Nl + col] = acc[i][j][e];
      }
    }
}

template <int BM_, int BN_, int WR, int WC, bool EPI = false, int NS = 2, bool DUAL = false, bool BKM = false, bool ROPE = false>
static hipError_t launch_gemm_dma(const LaunchCtx &lc, const GemmDesc &g, uint32_t grid) {
  // (ROPE: the f32 tile is exchanged through LDS at the end, BN_ + 8 floats per row)
  constexpr int stages = NS * (BM_ + BN_) * 64 * 2, smem = ROPE && BM_ * (BN_ + 8) * 4 > stages ? BM_ * (BN_ + 8) * 4 : stages;
  static bool configured = false;  // one attribute call per kernel and process
  if (!configured) {
    hipError_t e = hipFuncSetAttribute((const void *)gemm_bf16_dma_kernel<BM_, BN_, WR, WC, EPI, NS, DUAL, BKM, ROPE>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return e;
    configured = true;
  }
  cg_launch(lc, gemm_bf16_dma_kernel<BM_, BN_, WR, WC, EPI, NS, DUAL, BKM, ROPE>, dim3(grid), dim3(WR * WC * 64), smem, g);
  return hipGetLastError();
}

// C = sum over splits of workspace[split] (float4 per thread; sizes are multiples of 4 or the
// tail is handled scalar)
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const float *ws, float *c, uint64_t n,
                                                            uint32_t splits, const float *cadd) {
  const uint64_t n4 = n / 4;
  for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n4;
       i += (uint64_t)gridDim.x * 256) {
    float4 s = ((const float4 *)ws)[i];
    for (uint32_t k = 1; k < splits; ++k) {
      const float4 v = ((const float4 *)(ws + (uint64_t)k * n))[i];
      s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    if (cadd) {
      const float4 v = ((const float4 *)cadd)[i];
      s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    ((float4 *)c)[i] = s;
  }
  if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
    const uint64_t i = n4 * 4 + threadIdx.x;
    float s = ws[i];
    for (uint32_t k = 1; k < splits; ++k) s += ws[(uint64_t)k * n + i];
    c[i] = s + (cadd ? cadd[i] : 0.f);
  }
}

// f32 -> bf16 (round to nearest even, v_cvt_pk_bf16_f32), contiguous, 8 elements per thread
__global__ void __launch_bounds__(256) cast_bf16_kernel(const float *in, uint16_t *out, uint64_t n8) {
  for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n8;
       i += (uint64_t)gridDim.x * 256) {
    const float4 a = ((const float4 *)in)[2 * i], b = ((const float4 *)in)[2 * i + 1];
    bf16x2_t h0 = __builtin_convertvector((f32x2_t){a.x, a.y}, bf16x2_t);
    bf16x2_t h1 = __builtin_convertvector((f32x2_t){a.z, a.w}, bf16x2_t);
    bf16x2_t h2 = __builtin_convertvector((f32x2_t){b.x, b.y}, bf16x2_t);
    bf16x2_t h3 = __builtin_convertvector((f32x2_t){b.z, b.w}, bf16x2_t);
    uint4 q;
    q.x = *(uint32_t *)&h0; q.y = *(uint32_t *)&h1; q.z = *(uint32_t *)&h2; q.w = *(uint32_t *)&h3;
    ((uint4 *)out)[i] = q;
  }
}

// B[k, n] with unit stride along n (f32 or bf16)  ->  bf16 [batch][n][k], k-contiguous: the layout
// the direct-to-LDS GEMM wants.  64 x 64 tiles through LDS: reads run along n, writes along k.
template <typename TB, bool VEC>
__global__ void __launch_bounds__(256) transpose_cast_bf16_kernel(const TB *b, uint16_t *out, uint32_t K,
                                                                  uint32_t N, int64_t sbk, uint32_t nb1,
                                                                  int64_t sb_b0, int64_t sb_b1) {
  __shared__ __attribute__((aligned(8))) uint16_t tile[64][68];  // pitch 136 bytes keeps 8-byte alignment
  const uint32_t bz = blockIdx.z, b0 = bz / nb1, b1 = bz - b0 * nb1;
  const TB *src = b + b0 * sb_b0 + b1 * sb_b1;
  uint16_t *dst = out + (uint64_t)bz * N * K;
  const uint32_t n0 = blockIdx.x * 64, k0 = blockIdx.y * 64;
  const int r = threadIdx.x >> 4, c4 = (threadIdx.x & 15) * 4;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t k = k0 + r + i * 16, n = n0 + c4;
    uint16_t v[4] = {0, 0, 0, 0};
    if (VEC) {  // N % 4 == 0, 4-element groups aligned: all four in range or none
      if (k < K && n < N) {
        if (sizeof(TB) == 4) {
          const float4 q = *(const float4 *)((const float *)src + (int64_t)k * sbk + n);
          v[0] = (uint16_t)bf16_rne(q.x); v[1] = (uint16_t)bf16_rne(q.y);
          v[2] = (uint16_t)bf16_rne(q.z); v[3] = (uint16_t)bf16_rne(q.w);
        } else {
          const uint2 q = *(const uint2 *)((const uint16_t *)src + (int64_t)k * sbk + n);
          v[0] = (uint16_t)q.x; v[1] = (uint16_t)(q.x >> 16); v[2] = (uint16_t)q.y; v[3] = (uint16_t)(q.y >> 16);
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (k < K && n + j < N) {
          if (sizeof(TB) == 4) v[j] = (uint16_t)bf16_rne(widen(src[(int64_t)k * sbk + n + j]));
          else v[j] = (uint16_t)src[(int64_t)k * sbk + n + j];
        }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) tile[c4 + j][r + i * 16] = v[j];  // stored transposed: tile[n][k]
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t n = n0 + r + i * 16, k = k0 + c4;
    const uint16_t *t = &tile[r + i * 16][c4];
    if (VEC) {
      if (n < N && k < K) *(uint2 *)(dst + (uint64_t)n * K + k) = *(const uint2 *)t;
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (n < N && k + j < K) dst[(uint64_t)n * K + k + j] = t[j];
    }
  }
}

hipError_t launch_transpose_cast_bf16(const LaunchCtx &lc, const void *b, int b_stype, void *out, uint32_t K,
                                      uint32_t N, int64_t sbk, uint32_t nb0, uint32_t nb1, int64_t sb_b0,
                                      int64_t sb_b1) {
  if (!K || !N || !nb0 || !nb1) return hipSuccess;
  dim3 grid((N + 63) / 64, (K + 63) / 64, nb0 * nb1);
  const int es = b_stype == ST_BF16 ? 2 : 4;
  const bool vec = N % 4 == 0 && K % 4 == 0 && sbk % 4 == 0 && sb_b0 % 4 == 0 && sb_b1 % 4 == 0 &&
                   ((uintptr_t)b % (4 * es)) == 0 && ((uintptr_t)out % 8) == 0;
  if (b_stype == ST_BF16) {
    if (vec) CG_LAUNCH(lc, (transpose_cast_bf16_kernel<uint16_t, true>), grid, 256, (const uint16_t *)b, (uint16_t *)out, K, N, sbk, nb1, sb_b0, sb_b1);
    else CG_LAUNCH(lc, (transpose_cast_bf16_kernel<uint16_t, false>), grid, 256, (const uint16_t *)b, (uint16_t *)out, K, N, sbk, nb1, sb_b0, sb_b1);
  } else {
    if (vec) CG_LAUNCH(lc, (transpose_cast_bf16_kernel<float, true>), grid, 256, (const float *)b, (uint16_t *)out, K, N, sbk, nb1, sb_b0, sb_b1);
    else CG_LAUNCH(lc, (transpose_cast_bf16_kernel<float, false>), grid, 256, (const float *)b, (uint16_t *)out, K, N, sbk, nb1, sb_b0, sb_b1);
  }
  return hipGetLastError();
}

hipError_t launch_cast_bf16(const LaunchCtx &lc, const float *in, void *out, uint64_t n) {
  if (!n) return hipSuccess;
  const uint64_t n8 = n / 8;
  uint64_t blocks = (n8 + 255) / 256, cap = (uint64_t)lc.n_cus * 16;
  CG_LAUNCH(lc, (cast_bf16_kernel), (unsigned)(blocks < cap ? blocks : cap), 256, in, (uint16_t *)out, n8);
  return hipGetLastError();
}

// ---- GEMV, B k-contiguous (weights, K^T): y[m, n] = sum_k x[m, k] * B[n, k] ------------------------
// LPR lanes share one output column; each lane moves 16 bytes of B per load and keeps UNROLL
// loads in flight (HBM latency x bandwidth needs tens of KB outstanding per CU); B is streamed
// with non-temporal loads, x comes back from L1/L2.
typedef float f32x4n __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4n __attribute__((ext_vector_type(4)));
template <typename TB> struct WVec;
template <> struct WVec<float> {
  typedef f32x4n type;
  enum { EPL = 4 };
  static __device__ __forceinline__ void widen(const f32x4n &q, float (&w)[4]) {
    w[0] = q.x; w[1] = q.y; w[2] = q.z; w[3] = q.w;
  }
};
template <> struct WVec<uint16_t> {
  typedef u32x4n type;
  enum { EPL = 8 };
  static __device__ __forceinline__ void widen(const u32x4n &q, float (&w)[8]) {
    w[0] = __uint_as_float(q.x << 16); w[1] = __uint_as_float(q.x & 0xFFFF0000u);
    w[2] = __uint_as_float(q.y << 16); w[3] = __uint_as_float(q.y & 0xFFFF0000u);
    w[4] = __uint_as_float(q.z << 16); w[5] = __uint_as_float(q.z & 0xFFFF0000u);
    w[6] = __uint_as_float(q.w << 16); w[7] = __uint_as_float(q.w & 0xFFFF0000u);
  }
};

// R: column groups a wave keeps in flight at once; KSPLIT: waves of a workgroup that share one
// column group, each taking a contiguous 1/KSPLIT of k (for deep, narrow matrices).
template <typename TB, int LPR, int MROWS, int R, int KSPLIT>
__global__ void __launch_bounds__(256) gemv_rowdot_kernel(GemmDesc g, int b_vec, int a_vec) {
  warm_kernel_arguments<sizeof(GemmDesc)>();
  typedef typename WVec<TB>::type VT;
  constexpr int EPL = WVec<TB>::EPL;  // elements per 16-byte load
  constexpr int UNROLL = 4;
  constexpr int CPW = 64 / LPR;       // columns per wave per group
  __shared__ float red[KSPLIT > 1 ? 4 : 1][R][MROWS][CPW];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = lane % LPR, col_in_wave = lane / LPR;
  const uint32_t bz = blockIdx.y, b0 = bz / g.nb1, b1 = bz - b0 * g.nb1;
  const float *A = (const float *)g.a + b0 * g.sa_b0 + b1 * g.sa_b1;
  const TB *B = (const TB *)g.b + b_batch_offset(g, bz, b0, b1);
  float *C = g.c + (uint64_t)bz * g.M * g.N;
  const float *Cadd = g.c_add ? g.c_add + (uint64_t)bz * g.M * g.N : nullptr;
  // a "slot" is one wave (KSPLIT == 1) or one workgroup (KSPLIT == 4)
  const uint32_t slot = KSPLIT == 1 ? blockIdx.x * 4 + wave : blockIdx.x;
  const uint32_t n_slots = KSPLIT == 1 ? gridDim.x * 4 : gridDim.x;
  // this wave's share of k (multiples of the load width)
  uint32_t k_begin = 0, k_end = g.K;
  if (KSPLIT > 1) {
    const uint32_t per = ((g.K + KSPLIT - 1) / KSPLIT + EPL - 1) / EPL * EPL;
    k_begin = min(g.K, wave * per);
    k_end = min(g.K, k_begin + per);
  }
  const bool fast = b_vec && a_vec && (g.K % EPL == 0);
  for (uint32_t nb = slot * CPW * R; nb < g.N; nb += n_slots * CPW * R) {
    float acc[R][MROWS];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < MROWS; ++m) acc[r][m] = 0.f;
    // What is added at the end (a residual) is requested now, by every lane with its position clamped, so that
    // it is there when the sums are: loaded where it is used it costs the launch one more trip to memory.
    float cpre[R][MROWS];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < MROWS; ++m) cpre[r][m] = 0.f;
    if (Cadd) {
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < MROWS; ++m)
          cpre[r][m] = Cadd[(uint64_t)min((uint32_t)m, g.M - 1) * g.N + min(nb + r * CPW + col_in_wave, g.N - 1)];
    }
    if (fast) {
      for (uint32_t k0 = k_begin + sub * EPL; k0 < k_end; k0 += LPR * EPL * UNROLL) {
        VT q[R][UNROLL];
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const uint32_t n = nb + r * CPW + col_in_wave;
#pragma unroll
          for (int u = 0; u < UNROLL; ++u) {
            const uint32_t k = k0 + u * LPR * EPL;
            if (k < k_end && n < g.N)
              q[r][u] = __builtin_nontemporal_load((const VT *)(B + (int64_t)n * g.sbn + k));
          }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
          const uint32_t k = k0 + u * LPR * EPL;
          if (k < k_end) {
#pragma unroll
            for (int m = 0; m < MROWS; ++m) {
              if ((uint32_t)m < g.M) {
                const float *xr = A + (int64_t)m * g.sam + k;
                float xs[EPL];
#pragma unroll
                for (int j4 = 0; j4 < EPL; j4 += 4) {
                  const float4 xv = *(const float4 *)(xr + j4);
                  xs[j4] = xv.x; xs[j4 + 1] = xv.y; xs[j4 + 2] = xv.z; xs[j4 + 3] = xv.w;
                }
#pragma unroll
                for (int r = 0; r < R; ++r) {
                  if (nb + r * CPW + col_in_wave < g.N) {
                    float w[EPL];
                    WVec<TB>::widen(q[r][u], w);
#pragma unroll
                    for (int j = 0; j < EPL; ++j) acc[r][m] += w[j] * xs[j];
                  }
                }
              }
            }
          }
        }
      }
    } else {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const uint32_t n = nb + r * CPW + col_in_wave;
        if (n < g.N) {
          const TB *brow = B + (int64_t)n * g.sbn;
          for (uint32_t k = k_begin + sub; k < k_end; k += LPR) {
            const float w = widen(brow[(int64_t)k * g.sbk]);
#pragma unroll
            for (int m = 0; m < MROWS; ++m)
              if ((uint32_t)m < g.M) acc[r][m] += w * A[(int64_t)m * g.sam + (int64_t)k * g.sak];
          }
        }
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < MROWS; ++m)
        acc[r][m] = group_sum<LPR>(acc[r][m]);
    if (KSPLIT > 1) {
      __syncthreads();
      if (sub == 0)
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
          for (int m = 0; m < MROWS; ++m) red[wave][r][m][col_in_wave] = acc[r][m];
      __syncthreads();
      if (wave == 0 && sub == 0) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const uint32_t n = nb + r * CPW + col_in_wave;
#pragma unroll
          for (int m = 0; m < MROWS; ++m)
            if (n < g.N && (uint32_t)m < g.M)
              C[(uint64_t)m * g.N + n] = ((red[0][r][m][col_in_wave] + red[1][r][m][col_in_wave]) +
                                          (red[2][r][m][col_in_wave] + red[3][r][m][col_in_wave])) +
                                         cpre[r][m];
        }
      }
    } else if (sub == 0) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const uint32_t n = nb + r * CPW + col_in_wave;
#pragma unroll
        for (int m = 0; m < MROWS; ++m)
          if (n < g.N && (uint32_t)m < g.M)
            C[(uint64_t)m * g.N + n] = acc[r][m] + cpre[r][m];
      }
    }
  }
}

// ---- several GEMVs sharing x in one launch (q/k/v and gate/up of a decode step) -------------------
// Same streaming scheme as gemv_rowdot_kernel<.., 64, 1, 2, 1>; blockIdx.y selects the problem.
template <typename TB>
__global__ void __launch_bounds__(256) gemv_multi_kernel(GemvMultiDesc g) {
  warm_kernel_arguments<sizeof(GemvMultiDesc)>();
  typedef typename WVec<TB>::type VT;
  constexpr int EPL = WVec<TB>::EPL, UNROLL = 4, R = 2;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t N = g.p[blockIdx.y].N;
  const TB *B = (const TB *)g.p[blockIdx.y].b;
  const int64_t sbn = g.p[blockIdx.y].sbn;
  float *C = g.p[blockIdx.y].c;
  const float *Cadd = g.p[blockIdx.y].c_add;
  const uint32_t n_waves = gridDim.x * 4;
  for (uint32_t nb = (blockIdx.x * 4 + wave) * R; nb < N; nb += n_waves * R) {
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.f;
    for (uint32_t k0 = lane * EPL; k0 < g.K; k0 += 64 * EPL * UNROLL) {
      VT q[R][UNROLL];
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
          const uint32_t k = k0 + u * 64 * EPL;
          if (k < g.K && nb + r < N)
            q[r][u] = __builtin_nontemporal_load((const VT *)(B + (int64_t)(nb + r) * sbn + k));
        }
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const uint32_t k = k0 + u * 64 * EPL;
        if (k < g.K) {
          float xs[EPL];
#pragma unroll
          for (int j4 = 0; j4 < EPL; j4 += 4) {
            const float4 xv = *(const float4 *)(g.x + k + j4);
            xs[j4] = xv.x; xs[j4 + 1] = xv.y; xs[j4 + 2] = xv.z; xs[j4 + 3] = xv.w;
          }
#pragma unroll
          for (int r = 0; r < R; ++r) {
            if (nb + r < N) {
              float w[EPL];
              WVec<TB>::widen(q[r][u], w);
#pragma unroll
              for (int j = 0; j < EPL; ++j) acc[r] += w[j] * xs[j];
            }
          }
        }
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      acc[r] = wave_sum(acc[r]);
      if (lane == 0 && nb + r < N) C[nb + r] = acc[r] + (Cadd ? Cadd[nb + r] : 0.f);
    }
  }
}

hipError_t launch_gemv_multi(const LaunchCtx &lc, const GemvMultiDesc &g) {
  uint32_t max_n = 0;
  for (int i = 0; i < g.n_prob; ++i) max_n = g.p[i].N > max_n ? g.p[i].N : max_n;
  if (!max_n || !g.n_prob) return hipSuccess;
  uint32_t blocks = (max_n + 7) / 8;  // 4 waves x 2 columns per workgroup pass
  const uint32_t cap = (uint32_t)lc.n_cus * 16 / g.n_prob;
  if (blocks > cap) blocks = cap;
  dim3 grid(blocks, g.n_prob);
  if (g.b_stype == ST_BF16) CG_LAUNCH(lc, (gemv_multi_kernel<uint16_t>), grid, 256, g);
  else CG_LAUNCH(lc, (gemv_multi_kernel<float>), grid, 256, g);
  return hipGetLastError();
}

// ---- GEMVs whose input row is computed in the kernel --------------------------------------------------
// A decode step spends as much time launching its small kernels as running them.  The RMSNorm in
// front of q/k/v and gate/up, and the SwiGLU in front of down_proj, produce a single row of K
// floats: every workgroup recomputes that row into LDS (a few KB from L2, microseconds of ALU
// spread over all CUs) and then streams its share of the weight rows exactly like
// gemv_multi_kernel, reading x from LDS.  KSPLIT: the four waves of a workgroup share a column
// pair and take a quarter of k each (deep, narrow matrices).
// GLUEPI (two problems of equal N, no k-split): a wave computes column n of both and stores
// act(first) * second, i.e. gate_proj, up_proj and the SwiGLU / GeGLU between them in one pass.
// MR: input rows that share the weights (a decode step of a small batch): MR rows of K floats are
// staged (rows * K <= GEMV_PRO_MAX_K), every weight vector fetched is used for each of them, and the
// outputs are the rows of a contiguous [rows, N] matrix.
// XV: 16-byte pieces of the input rows per thread (rows * K <= XV * 1024 floats).
// MERGE (PRO_ATTN_MERGE): the input row is the result of a split decode attention that stopped at its
// partials; every workgroup merges them on its way in - the maxima and sums of all (head, split) records,
// one per thread, meet in LDS, and a thread combines the value pieces of its positions with the weights
// exp(max_s - max) / sum.  All of it is requested with the first loads, so the attention launch needs no
// hand-over between its workgroups (acknowledged stores, a counter, a second pass over the partials:
// 2.8 us of a 6.7 us kernel) and the merge costs this launch one LDS exchange.
// AMAX (one row, one problem, no k-split): a wave also keeps the largest value it stores - in the order of
// f32::total_cmp, the last of equal values winning, like Backend::argmax (ndarray.rs:469-480) - and leaves
// (key, column, any) in g.amax_part[wave of the grid]: the argmax over the row then only merges these records
// instead of reading the row back.
// ROUTER (batched over MoE slots, one row, a plain product): the expert of a (slot, token) pair is chosen here, by
// the softmax and top-k of the token's router logits (GemvProDesc::router_logits).
template <typename TB, bool KSPLIT, bool GLUEPI, int MR, int XV, bool MERGE = false, bool AMAX = false, bool ROUTER = false>
__global__ void __launch_bounds__(256) gemv_pro_kernel(GemvProDesc g) {
  typedef typename WVec<TB>::type VT;
  constexpr int EPL = WVec<TB>::EPL, UNROLL = 4, R = 2;
  __shared__ __attribute__((aligned(16))) float xs[GEMV_PRO_MAX_K];
  __shared__ float lds[4 * MR];
  __shared__ float part[4][R][MR];
  __shared__ float2 merge_ml[MERGE ? 256 : 1];
  static_assert(!MERGE || (MR == 1 && !GLUEPI && !KSPLIT), "the attention merge feeds one row to a plain product");
  static_assert(!AMAX || (MR == 1 && !GLUEPI && !KSPLIT && !MERGE), "argmax records: one row, a plain product");
  int32_t best_key = INT32_MIN;
  uint32_t best_col = 0, best_any = 0;
  warm_kernel_arguments<sizeof(GemvProDesc)>();
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t K = g.m.K, bz = blockIdx.z;
  const uint32_t rows = MR == 1 ? 1u : g.rows;
  // batch entry -> (slot, token) when several MoE slots share the launch
  const uint32_t tz = g.slot_tokens ? bz % g.slot_tokens : bz, sz = g.slot_tokens ? bz / g.slot_tokens : 0u;
  const uint32_t az = g.a_by_token ? tz : bz;
  const float *ga = g.a + (int64_t)az * g.a_bstride;
  const float *gaux = g.aux ? g.aux + (int64_t)az * g.aux_bstride : nullptr;
  // ---- which rows of which matrix
  const uint32_t N = g.m.p[blockIdx.y].N;
  const TB *B = (const TB *)g.m.p[blockIdx.y].b;
  const TB *B2 = GLUEPI ? (const TB *)g.m.p[1].b : nullptr;
  const int64_t sbn2 = GLUEPI ? g.m.p[1].sbn : 0;
  if (g.b_index || g.slot_tokens) {
    uint32_t ix = 0;
    if constexpr (ROUTER) {
      // the router's softmax and top-k for this token, by every wave alike
      const bool writer = blockIdx.x == 0 && blockIdx.y == 0 && sz == 0 && wave == 0 && lane == 0;
      const uint32_t want = g.router_col[sz];
      softmax_topk_row<1>(g.router_logits + (int64_t)tz * g.router_stride, g.router_n, g.router_k, (uint32_t)lane,
                          [&](uint32_t t, float bv, uint32_t bi) {
                            if (t == want) ix = bi;
                            if (writer) {
                              g.router_values[(uint64_t)tz * g.router_k + t] = bv;
                              g.router_indices[(uint64_t)tz * g.router_k + t] = bi;
                            }
                          });
      ix = __builtin_amdgcn_readfirstlane(ix);
    } else {
      const uint32_t *bi = g.slot_tokens ? g.b_index_slot[sz] : g.b_index;
      ix = bi[(int64_t)tz * g.b_index_stride];
    }
    if (ix >= g.b_index_limit) {  // the reference's select() panics; flag it and stay in bounds
      atomicOr(g.err, ERRF_INDEX_OOB);
      ix = g.b_index_limit - 1;
    }
    B += (int64_t)ix * g.sb_index;
  }
  const int64_t sbn = g.m.p[blockIdx.y].sbn;
  float *C = g.m.p[blockIdx.y].c + (uint64_t)bz * N;
  const float *Cadd = g.m.p[blockIdx.y].c_add ? g.m.p[blockIdx.y].c_add + (uint64_t)bz * N : nullptr;
  const uint32_t cadd_rs = g.m.p[blockIdx.y].c_add_is_row ? 0u : N;  // a bias vector or a [rows, N] residual
  const uint32_t slot = KSPLIT ? blockIdx.x : blockIdx.x * 4 + wave;
  const uint32_t n_slots = KSPLIT ? gridDim.x : gridDim.x * 4;
  uint32_t k_begin = 0, k_end = K;
  if (KSPLIT) {
    const uint32_t per = ((K + 3) / 4 + EPL - 1) / EPL * EPL;
    k_begin = min(K, wave * per);
    k_end = min(K, k_begin + per);
  }
  constexpr int CPS = GLUEPI ? 1 : R;  // output columns per slot
  // The weight rows of the first pass do not depend on the input row: request them before the
  // prologue so that their latency overlaps it.
  // Every request is R * UNROLL loads, no fewer (positions past the end repeat the last valid piece
  // and are not used): the prologue below waits for its own, older loads by count.
  VT q[R][UNROLL];
  auto request = [&](uint32_t nb, uint32_t k0) {
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const uint32_t k = min(k0 + u * 64 * EPL, k_end - EPL);
        if (GLUEPI) q[r][u] = __builtin_nontemporal_load((const VT *)((r == 0 ? B + (int64_t)nb * sbn : B2 + (int64_t)nb * sbn2) + k));
        else q[r][u] = __builtin_nontemporal_load((const VT *)(B + (int64_t)min(nb + r, N - 1) * sbn + k));
      }
  };
  // A workgroup with no column to compute (the narrower problems of a grouped launch) has nothing to stage.
  if ((KSPLIT ? blockIdx.x : blockIdx.x * 4) * CPS >= N) return;
  // The input rows first: rows * K floats are at most XV 16-byte pieces per thread (K % 8 == 0: a piece
  // lies in one row), requested together with what the prologue combines them with (RMSNorm: gamma, one
  // vector for every row; GLU: the up rows).  They are older than the weight requests that follow, so
  // they come back first, and - every load here being unconditional, positions past the end repeating
  // the last piece - the compiler's wait for them is a count that leaves the weight loads in flight: the
  // prologue's arithmetic runs while the weights are still on their way.
  const uint32_t pieces = rows * K / 4;
  const bool has_aux = g.pro == PRO_RMSNORM ? gaux != nullptr : g.pro != PRO_NONE;
  const float *aux_base = has_aux ? gaux : ga;  // no aux: the loads below repeat the row's own pieces
  const int64_t aux_rs = !has_aux ? g.a_rstride : g.pro == PRO_RMSNORM ? 0 : g.aux_rstride;
  float4 xv[XV], gv[XV];
  uint32_t pm[XV], pk[XV];
  constexpr int MS = MERGE ? ATTN_MERGE_MAX_SPLITS : 1;
  float4 mv[XV][MS];  // MERGE: the value pieces of every split
  float2 my_ml = make_float2(0.f, 0.f);
  if constexpr (MERGE) {
    const uint32_t pw = g.merge_d + 4, records = g.merge_heads * g.merge_splits;
    my_ml = *(const float2 *)(g.merge_part + (uint64_t)min((uint32_t)tid, records - 1) * pw + g.merge_d);
#pragma unroll
    for (int j = 0; j < XV; ++j) {
      const uint32_t e = min((uint32_t)tid + j * 256u, pieces - 1) * 4;
      pm[j] = 0u;
      pk[j] = e;
      const uint32_t h = e / g.merge_d, t = e % g.merge_d;
#pragma unroll
      for (int sp = 0; sp < MS; ++sp)
        mv[j][sp] = *(const float4 *)(g.merge_part + (uint64_t)(h * g.merge_splits + min((uint32_t)sp, g.merge_splits - 1)) * pw + t);
    }
  } else {
#pragma unroll
    for (int j = 0; j < XV; ++j) {
      const uint32_t e = min((uint32_t)tid + j * 256u, pieces - 1) * 4;
      pm[j] = MR == 1 ? 0u : e / K;
      pk[j] = MR == 1 ? e : e % K;
      xv[j] = *(const float4 *)(ga + (int64_t)pm[j] * g.a_rstride + pk[j]);
    }
#pragma unroll
    for (int j = 0; j < XV; ++j) gv[j] = *(const float4 *)(aux_base + (int64_t)pm[j] * aux_rs + pk[j]);
  }
  bool requested = true;
  request(min(slot * CPS, N - 1), k_begin + lane * EPL);
  // ---- prologue: the input rows, from the registers loaded above into LDS
  if constexpr (MERGE) {
    merge_ml[tid] = my_ml;  // record (head, split) = tid: (maximum, sum)
    __syncthreads();
#pragma unroll
    for (int j = 0; j < XV; ++j)
      if (tid + j * 256 < pieces) {
        const uint32_t h = pk[j] / g.merge_d;
        const float2 *ml = merge_ml + h * g.merge_splits;
        float mx = -3.40282347e+38f;
        for (uint32_t sp = 0; sp < g.merge_splits; ++sp) mx = fmaxf(mx, ml[sp].x);
        float l = 0.f;
        float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int sp = 0; sp < MS; ++sp)
          if ((uint32_t)sp < g.merge_splits) {
            const float w = __expf(ml[sp].x - mx);
            l += w * ml[sp].y;
            o.x += w * mv[j][sp].x; o.y += w * mv[j][sp].y; o.z += w * mv[j][sp].z; o.w += w * mv[j][sp].w;
          }
        o.x /= l; o.y /= l; o.z /= l; o.w /= l;
        *(float4 *)(xs + pk[j]) = o;
      }
  } else if (g.pro == PRO_RMSNORM) {
    float ssq[MR];
#pragma unroll
    for (int m = 0; m < MR; ++m) ssq[m] = 0.f;
#pragma unroll
    for (int j = 0; j < XV; ++j)
      if (tid + j * 256 < pieces) {
        const float s = xv[j].x * xv[j].x + xv[j].y * xv[j].y + xv[j].z * xv[j].z + xv[j].w * xv[j].w;
#pragma unroll
        for (int m = 0; m < MR; ++m) ssq[m] += (MR == 1 || pm[j] == (uint32_t)m) ? s : 0.f;
      }
#pragma unroll
    for (int m = 0; m < MR; ++m) ssq[m] = wave_sum(ssq[m]);
    if (lane == 0)
#pragma unroll
      for (int m = 0; m < MR; ++m) lds[wave * MR + m] = ssq[m];
    __syncthreads();
    float rms[MR];
#pragma unroll
    for (int m = 0; m < MR; ++m)
      rms[m] = sqrtf(((lds[m] + lds[MR + m]) + (lds[2 * MR + m] + lds[3 * MR + m])) / g.n_as_float + g.eps);
#pragma unroll
    for (int j = 0; j < XV; ++j)
      if (tid + j * 256 < pieces) {
        float r = rms[0];
#pragma unroll
        for (int m = 1; m < MR; ++m) r = pm[j] == (uint32_t)m ? rms[m] : r;
        float4 o;
        o.x = xv[j].x / r; o.y = xv[j].y / r; o.z = xv[j].z / r; o.w = xv[j].w / r;
        if (has_aux) {
          o.x *= g.gamma_offset + gv[j].x; o.y *= g.gamma_offset + gv[j].y;
          o.z *= g.gamma_offset + gv[j].z; o.w *= g.gamma_offset + gv[j].w;
        }
        *(float4 *)(xs + (size_t)pm[j] * K + pk[j]) = o;
      }
  } else {
#pragma unroll
    for (int j = 0; j < XV; ++j)
      if (tid + j * 256 < pieces) {
        float4 o = xv[j];
        if (g.pro == PRO_GEGLU) {
          o.x = gelu_ref(o.x) * gv[j].x; o.y = gelu_ref(o.y) * gv[j].y;
          o.z = gelu_ref(o.z) * gv[j].z; o.w = gelu_ref(o.w) * gv[j].w;
        } else if (g.pro == PRO_SWIGLU) {
          o.x = o.x * sigmoid_ref(o.x) * gv[j].x; o.y = o.y * sigmoid_ref(o.y) * gv[j].y;
          o.z = o.z * sigmoid_ref(o.z) * gv[j].z; o.w = o.w * sigmoid_ref(o.w) * gv[j].w;
        }
        *(float4 *)(xs + (size_t)pm[j] * K + pk[j]) = o;
      }
  }
  __syncthreads();
  // Several rows: a lane meets the same k positions in every column (K <= 64 * EPL * UNROLL, one pass
  // over k), so its share of the staged rows moves to registers once and the column loop reads no LDS.
  float xr[MR > 1 ? MR : 1][UNROLL][EPL];
  if (MR > 1) {
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const uint32_t k = lane * EPL + u * 64 * EPL;
#pragma unroll
        for (int j4 = 0; j4 < EPL; j4 += 4) {
          float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
          if ((uint32_t)m < rows && k < K) t = *(const float4 *)(xs + (size_t)m * K + k + j4);
          xr[MR > 1 ? m : 0][u][j4] = t.x; xr[MR > 1 ? m : 0][u][j4 + 1] = t.y;
          xr[MR > 1 ? m : 0][u][j4 + 2] = t.z; xr[MR > 1 ? m : 0][u][j4 + 3] = t.w;
        }
      }
  }
  // ---- the products
  for (uint32_t nb = slot * CPS; nb < N; nb += n_slots * CPS) {  // uniform per workgroup when KSPLIT
    // (what is added at the end is requested now, positions clamped: see gemv_rowdot_kernel)
    float cpre[R][MR];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < MR; ++m) cpre[r][m] = 0.f;
    if (Cadd && !KSPLIT && !GLUEPI) {
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < MR; ++m) cpre[r][m] = Cadd[(uint64_t)min((uint32_t)m, rows - 1) * cadd_rs + min(nb + r, N - 1)];
    }
    float acc[R][MR];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < MR; ++m) acc[r][m] = 0.f;
    for (uint32_t k0 = k_begin + lane * EPL; k0 < k_end; k0 += 64 * EPL * UNROLL) {
      if (!requested) request(nb, k0);
      requested = false;
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const uint32_t k = k0 + u * 64 * EPL;
        if (k < k_end) {
          float xv[EPL];
          if (MR == 1) {
#pragma unroll
            for (int j4 = 0; j4 < EPL; j4 += 4) {
              const float4 t = *(const float4 *)(xs + k + j4);
              xv[j4] = t.x; xv[j4 + 1] = t.y; xv[j4 + 2] = t.z; xv[j4 + 3] = t.w;
            }
          }
#pragma unroll
          for (int r = 0; r < R; ++r) {
            if (GLUEPI || nb + r < N) {
              float w[EPL];
              WVec<TB>::widen(q[r][u], w);
#pragma unroll
              for (int m = 0; m < MR; ++m)
#pragma unroll
                for (int j = 0; j < EPL; ++j) acc[r][m] += w[j] * (MR == 1 ? xv[j] : xr[MR > 1 ? m : 0][u][j]);
            }
          }
        }
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < MR; ++m) acc[r][m] = wave_sum(acc[r][m]);
    if (GLUEPI) {
      if (lane == 0)
#pragma unroll
        for (int m = 0; m < MR; ++m)
          if ((uint32_t)m < rows)
            C[(uint64_t)m * N + nb] =
                (g.glu_epilogue == PRO_GEGLU ? gelu_ref(acc[0][m]) : acc[0][m] * sigmoid_ref(acc[0][m])) * acc[1][m];
    } else if (KSPLIT) {
      __syncthreads();
      if (lane == 0)
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
          for (int m = 0; m < MR; ++m) part[wave][r][m] = acc[r][m];
      __syncthreads();
      if (tid < R * MR) {
        const int r = tid % R, m = tid / R;
        if ((uint32_t)m < rows && nb + r < N) {
          const uint64_t at = (uint64_t)m * N + nb + r;
          C[at] = ((part[0][r][m] + part[1][r][m]) + (part[2][r][m] + part[3][r][m])) +
                  (Cadd ? Cadd[(uint64_t)m * cadd_rs + nb + r] : 0.f);
        }
      }
    } else if (lane == 0) {
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < MR; ++m)
          if ((uint32_t)m < rows && nb + r < N) {
            const uint64_t at = (uint64_t)m * N + nb + r;
            const float v = acc[r][m] + cpre[r][m];
            C[at] = v;
            if (AMAX) {
              const int32_t b = __float_as_int(v), key = b ^ (int32_t)(((uint32_t)(b >> 31)) >> 1);
              if (!best_any || key > best_key || (key == best_key && nb + r > best_col)) {
                best_key = key;
                best_col = nb + r;
                best_any = 1;
              }
            }
          }
    }
  }
  if (AMAX && lane == 0) {  // (a wave without a column leaves any = 0)
    uint32_t *rec = g.amax_part + (uint64_t)(blockIdx.x * 4 + wave) * 3;
    rec[0] = (uint32_t)best_key;
    rec[1] = best_col;
    rec[2] = best_any;
  }
}

// workgroups along x of the plain (no GLU epilogue, no attention merge) form
static uint32_t gemv_pro_block_count(const LaunchCtx &lc, const GemvProDesc &g, uint32_t slots, bool ksplit, bool multi) {
  // `slots` = column pairs per problem; 256-thread workgroups (wider ones stream worse).  Long input
  // rows cost more to recompute, so fewer workgroups each take several column pairs.
  const uint32_t per_wg = ksplit ? 1 : 4;
  uint32_t blocks = (slots + per_wg - 1) / per_wg;
  const uint32_t batch = g.batch ? g.batch : 1;
  // (several rows: two workgroups fit a CU and staging the rows costs as much as a pass of columns - one round)
  const uint32_t cap = (uint32_t)lc.n_cus * (multi || g.m.K >= 4096 ? 2 : 4) / (g.m.n_prob * batch);
  if (blocks > cap) blocks = cap ? cap : 1;
  return blocks;
}

template <typename TB, bool KSPLIT, int MR>
static void launch_gemv_pro_block(const LaunchCtx &lc, const GemvProDesc &g, uint32_t slots) {
  const uint32_t blocks = gemv_pro_block_count(lc, g, slots, KSPLIT, MR > 1);
  const uint32_t batch = g.batch ? g.batch : 1;
  dim3 grid(blocks, g.m.n_prob, batch);
  const uint32_t xv = ((MR > 1 ? g.rows : 1u) * g.m.K / 4 + 255) / 256;  // 16-byte pieces of the input rows per thread
  if constexpr (!KSPLIT && MR == 1) {
    if (g.router_logits) {  // (launch_gemv_pro has checked the form)
      if (xv <= 2) CG_LAUNCH(lc, (gemv_pro_kernel<TB, false, false, 1, 2, false, false, true>), grid, 256, g);
      else if (xv <= 4) CG_LAUNCH(lc, (gemv_pro_kernel<TB, false, false, 1, 4, false, false, true>), grid, 256, g);
      else CG_LAUNCH(lc, (gemv_pro_kernel<TB, false, false, 1, 8, false, false, true>), grid, 256, g);
      return;
    }
    if (g.amax_part) {  // (launch_gemv_pro has checked gemv_pro_amax_records)
      if (xv <= 2) CG_LAUNCH(lc, (gemv_pro_kernel<TB, false, false, 1, 2, false, true>), grid, 256, g);
      else if (xv <= 4) CG_LAUNCH(lc, (gemv_pro_kernel<TB, false, false, 1, 4, false, true>), grid, 256, g);
      else CG_LAUNCH(lc, (gemv_pro_kernel<TB, false, false, 1, 8, false, true>), grid, 256, g);
      return;
    }
  }
  if (xv <= 2) CG_LAUNCH(lc, (gemv_pro_kernel<TB, KSPLIT, false, MR, 2>), grid, 256, g);
  else if (xv <= 4) CG_LAUNCH(lc, (gemv_pro_kernel<TB, KSPLIT, false, MR, 4>), grid, 256, g);
  else CG_LAUNCH(lc, (gemv_pro_kernel<TB, KSPLIT, false, MR, 8>), grid, 256, g);
}

template <typename TB, int MR>
static void launch_gemv_pro_glu(const LaunchCtx &lc, const GemvProDesc &g) {
  const uint32_t slots = g.m.p[0].N;  // one (gate, up) column pair per wave pass
  uint32_t blocks = (slots + 3) / 4;
  // two workgroups per CU, each wave walking several column pairs: swept on the whole decode loop (workgroups
  // per CU: 1 -> 1344, 2 -> 1400-1407, 3 -> 1401, 4 -> 1383 tokens/s; more than four, with LDS sized per launch, 1323)
  const uint32_t cap = (uint32_t)lc.n_cus * 2;
  if (blocks > cap) blocks = cap;
  const uint32_t xv = ((MR > 1 ? g.rows : 1u) * g.m.K / 4 + 255) / 256;
  if (xv <= 2) CG_LAUNCH(lc, (gemv_pro_kernel<TB, false, true, MR, 2>), dim3(blocks, 1, 1), 256, g);
  else if (xv <= 4) CG_LAUNCH(lc, (gemv_pro_kernel<TB, false, true, MR, 4>), dim3(blocks, 1, 1), 256, g);
  else CG_LAUNCH(lc, (gemv_pro_kernel<TB, false, true, MR, 8>), dim3(blocks, 1, 1), 256, g);
}

uint32_t gemv_pro_multi_row_max_k(int b_stype) { return 64u * (b_stype == ST_BF16 ? 8u : 4u) * 4u; }

// ---- a few input rows against shared bf16 weights, on the matrix cores ---------------------------------
// A decode step of a small batch multiplies 2 to 16 rows by every weight matrix.  The kernel above does
// that with one multiply-add per lane, weight and row, and at four rows its arithmetic, not the stream of
// weights, sets the pace (17 us for 25 MB).  Here v_mfma_f32_16x16x32_bf16 does the arithmetic: its A
// operand is 16 weight columns - lane (n = lane & 15, kb = lane >> 4) holds k = kb * 8 .. + 7 of column n -
// and its B operand the input rows, narrowed to bf16 in LDS by the prologue (RMSNorm, SwiGLU / GeGLU or
// none, as above): lane (m, kb) reads row m, or zeros past the last row.  D[n][m] sits in lane
// m + 16 * (n / 4), register n % 4.
// Memory wants long runs: a load instruction whose lanes follow the operand layout touches 16 weight rows,
// 64 bytes of each, and streams at 5 TB/s; one that reads 512 contiguous bytes of two rows reaches 6.5.  So
// a lane loads piece lane & 31 (8 values) of row 2u + (lane >> 5) of a window of 256 k, 8 instructions a
// window, and the wave turns the window around in 8 KB of LDS of its own (rows 528 bytes apart, free of
// bank conflicts both ways) before it reads the operands.  Two windows are in flight per lane.
// A workgroup owns groups of 16 output columns; its four waves take a quarter of k each (K % 128 == 0) and
// meet in LDS, where thread (m, n) adds the four quarters, applies the epilogue and stores.  GLUEPI: a
// group is 8 columns of gate_proj and the same 8 of up_proj, rows 0-7 and 8-15 of one operand, and thread
// (m, n < 8) stores act(gate) * up.
// The inputs are rounded to bf16 like those of every many-row product in bf16 mode.
// RS, PP: the prologue keeps the rows of a wave - rows wave, wave + 4, ... (RS of them), so that a row's sum
// of squares never leaves the wave - as PP 16-byte pieces per lane and row in registers; RMSNorm needs the
// whole row at once (K <= 256 * PP), the elementwise prologues take K in several passes.
enum { GEMV_ROWS_MAX = 16, GEMV_ROWS_LDS = 20480, GEMV_ROWS_TP = 264 };
// The work of one workgroup: problem `prob` (GLUEPI: problems 0 and 1), groups first_group, first_group +
// group_step, ...
template <bool GLUEPI, int RS, int PP>
__device__ __forceinline__ void gemv_rows_mfma_body(const GemvProDesc &g, const uint32_t prob, const uint32_t first_group,
                                                    const uint32_t group_step, uint16_t *xs,
                                                    uint16_t (*turn)[16 * GEMV_ROWS_TP], float (*red)[16][17]) {
  typedef WVec<uint16_t>::type VT;
  constexpr int UN = 16;               // 16-byte loads in flight per lane: two windows of 8
  constexpr int CG = GLUEPI ? 8 : 16;  // output columns per group
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, kb = lane >> 4;
  const uint32_t K = g.m.K, rows = g.rows, pitch = K + 8;
  const uint32_t N = g.m.p[prob].N, groups = (N + CG - 1) / CG;
  if (first_group >= groups) return;  // the narrower problems of a grouped launch
  const uint16_t *B = (const uint16_t *)g.m.p[prob].b;
  const uint16_t *B2 = GLUEPI ? (const uint16_t *)g.m.p[1].b : nullptr;
  const int64_t sbn = g.m.p[prob].sbn, sbn2 = GLUEPI ? g.m.p[1].sbn : 0;
  float *C = g.m.p[prob].c;
  const float *Cadd = g.m.p[prob].c_add;
  const uint32_t cadd_rs = g.m.p[prob].c_add_is_row ? 0u : N;
  const uint32_t kw = K / 4, k_begin = wave * kw;  // this wave's share of k
  const uint32_t nbatch = (kw + 511) / 512;        // requests (two windows of 256) per group
  const uint32_t lrow = lane >> 5, lk = (lane & 31) * 8;
  // Every request is UN loads, no fewer (pieces past the end of the wave's share repeat its last and are not
  // used), so the prologue's wait for its own, older loads is a count that leaves these in flight.
  VT q[UN];
  auto request_window = [&](uint32_t group, uint32_t batch, int w2) {
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const uint32_t v = 2 * u + lrow;  // row of the operand
      const uint16_t *row;
      if (GLUEPI) row = u < 4 ? B + (int64_t)min(group * 8 + v, N - 1) * sbn : B2 + (int64_t)min(group * 8 + v - 8, N - 1) * sbn2;
      else row = B + (int64_t)min(group * 16 + v, N - 1) * sbn;
      const uint32_t kl = min((batch * 2 + w2) * 256 + lk, kw - 8);
      q[w2 * 8 + u] = __builtin_nontemporal_load((const VT *)(row + k_begin + kl));
    }
  };
  auto request = [&](uint32_t group, uint32_t batch) {
    request_window(group, batch, 0);
    request_window(group, batch, 1);
  };
  // Everything the prologue loads is used in straight-line code, down to the LDS store (pieces past the end of
  // a row or of the rows go to a spare location): a load whose only use sits inside a branch - gamma under
  // `if (aux)`, or the whole piece under `if (k < K)` - is moved there by the compiler, behind the request for
  // the weights, where it waits for them to arrive.
  auto early_load = [](const float *p) { return *(const float4 *)p; };
  uint16_t *spare = turn[wave] + lane * 4;  // (the wave's window buffer is not in use yet)
  auto narrow = [](const float4 &o) {
    union { bf16x2_t h[2]; uint2 u; } pk;
    pk.h[0] = __builtin_convertvector((f32x2_t){o.x, o.y}, bf16x2_t);
    pk.h[1] = __builtin_convertvector((f32x2_t){o.z, o.w}, bf16x2_t);
    return pk.u;
  };
  // ---- the input rows, to LDS as bf16
  if (g.pro == PRO_RMSNORM) {
    float4 xv[RS][PP], gv[PP];
#pragma unroll
    for (int i = 0; i < PP; ++i) {
      const uint32_t k = min((lane + 64 * i) * 4u, K - 4);
      gv[i] = early_load((g.aux ? g.aux : g.a) + k);  // gamma: one vector for every row
#pragma unroll
      for (int rs = 0; rs < RS; ++rs) xv[rs][i] = early_load(g.a + (int64_t)min(wave + 4u * rs, rows - 1) * g.a_rstride + k);
    }
    request(first_group, 0);
    const float has_gamma = g.aux ? 1.f : 0.f, no_gamma = 1.f - has_gamma;
#pragma unroll
    for (int rs = 0; rs < RS; ++rs) {
      float ssq = 0.f;
#pragma unroll
      for (int i = 0; i < PP; ++i)
        if ((lane + 64 * i) * 4u < K) ssq += xv[rs][i].x * xv[rs][i].x + xv[rs][i].y * xv[rs][i].y + xv[rs][i].z * xv[rs][i].z + xv[rs][i].w * xv[rs][i].w;
      const float inv = 1.0f / sqrtf(wave_sum(ssq) / g.n_as_float + g.eps);
      const uint32_t row = wave + 4u * rs;
#pragma unroll
      for (int i = 0; i < PP; ++i) {
        const uint32_t k = (lane + 64 * i) * 4u;
        float4 o;  // x / rms * (offset + gamma), or x / rms without a gamma (has_gamma = 0: the factor is 1)
        o.x = xv[rs][i].x * inv * (has_gamma * (g.gamma_offset + gv[i].x) + no_gamma);
        o.y = xv[rs][i].y * inv * (has_gamma * (g.gamma_offset + gv[i].y) + no_gamma);
        o.z = xv[rs][i].z * inv * (has_gamma * (g.gamma_offset + gv[i].z) + no_gamma);
        o.w = xv[rs][i].w * inv * (has_gamma * (g.gamma_offset + gv[i].w) + no_gamma);
        *(uint2 *)(row < rows && k < K ? xs + (size_t)row * pitch + k : spare) = narrow(o);
      }
    }
  } else {
    // elementwise prologues: PP pieces per lane and row at a time
    const bool glu = g.pro != PRO_NONE;
    const float is_glu = glu ? 1.f : 0.f, not_glu = 1.f - is_glu;
    const uint32_t ppr = (K + 255) / 256;
    float4 xv[RS][PP], gv[RS][PP];
    auto load_pass = [&](uint32_t i0) {
#pragma unroll
      for (int rs = 0; rs < RS; ++rs) {
        const uint32_t row = min(wave + 4u * rs, rows - 1);
        const float *xa = g.a + (int64_t)row * g.a_rstride;
        const float *xb = glu ? g.aux + (int64_t)row * g.aux_rstride : xa;  // no second operand: the row's own pieces again
#pragma unroll
        for (int i = 0; i < PP; ++i) {
          const uint32_t k = min((lane + 64 * (i0 + i)) * 4u, K - 4);
          xv[rs][i] = early_load(xa + k);
          gv[rs][i] = early_load(xb + k);
        }
      }
    };
    auto store_pass = [&](uint32_t i0) {
#pragma unroll
      for (int rs = 0; rs < RS; ++rs) {
        const uint32_t row = wave + 4u * rs;
#pragma unroll
        for (int i = 0; i < PP; ++i) {
          const uint32_t k = (lane + 64 * (i0 + i)) * 4u;
          float4 o = xv[rs][i];
          if (g.pro == PRO_GEGLU) {
            o.x = gelu_ref(o.x); o.y = gelu_ref(o.y); o.z = gelu_ref(o.z); o.w = gelu_ref(o.w);
          } else if (g.pro == PRO_SWIGLU) {
            o.x *= sigmoid_ref(o.x); o.y *= sigmoid_ref(o.y); o.z *= sigmoid_ref(o.z); o.w *= sigmoid_ref(o.w);
          }
          // times the second operand, or times 1 without one (is_glu = 0)
          o.x *= is_glu * gv[rs][i].x + not_glu; o.y *= is_glu * gv[rs][i].y + not_glu;
          o.z *= is_glu * gv[rs][i].z + not_glu; o.w *= is_glu * gv[rs][i].w + not_glu;
          *(uint2 *)(row < rows && k < K ? xs + (size_t)row * pitch + k : spare) = narrow(o);
        }
      }
    };
    load_pass(0);
    request(first_group, 0);
    store_pass(0);
    for (uint32_t i0 = PP; i0 < ppr; i0 += PP) {
      load_pass(i0);
      store_pass(i0);
    }
  }
  __syncthreads();
  // ---- the products
  const bool live = (uint32_t)r < rows;
  const uint16_t *xrow = xs + (size_t)min((uint32_t)r, rows - 1) * pitch + k_begin + kb * 8;
  uint16_t *mine = turn[wave];
  for (uint32_t group = first_group; group < groups; group += group_step) {
    f32x4n acc = {0.f, 0.f, 0.f, 0.f};
    for (uint32_t batch = 0; batch < nbatch; ++batch) {
#pragma unroll
      for (int w2 = 0; w2 < 2; ++w2) {
        const uint32_t wk = (batch * 2 + w2) * 256;  // where the window starts in the wave's share of k
        if (wk < kw) {
          // (LDS serves a wave's accesses in order: these stores follow the previous window's reads)
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
#pragma unroll
          for (int u = 0; u < 8; ++u) *(VT *)(mine + (2 * u + lrow) * GEMV_ROWS_TP + lk) = q[w2 * 8 + u];
          __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        }
        // The window's registers are free again: the same window of the next vectors - of this group, or the first
        // of the workgroup's next group - is requested into them while this one multiplies.
        if (batch + 1 < nbatch) request_window(group, batch + 1, w2);
        else if (group + group_step < groups) request_window(group + group_step, 0, w2);
        if (wk < kw) {
#pragma unroll
          for (int s = 0; s < 8; ++s)
            if (wk + s * 32 < kw) {
              union { uint4 u4; bf16x8 h; } xb, w;
              w.u4 = *(const uint4 *)(mine + r * GEMV_ROWS_TP + s * 32 + kb * 8);
              xb.u4 = *(const uint4 *)(xrow + wk + s * 32);
              if (!live) xb.u4 = make_uint4(0u, 0u, 0u, 0u);
              acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w.h, xb.h, acc, 0, 0, 0);
            }
        }
      }
    }
    __syncthreads();  // the previous group's sums have been read
#pragma unroll
    for (int v = 0; v < 4; ++v) red[wave][kb * 4 + v][r] = acc[v];
    __syncthreads();
    const uint32_t m = tid >> 4, n = tid & 15, col = group * CG + n;
    if (m < rows && n < (uint32_t)CG && col < N) {
      float v0 = (red[0][n][m] + red[1][n][m]) + (red[2][n][m] + red[3][n][m]);
      if (GLUEPI) {
        const float v1 = (red[0][n + 8][m] + red[1][n + 8][m]) + (red[2][n + 8][m] + red[3][n + 8][m]);
        v0 = (g.glu_epilogue == PRO_GEGLU ? gelu_ref(v0) : v0 * sigmoid_ref(v0)) * v1;
      } else if (Cadd) {
        v0 += Cadd[(uint64_t)m * cadd_rs + col];
      }
      C[(uint64_t)m * N + col] = v0;
    }
  }
}

// GLUEPI with glu_extra_blocks > 0: the first workgroups of the grid take one group each of the plain problems
// 2, 3 (narrow products on the same input rows: a MoE block's router and the gate of its shared expert), with
// the same prologue; the gated pair has as many workgroups fewer, so that the whole grid is resident at once.
template <bool GLUEPI, int RS, int PP>
__global__ void __launch_bounds__(256) gemv_rows_mfma_kernel(GemvProDesc g) {
  __shared__ __attribute__((aligned(16))) uint16_t xs[GEMV_ROWS_LDS];  // [rows][K + 8] bf16
  __shared__ __attribute__((aligned(16))) uint16_t turn[4][16 * GEMV_ROWS_TP];
  __shared__ float red[4][16][17];
  warm_kernel_arguments<sizeof(GemvProDesc)>();
  if constexpr (GLUEPI) {
    if (blockIdx.x >= g.glu_extra_blocks) {
      gemv_rows_mfma_body<true, RS, PP>(g, 0u, blockIdx.x - g.glu_extra_blocks, gridDim.x - g.glu_extra_blocks, xs, turn, red);
    } else {
      uint32_t at = blockIdx.x, prob = 2;
      while (prob + 1 < (uint32_t)g.m.n_prob && at >= (g.m.p[prob].N + 15) / 16) {
        at -= (g.m.p[prob].N + 15) / 16;
        ++prob;
      }
      gemv_rows_mfma_body<false, RS, PP>(g, prob, at, 0x40000000u, xs, turn, red);
    }
  } else {
    gemv_rows_mfma_body<false, RS, PP>(g, blockIdx.y, blockIdx.x, gridDim.x, xs, turn, red);
  }
}

// Whether the kernel above takes `rows` input rows of K values with prologue `pro`.
bool gemv_rows_mfma_ok(int b_stype, uint32_t rows, uint32_t K, int pro) {
  if (b_stype != ST_BF16 || rows < 2 || rows > GEMV_ROWS_MAX || K < 128 || K % 128) return false;
  if ((uint64_t)rows * (K + 8) > GEMV_ROWS_LDS) return false;
  // RMSNorm keeps a wave's rows whole in registers: 16 pieces of 16 bytes per lane
  if (pro == PRO_RMSNORM && (rows <= 4 ? 1u : rows <= 8 ? 2u : 4u) * ((K + 255) / 256) > 16) return false;
  return pro == PRO_NONE || pro == PRO_RMSNORM || pro == PRO_SWIGLU || pro == PRO_GEGLU;
}

bool gemv_pro_rows_ok(int b_stype, uint32_t rows, uint32_t K, int pro) {
  if (rows <= 1) return rows == 1 && K <= GEMV_PRO_MAX_K;
  if (gemv_rows_mfma_ok(b_stype, rows, K, pro)) return true;
  return rows <= 4 && (uint64_t)rows * K <= GEMV_PRO_MAX_K && K <= gemv_pro_multi_row_max_k(b_stype);
}

template <bool GLUEPI>
static void launch_gemv_rows_mfma_as(const LaunchCtx &lc, const GemvProDesc &g, dim3 grid) {
  if (g.rows > 8) CG_LAUNCH(lc, (gemv_rows_mfma_kernel<GLUEPI, 4, 4>), grid, 256, g);
  else if (g.rows > 4) CG_LAUNCH(lc, (gemv_rows_mfma_kernel<GLUEPI, 2, 8>), grid, 256, g);
  else if (g.m.K > 2048) CG_LAUNCH(lc, (gemv_rows_mfma_kernel<GLUEPI, 1, 16>), grid, 256, g);
  else CG_LAUNCH(lc, (gemv_rows_mfma_kernel<GLUEPI, 1, 8>), grid, 256, g);
}

static hipError_t launch_gemv_rows_mfma(const LaunchCtx &lc, const GemvProDesc &g, uint32_t max_n) {
  if (g.glu_epilogue) max_n = g.m.p[0].N;  // (further problems ride along as extra workgroups)
  const uint32_t groups = g.glu_epilogue ? (max_n + 7) / 8 : (max_n + 15) / 16;
  // Two workgroups per CU is what the kernel's registers (under 256 per lane) and its 77 KB of LDS allow: a larger
  // grid only queues behind the resident workgroups and stages the rows again.  A workgroup stages the rows once and
  // walks its groups, the next group's vectors requested while the current ones multiply.  (While the kernel kept a
  // register copy of the vectors in flight it held 270-280 registers, one workgroup per CU, and a grid sized for
  // two cost q/k/v of a four-row step 11.1 us instead of 9.5; without the copy and with two resident: 8.7 us.)
  uint32_t cap = (uint32_t)lc.n_cus * 2 / (g.glu_epilogue ? 1 : g.m.n_prob);
  if (!cap) cap = 1;
  const uint32_t blocks = groups < cap ? groups : cap;
  if (g.glu_epilogue) {
    GemvProDesc gg = g;
    gg.glu_extra_blocks = 0;
    for (int i = 2; i < g.m.n_prob; ++i) gg.glu_extra_blocks += (g.m.p[i].N + 15) / 16;
    const uint32_t glu_blocks = blocks + gg.glu_extra_blocks > cap && blocks > gg.glu_extra_blocks ? cap - gg.glu_extra_blocks : blocks;
    launch_gemv_rows_mfma_as<true>(lc, gg, dim3(glu_blocks + gg.glu_extra_blocks, 1, 1));
  } else {
    launch_gemv_rows_mfma_as<false>(lc, g, dim3(blocks, g.m.n_prob, 1));
  }
  return hipGetLastError();
}


// Whether (and how finely) launch_gemv_pro can leave argmax records: the number of records the launch writes
// to GemvProDesc::amax_part (3 words each), or 0 when this product takes another form.
uint32_t gemv_pro_amax_records(const LaunchCtx &lc, const GemvProDesc &g) {
  if (g.m.n_prob != 1 || g.rows > 1 || g.batch > 1 || g.b_index || g.slot_tokens || g.glu_epilogue || g.pro == PRO_ATTN_MERGE ||
      !g.m.p[0].N || g.m.K > GEMV_PRO_MAX_K)
    return 0;
  const uint32_t slots = (g.m.p[0].N + 1) / 2;
  if (g.m.K >= 4096 && slots <= (uint32_t)lc.n_cus * 8) return 0;  // k split over the waves
  return gemv_pro_block_count(lc, g, slots, false, false) * 4;
}

hipError_t launch_gemv_pro(const LaunchCtx &lc, const GemvProDesc &g) {
  uint32_t max_n = 0;
  for (int i = 0; i < g.m.n_prob; ++i) max_n = g.m.p[i].N > max_n ? g.m.p[i].N : max_n;
  if (!max_n || !g.m.n_prob) return hipSuccess;
  if (g.amax_part && !gemv_pro_amax_records(lc, g)) return hipErrorInvalidValue;
  if (g.pro == PRO_ATTN_MERGE) {
    if (!g.merge_part || g.merge_splits < 1 || g.merge_splits > ATTN_MERGE_MAX_SPLITS || g.merge_d % 4 || !g.merge_d ||
        g.merge_heads * g.merge_splits > 256 || g.m.K != g.merge_heads * g.merge_d || g.m.K > 2048 || g.m.K % 8 ||
        g.rows > 1 || g.batch > 1 || g.b_index || g.slot_tokens || g.glu_epilogue)
      return hipErrorInvalidValue;
    const uint32_t slots = (max_n + 1) / 2;
    uint32_t blocks = (slots + 3) / 4;
    const uint32_t cap = (uint32_t)lc.n_cus * 4 / g.m.n_prob;
    if (blocks > cap) blocks = cap ? cap : 1;
    dim3 grid(blocks, g.m.n_prob, 1);
    if (g.m.b_stype == ST_BF16) CG_LAUNCH(lc, (gemv_pro_kernel<uint16_t, false, false, 1, 2, true>), grid, 256, g);
    else CG_LAUNCH(lc, (gemv_pro_kernel<float, false, false, 1, 2, true>), grid, 256, g);
    return hipGetLastError();
  }
  const bool multi = g.rows > 1;  // several input rows share the weights
  if (multi && g.batch <= 1 && !g.b_index && !g.slot_tokens && gemv_rows_mfma_ok(g.m.b_stype, g.rows, g.m.K, g.pro)) {
    if (g.glu_epilogue && (g.m.n_prob < 2 || g.m.p[0].N != g.m.p[1].N)) return hipErrorInvalidValue;
    if ((uintptr_t)g.a % 16 || g.a_rstride % 4 || (g.aux && ((uintptr_t)g.aux % 16 || g.aux_rstride % 4))) return hipErrorInvalidValue;
    for (int i = 0; i < g.m.n_prob; ++i)
      if ((uintptr_t)g.m.p[i].b % 16 || g.m.p[i].sbn % 8) return hipErrorInvalidValue;
    return launch_gemv_rows_mfma(lc, g, max_n);
  }
  // several rows: one pass over k per column (K <= 64 lanes x 16 bytes x 4 loads)
  if (multi && (g.rows > 4 || (uint64_t)g.rows * g.m.K > GEMV_PRO_MAX_K || g.batch > 1 || g.b_index || g.slot_tokens ||
                g.m.K > gemv_pro_multi_row_max_k(g.m.b_stype)))
    return hipErrorInvalidValue;
  if (g.glu_epilogue) {
    if (g.m.n_prob != 2 || g.m.p[0].N != g.m.p[1].N || g.batch > 1 || g.b_index || g.slot_tokens) return hipErrorInvalidValue;
    if (g.m.b_stype == ST_BF16) multi ? launch_gemv_pro_glu<uint16_t, 4>(lc, g) : launch_gemv_pro_glu<uint16_t, 1>(lc, g);
    else multi ? launch_gemv_pro_glu<float, 4>(lc, g) : launch_gemv_pro_glu<float, 1>(lc, g);
    return hipGetLastError();
  }
  const uint32_t slots = (max_n + 1) / 2;
  const bool ksplit = g.m.K >= 4096 && slots * (uint32_t)g.m.n_prob <= (uint32_t)lc.n_cus * 8;
  if (g.router_logits && (multi || ksplit || !g.slot_tokens || g.amax_part || g.router_n < 1 || g.router_n > 64 || g.router_k < 1 ||
                          g.router_k > 8 || g.router_k > g.router_n || !g.router_values || !g.router_indices))
    return hipErrorInvalidValue;
  if (g.m.b_stype == ST_BF16) {
    if (multi) launch_gemv_pro_block<uint16_t, false, 4>(lc, g, slots);  // rows * K <= 8192: K < 4096
    else if (ksplit) launch_gemv_pro_block<uint16_t, true, 1>(lc, g, slots);
    else launch_gemv_pro_block<uint16_t, false, 1>(lc, g, slots);
  } else {
    if (multi) launch_gemv_pro_block<float, false, 4>(lc, g, slots);
    else if (ksplit) launch_gemv_pro_block<float, true, 1>(lc, g, slots);
    else launch_gemv_pro_block<float, false, 1>(lc, g, slots);
  }
  return hipGetLastError();
}

// ---- routed experts over many tokens (a MoE prefill) ----------------------------------------------------
// The batched, expert-indexed product above once there are enough tokens for an expert's matrix to
// be worth reading once instead of once per token: a workgroup owns (128 output columns, one
// expert, one problem).  It walks the (slot, token) pairs in segments of 4096, collects those
// routed to its expert in LDS, and multiplies them 128 at a time against its weight tile with
// v_mfma_f32_32x32x16_bf16 (token rows gathered, narrowed to bf16 and - for down_proj - computed
// from gate and up on the way into LDS); rows are scattered back to their slot's output.  Every
// (slot, token) pair belongs to exactly one expert, so every output row is written once.  An index
// past the last expert is flagged and served by the last expert, like the one-row kernel's clamp.
// NP weight tiles per workgroup: 1, or 2 for the fused gate / up form (fuse_glu).
template <int NP>
__global__ void __launch_bounds__(256) moe_gemm_kernel(MoeGemmDesc g) {
  constexpr int BM_ = 128, BN_ = 128, BK = 64, LD = BK + 8, SEG = 4096, MT = BM_ / 32;
  __shared__ __attribute__((aligned(16))) uint16_t As[BM_ * LD];
  __shared__ __attribute__((aligned(16))) uint16_t Bs[NP][BN_ * LD];
  __shared__ uint32_t list[SEG];  // slot << 16 | token
  __shared__ uint32_t count;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t e = blockIdx.y, n0 = blockIdx.x * BN_, prob = NP == 2 ? 0 : blockIdx.z;
  const uint32_t K = g.K, N = g.prob[prob].N, S = g.S;
  if (n0 >= N) return;  // the other problem is wider
  const uint16_t *W[NP];
  int64_t sbn[NP];
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    W[p] = (const uint16_t *)g.prob[prob + p].w + (int64_t)e * g.sb_index;
    sbn[p] = g.prob[prob + p].sbn;
  }
  const bool last = e + 1 == g.n_expert;
  const uint32_t pairs = S * g.n_slot;
  const int a_k8 = (tid & 7) * 8;  // this thread's 8 k of the staged rows tid >> 3, + 32, + 64, + 96
  for (uint32_t s0 = 0; s0 < pairs; s0 += SEG) {
    if (tid == 0) count = 0;
    __syncthreads();
    for (uint32_t p = s0 + tid; p < min(pairs, s0 + SEG); p += 256) {
      const uint32_t sl = p / S, t = p - sl * S;
      const uint32_t ix = g.slot[sl].idx[(int64_t)t * g.slot[sl].idx_stride];
      if (ix >= g.n_expert) atomicOr(g.err, ERRF_INDEX_OOB);
      if (ix == e || (last && ix >= g.n_expert)) list[atomicAdd(&count, 1u)] = sl << 16 | t;
    }
    __syncthreads();
    const uint32_t cnt = count;
    for (uint32_t m0 = 0; m0 < cnt; m0 += BM_) {
      const int live_tiles = (int)min((uint32_t)MT, (cnt - m0 + 31) / 32);  // 32-row tiles with any row (uniform)
      f32x16 acc[NP][MT];
#pragma unroll
      for (int p = 0; p < NP; ++p)
#pragma unroll
        for (int h = 0; h < MT; ++h)
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[p][h][i] = 0.f;
      const float *arow[MT], *xrow[MT];
      const uint16_t *hrow[MT];
      bool a_live[MT];
#pragma unroll
      for (int h = 0; h < MT; ++h) {
        const uint32_t r = m0 + (tid >> 3) + h * 32;
        a_live[h] = r < cnt;
        const uint32_t ent = a_live[h] ? list[r] : 0u, sl = ent >> 16, tok = ent & 0xFFFFu;
        arow[h] = g.slot[sl].a ? g.slot[sl].a + (int64_t)tok * g.slot[sl].a_bs : nullptr;
        xrow[h] = g.slot[sl].aux ? g.slot[sl].aux + (int64_t)tok * g.slot[sl].aux_bs : nullptr;
        hrow[h] = g.slot[sl].a16 ? g.slot[sl].a16 + (int64_t)tok * g.slot[sl].a_bs : nullptr;
      }
      // registers of the k-step in flight: token rows (as bf16) and the weight tiles
      uint4 q[MT];
      u32x4n wq[NP][4];
      auto fetch = [&](uint32_t k0) {
#pragma unroll
        for (int h = 0; h < MT; ++h) {
          if (!a_live[h] || k0 + a_k8 >= K) {
            q[h] = make_uint4(0u, 0u, 0u, 0u);
          } else if (hrow[h]) {
            q[h] = *(const uint4 *)(hrow[h] + k0 + a_k8);
          } else {
            const float4 x0 = *(const float4 *)(arow[h] + k0 + a_k8), x1 = *(const float4 *)(arow[h] + k0 + a_k8 + 4);
            float v[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
            if (g.pro == PRO_SWIGLU || g.pro == PRO_GEGLU) {
              const float4 u0 = *(const float4 *)(xrow[h] + k0 + a_k8), u1 = *(const float4 *)(xrow[h] + k0 + a_k8 + 4);
              const float u[8] = {u0.x, u0.y, u0.z, u0.w, u1.x, u1.y, u1.z, u1.w};
#pragma unroll
              for (int i = 0; i < 8; ++i) v[i] = (g.pro == PRO_GEGLU ? gelu_ref(v[i]) : v[i] * sigmoid_ref(v[i])) * u[i];
            }
            const uint2 lo = bf16_pack4(make_float4(v[0], v[1], v[2], v[3])), hi = bf16_pack4(make_float4(v[4], v[5], v[6], v[7]));
            q[h] = make_uint4(lo.x, lo.y, hi.x, hi.y);
          }
        }
#pragma unroll
        for (int p = 0; p < NP; ++p)
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            const int ch = tid + c * 256, col = ch >> 3, k8 = (ch & 7) * 8;
            wq[p][c] = (k0 + k8 < K)
                           ? __builtin_nontemporal_load((const u32x4n *)(W[p] + (int64_t)min(n0 + col, N - 1) * sbn[p] + k0 + k8))
                           : (u32x4n){0u, 0u, 0u, 0u};
          }
      };
      fetch(0);
      for (uint32_t k0 = 0; k0 < K; k0 += BK) {
        __syncthreads();  // the previous step's fragments have been read
#pragma unroll
        for (int h = 0; h < MT; ++h) *(uint4 *)(&As[((tid >> 3) + h * 32) * LD + a_k8]) = q[h];
#pragma unroll
        for (int p = 0; p < NP; ++p)
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            const int ch = tid + c * 256, col = ch >> 3, k8 = (ch & 7) * 8;
            *(u32x4n *)(&Bs[p][col * LD + k8]) = wq[p][c];
          }
        __syncthreads();
        if (k0 + BK < K) fetch(k0 + BK);  // in flight during the products below
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
          bf16x8 bf[NP];
#pragma unroll
          for (int p = 0; p < NP; ++p)
            bf[p] = *(const bf16x8 *)(&Bs[p][(wave * 32 + (lane & 31)) * LD + ks * 16 + (lane >> 5) * 8]);
#pragma unroll
          for (int h = 0; h < MT; ++h) {
            if (h < live_tiles) {
              const bf16x8 af = *(const bf16x8 *)(&As[(h * 32 + (lane & 31)) * LD + ks * 16 + (lane >> 5) * 8]);
#pragma unroll
              for (int p = 0; p < NP; ++p) acc[p][h] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, bf[p], acc[p][h], 0, 0, 0);
            }
          }
        }
      }
      // ---- rows back to their slot and token: register i of tile h is row
      // h * 32 + (i >> 2) * 8 + (lane >> 5) * 4 + (i & 3), column lane & 31
      const uint32_t col = n0 + wave * 32 + (lane & 31);
#pragma unroll
      for (int h = 0; h < MT; ++h)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const uint32_t r = m0 + h * 32 + (i >> 2) * 8 + (lane >> 5) * 4 + (i & 3);
          if (r < cnt && col < N) {
            const uint32_t ent = list[r];
            const uint64_t at = (uint64_t)(ent & 0xFFFFu) * N + col;
            if (NP == 2) {
              const float gt = acc[0][h][i];
              const float hv = (g.fuse_glu == PRO_GEGLU ? gelu_fast(gt) : silu_fast(gt)) * acc[NP - 1][h][i];  // (leaves as bf16)
              g.slot[ent >> 16].h16[at] = (uint16_t)bf16_bits(hv);
            } else {
              g.slot[ent >> 16].c[prob][at] = acc[0][h][i];
            }
          }
        }
      __syncthreads();  // As / Bs and the list are reused
    }
    __syncthreads();
  }
}

// ---- the same with the routing done once and the operands streamed like the dense GEMM ------------------
// One workgroup of 1024 threads sorts the (slot, token) pairs by expert: a histogram in LDS, a scan,
// and a scatter through per-expert cursors.  The order of an expert's pairs depends on the order
// the atomics land in, which only decides the tile row a token occupies, never its result.
// tiles (optional): tiles[0] = the number of 128-pair row tiles over all experts, tiles[1 + t] = expert << 16 |
// row tile within the expert, expert by expert - the work list of the GEMM, one workgroup per (row tile, column
// tile), so that an expert most tokens chose is spread over the device instead of walked by one workgroup.
__global__ void __launch_bounds__(1024) moe_route_kernel(MoeGemmDesc g, uint32_t *count, uint32_t *offset, uint32_t *list,
                                                         uint32_t *tiles) {
  __shared__ uint32_t hist[MOE_ROUTE_MAX_EXPERTS], cursor[MOE_ROUTE_MAX_EXPERTS], scan[1024];
  const uint32_t tid = threadIdx.x, E = g.n_expert, S = g.S, pairs = S * g.n_slot;
  for (uint32_t i = tid; i < E; i += 1024) hist[i] = 0;
  __syncthreads();
  for (uint32_t p = tid; p < pairs; p += 1024) {
    const uint32_t sl = p / S, t = p - sl * S;
    uint32_t ix = g.slot[sl].idx[(int64_t)t * g.slot[sl].idx_stride];
    if (ix >= E) {
      atomicOr(g.err, ERRF_INDEX_OOB);
      ix = E - 1;
    }
    atomicAdd(&hist[ix], 1u);
  }
  __syncthreads();
  const uint32_t per = (E + 1023) / 1024, first = tid * per;
  uint32_t local = 0;
  for (uint32_t i = first; i < min(E, first + per); ++i) local += hist[i];
  scan[tid] = local;
  __syncthreads();
  for (uint32_t d = 1; d < 1024; d <<= 1) {
    const uint32_t v = tid >= d ? scan[tid - d] : 0u;
    __syncthreads();
    scan[tid] += v;
    __syncthreads();
  }
  uint32_t at = scan[tid] - local;
  for (uint32_t i = first; i < min(E, first + per); ++i) {
    count[i] = hist[i];
    offset[i] = at;
    cursor[i] = at;
    at += hist[i];
  }
  __syncthreads();
  for (uint32_t p = tid; p < pairs; p += 1024) {
    const uint32_t sl = p / S, t = p - sl * S;
    const uint32_t ix = min(g.slot[sl].idx[(int64_t)t * g.slot[sl].idx_stride], E - 1);
    list[atomicAdd(&cursor[ix], 1u)] = sl << 16 | t;
  }
  if (!tiles) return;
  // the same scan over row tiles per expert
  uint32_t my_tiles = 0;
  for (uint32_t i = first; i < min(E, first + per); ++i) my_tiles += (hist[i] + 127) / 128;
  scan[tid] = my_tiles;
  __syncthreads();
  for (uint32_t d = 1; d < 1024; d <<= 1) {
    const uint32_t v = tid >= d ? scan[tid - d] : 0u;
    __syncthreads();
    scan[tid] += v;
    __syncthreads();
  }
  uint32_t tt = scan[tid] - my_tiles;
  for (uint32_t i = first; i < min(E, first + per); ++i)
    for (uint32_t j = 0; j < (hist[i] + 127) / 128; ++j) tiles[1 + tt++] = i << 16 | j;
  if (tid == 1023) tiles[0] = scan[1023];
}

// most row tiles launch_moe_route can list for g: every expert may end in a partly filled one
uint32_t moe_route_max_tiles(const MoeGemmDesc &g) { return (g.S * g.n_slot + 127) / 128 + g.n_expert; }

hipError_t launch_moe_route(const LaunchCtx &lc, const MoeGemmDesc &g, uint32_t *count, uint32_t *offset, uint32_t *list,
                            uint32_t *tiles) {
  if (!g.S || !g.n_slot || !g.n_expert) return hipSuccess;
  if (g.n_expert > MOE_ROUTE_MAX_EXPERTS || g.S > 65535 || g.n_slot > 8) return hipErrorInvalidValue;
  CG_LAUNCH(lc, moe_route_kernel, 1, 1024, g, count, offset, list, tiles);
  return hipGetLastError();
}

// A workgroup owns (128 output columns of NP problems, one expert) and walks that expert's pairs 128
// at a time.  Token rows (gathered through the sorted list, bf16) and weight rows travel to LDS with
// global_load_lds_dwordx4 exactly as in gemm_bf16_dma_kernel - same 1 KB wave loads, same XOR
// swizzle, NS stages in flight - so a k-step no longer waits out a trip to memory.  Wavefront w
// computes columns [32 w, 32 w + 32) of every 32-row tile that has a live row.
template <int NP, int NS>
__global__ void __launch_bounds__(256) moe_gemm_dma_kernel(MoeGemmDesc g) {
  constexpr int BM_ = 128, BN_ = 128, BK = 64, MT = BM_ / 32;
  constexpr int ROWS = BM_ + NP * BN_;    // the stacked [A; B0; B1] tile of a stage
  constexpr int LPW = ROWS / 8 / 4;       // 1 KB loads per wave per stage
  constexpr int STAGE = ROWS * BK * 2;    // bytes
  extern __shared__ __attribute__((aligned(16))) uint16_t dma_smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t prob = NP == 2 ? 0 : blockIdx.y;
  const uint32_t K = g.K, N = g.prob[prob].N;
  const uint32_t tiles_n = (N + BN_ - 1) / BN_;
  // consecutive workgroups (dealt round-robin to the 8 XCDs) take the column tiles of one expert: giving an
  // XCD a contiguous range of experts instead measured 10 % slower
  const uint32_t id = blockIdx.x;
  uint32_t e = id / tiles_n, m_first = 0, m_last = UINT32_MAX;
  const uint32_t n0 = (id - e * tiles_n) * BN_;
  if (g.route_tiles) {  // one row tile of one expert
    if (e >= g.route_tiles[0]) return;  // the grid is sized for the most tiles there can be
    const uint32_t ent = g.route_tiles[1 + e];
    e = ent >> 16;
    m_first = (ent & 0xFFFFu) * BM_;
    m_last = m_first + BM_;
  }
  if (e >= g.n_expert) return;  // the grid is sized for the wider problem
  const uint32_t cnt = min(g.route_count[e], m_last);
  const uint32_t *list = g.route_list + g.route_offset[e];
  const uint16_t *W[NP];
  int64_t sbn[NP];
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    W[p] = (const uint16_t *)g.prob[prob + p].w + (int64_t)e * g.sb_index;
    sbn[p] = g.prob[prob + p].sbn;
  }
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint16_t *)dma_smem;
  const int sw = (lane >> 1) & 7, half = lane >> 5;
  const int n_steps = (int)(K / BK);
  for (uint32_t m0 = m_first; m0 < cnt; m0 += BM_) {
    const int live_tiles = (int)min((uint32_t)MT, (cnt - m0 + 31) / 32);  // wave-uniform
    f32x16 acc[NP][MT];
#pragma unroll
    for (int p = 0; p < NP; ++p)
#pragma unroll
      for (int h = 0; h < MT; ++h)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[p][h][i] = 0.f;
    const uint16_t *gp[LPW];  // per-lane source of each of this wave's loads; advances by BK per stage
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
      const int q = wave * LPW + i;  // 8-row block of the stacked tile
      const int R = q * 8 + (lane >> 3);
      const int c = (lane & 7) ^ ((R >> 1) & 7);
      if (q * 8 < BM_) {
        // rows past the expert's last pair repeat it: loaded, multiplied, never stored
        const uint32_t ent = list[min(m0 + (uint32_t)R, cnt - 1)], sl = ent >> 16, tok = ent & 0xFFFFu;
        const uint16_t *rows = g.slot[0].a16;
        int64_t bs = g.slot[0].a_bs;
#pragma unroll
        for (int s = 1; s < 8; ++s)
          if (sl == (uint32_t)s) {
            rows = g.slot[s].a16;
            bs = g.slot[s].a_bs;
          }
        gp[i] = rows + (int64_t)tok * bs + c * 8;
      } else {
        const int rb = R - BM_, p = rb / BN_, col = rb - p * BN_;
        gp[i] = W[p < NP ? p : 0] + (int64_t)min(n0 + (uint32_t)col, N - 1) * sbn[p < NP ? p : 0] + c * 8;
      }
    }
    auto issue = [&](int buf) {
#pragma unroll
      for (int i = 0; i < LPW; ++i) {
        if ((wave * LPW + i) * 8 < BM_) lds_dma16(gp[i], lds0 + buf * STAGE + (wave * LPW + i) * 1024);
        else lds_dma16_stream(gp[i], lds0 + buf * STAGE + (wave * LPW + i) * 1024);
        gp[i] += BK;
      }
    };
    auto compute = [&](int buf) {
      const uint16_t *As = dma_smem + buf * (STAGE / 2), *Bs = As + BM_ * BK;
      bf16x8 af[2][MT], bfr[2][NP];
      auto frags = [&](int ks, int set) {
        const int o = ((ks * 2 + half) ^ sw) * 8;
#pragma unroll
        for (int h = 0; h < MT; ++h)
          if (h < live_tiles) af[set][h] = *(const bf16x8 *)(&As[(h * 32 + (lane & 31)) * BK + o]);
#pragma unroll
        for (int p = 0; p < NP; ++p) bfr[set][p] = *(const bf16x8 *)(&Bs[(p * BN_ + wave * 32 + (lane & 31)) * BK + o]);
      };
      frags(0, 0);
#pragma unroll
      for (int ks = 0; ks < BK / 16; ++ks) {
        if (ks + 1 < BK / 16) frags(ks + 1, (ks + 1) & 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int h = 0; h < MT; ++h)
          if (h < live_tiles)
#pragma unroll
            for (int p = 0; p < NP; ++p)
              acc[p][h] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[ks & 1][h], bfr[ks & 1][p], acc[p][h], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
#pragma unroll
    for (int s0 = 0; s0 < NS - 1; ++s0)
      if (s0 < n_steps) issue(s0);
    for (int step = 0; step < n_steps; ++step) {
      if (step + NS - 1 <= n_steps) wait_vmcnt<(NS - 2) * LPW>();
      else wait_vmcnt<0>();
      __syncthreads();
      if (step + NS - 1 < n_steps) issue((step + NS - 1) % NS);
      compute(step % NS);
    }
    // ---- rows back to their slot and token.  Register i of tile h is row
    // h * 32 + (i >> 2) * 8 + (lane >> 5) * 4 + (i & 3), column lane & 31.  The tile is staged in LDS
    // (the operand stages are free now) so that a row leaves as 16-byte pieces: f32 for a plain
    // product, bf16 act(gate) * up for the fused pair.
    __syncthreads();  // every wave is done reading the last stage
    constexpr int TP = NP == 2 ? BN_ + 8 : BN_ + 4;  // row pitch in elements (keeps 16-byte alignment)
    if (NP == 2) {
      uint16_t *T = dma_smem;
#pragma unroll
      for (int h = 0; h < MT; ++h)
        if (h < live_tiles)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const float gt = acc[0][h][i];
            const float hv = (g.fuse_glu == PRO_GEGLU ? gelu_fast(gt) : silu_fast(gt)) * acc[NP - 1][h][i];  // (leaves as bf16)
            T[(h * 32 + (i >> 2) * 8 + (lane >> 5) * 4 + (i & 3)) * TP + wave * 32 + (lane & 31)] = (uint16_t)bf16_bits(hv);
          }
    } else {
      float *T = (float *)dma_smem;
#pragma unroll
      for (int h = 0; h < MT; ++h)
        if (h < live_tiles)
#pragma unroll
          for (int i = 0; i < 16; ++i)
            T[(h * 32 + (i >> 2) * 8 + (lane >> 5) * 4 + (i & 3)) * TP + wave * 32 + (lane & 31)] = acc[0][h][i];
    }
    __syncthreads();
    {
      constexpr int EPV = NP == 2 ? 8 : 4;        // elements per 16-byte piece
      constexpr int PPR = BN_ / EPV;              // pieces per row
      const uint32_t rows_here = min((uint32_t)BM_, cnt - m0);
      for (uint32_t idx = tid; idx < rows_here * PPR; idx += 256) {
        const uint32_t r = idx / PPR, c = (idx - r * PPR) * EPV;
        if (n0 + c >= N) continue;  // N % 8 == 0: a piece is inside or outside
        const uint32_t ent = list[m0 + r], sl = ent >> 16;
        const uint64_t at = (uint64_t)(ent & 0xFFFFu) * N + n0 + c;
        if (NP == 2) {
          uint16_t *out = g.slot[0].h16;
#pragma unroll
          for (int s2 = 1; s2 < 8; ++s2)
            if (sl == (uint32_t)s2) out = g.slot[s2].h16;
          *(uint4 *)(out + at) = *(const uint4 *)(dma_smem + r * TP + c);
        } else {
          float *out = g.slot[0].c[prob];
#pragma unroll
          for (int s2 = 1; s2 < 8; ++s2)
            if (sl == (uint32_t)s2) out = g.slot[s2].c[prob];
          *(float4 *)(out + at) = *(const float4 *)((const float *)dma_smem + r * TP + c);
        }
      }
    }
    wait_vmcnt<0>();
    __syncthreads();  // the stages are refilled for the next 128 pairs
  }
}

bool moe_gemm_pipelined_ok(const MoeGemmDesc &g) {
  if (!g.route_count || !g.route_offset || !g.route_list || g.K % 64 || g.K < 64 || g.pro != PRO_NONE) return false;
  for (uint32_t s = 0; s < g.n_slot; ++s)
    if (!g.slot[s].a16 || (uintptr_t)g.slot[s].a16 % 16 || g.slot[s].a_bs % 8) return false;
  for (uint32_t p = 0; p < g.n_prob; ++p)
    if ((uintptr_t)g.prob[p].w % 16 || g.prob[p].sbn % 8 || g.sb_index % 8 || g.prob[p].N % 8) return false;
  for (uint32_t s = 0; s < g.n_slot; ++s)  // rows leave as 16-byte pieces
    if (g.fuse_glu ? (uintptr_t)g.slot[s].h16 % 16 != 0 : ((uintptr_t)g.slot[s].c[0] % 16 != 0 || (g.n_prob > 1 && (uintptr_t)g.slot[s].c[1] % 16 != 0)))
      return false;
  return true;
}

template <int NP, int NS>
static hipError_t launch_moe_gemm_dma(const LaunchCtx &lc, const MoeGemmDesc &g, dim3 grid) {
  // the operand stages, or the staged output tile (f32 rows of 128 + 4, or bf16 rows of 128 + 8) if that is larger
  constexpr int stages = NS * (128 + NP * 128) * 64 * 2, tile = NP == 2 ? 128 * (128 + 8) * 2 : 128 * (128 + 4) * 4;
  constexpr int smem = stages > tile ? stages : tile;
  static bool configured = false;  // one attribute call per kernel and process
  if (!configured) {
    hipError_t e = hipFuncSetAttribute((const void *)moe_gemm_dma_kernel<NP, NS>, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return e;
    configured = true;
  }
  cg_launch(lc, moe_gemm_dma_kernel<NP, NS>, grid, dim3(256), smem, g);
  return hipGetLastError();
}

hipError_t launch_moe_gemm(const LaunchCtx &lc, const MoeGemmDesc &g) {
  if (!g.S || !g.n_prob || !g.n_slot || !g.n_expert) return hipSuccess;
  if (g.S > 65535 || g.n_slot > 8 || g.n_prob > 2 || g.n_expert > 65535 || g.K % 8 || g.pro == PRO_RMSNORM)
    return hipErrorInvalidValue;
  uint32_t max_n = 0;
  for (uint32_t i = 0; i < g.n_prob; ++i) max_n = g.prob[i].N > max_n ? g.prob[i].N : max_n;
  if (!max_n) return hipSuccess;
  if (g.fuse_glu) {
    if (g.n_prob != 2 || g.prob[0].N != g.prob[1].N || g.pro != PRO_NONE) return hipErrorInvalidValue;
    if (moe_gemm_pipelined_ok(g))
      return launch_moe_gemm_dma<2, 3>(lc, g, dim3((max_n + 127) / 128 * (g.route_tiles ? moe_route_max_tiles(g) : g.n_expert), 1, 1));
    dim3 grid((max_n + 127) / 128, g.n_expert, 1);
    CG_LAUNCH(lc, moe_gemm_kernel<2>, grid, 256, g);
  } else if (moe_gemm_pipelined_ok(g)) {
    return launch_moe_gemm_dma<1, 2>(lc, g, dim3((max_n + 127) / 128 * (g.route_tiles ? moe_route_max_tiles(g) : g.n_expert), g.n_prob, 1));
  } else {
    dim3 grid((max_n + 127) / 128, g.n_expert, g.n_prob);
    CG_LAUNCH(lc, moe_gemm_kernel<1>, grid, 256, g);
  }
  return hipGetLastError();
}

// ---- GEMV, B n-contiguous (V of attention): y[m, n] = sum_k x[m, k] * B[k, n] ---------------------
// 16 column groups of 4 columns x KS k-slices per workgroup; slices meet in LDS.
template <typename TB, int MROWS, int KS>
__global__ void __launch_bounds__(16 * KS) gemv_col_kernel(GemmDesc g, int b_vec) {
  warm_kernel_arguments<sizeof(GemmDesc)>();
  __shared__ float part[KS][MROWS][64 + 4];
  const int cg = threadIdx.x & 15, ks = threadIdx.x >> 4;
  const uint32_t bz = blockIdx.y, b0 = bz / g.nb1, b1 = bz - b0 * g.nb1;
  const float *A = (const float *)g.a + b0 * g.sa_b0 + b1 * g.sa_b1;
  const TB *B = (const TB *)g.b + b_batch_offset(g, bz, b0, b1);
  float *C = g.c + (uint64_t)bz * g.M * g.N;
  const float *Cadd = g.c_add ? g.c_add + (uint64_t)bz * g.M * g.N : nullptr;
  const uint32_t n = blockIdx.x * 64 + cg * 4;
  float acc[MROWS][4];
#pragma unroll
  for (int m = 0; m < MROWS; ++m)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[m][j] = 0.f;
  for (uint32_t k = ks; k < g.K; k += KS) {
    const TB *brow = B + (int64_t)k * g.sbk + n;
    float w[4];
    if (b_vec && n + 4 <= g.N) {
      if (sizeof(TB) == 4) {
        float4 q = *(const float4 *)brow;
        w[0] = q.x; w[1] = q.y; w[2] = q.z; w[3] = q.w;
      } else {
        uint2 q = *(const uint2 *)brow;
        w[0] = __uint_as_float(q.x << 16); w[1] = __uint_as_float(q.x & 0xFFFF0000u);
        w[2] = __uint_as_float(q.y << 16); w[3] = __uint_as_float(q.y & 0xFFFF0000u);
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = n + j < g.N ? widen(brow[j]) : 0.f;
    }
#pragma unroll
    for (int m = 0; m < MROWS; ++m) {
      if ((uint32_t)m < g.M) {
        const float xv = A[(int64_t)m * g.sam + (int64_t)k * g.sak];
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[m][j] += xv * w[j];
      }
    }
  }
#pragma unroll
  for (int m = 0; m < MROWS; ++m)
#pragma unroll
    for (int j = 0; j < 4; ++j) part[ks][m][cg * 4 + j] = acc[m][j];
  __syncthreads();
  for (int o = threadIdx.x; o < MROWS * 64; o += 16 * KS) {
    const int m = o / 64, c = o % 64;
    float s = 0.f;
#pragma unroll
    for (int q = 0; q < KS; ++q) s += part[q][m][c];
    const uint32_t col = blockIdx.x * 64 + c;
    if ((uint32_t)m < g.M && col < g.N)
      C[(uint64_t)m * g.N + col] = s + (Cadd ? Cadd[(uint64_t)m * g.N + col] : 0.f);
  }
}

// ---- u32 matmul (wrapping), contiguous operands: correctness path only -------------------------
__global__ void __launch_bounds__(256) matmul_u32_kernel(const uint32_t *a, const uint32_t *b,
                                                         uint32_t *c, uint32_t batch, uint32_t M,
                                                         uint32_t N, uint32_t K) {
  const uint64_t total = (uint64_t)batch * M * N;
  for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < total;
       i += (uint64_t)gridDim.x * 256) {
    const uint32_t n = i % N, m = (i / N) % M, bz = i / ((uint64_t)M * N);
    const uint32_t *ar = a + ((uint64_t)bz * M + m) * K, *bc = b + (uint64_t)bz * K * N + n;
    uint32_t s = 0;
    for (uint32_t k = 0; k < K; ++k) s += ar[k] * bc[(uint64_t)k * N];
    c[i] = s;
  }
}

hipError_t launch_matmul_u32(const LaunchCtx &lc, const uint32_t *a, const uint32_t *b, uint32_t *c,
                             uint32_t batch, uint32_t M, uint32_t N, uint32_t K) {
  uint64_t total = (uint64_t)batch * M * N;
  if (!total) return hipSuccess;
  uint64_t blocks = (total + 255) / 256, cap = (uint64_t)lc.n_cus * 8;
  CG_LAUNCH(lc, (matmul_u32_kernel), (unsigned)(blocks < cap ? blocks : cap), 256, a, b, c, batch,
                                                                                   M, N, K);
  return hipGetLastError();
}

// ---- dispatch ------------------------------------------------------------------------------
static bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

// 16-byte loads along the unit-stride axis are legal when the base, the other matrix stride and
// the batch strides all keep 16-byte alignment
static int vec_ok(const void *base, int esize, int64_t other_stride, int64_t sb0, int64_t sb1) {
  const int64_t q = 16 / esize;
  return aligned16(base) && other_stride % q == 0 && sb0 % q == 0 && sb1 % q == 0;
}

template <typename TA, typename TB, bool BF16>
static void launch_gemm_layout(const LaunchCtx &lc, const GemmDesc &g, dim3 grid, int av, int bv) {
  const bool akc = g.sak == 1 || g.K == 1, bkc = g.sbk == 1 && !(g.sbn == 1 && g.N > 1 && false);
  if (akc && bkc) CG_LAUNCH(lc, (gemm_kernel<TA, TB, true, true, BF16>), grid, 256, g, av, bv);
  else if (akc) CG_LAUNCH(lc, (gemm_kernel<TA, TB, true, false, BF16>), grid, 256, g, av, bv);
  else if (bkc) CG_LAUNCH(lc, (gemm_kernel<TA, TB, false, true, BF16>), grid, 256, g, av, bv);
  else CG_LAUNCH(lc, (gemm_kernel<TA, TB, false, false, BF16>), grid, 256, g, av, bv);
}

template <typename TB, int MROWS>
static void launch_rowdot(const LaunchCtx &lc, const GemmDesc &g, int bv, int av) {
  constexpr int EPL = 16 / sizeof(TB);
  constexpr int R = MROWS == 1 ? 2 : 1;
  const uint32_t batch = g.nb0 * g.nb1;
  uint32_t lanes = (g.K + EPL - 1) / EPL;
  int lpr = lanes >= 64 ? 64 : lanes >= 32 ? 32 : lanes >= 16 ? 16 : 8;
  const uint32_t cpw = 64 / lpr;
  const uint32_t groups = (g.N + cpw * R - 1) / (cpw * R);  // column groups of one wave-pass
  // deep and narrow (down_proj: K = 8192, N = 2048): four waves share a column group
  const bool ksplit = lpr == 64 && g.K >= 4096 && (uint64_t)groups * batch <= (uint64_t)lc.n_cus * 16;
  uint32_t blocks = ksplit ? groups : (groups + 3) / 4;
  const uint32_t cap = (uint32_t)lc.n_cus * 16;
  if ((uint64_t)blocks * batch > cap) blocks = (cap + batch - 1) / batch;
  if (blocks < 1) blocks = 1;
  dim3 grid(blocks, batch);
  if (ksplit) {
    // Up to four rows (the shared expert's down_proj of a MoE decode step, 4 x 5632 x 2048): a wave reads its share of
    // every input row from L2 once per column group - with one column in a group that is eight times the weights'
    // bytes.  Two columns share it (10.7 us against 14.0; four columns 12.3, eight 16.2: too few workgroups).
    if constexpr (MROWS == 4) {
      CG_LAUNCH(lc, (gemv_rowdot_kernel<TB, 64, 4, 2, 4>), dim3((g.N + 1) / 2, batch), 256, g, bv, av);
      return;
    }
    CG_LAUNCH(lc, (gemv_rowdot_kernel<TB, 64, MROWS, R, 4>), grid, 256, g, bv, av);
    return;
  }
  switch (lpr) {
    case 64: CG_LAUNCH(lc, (gemv_rowdot_kernel<TB, 64, MROWS, R, 1>), grid, 256, g, bv, av); break;
    case 32: CG_LAUNCH(lc, (gemv_rowdot_kernel<TB, 32, MROWS, R, 1>), grid, 256, g, bv, av); break;
    case 16: CG_LAUNCH(lc, (gemv_rowdot_kernel<TB, 16, MROWS, R, 1>), grid, 256, g, bv, av); break;
    default: CG_LAUNCH(lc, (gemv_rowdot_kernel<TB, 8, MROWS, R, 1>), grid, 256, g, bv, av); break;
  }
}

// the direct-to-LDS kernel: both operands unit-stride along k, K (and each split) a multiple of 64
static bool gemm_dma_ok(const GemmDesc &g) {
  return g.sak == 1 && g.sbk == 1 && g.K % 64 == 0 && g.K >= 64 && g.M >= 64 && g.N >= 64;
}

// B [K, N] with unit stride along n, used as it lies by the k-major form of the direct-to-LDS kernel
bool gemm_dma_bkm_ok(const GemmDesc &g) {
  return g.bf16_math && g.a_stype == ST_BF16 && g.b_stype == ST_BF16 && g.sak == 1 && g.sbn == 1 && g.sbk != 1 && g.sbk % 8 == 0 &&
         g.K % 64 == 0 && g.K >= 64 && g.M >= 64 && g.N >= 64 && g.N % 8 == 0 && ((uintptr_t)g.a & 15) == 0 &&
         ((uintptr_t)g.b & 15) == 0 && g.sam % 8 == 0 && g.sa_b0 % 8 == 0 && g.sa_b1 % 8 == 0 && g.sb_b0 % 8 == 0 &&
         g.sb_b1 % 8 == 0 && !g.b_index && !g.n_group && !g.glu_gate && !g.c16 && !g.dual_b && !g.c_add;
}

static bool gemm_fast_path(const GemmDesc &g, int av, int bv) {
  return g.bf16_math && g.M > 8 && g.a_stype == ST_BF16 && g.b_stype == ST_BF16 && g.sak == 1 &&
         (g.sbk == 1 || g.sbn == 1) && g.K % 8 == 0 && (g.sbk == 1 || g.N % 8 == 0) && av && bv;
}

bool gemm_epilogue_ok(const GemmDesc &g) {
  const int asz = g.a_stype == ST_BF16 ? 2 : 4, bsz = g.b_stype == ST_BF16 ? 2 : 4;
  const int av = vec_ok(g.a, asz, g.sak == 1 ? g.sam : g.sak, g.sa_b0, g.sa_b1);
  const int bv = vec_ok(g.b, bsz, g.sbk == 1 ? g.sbn : g.sbk, g.sb_b0, g.sb_b1);
  return gemm_fast_path(g, av, bv) && gemm_dma_ok(g) && g.splits <= 1 && !g.b_index && !g.c_add && g.N % 4 == 0;
}

bool gemm_rope_epilogue_ok(const LaunchCtx &lc, const GemmDesc &g) {
  if (!g.rope_s || !g.n_group || !gemm_epilogue_ok(g)) return false;
  if (g.rope_hd != 64 && g.rope_hd != 128) return false;
  if (g.nb0 * g.nb1 != 1 || g.glu_gate || g.c16 || g.dual_b || g.M % g.rope_s || g.rope_s % 4 || g.M < 64) return false;
  bool grp256 = true;
  for (uint32_t p = 0; p < g.n_group; ++p) {
    if (g.grp_n[p] % 128) return false;
    grp256 = grp256 && g.grp_n[p] % 256 == 0;
    if (g.rope_role[p] == 1) {
      if (!g.rope_out[p] || !g.rope_cos[p] || !g.rope_sin[p]) return false;
    } else if (g.rope_role[p] == 2) {
      if (!g.rope_out16[p] || (uintptr_t)g.rope_out16[p] % 8 || !g.grp_c[p]) return false;
    } else if (g.rope_role[p] != 0 || !g.grp_c[p]) {
      return false;
    }
  }
  // launch_matmul's tiles of 128 rows have this epilogue (128 columns, or 64 - for heads of 64 - where those are
  // too few for the CUs); the 256 x 256 tile of the largest problems has not
  const uint64_t t256 = (uint64_t)((g.M + 255) / 256) * ((g.N + 255) / 256);
  if (t256 >= (uint64_t)lc.n_cus && grp256) return false;
  return g.N >= 128;
}

// A plain product of 2 to 16 rows with bf16 weights [N][K] that gemv_rows_mfma_kernel takes.
// (any number of columns: the caller may group several narrow products into one launch)
bool gemv_rows_group_ok(const GemmDesc &g) {
  if (g.M < 2 || g.M > GEMV_ROWS_MAX || g.nb0 * g.nb1 != 1 || g.b_index || g.splits > 1 || g.K >= 4096) return false;
  if (g.a_stype != ST_F32 || g.b_stype != ST_BF16 || !g.bf16_math || g.sak != 1 || g.sbk != 1 || g.N < 1) return false;
  if (g.glu_gate || g.c16 || g.n_group || g.dual_b || (g.c_add && g.M > 8)) return false;
  if ((uintptr_t)g.a % 16 || g.sam % 4 || (uintptr_t)g.b % 16 || (g.N > 1 && g.sbn % 8)) return false;
  return gemv_rows_mfma_ok(ST_BF16, g.M, g.K, PRO_NONE);
}
bool gemv_rows_plain_ok(const LaunchCtx &lc, const GemmDesc &g) {
  // deep and narrow (down_proj of a wide MLP, 4 x 5632 x 2048): fewer 16-column groups than half the CUs, each
  // a chain of several trips to memory - the vector kernel splits k further and is faster there (12.6 against 16.7 us)
  if (g.K >= 4096 && (g.N + 15) / 16 * 2 <= (uint32_t)lc.n_cus && g.M <= 8) return false;
  if (g.M < 2 || g.M > GEMV_ROWS_MAX || g.nb0 * g.nb1 != 1 || g.b_index || g.splits > 1) return false;
  if (g.a_stype != ST_F32 || g.b_stype != ST_BF16 || !g.bf16_math || g.sak != 1 || g.sbk != 1 || g.N < 64) return false;
  if (g.glu_gate || g.c16 || g.n_group || g.dual_b || (g.c_add && g.M > 8)) return false;
  if ((uintptr_t)g.a % 16 || g.sam % 4 || (uintptr_t)g.b % 16 || g.sbn % 8) return false;
  return gemv_rows_mfma_ok(ST_BF16, g.M, g.K, PRO_NONE);
}

hipError_t launch_splitk_sum(const LaunchCtx &lc, const float *ws, float *c, uint64_t n, uint32_t splits, const float *cadd) {
  if (!n || !splits) return hipSuccess;
  if ((uintptr_t)ws % 16 || (uintptr_t)c % 16 || (cadd && (uintptr_t)cadd % 16) || (splits > 1 && n % 4)) return hipErrorInvalidValue;
  uint64_t blocks = (n / 4 + 255) / 256, cap = (uint64_t)lc.n_cus * 16;
  CG_LAUNCH(lc, (splitk_reduce_kernel), (unsigned)(blocks < cap ? (blocks ? blocks : 1) : cap), 256, ws, c, n, splits, cadd);
  return hipGetLastError();
}

// Split-K factor for a problem too small to fill the CUs with 128x128 tiles (0/1 = none).
// The caller provides g.workspace of splits * batch * M * N floats and sets g.splits/k_per_split.
uint32_t gemm_split_k(const LaunchCtx &lc, const GemmDesc &g) {
  const uint32_t batch = g.nb0 * g.nb1;
  const int asz = g.a_stype == ST_BF16 ? 2 : 4, bsz = g.b_stype == ST_BF16 ? 2 : 4;
  const int av = vec_ok(g.a, asz, g.sak == 1 ? g.sam : g.sak, g.sa_b0, g.sa_b1);
  const int bv = vec_ok(g.b, bsz, g.sbk == 1 ? g.sbn : g.sbk, g.sb_b0, g.sb_b1);
  const uint64_t tiles = (uint64_t)((g.M + 127) / 128) * ((g.N + 127) / 128) * batch;
  uint32_t splits = 1;
  if (gemv_rows_plain_ok(lc, g)) return 1;
  if (gemm_small_ok(lc, g)) {
    // deep and tiny: more workgroups along k while each wavefront keeps two 32-wide chunks
    const uint64_t t32 = (uint64_t)((g.M + 31) / 32) * ((g.N + 31) / 32) * batch;
    while (t32 * splits * 2 <= (uint64_t)lc.n_cus && g.K / (splits * 2) >= 256 && splits < 64) splits *= 2;
    return splits;
  }
  if (!gemm_fast_path(g, av, bv)) {
    // the generic kernel (f32 products): same idea, shorter k-steps, so thinner slices still pay
    if (g.M <= 8 || g.b_index || !g.K) return 1;
    while (tiles * splits * 2 <= (uint64_t)lc.n_cus && g.K / (splits * 2) >= 256 && splits < 16) splits *= 2;
    return splits;
  }
  // (a narrow product - the router of a MoE prefill, 1024 x 60 x 2048: 16 tiles of 64 x 64 walking all of k, 27 us -
  // is split like any other when its slices stay 16-byte aligned for the summing pass)
  if (g.N <= 64 && ((uint64_t)batch * g.M * g.N) % 4) return 1;
  while (tiles * splits * 2 <= (uint64_t)lc.n_cus && g.K / (splits * 2) >= 512 && splits < 8) splits *= 2;
  return splits;
}

hipError_t launch_matmul(const LaunchCtx &lc_in, const GemmDesc &g, const char **kernel_name) {
  const uint32_t batch = g.nb0 * g.nb1;
  if (!batch || !g.M || !g.N) return hipSuccess;
  // A product split along k is two launches (the slices, then their sum): when the launch is timed, the
  // start event goes with the first and the stop event with the second, so the record covers both.
  LaunchCtx lc = lc_in, tail = lc_in;
  if (g.splits > 1 && !g.defer_reduce) {
    lc.ev_stop = nullptr;
    tail.ev_start = nullptr;
  }
  const int asz = g.a_stype == ST_BF16 ? 2 : 4, bsz = g.b_stype == ST_BF16 ? 2 : 4;
  const bool a_unit_k = g.sak == 1 || g.K == 1, b_unit_k = g.sbk == 1 || g.K == 1;
  const bool b_unit_n = g.sbn == 1 || g.N == 1;
  // the stride of an axis of length 1 is never used: it must not spoil the alignment test
  const int av = vec_ok(g.a, asz, a_unit_k ? (g.M == 1 ? 0 : g.sam) : (g.K == 1 ? 0 : g.sak), g.sa_b0, g.sa_b1);
  const int bv = vec_ok(g.b, bsz, b_unit_k ? (g.N == 1 ? 0 : g.sbn) : (g.K == 1 ? 0 : g.sbk),
                        g.b_index ? g.sb_index : g.sb_b0, g.sb_b1);
  // only the one-row kernels follow b_index and c_add (and the k-slice sum of a split GEMM adds c_add)
  const bool one_row = g.M <= 8 && g.a_stype == ST_F32 && g.K > 0 && (b_unit_k || b_unit_n);
  if (g.b_index && !one_row) return hipErrorInvalidValue;
  if (g.c_add && !one_row && g.splits <= 1) return hipErrorInvalidValue;
  if ((g.glu_gate || g.c16 || g.n_group || g.dual_b) && !gemm_epilogue_ok(g)) return hipErrorInvalidValue;
  if (g.rope_s && !gemm_rope_epilogue_ok(lc_in, g)) return hipErrorInvalidValue;

  if (gemv_rows_plain_ok(lc_in, g)) {
    // a few rows against bf16 weights: the matrix-core kernel, without a prologue
    if (kernel_name) *kernel_name = "gemv_rows_bf16";
    GemvProDesc p;
    std::memset(&p, 0, sizeof(p));
    p.m.K = g.K;
    p.m.n_prob = 1;
    p.m.b_stype = g.b_stype;
    p.m.p[0].b = g.b;
    p.m.p[0].c = g.c;
    p.m.p[0].c_add = g.c_add;
    p.m.p[0].sbn = g.sbn;
    p.m.p[0].N = g.N;
    p.pro = PRO_NONE;
    p.a = (const float *)g.a;
    p.rows = g.M;
    p.a_rstride = g.sam;
    return launch_gemv_pro(lc, p);
  }
  if (g.M <= 8 && g.a_stype == ST_F32 && g.K > 0) {
    if (b_unit_k) {
      if (kernel_name) *kernel_name = g.b_stype == ST_BF16 ? "gemv_rowdot_bf16" : "gemv_rowdot_f32";
      const int avx = av && a_unit_k;
      // One row against a matrix of a few MB (o_proj of a decode step): the kernel that stages the row in
      // LDS asks for it before the weights and runs with every load in flight from the start; it beats
      // this one by ~2 us per launch at that size (5.5 -> 3.5 us).  Deep or long matrices stream the same
      // either way and stay here.
      if (g.M == 1 && batch == 1 && !g.b_index && avx && bv && g.K % 8 == 0 && g.K >= 256 && g.K < 4096 &&
          g.N <= 16384 && g.N >= 64) {
        GemvProDesc p;
        std::memset(&p, 0, sizeof(p));
        p.m.K = g.K;
        p.m.n_prob = 1;
        p.m.b_stype = g.b_stype;
        p.m.p[0].b = g.b;
        p.m.p[0].c = g.c;
        p.m.p[0].c_add = g.c_add;
        p.m.p[0].sbn = g.sbn;
        p.m.p[0].N = g.N;
        p.pro = PRO_NONE;
        p.a = (const float *)g.a;
        p.err = g.err;
        p.b_index_limit = 1;
        return launch_gemv_pro(lc, p);
      }
      if (g.M == 1) {
        if (g.b_stype == ST_BF16) launch_rowdot<uint16_t, 1>(lc, g, bv, avx);
        else launch_rowdot<float, 1>(lc, g, bv, avx);
      } else if (g.M <= 4) {
        if (g.b_stype == ST_BF16) launch_rowdot<uint16_t, 4>(lc, g, bv, avx);
        else launch_rowdot<float, 4>(lc, g, bv, avx);
      } else {
        if (g.b_stype == ST_BF16) launch_rowdot<uint16_t, 8>(lc, g, bv, avx);
        else launch_rowdot<float, 8>(lc, g, bv, avx);
      }
      return hipGetLastError();
    }
    if (b_unit_n) {
      if (kernel_name) *kernel_name = g.b_stype == ST_BF16 ? "gemv_col_bf16" : "gemv_col_f32";
      dim3 grid((g.N + 63) / 64, batch);
      if (g.M == 1) {
        // one output row: 64 k-slices per workgroup keep enough loads in flight
        if (g.b_stype == ST_BF16) CG_LAUNCH(lc, (gemv_col_kernel<uint16_t, 1, 64>), grid, 1024, g, bv);
        else CG_LAUNCH(lc, (gemv_col_kernel<float, 1, 64>), grid, 1024, g, bv);
      } else {
        if (g.b_stype == ST_BF16) CG_LAUNCH(lc, (gemv_col_kernel<uint16_t, 8, 16>), grid, 256, g, bv);
        else CG_LAUNCH(lc, (gemv_col_kernel<float, 8, 16>), grid, 256, g, bv);
      }
      return hipGetLastError();
    }
  }

  if (gemm_fast_path(g, av, bv)) {
    if (kernel_name) *kernel_name = "gemm_mfma_bf16";
    const bool bkc = g.sbk == 1;
    const uint32_t splits = g.splits > 1 ? g.splits : 1;
    GemmDesc gg = g;
    gg.splits = splits;
    if (splits == 1) gg.k_per_split = g.K;
    if (gemm_dma_ok(g)) {
      const uint64_t t256 = (uint64_t)((g.M + 255) / 256) * ((g.N + 255) / 256) * batch * splits;
      hipError_t e;
      bool grp256 = true;  // 256-column tiles must not straddle two grouped products
      for (uint32_t p = 0; p < g.n_group; ++p) grp256 = grp256 && g.grp_n[p] % 256 == 0;
      if (g.n_group && (batch != 1 || splits != 1 || g.glu_gate || g.c16)) return hipErrorInvalidValue;
      const uint64_t t128 = (uint64_t)((g.M + 127) / 128) * ((g.N + 127) / 128) * batch * splits;
      const bool deep = t128 < 2 * (uint64_t)lc.n_cus;  // at most one workgroup per CU at a time: four stages
      if (g.dual_b) {  // gate and up stacked: 128 output columns per tile, 256 rows when that still fills the CUs
        if (g.n_group || g.glu_gate || splits != 1) return hipErrorInvalidValue;
        const uint64_t d256 = (uint64_t)((g.M + 255) / 256) * ((g.N + 127) / 128) * batch;
        const uint64_t d128 = (uint64_t)((g.M + 127) / 128) * ((g.N + 127) / 128) * batch;
        if (d256 >= (uint64_t)lc.n_cus) e = launch_gemm_dma<256, 256, 2, 4, true, 2, true>(lc, gg, (uint32_t)d256);
        else e = launch_gemm_dma<128, 256, 2, 4, true, 3, true>(lc, gg, (uint32_t)d128);
      } else if (g.glu_gate || g.c16) {  // the epilogue variant stages a 128 x 128 tile
        if (deep) e = launch_gemm_dma<128, 128, 2, 4, true, 4>(lc, gg, (uint32_t)t128);
        else e = launch_gemm_dma<128, 128, 2, 2, true, 2>(lc, gg, (uint32_t)t128);
      } else if (t256 >= (uint64_t)lc.n_cus && grp256) {
        // 256 x 256 tiles run one to a CU, 128 x 128 two to a CU: when the big tiles leave the last round of
        // workgroups mostly empty (320 tiles on 256 CUs), the small ones fill the machine better
        auto fill = [&](uint64_t tiles, uint64_t slots) { return (double)tiles / (double)((tiles + slots - 1) / slots * slots); };
        // A deep product whose last round of big tiles would leave most CUs idle (Gemma's down_proj,
        // 16384 x 1152 x 6912: 320 tiles): whole rounds over the leading rows, the remaining rows as a product of
        // their own with the tiling that suits them (347 -> 307 us; with K = 1024 the second launch costs what
        // the idle CUs did)
        const uint64_t tiles_n = (g.N + 255) / 256, tiles_m = (g.M + 255) / 256;
        const uint64_t lead_m = t256 / (uint64_t)lc.n_cus * (uint64_t)lc.n_cus / tiles_n;  // tile rows of the whole rounds
        if (!g.n_group && batch == 1 && splits == 1 && g.K >= 2048 && fill(t256, (uint64_t)lc.n_cus) < 0.8 && lead_m >= 1 &&
            lead_m < tiles_m && g.a_stype == ST_BF16) {
          GemmDesc lead = gg, rest = g;
          lead.M = (uint32_t)(lead_m * 256);
          rest.M = g.M - lead.M;
          rest.a = (const uint16_t *)g.a + (int64_t)lead.M * g.sam;
          rest.c = g.c + (uint64_t)lead.M * g.N;
          LaunchCtx first = lc, second = lc_in;
          first.ev_stop = nullptr;
          second.ev_start = nullptr;
          e = launch_gemm_dma<256, 256, 2, 4>(first, lead, (uint32_t)(lead_m * tiles_n));
          if (e != hipSuccess) return e;
          return launch_matmul(second, rest, nullptr);
        }
        if (!g.n_group && fill(t128, 2 * (uint64_t)lc.n_cus) > 1.15 * fill(t256, (uint64_t)lc.n_cus))
          e = launch_gemm_dma<128, 128, 2, 2>(lc, gg, (uint32_t)t128);
        else
          e = launch_gemm_dma<256, 256, 2, 4>(lc, gg, (uint32_t)t256);
      } else if (splits == 1 && t128 * 2 <= (uint64_t)lc.n_cus && g.N >= 128) {
        // too few 128 x 128 tiles for the CUs and no split-K to multiply them: halve the tile
        const uint32_t t64 = (uint32_t)((uint64_t)((g.M + 127) / 128) * ((g.N + 63) / 64) * batch);
        // (heads of 128 columns need the whole head in one tile)
        if (g.rope_s && g.rope_hd > 64) e = launch_gemm_dma<128, 128, 2, 4, false, 4, false, false, true>(lc, gg, (uint32_t)t128);
        else if (g.rope_s) e = launch_gemm_dma<128, 64, 4, 2, false, 4, false, false, true>(lc, gg, t64);
        else e = launch_gemm_dma<128, 64, 4, 2, false, 4>(lc, gg, t64);
      } else if (deep) {
        // more tiles than CUs and an epilogue that takes a while: two workgroups of two stages share a CU, and the
        // epilogue of one runs under the main loop of the other (1024 x 6144 x 2048: 59.7 -> 47.6 us, what the plain
        // grouped product takes; the plain product itself gains nothing from it)
        const bool two = t128 > (uint64_t)lc.n_cus;
        if (g.rope_s && two) e = launch_gemm_dma<128, 128, 2, 4, false, 2, false, false, true>(lc, gg, (uint32_t)t128);
        else if (g.rope_s) e = launch_gemm_dma<128, 128, 2, 4, false, 4, false, false, true>(lc, gg, (uint32_t)t128);
        else e = launch_gemm_dma<128, 128, 2, 4, false, 4>(lc, gg, (uint32_t)t128);
      } else {
        if (g.rope_s) e = launch_gemm_dma<128, 128, 2, 2, false, 2, false, false, true>(lc, gg, (uint32_t)t128);
        else e = launch_gemm_dma<128, 128, 2, 2>(lc, gg, (uint32_t)t128);
      }
      if (e != hipSuccess) return e;
    } else if (gemm_dma_bkm_ok(g)) {
      const uint64_t t256 = (uint64_t)((g.M + 255) / 256) * ((g.N + 255) / 256) * batch * splits;
      const uint64_t t128 = (uint64_t)((g.M + 127) / 128) * ((g.N + 127) / 128) * batch * splits;
      hipError_t e = t256 >= (uint64_t)lc.n_cus ? launch_gemm_dma<256, 256, 2, 4, false, 2, false, true>(lc, gg, (uint32_t)t256)
                                                : launch_gemm_dma<128, 128, 2, 2, false, 2, false, true>(lc, gg, (uint32_t)t128);
      if (e != hipSuccess) return e;
    } else {
    if (g.n_group) return hipErrorInvalidValue;
    const uint64_t big_tiles = (uint64_t)((g.M + 127) / 128) * ((g.N + 127) / 128) * batch * splits;
    if (big_tiles * 2 >= (uint64_t)lc.n_cus && g.N > 64) {
      dim3 gr((g.N + 127) / 128, (g.M + 127) / 128, batch * splits);
      if (bkc) CG_LAUNCH(lc, (gemm_bf16_nt_kernel<128, 128, true>), gr, 256, gg);
      else CG_LAUNCH(lc, (gemm_bf16_nt_kernel<128, 128, false>), gr, 256, gg);
    } else {
      dim3 gr((g.N + 63) / 64, (g.M + 63) / 64, batch * splits);
      if (bkc) CG_LAUNCH(lc, (gemm_bf16_nt_kernel<64, 64, true>), gr, 256, gg);
      else CG_LAUNCH(lc, (gemm_bf16_nt_kernel<64, 64, false>), gr, 256, gg);
    }
    }
    if (splits > 1 && !g.defer_reduce) {
      const uint64_t n = (uint64_t)batch * g.M * g.N;
      uint64_t blocks = (n / 4 + 255) / 256, cap = (uint64_t)lc.n_cus * 16;
      CG_LAUNCH(tail, (splitk_reduce_kernel), (unsigned)(blocks < cap ? (blocks ? blocks : 1) : cap), 256,
                (const float *)g.workspace, g.c, n, splits, g.c_add);
    }
    return hipGetLastError();
  }
  const uint32_t gsplits = g.splits > 1 ? g.splits : 1;
  auto sum_slices = [&]() {
    if (gsplits > 1 && !g.defer_reduce) {
      const uint64_t n = (uint64_t)batch * g.M * g.N;
      uint64_t blocks = (n / 4 + 255) / 256, cap = (uint64_t)lc.n_cus * 16;
      CG_LAUNCH(tail, (splitk_reduce_kernel), (unsigned)(blocks < cap ? (blocks ? blocks : 1) : cap), 256,
                (const float *)g.workspace, g.c, n, gsplits, g.c_add);
    }
  };
  if (gemm_small_ok(lc, g)) {
    if (kernel_name) *kernel_name = "gemm_mfma_f32";
    dim3 gr((g.N + 31) / 32, (g.M + 31) / 32, batch * gsplits);
    const bool akc = a_unit_k, bkc = b_unit_k;
    if (akc && bkc) CG_LAUNCH(lc, (gemm_small_f32_kernel<true, true>), gr, 256, g, av, bv);
    else if (akc) CG_LAUNCH(lc, (gemm_small_f32_kernel<true, false>), gr, 256, g, av, 0);
    else if (bkc) CG_LAUNCH(lc, (gemm_small_f32_kernel<false, true>), gr, 256, g, 0, bv);
    else CG_LAUNCH(lc, (gemm_small_f32_kernel<false, false>), gr, 256, g, 0, 0);
    sum_slices();
    return hipGetLastError();
  }
  dim3 grid((g.N + BN - 1) / BN, (g.M + BM - 1) / BM, batch * gsplits);
  if (g.bf16_math) {
    if (kernel_name) *kernel_name = "gemm_mfma_bf16";
    if (g.a_stype == ST_F32 && g.b_stype == ST_BF16) launch_gemm_layout<float, uint16_t, true>(lc, g, grid, av, bv);
    else if (g.a_stype == ST_F32 && g.b_stype == ST_F32) launch_gemm_layout<float, float, true>(lc, g, grid, av, bv);
    else if (g.a_stype == ST_BF16 && g.b_stype == ST_BF16) launch_gemm_layout<uint16_t, uint16_t, true>(lc, g, grid, av, bv);
    else launch_gemm_layout<uint16_t, float, true>(lc, g, grid, av, bv);
  } else {
    if (kernel_name) *kernel_name = "gemm_mfma_f32";
    if (g.a_stype != ST_F32 || g.b_stype != ST_F32) return hipErrorInvalidValue;
    launch_gemm_layout<float, float, false>(lc, g, grid, av, bv);
  }
  sum_slices();
  return hipGetLastError();
}

}  // namespace cgk
