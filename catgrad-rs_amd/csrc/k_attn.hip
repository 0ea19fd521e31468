// k_attn.hip — attention over many query rows (prefill) in one pass: bf16 MFMA with f32 accumulation,
// and an all-f32 variant for a backend without the bf16 flag.
//
// The op sequence of catgrad-llm/src/models/llama.rs:95-107 (also gemma3.rs:153-186):
//   scores = matmul(q, transpose(k));  scores / sqrt(d);  + mask;  softmax;  matmul(., v)
// materialises [b, h, S, T] twice on the generic path.  Here a workgroup takes 128 (or 64) query rows of one
// (batch, head) and walks the keys 64 at a time with the running maximum / sum of the row
// (online softmax); scores and probabilities only ever exist in registers.
//
// Everything is computed transposed so that a lane owns one query for the whole kernel:
//   S^T[key, query]   = K[key, :] . Q[query, :]       A = K tile (LDS), B = Q rows (registers)
//   O^T[dim, query]  += V^T[dim, key] . P^T[key, query]  A = V^T tile (LDS), B = P^T (registers)
// In the 32x32 MFMA result layout a lane holds column (lane & 31) = its query, so the row
// statistics are in-lane reductions plus one exchange with lane ^ 32, the rescaling of O by
// exp(m_old - m_new) is a per-lane scalar, and P^T feeds the second product straight from the
// registers of the first: the key order inside each 16-key block is permuted the same way for
// both operands (a lane's eight values are keys {4h..4h+3, 8+4h..8+4h+3}, h = lane >> 5), which
// the V^T fragment mirrors with two 8-byte LDS reads.
#include <hip/hip_runtime.h>
#include <math.h>
#include "launch.hpp"
#include "dev_common.hpp"

namespace cgk {

typedef __attribute__((ext_vector_type(8))) __bf16 a_bf16x8;
typedef __attribute__((ext_vector_type(16))) float a_f32x16;

typedef __attribute__((ext_vector_type(2))) __bf16 a_bf16x2;
typedef __attribute__((ext_vector_type(2))) float a_f32x2;

// eight floats -> eight bf16 (round to nearest even: v_cvt_pk_bf16_f32, one instruction per pair)
__device__ __forceinline__ a_bf16x8 pack8(const float *v) {
  union {
    a_bf16x2 h2[4];
    a_bf16x8 h;
  } r;
#pragma unroll
  for (int i = 0; i < 4; ++i) r.h2[i] = __builtin_convertvector((a_f32x2){v[2 * i], v[2 * i + 1]}, a_bf16x2);
  return r.h;
}

// The classes of one query tile's key tiles (AttnPrefillDesc::tile_class), as the kernels walk them.  A row
// of up to 64 entries is read once, by the lanes of a wave, and kept as two bit masks: finding the next
// live tile is then bit arithmetic, not a chain of dependent loads.
template <int BN>
struct KeyTiles {
  const uint8_t *cls;  // null: no table, every tile is visited and reads its mask values
  uint32_t cols, t;
  uint64_t live, zero;  // bit i: tile i is not dead / needs no mask values
  bool bits;
  __device__ __forceinline__ KeyTiles(const AttnPrefillDesc &a, uint32_t q_tile, int lane) {
    cls = a.tile_class ? a.tile_class + (size_t)q_tile * a.tile_cols : nullptr;
    cols = a.tile_cols;
    t = a.t;
    bits = cls && cols <= 64;
    live = zero = 0;
    if (bits) {
      const uint8_t c = (uint32_t)lane < cols ? cls[lane] : 0;
      live = __ballot(c != 0);
      zero = __ballot(c == 2);
    }
  }
  // the first step at or after t0 that is not dead (>= t: none)
  __device__ __forceinline__ uint32_t next_step(uint32_t t0) const {
    if (!cls) return t0;
    uint32_t i = t0 / BN;
    if (bits) {
      const uint64_t m = i < 64 ? live >> i : 0;
      return m ? (i + (uint32_t)__builtin_ctzll(m)) * (uint32_t)BN : cols * (uint32_t)BN;
    }
    while (i < cols && cls[i] == 0) ++i;
    return i * (uint32_t)BN;
  }
  // does the step at t0 read mask values (given that there is a mask)?
  __device__ __forceinline__ bool reads_mask(uint32_t t0) const {
    if (!cls || t0 >= t) return true;
    return bits ? !((zero >> (t0 / BN)) & 1) : cls[t0 / BN] != 2;
  }
};

constexpr float ATTN_MAX_SLACK = 8.0f;

// BN keys per step; the K / V rows and the mask values of step i+1 are fetched into registers while
// step i is being computed, so global latency is paid once per workgroup, not once per step.
// NW waves of 32 queries each per workgroup (4, or 2 when that is what it takes to occupy the CUs).
template <int D, int BN, int NW>
__global__ void __launch_bounds__(NW * 64) attn_prefill_kernel(AttnPrefillDesc a) {
  constexpr int NT = NW * 64;
  constexpr int KP = D + 8;              // K tile row pitch (bf16 elements)
  constexpr int VP = BN + 8;             // V^T tile row pitch
  constexpr int DT = D / 32;             // 32-row tiles of O^T
  constexpr int KT = BN / 32;            // 32-key tiles of S^T
  constexpr int KCH = BN * D / 8 / NT;   // 16-byte chunks of the K tile / of the V^T tile per thread
  __shared__ __attribute__((aligned(16))) uint16_t Ks[BN * KP];
  __shared__ __attribute__((aligned(16))) uint16_t Vt[D * VP];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 31, half = lane >> 5;
  const uint32_t h = blockIdx.y, b = blockIdx.z;
  const uint32_t kvh = h / a.rep, rp = h % a.rep;
  const uint32_t query = blockIdx.x * (NW * 32) + wave * 32 + col;
  const bool q_ok = query < a.s;
  const uint32_t qc = q_ok ? query : a.s - 1;  // loads of lanes past the end go to a valid row
  const float *Q = a.q + (int64_t)b * a.q_sb + (int64_t)h * a.q_sh + (int64_t)qc * a.q_ss;
  // K rows as bf16 (the twin of the rotated keys), V as bf16 V^T [b, kv, d, T]: both were narrowed
  // once, not once per query block
  const uint16_t *K = a.k16 + (int64_t)b * a.k_sb + (int64_t)kvh * a.k_skv + (int64_t)rp * a.k_srep;
  const uint16_t *VT = a.vt16 + ((int64_t)b * (a.heads / a.rep) + kvh) * D * (int64_t)a.t;
  const float *V = a.v + (int64_t)b * a.v_sb + (int64_t)kvh * a.v_skv + (int64_t)rp * a.v_srep;
  const float *M = a.mask ? a.mask + (int64_t)b * a.m_sb + (int64_t)h * a.m_sh + (int64_t)qc * a.m_ss : nullptr;

  // this lane's query row as B fragments: k-step ks covers dims 16 ks .. 16 ks + 15, half h takes 8
  a_bf16x8 qf[D / 16];
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) {
    float v[8];
    if (q_ok) {
      const float4 x0 = *(const float4 *)(Q + ks * 16 + half * 8), x1 = *(const float4 *)(Q + ks * 16 + half * 8 + 4);
      v[0] = x0.x; v[1] = x0.y; v[2] = x0.z; v[3] = x0.w; v[4] = x1.x; v[5] = x1.y; v[6] = x1.z; v[7] = x1.w;
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = 0.f;
    }
    qf[ks] = pack8(v);
  }
  a_f32x16 o[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[t][e] = 0.f;
  float m_run = -3.40282347e+38f, l_run = 0.f;
  const float inv_scale = a.has_scale ? 1.0f / a.scale : 1.0f;  // bf16 mode: a product, not the reference's quotient

  // registers of the step in flight
  uint4 kreg[KCH], vreg[KCH];
  float4 mreg[KT][4];
  // All loads are unconditional (indices clamped into range) so that they are issued back to back;
  // chunks past the end are zeroed when the registers are consumed.
  // With a class table, dead key tiles are never visited and all-zero ones need no mask values.
  const KeyTiles<BN> tiles(a, blockIdx.x, lane);
  auto next_step = [&](uint32_t t0) { return tiles.next_step(t0); };
  auto step_mask = [&](uint32_t t0) { return M && tiles.reads_mask(t0); };
  auto fetch = [&](uint32_t t0) {
#pragma unroll
    for (int c = 0; c < KCH; ++c) {
      const int ch = tid + c * NT, key = ch / (D / 8), d8 = (ch % (D / 8)) * 8;
      kreg[c] = *(const uint4 *)(K + (int64_t)min(t0 + key, a.t - 1) * a.k_st + d8);
    }
#pragma unroll
    for (int c = 0; c < KCH; ++c) {
      const int ch = tid + c * NT, dim = ch / (BN / 8), k8 = (ch % (BN / 8)) * 8;
      vreg[c] = *(const uint4 *)(VT + (int64_t)dim * a.t + min(t0 + k8, a.t - 8));
    }
    if (step_mask(t0)) {  // mask rows allow 16-byte loads and T % 8 == 0 (checked by the host)
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          mreg[kt][j] = *(const float4 *)(M + min(t0 + kt * 32 + j * 8 + half * 4, a.t - 4));
    }
  };
  uint32_t t0 = next_step(0);
  if (t0 < a.t) fetch(t0);
  for (; t0 < a.t;) {
    const uint32_t t_next = next_step(t0 + BN);
    const bool use_mask = step_mask(t0);  // uniform
    // ---- is any (query, key) pair of this step unmasked?  A causal or sliding-window mask kills
    // most steps; a dead step only adds terms that the first live step rescales to zero.
    const bool tail = t0 + BN > a.t;  // the only step with keys past the end (uniform)
    bool live_pair = !use_mask;
    float4 mcur[KT][4];
    if (use_mask) {
      float mmax = -3.40282347e+38f;
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          mcur[kt][j] = mreg[kt][j];
          float4 mk = mcur[kt][j];
          if (tail) {
            const uint32_t key = t0 + kt * 32 + j * 8 + half * 4;
            if (key >= a.t) mk.x = -3.40282347e+38f;
            if (key + 1 >= a.t) mk.y = -3.40282347e+38f;
            if (key + 2 >= a.t) mk.z = -3.40282347e+38f;
            if (key + 3 >= a.t) mk.w = -3.40282347e+38f;
          }
          mmax = fmaxf(mmax, fmaxf(fmaxf(mk.x, mk.y), fmaxf(mk.z, mk.w)));
        }
      live_pair = q_ok && mmax > -3.0e38f;
    }
    const bool live = __syncthreads_or(live_pair);  // also: the previous step's fragments have been read
    if (live) {
      // ---- registers -> LDS: K [BN, D] and V^T [D, BN]
#pragma unroll
      for (int c = 0; c < KCH; ++c) {
        const int ch = tid + c * NT, key = ch / (D / 8), d8 = (ch % (D / 8)) * 8;
        *(uint4 *)(&Ks[key * KP + d8]) = (t0 + key < a.t) ? kreg[c] : make_uint4(0u, 0u, 0u, 0u);
      }
#pragma unroll
      for (int c = 0; c < KCH; ++c) {
        const int ch = tid + c * NT, dim = ch / (BN / 8), k8 = (ch % (BN / 8)) * 8;
        *(uint4 *)(&Vt[dim * VP + k8]) = (t0 + k8 < a.t) ? vreg[c] : make_uint4(0u, 0u, 0u, 0u);
      }
    }
    __syncthreads();
    if (t_next < a.t) fetch(t_next);  // in flight during the arithmetic below
    const uint32_t t_cur = t0;
    t0 = t_next;
    if (!live) continue;
    // ---- S^T = K . Q^T
    a_f32x16 st[KT];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
      for (int e = 0; e < 16; ++e) st[kt][e] = 0.f;
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) {
        const a_bf16x8 kf = *(const a_bf16x8 *)(&Ks[(kt * 32 + col) * KP + ks * 16 + half * 8]);
        st[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[ks], st[kt], 0, 0, 0);
      }
    }
    // ---- scale, mask, running maximum.  Register e of tile kt is key t0 + kt*32 + (e>>2)*8 + half*4 + (e&3)
    float tmax = -3.40282347e+38f;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t key = t_cur + kt * 32 + j * 8 + half * 4;
        float mv[4] = {0.f, 0.f, 0.f, 0.f};
        if (use_mask) { mv[0] = mcur[kt][j].x; mv[1] = mcur[kt][j].y; mv[2] = mcur[kt][j].z; mv[3] = mcur[kt][j].w; }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float s = st[kt][j * 4 + i];
          if (a.has_scale) s = s * inv_scale;
          if (use_mask) s = s + mv[i];
          else if (!M && a.has_mask_const) s = s + a.mask_const;
          if (tail && key + i >= a.t) s = -3.40282347e+38f;  // past the end: contributes exp(..) = 0
          st[kt][j * 4 + i] = s;
          tmax = fmaxf(tmax, s);
        }
      }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    // The reference point of the exponentials only follows the maximum when that has moved by more than
    // ATTN_MAX_SLACK: the quotient O / l at the end does not depend on it, weights of up to e^slack are as
    // exact in f32 and bf16 as weights of up to 1, and O is rescaled on a few steps instead of on most.
    const float m_new = tmax > m_run + ATTN_MAX_SLACK ? tmax : m_run;
    const float alpha = __expf(m_run - m_new);
    float psum = 0.f;
    a_bf16x8 pf[KT * 2];  // P^T as B fragments of the 16-key blocks
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int blk = 0; blk < 2; ++blk) {
        float p[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const uint32_t key = t_cur + kt * 32 + (blk * 2 + (i >> 2)) * 8 + half * 4 + (i & 3);
          p[i] = __expf(st[kt][blk * 8 + i] - m_new);
          if (tail && key >= a.t) p[i] = 0.f;
          psum += p[i];
        }
        pf[kt * 2 + blk] = pack8(p);
      }
    psum += __shfl_xor(psum, 32, 64);
    l_run = l_run * alpha + psum;
    m_run = m_new;
    // ---- O^T = O^T * alpha + V^T . P^T
    if (__any(alpha != 1.0f)) {  // the running maximum moved for some query of this wave
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[t][e] *= alpha;
    }
#pragma unroll
    for (int t = 0; t < DT; ++t) {
#pragma unroll
      for (int blk = 0; blk < KT * 2; ++blk) {
        // A fragment: row = dim t*32 + col, the lane's eight keys of this block in the permuted order
        const uint16_t *vr = &Vt[(t * 32 + col) * VP + blk * 16 + half * 4];
        union {
          uint2 u[2];
          a_bf16x8 hv;
        } vf;
        vf.u[0] = *(const uint2 *)vr;
        vf.u[1] = *(const uint2 *)(vr + 8);
        o[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf.hv, pf[blk], o[t], 0, 0, 0);
      }
    }
  }
  // A row whose every key is masked has all scores equal to f32::MIN on the reference path:
  // uniform weights, i.e. the mean of V.  Dead steps were skipped above, so rebuild that here.
  if (M && q_ok && m_run <= -3.0e38f) {
    l_run = (float)a.t;
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int e = 0; e < 16; ++e) o[t][e] = 0.f;
    for (uint32_t key = 0; key < a.t; ++key)
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float4 vv = *(const float4 *)(V + (int64_t)key * a.v_st + t * 32 + j * 8 + half * 4);
          o[t][j * 4 + 0] += vv.x; o[t][j * 4 + 1] += vv.y; o[t][j * 4 + 2] += vv.z; o[t][j * 4 + 3] += vv.w;
        }
  }
  // ---- normalise and store: O^T register e of tile t is dim t*32 + (e>>2)*8 + half*4 + (e&3)
  if (q_ok) {
    const int64_t o_off = (int64_t)b * a.o_sb + (int64_t)h * a.o_sh + (int64_t)query * a.o_ss;
    float *out = a.out + o_off;
    uint16_t *out16 = a.out16 ? a.out16 + o_off : nullptr;
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float4 r;
        r.x = o[t][j * 4 + 0] / l_run; r.y = o[t][j * 4 + 1] / l_run;
        r.z = o[t][j * 4 + 2] / l_run; r.w = o[t][j * 4 + 3] / l_run;
        const int dim = t * 32 + j * 8 + half * 4;
        *(float4 *)(out + dim) = r;
        if (out16) *(uint2 *)(out16 + dim) = bf16_pack4(r);
      }
  }
}

// Few query rows (a 512-token prompt: 256 workgroups of 64 queries, one per CU, each walking up to eight
// key tiles one memory round trip at a time): the keys are divided instead.  The NW waves of a workgroup
// all own the same 32 queries; wave w takes every NW-th live key tile into an LDS region of its own, so
// the main loop needs no workgroup barrier and the waves' memory waits overlap each other's arithmetic.
// Each wave ends with its own running maximum, sum and O^T; they meet once, in LDS, and wave 0 merges
// them (the same rescaling as between two steps of one wave).
template <int D, int BN, int NW>
__global__ void __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(2, 2)))  // two workgroups per CU
attn_prefill_keysplit_kernel(AttnPrefillDesc a) {
  constexpr int KP = D + 8;
  constexpr int VP = BN + 8;
  constexpr int DT = D / 32;
  constexpr int KT = BN / 32;
  constexpr int KCH = BN * D / 8 / 64;   // 16-byte chunks of the K tile / of the V^T tile per lane
  constexpr int REGION = BN * KP + D * VP;  // bf16 elements of one wave's tiles
  static_assert(REGION * 2 >= (DT * 16 + 2) * 64 * 4, "a wave's partial result must fit in its tile region");
  __shared__ __attribute__((aligned(16))) uint16_t lds[NW * REGION];
  __shared__ __attribute__((aligned(16))) uint16_t qs[32 * (D + 8)];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 31, half = lane >> 5;
  uint16_t *Ks = lds + wave * REGION, *Vt = Ks + BN * KP;
  const uint32_t h = blockIdx.y, b = blockIdx.z;
  const uint32_t kvh = h / a.rep, rp = h % a.rep;
  const uint32_t query = blockIdx.x * 32 + col;
  const bool q_ok = query < a.s;
  const uint32_t qc = q_ok ? query : a.s - 1;
  const uint16_t *K = a.k16 + (int64_t)b * a.k_sb + (int64_t)kvh * a.k_skv + (int64_t)rp * a.k_srep;
  const uint16_t *VT = a.vt16 + ((int64_t)b * (a.heads / a.rep) + kvh) * D * (int64_t)a.t;
  const float *V = a.v + (int64_t)b * a.v_sb + (int64_t)kvh * a.v_skv + (int64_t)rp * a.v_srep;
  const float *M = a.mask ? a.mask + (int64_t)b * a.m_sb + (int64_t)h * a.m_sh + (int64_t)qc * a.m_ss : nullptr;

  const KeyTiles<BN> tiles(a, blockIdx.x, lane);
  auto skip_steps = [&](uint32_t t0, int n) {  // the n-th live step after the one at t0
    for (int i = 0; i < n && t0 < a.t; ++i) t0 = tiles.next_step(t0 + BN);
    return t0;
  };
  auto step_mask = [&](uint32_t t0) { return M && tiles.reads_mask(t0); };
  uint4 kreg[KCH], vreg[KCH];
  auto fetch = [&](uint32_t t0) {
#pragma unroll
    for (int c = 0; c < KCH; ++c) {
      const int ch = lane + c * 64, key = ch / (D / 8), d8 = (ch % (D / 8)) * 8;
      kreg[c] = *(const uint4 *)(K + (int64_t)min(t0 + key, a.t - 1) * a.k_st + d8);
    }
#pragma unroll
    for (int c = 0; c < KCH; ++c) {
      const int ch = lane + c * 64, dim = ch / (BN / 8), k8 = (ch % (BN / 8)) * 8;
      vreg[c] = *(const uint4 *)(VT + (int64_t)dim * a.t + min(t0 + k8, a.t - 8));
    }
  };
  uint32_t t0 = skip_steps(tiles.next_step(0), wave);
  if (t0 < a.t) fetch(t0);  // asked for before the queries: one round trip for both

  // The queries: each wave converts a quarter of the workgroup's 32 rows (16 bytes of bf16 per lane and
  // piece), the rows meet in LDS, and every wave reads its B fragments from there - a quarter of the loads
  // of every wave fetching every row.
  constexpr int QP = D + 8;  // row pitch (bf16 elements)
  {
    const float *Q0 = a.q + (int64_t)b * a.q_sb + (int64_t)h * a.q_sh;
#pragma unroll
    for (int c = 0; c < 32 * D / 8 / (NW * 64); ++c) {
      const int ch = tid + c * NW * 64, r = ch / (D / 8), d8 = (ch % (D / 8)) * 8;
      const uint32_t row = blockIdx.x * 32 + r;
      float v[8];
      if (row < a.s) {
        const float *qr = Q0 + (int64_t)row * a.q_ss + d8;
        const float4 x0 = *(const float4 *)qr, x1 = *(const float4 *)(qr + 4);
        v[0] = x0.x; v[1] = x0.y; v[2] = x0.z; v[3] = x0.w; v[4] = x1.x; v[5] = x1.y; v[6] = x1.z; v[7] = x1.w;
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = 0.f;
      }
      *(a_bf16x8 *)(&qs[r * QP + d8]) = pack8(v);
    }
  }
  __syncthreads();
  a_bf16x8 qf[D / 16];
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) qf[ks] = *(const a_bf16x8 *)(&qs[col * QP + ks * 16 + half * 8]);
  a_f32x16 o[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[t][e] = 0.f;
  float m_run = -3.40282347e+38f, l_run = 0.f;
  const float inv_scale = a.has_scale ? 1.0f / a.scale : 1.0f;

  while (t0 < a.t) {
    const uint32_t t_next = skip_steps(t0, NW);
    const bool use_mask = step_mask(t0);  // uniform over the wave
    const bool tail = t0 + BN > a.t;
    const uint32_t t_cur = t0;
    t0 = t_next;
    // The mask values of this step are asked for here and used after the score product.  (A step whose
    // every pair is masked - possible only without a class table - needs no special case: its terms
    // carry the weight exp(f32::MIN - m), which is zero once any live key has been seen, and a row
    // that never sees one is rebuilt at the end.)
    float4 mcur[KT][4];
    if (use_mask) {
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          mcur[kt][j] = *(const float4 *)(M + min(t_cur + kt * 32 + j * 8 + half * 4, a.t - 4));
    }
    // registers -> this wave's LDS region.  Its LDS instructions run in program order, so the fragment
    // reads of the previous step are behind these writes and the reads below are ahead of them; the
    // fences keep the compiler from reordering across them.
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
#pragma unroll
    for (int c = 0; c < KCH; ++c) {
      const int ch = lane + c * 64, key = ch / (D / 8), d8 = (ch % (D / 8)) * 8;
      *(uint4 *)(&Ks[key * KP + d8]) = (t_cur + key < a.t) ? kreg[c] : make_uint4(0u, 0u, 0u, 0u);
    }
#pragma unroll
    for (int c = 0; c < KCH; ++c) {
      const int ch = lane + c * 64, dim = ch / (BN / 8), k8 = (ch % (BN / 8)) * 8;
      *(uint4 *)(&Vt[dim * VP + k8]) = (t_cur + k8 < a.t) ? vreg[c] : make_uint4(0u, 0u, 0u, 0u);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    if (t_next < a.t) fetch(t_next);  // in flight during the arithmetic below
    a_f32x16 st[KT];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
      for (int e = 0; e < 16; ++e) st[kt][e] = 0.f;
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) {
        const a_bf16x8 kf = *(const a_bf16x8 *)(&Ks[(kt * 32 + col) * KP + ks * 16 + half * 8]);
        st[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[ks], st[kt], 0, 0, 0);
      }
    }
    float tmax = -3.40282347e+38f;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t key = t_cur + kt * 32 + j * 8 + half * 4;
        float mv[4] = {0.f, 0.f, 0.f, 0.f};
        if (use_mask) { mv[0] = mcur[kt][j].x; mv[1] = mcur[kt][j].y; mv[2] = mcur[kt][j].z; mv[3] = mcur[kt][j].w; }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float s = st[kt][j * 4 + i];
          if (a.has_scale) s = s * inv_scale;
          if (use_mask) s = s + mv[i];
          else if (!M && a.has_mask_const) s = s + a.mask_const;
          if (tail && key + i >= a.t) s = -3.40282347e+38f;
          st[kt][j * 4 + i] = s;
          tmax = fmaxf(tmax, s);
        }
      }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    // The reference point of the exponentials only follows the maximum when that has moved by more than
    // ATTN_MAX_SLACK: the quotient O / l at the end does not depend on it, weights of up to e^slack are as
    // exact in f32 and bf16 as weights of up to 1, and O is rescaled on a few steps instead of on most.
    const float m_new = tmax > m_run + ATTN_MAX_SLACK ? tmax : m_run;
    const float alpha = __expf(m_run - m_new);
    float psum = 0.f;
    a_bf16x8 pf[KT * 2];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int blk = 0; blk < 2; ++blk) {
        float p[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const uint32_t key = t_cur + kt * 32 + (blk * 2 + (i >> 2)) * 8 + half * 4 + (i & 3);
          p[i] = __expf(st[kt][blk * 8 + i] - m_new);
          if (tail && key >= a.t) p[i] = 0.f;
          psum += p[i];
        }
        pf[kt * 2 + blk] = pack8(p);
      }
    psum += __shfl_xor(psum, 32, 64);
    l_run = l_run * alpha + psum;
    m_run = m_new;
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[t][e] *= alpha;
    }
#pragma unroll
    for (int t = 0; t < DT; ++t) {
#pragma unroll
      for (int blk = 0; blk < KT * 2; ++blk) {
        const uint16_t *vr = &Vt[(t * 32 + col) * VP + blk * 16 + half * 4];
        union {
          uint2 u[2];
          a_bf16x8 hv;
        } vf;
        vf.u[0] = *(const uint2 *)vr;
        vf.u[1] = *(const uint2 *)(vr + 8);
        o[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf.hv, pf[blk], o[t], 0, 0, 0);
      }
    }
  }
  // ---- the waves' partial results meet: [register][lane] floats in each wave's own region
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  float *mine = (float *)(lds + wave * REGION);
  if (wave) {
    mine[lane] = m_run;
    mine[64 + lane] = l_run;
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int e = 0; e < 16; ++e) mine[(2 + t * 16 + e) * 64 + lane] = o[t][e];
  }
  __syncthreads();
  if (wave) return;
#pragma unroll 1
  for (int w = 1; w < NW; ++w) {
    const float *other = (const float *)(lds + w * REGION);
    const float m_w = other[lane], l_w = other[64 + lane];
    const float m_new = fmaxf(m_run, m_w);
    const float f0 = __expf(m_run - m_new), f1 = __expf(m_w - m_new);
    l_run = l_run * f0 + l_w * f1;
    m_run = m_new;
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int e = 0; e < 16; ++e) o[t][e] = o[t][e] * f0 + other[(2 + t * 16 + e) * 64 + lane] * f1;
  }
  if (M && q_ok && m_run <= -3.0e38f) {  // every key masked: uniform weights, as on the reference path
    l_run = (float)a.t;
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int e = 0; e < 16; ++e) o[t][e] = 0.f;
    for (uint32_t key = 0; key < a.t; ++key)
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float4 vv = *(const float4 *)(V + (int64_t)key * a.v_st + t * 32 + j * 8 + half * 4);
          o[t][j * 4 + 0] += vv.x; o[t][j * 4 + 1] += vv.y; o[t][j * 4 + 2] += vv.z; o[t][j * 4 + 3] += vv.w;
        }
  }
  if (q_ok) {
    const int64_t o_off = (int64_t)b * a.o_sb + (int64_t)h * a.o_sh + (int64_t)query * a.o_ss;
    float *out = a.out + o_off;
    uint16_t *out16 = a.out16 ? a.out16 + o_off : nullptr;
    const float inv_l = 1.0f / l_run;  // bf16 products: a reciprocal and a product, not 64 quotients
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float4 r;
        r.x = o[t][j * 4 + 0] * inv_l; r.y = o[t][j * 4 + 1] * inv_l;
        r.z = o[t][j * 4 + 2] * inv_l; r.w = o[t][j * 4 + 3] * inv_l;
        const int dim = t * 32 + j * 8 + half * 4;
        *(float4 *)(out + dim) = r;
        if (out16) *(uint2 *)(out16 + dim) = bf16_pack4(r);
      }
  }
}

// The same pass with every product in f32 (v_mfma_f32_32x32x2_f32), for a backend without the bf16 flag:
// the results stay within the f32 bar of the reference's three-step sequence, and the [b, h, S, T]
// scores are still never written.  One MFMA consumes two values of the reduction axis, one per lane
// half, so
//   S^T: A = K[key kt*32 + col][dim 2 ks + half] (LDS, row pitch D + 2: 64 lanes, 64 banks),
//        B = the lane's query, dim 2 ks + half (registers);
//   O^T: B = register i of the lane's probabilities, which is key (i>>2)*8 + half*4 + (i&3) of the tile,
//        A = V[that key][dim t*32 + col] (LDS, rows as they lie in memory: no transpose).
// K and V take turns in one LDS tile: the V rows of a step are fetched while its scores are computed,
// the K rows of the next step while the V product runs.
// QLDS: the queries of the workgroup stay in LDS instead of registers (a 256-wide head would need 128
// registers per lane for them, on top of 128 for O^T).
template <bool QLDS, int D, int BN, int NW>
__global__ void __launch_bounds__(NW * 64) attn_prefill_f32_kernel(AttnPrefillDesc a) {
  constexpr int NT = NW * 64;
  constexpr int KP = D + 2;              // K tile row pitch (floats)
  constexpr int VP = D + 8;              // V tile row pitch
  constexpr int DT = D / 32;
  constexpr int KT = BN / 32;
  constexpr int CH = BN * D / 4 / NT;    // 16-byte chunks of a tile per thread
  constexpr bool AHEAD = !QLDS;          // fetch the next tile during the arithmetic (costs CH x 4 registers throughout)
  __shared__ __attribute__((aligned(16))) float tile[BN * VP];
  __shared__ __attribute__((aligned(16))) float qs[QLDS ? NW * 32 * KP : 2];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 31, half = lane >> 5;
  const uint32_t h = blockIdx.y, b = blockIdx.z;
  const uint32_t kvh = h / a.rep, rp = h % a.rep;
  const uint32_t query = blockIdx.x * (NW * 32) + wave * 32 + col;
  const bool q_ok = query < a.s;
  const uint32_t qc = q_ok ? query : a.s - 1;
  const float *Q = a.q + (int64_t)b * a.q_sb + (int64_t)h * a.q_sh + (int64_t)qc * a.q_ss;
  const float *K = a.k + (int64_t)b * a.k_sb + (int64_t)kvh * a.k_skv + (int64_t)rp * a.k_srep;
  const float *V = a.v + (int64_t)b * a.v_sb + (int64_t)kvh * a.v_skv + (int64_t)rp * a.v_srep;
  const float *M = a.mask ? a.mask + (int64_t)b * a.m_sb + (int64_t)h * a.m_sh + (int64_t)qc * a.m_ss : nullptr;

  float qf[QLDS ? 1 : D / 2];
  if constexpr (QLDS) {  // the workgroup's rows, zero past the end; first read after the loop's first barrier
    const float *Q0 = a.q + (int64_t)b * a.q_sb + (int64_t)h * a.q_sh;
#pragma unroll
    for (int c = 0; c < NW * 32 * D / 4 / NT; ++c) {
      const int ch = tid + c * NT, r = ch / (D / 4), d4 = (ch % (D / 4)) * 4;
      const uint32_t row = blockIdx.x * (NW * 32) + r;
      float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
      if (row < a.s) x = *(const float4 *)(Q0 + (int64_t)row * a.q_ss + d4);
      *(float2 *)(&qs[r * KP + d4]) = make_float2(x.x, x.y);
      *(float2 *)(&qs[r * KP + d4 + 2]) = make_float2(x.z, x.w);
    }
  } else {
#pragma unroll
    for (int c = 0; c < D / 4; ++c) {  // dims 4c .. 4c+3: k-steps 2c (x, y) and 2c+1 (z, w)
      float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
      if (q_ok) x = *(const float4 *)(Q + c * 4);
      qf[2 * c] = half ? x.y : x.x;
      qf[2 * c + 1] = half ? x.w : x.z;
    }
  }
  a_f32x16 o[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[t][e] = 0.f;
  float m_run = -3.40282347e+38f, l_run = 0.f;

  float4 treg[CH];
  float4 mreg[KT][4];
  const KeyTiles<BN> tiles(a, blockIdx.x, lane);
  auto next_step = [&](uint32_t t0) { return tiles.next_step(t0); };
  auto step_mask = [&](uint32_t t0) { return M && tiles.reads_mask(t0); };
  // rows of K (or V) of the step at t0 into registers; rows past the end repeat the last one and are
  // zeroed when they are written to LDS
  auto fetch_rows = [&](const float *base, int64_t row_stride, uint32_t t0) {
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int ch = tid + c * NT, key = ch / (D / 4), d4 = (ch % (D / 4)) * 4;
      treg[c] = *(const float4 *)(base + (int64_t)min(t0 + key, a.t - 1) * row_stride + d4);
    }
  };
  auto fetch_mask = [&](uint32_t t0) {
    if (step_mask(t0)) {
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          mreg[kt][j] = *(const float4 *)(M + min(t0 + kt * 32 + j * 8 + half * 4, a.t - 4));
    }
  };
  uint32_t t0 = next_step(0);
  if (t0 < a.t) {
    if (AHEAD) fetch_rows(K, a.k_st, t0);
    fetch_mask(t0);
  }
  for (; t0 < a.t;) {
    const uint32_t t_next = next_step(t0 + BN);
    const bool use_mask = step_mask(t0);
    const bool tail = t0 + BN > a.t;
    bool live_pair = !use_mask;
    float4 mcur[KT][4];
    if (use_mask) {
      float mmax = -3.40282347e+38f;
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          mcur[kt][j] = mreg[kt][j];
          float4 mk = mcur[kt][j];
          if (tail) {
            const uint32_t key = t0 + kt * 32 + j * 8 + half * 4;
            if (key >= a.t) mk.x = -3.40282347e+38f;
            if (key + 1 >= a.t) mk.y = -3.40282347e+38f;
            if (key + 2 >= a.t) mk.z = -3.40282347e+38f;
            if (key + 3 >= a.t) mk.w = -3.40282347e+38f;
          }
          mmax = fmaxf(mmax, fmaxf(fmaxf(mk.x, mk.y), fmaxf(mk.z, mk.w)));
        }
      live_pair = q_ok && mmax > -3.0e38f;
    }
    const bool live = __syncthreads_or(live_pair);  // also: the V rows of the previous step have been read
    const uint32_t t_cur = t0;
    t0 = t_next;
    if (!live) {  // uniform
      if (t_next < a.t) {
        if (AHEAD) fetch_rows(K, a.k_st, t_next);
        fetch_mask(t_next);
      }
      continue;
    }
    if (!AHEAD) fetch_rows(K, a.k_st, t_cur);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int ch = tid + c * NT, key = ch / (D / 4), d4 = (ch % (D / 4)) * 4;
      const float4 x = (t_cur + key < a.t) ? treg[c] : make_float4(0.f, 0.f, 0.f, 0.f);
      *(float2 *)(&tile[key * KP + d4]) = make_float2(x.x, x.y);
      *(float2 *)(&tile[key * KP + d4 + 2]) = make_float2(x.z, x.w);
    }
    __syncthreads();
    if (AHEAD) fetch_rows(V, a.v_st, t_cur);  // in flight during the score product
    // ---- S^T = K . Q^T
    a_f32x16 st[KT];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
      for (int e = 0; e < 16; ++e) st[kt][e] = 0.f;
#pragma unroll
      for (int ks = 0; ks < D / 2; ++ks) {
        float qv;
        if constexpr (QLDS) qv = qs[(wave * 32 + col) * KP + 2 * ks + half];
        else qv = qf[ks];
        st[kt] = __builtin_amdgcn_mfma_f32_32x32x2f32(tile[(kt * 32 + col) * KP + 2 * ks + half], qv, st[kt], 0, 0, 0);
        // keep the scheduler from hoisting a whole tile's LDS reads above the MFMAs (registers)
        if (ks % 16 == 15) __builtin_amdgcn_sched_barrier(0);
      }
    }
    // ---- scale, mask, running maximum.  Register e of tile kt is key t_cur + kt*32 + (e>>2)*8 + half*4 + (e&3)
    float tmax = -3.40282347e+38f;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t key = t_cur + kt * 32 + j * 8 + half * 4;
        float mv[4] = {0.f, 0.f, 0.f, 0.f};
        if (use_mask) { mv[0] = mcur[kt][j].x; mv[1] = mcur[kt][j].y; mv[2] = mcur[kt][j].z; mv[3] = mcur[kt][j].w; }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float s = st[kt][j * 4 + i];
          if (a.has_scale) s = s / a.scale;  // the reference's quotient
          if (use_mask) s = s + mv[i];
          else if (!M && a.has_mask_const) s = s + a.mask_const;
          if (tail && key + i >= a.t) s = -3.40282347e+38f;
          st[kt][j * 4 + i] = s;
          tmax = fmaxf(tmax, s);
        }
      }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float m_new = fmaxf(m_run, tmax);
    const float alpha = expf(m_run - m_new);
    float psum = 0.f;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const uint32_t key = t_cur + kt * 32 + (e >> 2) * 8 + half * 4 + (e & 3);
        float p = expf(st[kt][e] - m_new);
        if (tail && key >= a.t) p = 0.f;
        st[kt][e] = p;
        psum += p;
      }
    psum += __shfl_xor(psum, 32, 64);
    l_run = l_run * alpha + psum;
    m_run = m_new;
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int t = 0; t < DT; ++t) {
#pragma unroll
        for (int e = 0; e < 16; ++e) o[t][e] *= alpha;
        __builtin_amdgcn_sched_barrier(0);  // one tile of O^T at a time through the VALU registers
      }
    }
    if (!AHEAD) fetch_rows(V, a.v_st, t_cur);
    __syncthreads();  // every wave has read its K fragments
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int ch = tid + c * NT, key = ch / (D / 4), d4 = (ch % (D / 4)) * 4;
      *(float4 *)(&tile[key * VP + d4]) = (t_cur + key < a.t) ? treg[c] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    __syncthreads();
    if (t_next < a.t) {  // in flight during the value product
      if (AHEAD) fetch_rows(K, a.k_st, t_next);
      fetch_mask(t_next);
    }
    // ---- O^T += V^T . P^T
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = kt * 32 + (i >> 2) * 8 + half * 4 + (i & 3);
          o[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(tile[key * VP + t * 32 + col], st[kt][i], o[t], 0, 0, 0);
          if (i == 15) __builtin_amdgcn_sched_barrier(0);
        }
  }
  if (M && q_ok && m_run <= -3.0e38f) {  // every key masked: uniform weights, as on the reference path
    l_run = (float)a.t;
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int e = 0; e < 16; ++e) o[t][e] = 0.f;
    for (uint32_t key = 0; key < a.t; ++key)
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float4 vv = *(const float4 *)(V + (int64_t)key * a.v_st + t * 32 + j * 8 + half * 4);
          o[t][j * 4 + 0] += vv.x; o[t][j * 4 + 1] += vv.y; o[t][j * 4 + 2] += vv.z; o[t][j * 4 + 3] += vv.w;
        }
  }
  if (q_ok) {
    float *out = a.out + (int64_t)b * a.o_sb + (int64_t)h * a.o_sh + (int64_t)query * a.o_ss;
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float4 r;
        r.x = o[t][j * 4 + 0] / l_run; r.y = o[t][j * 4 + 1] / l_run;
        r.z = o[t][j * 4 + 2] / l_run; r.w = o[t][j * 4 + 3] / l_run;
        *(float4 *)(out + t * 32 + j * 8 + half * 4) = r;
      }
  }
}

// bf16 products, few query rows: 64-query workgroups would not give every CU two of them
static bool attn_prefill_keysplit(const LaunchCtx &lc, const AttnPrefillDesc &d) {
  return !d.f32 && d.d == 64 && (uint64_t)((d.s + 63) / 64) * d.heads * d.b < 2 * (uint64_t)lc.n_cus;
}

static bool attn_prefill_small_tiles(const LaunchCtx &lc, const AttnPrefillDesc &d) {
  if (d.f32 && d.d == 256) return true;  // its queries live in LDS: 64 of them fit beside the K / V tile
  return (uint64_t)((d.s + 127) / 128) * d.heads * d.b < (uint64_t)lc.n_cus;  // too few workgroups of 128 queries: 64 each
}

void attn_prefill_tiling(const LaunchCtx &lc, const AttnPrefillDesc &d, uint32_t *q_rows, uint32_t *keys) {
  *q_rows = attn_prefill_keysplit(lc, d) ? 32 : attn_prefill_small_tiles(lc, d) ? 64 : 128;
  *keys = (d.d == 256 || (d.f32 && d.d == 128)) ? 32 : 64;
}

// one workgroup per (key tile, query tile): any value above the masked level, any value that is not zero
__global__ void __launch_bounds__(256) mask_tiles_kernel(const float *mask, int64_t m_ss, uint32_t s, uint32_t t, uint32_t q_rows,
                                                         uint32_t keys, uint8_t *out) {
  __shared__ uint32_t flags;
  if (threadIdx.x == 0) flags = 0;
  __syncthreads();
  const uint32_t q0 = blockIdx.y * q_rows, k0 = blockIdx.x * keys;
  uint32_t f = 0;  // bit 0: some pair is not masked, bit 1: some value is not zero
  for (uint32_t i = threadIdx.x; i < q_rows * keys; i += 256) {
    const uint32_t q = q0 + i / keys, k = k0 + i % keys;
    if (q < s && k < t) {
      const float v = mask[(int64_t)q * m_ss + k];
      if (v > -3.0e38f) f |= 1u;
      if (v != 0.f) f |= 2u;
    }
  }
  if (f) atomicOr(&flags, f);
  __syncthreads();
  if (threadIdx.x == 0) out[(size_t)blockIdx.y * gridDim.x + blockIdx.x] = !(flags & 1u) ? 0 : (flags & 2u) ? 1 : 2;
}

hipError_t launch_mask_tiles(const LaunchCtx &lc, const float *mask, int64_t m_ss, uint32_t s, uint32_t t, uint32_t q_rows,
                             uint32_t keys, uint8_t *out) {
  if (!s || !t) return hipSuccess;
  CG_LAUNCH(lc, mask_tiles_kernel, dim3((t + keys - 1) / keys, (s + q_rows - 1) / q_rows), 256, mask, m_ss, s, t, q_rows, keys, out);
  return hipGetLastError();
}

hipError_t launch_attn_prefill(const LaunchCtx &lc, const AttnPrefillDesc &d) {
  if (!d.b || !d.heads || !d.s) return hipSuccess;
  if (d.f32 ? !d.k : (!d.k16 || !d.vt16)) return hipErrorInvalidValue;
  if (attn_prefill_keysplit(lc, d)) {
    dim3 g32((d.s + 31) / 32, d.heads, d.b);
    CG_LAUNCH(lc, (attn_prefill_keysplit_kernel<64, 64, 4>), g32, 256, d);
    return hipGetLastError();
  }
  dim3 grid((d.s + 127) / 128, d.heads, d.b);
  const bool small = attn_prefill_small_tiles(lc, d);
  if (small) grid.x = (d.s + 63) / 64;
#define CG_ATTN_CASE(DD, ...)                                               \
  case DD:                                                                  \
    if (small) CG_LAUNCH(lc, (__VA_ARGS__, 2>), grid, 128, d);              \
    else CG_LAUNCH(lc, (__VA_ARGS__, 4>), grid, 256, d);                    \
    break;
  if (d.f32) {
    switch (d.d) {
      CG_ATTN_CASE(64, attn_prefill_f32_kernel<false, 64, 64)
      CG_ATTN_CASE(128, attn_prefill_f32_kernel<false, 128, 32)
      case 256: CG_LAUNCH(lc, (attn_prefill_f32_kernel<true, 256, 32, 2>), grid, 128, d); break;
      default: return hipErrorInvalidValue;
    }
  } else {
    switch (d.d) {
      CG_ATTN_CASE(64, attn_prefill_kernel<64, 64)
      CG_ATTN_CASE(128, attn_prefill_kernel<128, 64)
      CG_ATTN_CASE(256, attn_prefill_kernel<256, 32)
      default: return hipErrorInvalidValue;
    }
  }
#undef CG_ATTN_CASE
  return hipGetLastError();
}

}  // namespace cgk
