// k_fused.hip — hand-written fused kernels for the op patterns catgrad-llm emits.
//
// The deferred graph behind the Backend interface is matched (rt.cpp) against the exact op
// sequences of the reference's emitters and, on a match, one of these kernels replaces the
// generic program interpreter:
//   softmax  (+ the scale and additive mask attention puts in front of it)
//            catgrad/src/stdlib/nn/mod.rs:162-171, catgrad-llm/src/models/llama.rs:97-107
//   rmsnorm  catgrad-llm/src/helpers.rs:120-145 (and the (1 + gamma) form of gemma3.rs:41-68)
//   rope     catgrad-llm/src/helpers.rs:195-221 (half-split rotate, tables sliced at `pos`)
//   swiglu   silu(gate) * up, catgrad/src/stdlib/nn/mod.rs:130-148, models/llama.rs:26
//   geglu    gelu(gate) * up, nn/mod.rs:150-160, models/gemma3.rs
//   binary   a single add/sub/mul/div over contiguous operands (the residual adds)
// All are HBM- or latency-bound: one read of every operand, one write, 16-byte accesses,
// short straight-line code (a decode step runs each of them on a few KB, where instruction
// fetch and launch latency dominate).
#include <hip/hip_runtime.h>
#include <math.h>
#include "launch.hpp"
#include "dev_common.hpp"

namespace cgk {

// ---- rmsnorm ----------------------------------------------------------------------------------
// y = x / sqrt(sum(x*x) / n + eps) * (gamma_offset + gamma), rows contiguous along the last axis.
// One workgroup per row; the row lives in registers between the two phases.
// PAIR (gemma3.rs:198-240, sandwich norms): the row with its residual added is the stream the next
// norm reads; it is written to y_mid and normed a second time (gamma2) from the registers it sits in.
// RPW rows per workgroup: with many short rows (a prefill) a wave takes a whole row (BLOCK = 64) - no
// barrier, no LDS - and four such waves share a workgroup.
template <int BLOCK, int EPT, bool PAIR, int RPW = 1>  // BLOCK = threads per row, EPT = float4 chunks per thread
__global__ void __launch_bounds__(BLOCK * RPW) rmsnorm_kernel(RmsNormDesc d) {
  static_assert(RPW == 1 || BLOCK == 64, "several rows per workgroup: one wave each");
  __shared__ float lds[BLOCK / 64];
  const uint32_t row = blockIdx.x * RPW + (RPW > 1 ? threadIdx.x / BLOCK : 0);
  const uint32_t tid = RPW > 1 ? threadIdx.x % BLOCK : threadIdx.x;
  if (RPW > 1 && row >= d.rows) return;  // whole waves leave; the one-wave-per-row form has no barrier
  int64_t xoff;
  if (d.x_d1 <= 1 && d.x_d2 <= 1) {
    xoff = (int64_t)row * d.x_row_stride;
  } else {
    const uint32_t d2 = d.x_d2 ? d.x_d2 : 1, d1 = d.x_d1 ? d.x_d1 : 1, q = row / d2;
    xoff = (int64_t)(q / d1) * d.x_row_stride + (int64_t)(q % d1) * d.x_s1 + (int64_t)(row % d2) * d.x_s2;
  }
  const float *x = d.x + xoff;
  float *y = d.y ? d.y + (int64_t)row * d.n : nullptr;
  float4 v[EPT];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const uint32_t c = (tid + e * BLOCK) * 4;
    if (c < d.n) {
      if (d.x_slices) {  // the row is still the k-slices of a split product: sum them, keep the sum
        const uint64_t at = (uint64_t)row * d.n + c;
        float4 s = *(const float4 *)(d.x_slices + at);
        for (uint32_t k = 1; k < d.x_n_slices; ++k) {
          const float4 t = *(const float4 *)(d.x_slices + k * d.x_slice_stride + at);
          s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
        }
        if (d.x_add) {
          const float4 t = *(const float4 *)(d.x_add + at);
          s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
        }
        *(float4 *)(d.x_out + at) = s;
        v[e] = s;
      } else {
        v[e] = *(const float4 *)(x + c);
      }
      ss += v[e].x * v[e].x + v[e].y * v[e].y + v[e].z * v[e].z + v[e].w * v[e].w;
    }
  }
  ss = block_reduce<BLOCK, false>(ss, lds);
  // the reference divides by sqrt (pow(.., 0.5)); keep a true division for the 1e-4 bar
  const float rms = sqrtf(ss / d.n_as_float + d.eps);
  float ss2 = 0.f;
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const uint32_t c = (tid + e * BLOCK) * 4;
    if (c < d.n) {
      float4 o;
      o.x = v[e].x / rms; o.y = v[e].y / rms; o.z = v[e].z / rms; o.w = v[e].w / rms;
      if (d.gamma) {
        const float4 g = *(const float4 *)(d.gamma + c);
        o.x *= d.gamma_offset + g.x; o.y *= d.gamma_offset + g.y;
        o.z *= d.gamma_offset + g.z; o.w *= d.gamma_offset + g.w;
      }
      if (d.residual) {
        const float4 r = *(const float4 *)(d.residual + (int64_t)row * d.n + c);
        o.x += r.x; o.y += r.y; o.z += r.z; o.w += r.w;
      }
      if (PAIR) {
        *(float4 *)(d.y_mid + (int64_t)row * d.n + c) = o;
        v[e] = o;
        ss2 += o.x * o.x + o.y * o.y + o.z * o.z + o.w * o.w;
      } else {
        if (y) *(float4 *)(y + c) = o;
        if (d.y16) *(uint2 *)(d.y16 + (int64_t)row * d.n + c) = bf16_pack4(o);
      }
    }
  }
  if (!PAIR) return;
  ss2 = block_reduce<BLOCK, false>(ss2, lds);
  const float rms2 = sqrtf(ss2 / d.n_as_float + d.eps2);
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const uint32_t c = (tid + e * BLOCK) * 4;
    if (c < d.n) {
      const float4 g = *(const float4 *)(d.gamma2 + c);
      float4 o;
      o.x = v[e].x / rms2 * (d.gamma2_offset + g.x); o.y = v[e].y / rms2 * (d.gamma2_offset + g.y);
      o.z = v[e].z / rms2 * (d.gamma2_offset + g.z); o.w = v[e].w / rms2 * (d.gamma2_offset + g.w);
      if (y) *(float4 *)(y + c) = o;
      if (d.y16) *(uint2 *)(d.y16 + (int64_t)row * d.n + c) = bf16_pack4(o);
    }
  }
}

template <bool PAIR>
static void launch_rmsnorm_as(const LaunchCtx &lc, const RmsNormDesc &d) {
  // n % 4 == 0 and n <= 16384 are checked by the caller
  if (d.rows >= 2048 && d.n <= 2048) {  // a wave per row, four rows per workgroup
    const uint32_t wgs = (d.rows + 3) / 4;
    if (d.n <= 256) CG_LAUNCH(lc, (rmsnorm_kernel<64, 1, PAIR, 4>), wgs, 256, d);
    else if (d.n <= 512) CG_LAUNCH(lc, (rmsnorm_kernel<64, 2, PAIR, 4>), wgs, 256, d);
    else if (d.n <= 1024) CG_LAUNCH(lc, (rmsnorm_kernel<64, 4, PAIR, 4>), wgs, 256, d);
    else if (d.n <= 1280) CG_LAUNCH(lc, (rmsnorm_kernel<64, 5, PAIR, 4>), wgs, 256, d);
    else CG_LAUNCH(lc, (rmsnorm_kernel<64, 8, PAIR, 4>), wgs, 256, d);
    return;
  }
  if (d.n <= 256) CG_LAUNCH(lc, (rmsnorm_kernel<64, 1, PAIR>), d.rows, 64, d);
  else if (d.n <= 1024) CG_LAUNCH(lc, (rmsnorm_kernel<256, 1, PAIR>), d.rows, 256, d);
  else if (d.n <= 2048) CG_LAUNCH(lc, (rmsnorm_kernel<256, 2, PAIR>), d.rows, 256, d);
  else if (d.n <= 4096) CG_LAUNCH(lc, (rmsnorm_kernel<256, 4, PAIR>), d.rows, 256, d);
  else CG_LAUNCH(lc, (rmsnorm_kernel<1024, 4, PAIR>), d.rows, 1024, d);
}

hipError_t launch_rmsnorm(const LaunchCtx &lc, const RmsNormDesc &d) {
  if (!d.rows || !d.n) return hipSuccess;
  if (d.x_slices && (!d.x_out || !d.x_n_slices || d.n % 4 || d.x_slice_stride % 4 || d.x_d1 > 1 || d.x_d2 > 1 ||
                     (uintptr_t)d.x_slices % 16 || (uintptr_t)d.x_out % 16 || (uintptr_t)d.x_add % 16))
    return hipErrorInvalidValue;
  if (d.y_mid) launch_rmsnorm_as<true>(lc, d);
  else launch_rmsnorm_as<false>(lc, d);
  return hipGetLastError();
}

// ---- softmax(x / scale + mask) ------------------------------------------------------------------------
// x rows contiguous; mask (optional) is read through (row-group, row, col) strides so that the
// [S, S] causal mask broadcast over batch and heads is never materialised.  The row is kept in
// registers: EPT elements per thread, lanes strided for coalescing.
template <int BLOCK, int EPT>
__global__ void __launch_bounds__(BLOCK == 64 ? 256 : BLOCK) softmax_kernel(SoftmaxDesc d) {
  __shared__ float lds[BLOCK / 64];
  constexpr int RPB = BLOCK == 64 ? 4 : 1;  // rows per workgroup (one wave each) for short rows
  const uint32_t row = blockIdx.x * RPB + (RPB == 4 ? threadIdx.y : 0);
  if (row >= d.rows) return;  // whole wave exits together (RPB == 4) or never (RPB == 1)
  const uint32_t tid = threadIdx.x;
  const float *x = d.x + (int64_t)row * d.x_row_stride;
  float *y = d.y + (int64_t)row * d.n;
  const float *mk = nullptr;
  if (d.mask) {
    const uint32_t r_in = row % d.mask_rows, grp = row / d.mask_rows;
    mk = d.mask + (int64_t)grp * d.mask_group_stride + (int64_t)r_in * d.mask_row_stride;
  }
  float v[EPT];
  float mx = -3.40282347e+38f;  // max folds from f32::MIN (ndarray.rs:455-460)
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const uint32_t c = tid + e * BLOCK;
    if (c < d.n) {
      float t = x[c];
      if (d.has_scale) t = t / d.scale;
      if (mk) t = t + mk[(int64_t)c * d.mask_col_stride];
      else if (d.has_mask_const) t = t + d.mask_const;
      v[e] = t;
      mx = fmaxf(mx, t);
    }
  }
  mx = block_reduce<BLOCK, true>(mx, lds);
  float sum = 0.f;
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const uint32_t c = tid + e * BLOCK;
    if (c < d.n) {
      v[e] = expf(v[e] - mx);
      sum += v[e];
    }
  }
  sum = block_reduce<BLOCK, false>(sum, lds);
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const uint32_t c = tid + e * BLOCK;
    if (c < d.n) {
      const float o = v[e] / sum;
      y[c] = o;
      if (d.y16) d.y16[(int64_t)row * d.n + c] = (uint16_t)bf16_bits(o);
    }
  }
}

// Same, 16 bytes per access (n % 4 == 0, rows and mask rows 16-byte aligned, unit mask column stride);
// the row stays in registers between the passes: CH float4 chunks per thread.
template <int BLOCK, int CH>
__global__ void __launch_bounds__(BLOCK) softmax_vec_kernel(SoftmaxDesc d) {
  __shared__ float lds[BLOCK / 64];
  const uint32_t row = blockIdx.x, tid = threadIdx.x;
  const float *x = d.x + (int64_t)row * d.x_row_stride;
  const uint16_t *x16 = (const uint16_t *)d.x + (int64_t)row * d.x_row_stride;  // when the rows are stored as bf16
  float *y = d.y + (int64_t)row * d.n;
  const float *mk = nullptr;
  if (d.mask) {
    const uint32_t r_in = row % d.mask_rows, grp = row / d.mask_rows;
    mk = d.mask + (int64_t)grp * d.mask_group_stride + (int64_t)r_in * d.mask_row_stride;
  }
  float4 v[CH];
  float mx = -3.40282347e+38f;
#pragma unroll
  for (int e = 0; e < CH; ++e) {
    const uint32_t c = (tid + e * BLOCK) * 4;
    if (c < d.n) {
      if (d.x_bf16) {
        const uint2 h = *(const uint2 *)(x16 + c);
        v[e] = make_float4(__uint_as_float(h.x << 16), __uint_as_float(h.x & 0xFFFF0000u), __uint_as_float(h.y << 16),
                           __uint_as_float(h.y & 0xFFFF0000u));
      } else {
        v[e] = *(const float4 *)(x + c);
      }
    }
  }
#pragma unroll
  for (int e = 0; e < CH; ++e) {
    const uint32_t c = (tid + e * BLOCK) * 4;
    if (c < d.n) {
      float4 t = v[e];
      if (d.has_scale) { t.x = t.x / d.scale; t.y = t.y / d.scale; t.z = t.z / d.scale; t.w = t.w / d.scale; }
      if (mk) {
        const float4 m = *(const float4 *)(mk + c);
        t.x += m.x; t.y += m.y; t.z += m.z; t.w += m.w;
      } else if (d.has_mask_const) {
        t.x += d.mask_const; t.y += d.mask_const; t.z += d.mask_const; t.w += d.mask_const;
      }
      v[e] = t;
      mx = fmaxf(fmaxf(mx, t.x), fmaxf(t.y, fmaxf(t.z, t.w)));
    }
  }
  mx = block_reduce<BLOCK, true>(mx, lds);
  float sum = 0.f;
#pragma unroll
  for (int e = 0; e < CH; ++e) {
    const uint32_t c = (tid + e * BLOCK) * 4;
    if (c < d.n) {
      float4 t = v[e];
      t.x = expf(t.x - mx); t.y = expf(t.y - mx); t.z = expf(t.z - mx); t.w = expf(t.w - mx);
      v[e] = t;
      sum += (t.x + t.y) + (t.z + t.w);
    }
  }
  sum = block_reduce<BLOCK, false>(sum, lds);
#pragma unroll
  for (int e = 0; e < CH; ++e) {
    const uint32_t c = (tid + e * BLOCK) * 4;
    if (c < d.n) {
      float4 t = v[e];
      t.x = t.x / sum; t.y = t.y / sum; t.z = t.z / sum; t.w = t.w / sum;
      *(float4 *)(y + c) = t;
      if (d.y16) *(uint2 *)(d.y16 + (int64_t)row * d.n + c) = bf16_pack4(t);
    }
  }
}

hipError_t launch_softmax(const LaunchCtx &lc, const SoftmaxDesc &d) {
  if (!d.rows || !d.n) return hipSuccess;
  // n <= 16384 checked by the caller
  const bool vec = d.n % 4 == 0 && d.n >= 256 && (uintptr_t)d.x % 16 == 0 && d.x_row_stride % 4 == 0 &&
                   (uintptr_t)d.y % 16 == 0 &&
                   (!d.mask || (d.mask_col_stride == 1 && (uintptr_t)d.mask % 16 == 0 && d.mask_row_stride % 4 == 0 &&
                                d.mask_group_stride % 4 == 0));
  if (d.x_bf16 && !vec) return hipErrorInvalidValue;
  if (vec) {
    if (d.n <= 512) CG_LAUNCH(lc, (softmax_vec_kernel<64, 2>), d.rows, 64, d);
    else if (d.n <= 1024) CG_LAUNCH(lc, (softmax_vec_kernel<256, 1>), d.rows, 256, d);
    else if (d.n <= 2048) CG_LAUNCH(lc, (softmax_vec_kernel<256, 2>), d.rows, 256, d);
    else if (d.n <= 4096) CG_LAUNCH(lc, (softmax_vec_kernel<256, 4>), d.rows, 256, d);
    else if (d.n <= 8192) CG_LAUNCH(lc, (softmax_vec_kernel<512, 4>), d.rows, 512, d);
    else CG_LAUNCH(lc, (softmax_vec_kernel<1024, 4>), d.rows, 1024, d);
    return hipGetLastError();
  }
  if (d.n <= 64) CG_LAUNCH(lc, (softmax_kernel<64, 1>), (d.rows + 3) / 4, dim3(64, 4), d);
  else if (d.n <= 256) CG_LAUNCH(lc, (softmax_kernel<64, 4>), (d.rows + 3) / 4, dim3(64, 4), d);
  else if (d.n <= 512) CG_LAUNCH(lc, (softmax_kernel<64, 8>), (d.rows + 3) / 4, dim3(64, 4), d);
  else if (d.n <= 1024) CG_LAUNCH(lc, (softmax_kernel<256, 4>), d.rows, 256, d);
  else if (d.n <= 4096) CG_LAUNCH(lc, (softmax_kernel<256, 16>), d.rows, 256, d);
  else CG_LAUNCH(lc, (softmax_kernel<1024, 16>), d.rows, 1024, d);
  return hipGetLastError();
}

// ---- one-query attention ----------------------------------------------------------------------------------
// The decode step of models/llama.rs:77-112: scores = q . K^T, / sqrt(d), + mask, softmax, . V, for one
// query row per head.  One workgroup per (batch, head); LPK lanes share a key/value row (16 bytes
// each), so a wave covers 64 / LPK rows per load.  Scores live in LDS between the three phases
// (dot products + max, exp + sum, weighted sum of V rows); nothing of size T goes to HBM.
template <int LPK, int BLOCK>
__global__ void __launch_bounds__(BLOCK) attn_decode_kernel(AttnDecodeDesc a) {
  constexpr int NW = BLOCK / 64;
  constexpr int KPW = 64 / LPK;       // rows per wave per load
  constexpr int STRIDE = NW * KPW;    // rows per workgroup per load
  constexpr int U = 4;                // independent row loads in flight per lane
  __shared__ float sc[ATTN_DECODE_MAX_T];
  __shared__ float red[STRIDE][LPK * 4];
  __shared__ float lds[NW];
  const uint32_t h = blockIdx.x, b = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int sub = lane % LPK, kg = lane / LPK;
  const uint32_t kv = h / a.rep, rp = h % a.rep;
  const float *q = a.q + (int64_t)b * a.q_sb + (int64_t)h * a.q_sh;
  const float *K = a.k + (int64_t)b * a.k_sb + (int64_t)kv * a.k_skv + (int64_t)rp * a.k_srep;
  const float *V = a.v + (int64_t)b * a.v_sb + (int64_t)kv * a.v_skv + (int64_t)rp * a.v_srep;
  const bool live = (uint32_t)sub * 4 < a.d;
  float4 qv = make_float4(0.f, 0.f, 0.f, 0.f);
  if (live) {
    qv = *(const float4 *)(q + sub * 4);
    if (a.q_cos) {  // apply_rope_embedding on the fly, same arithmetic as rope_kernel
      const uint32_t j = sub * 4, half = a.d / 2;
      const bool lo = j < half;
      float4 pv = *(const float4 *)(q + (lo ? j + half : j - half));
      if (lo) { pv.x = -pv.x; pv.y = -pv.y; pv.z = -pv.z; pv.w = -pv.w; }
      const float4 c = *(const float4 *)(a.q_cos + j), sn = *(const float4 *)(a.q_sin + j);
      qv.x = c.x * qv.x + sn.x * pv.x; qv.y = c.y * qv.y + sn.y * pv.y;
      qv.z = c.z * qv.z + sn.z * pv.z; qv.w = c.w * qv.w + sn.w * pv.w;
    }
  }
  // this step's own key / value row: from the projections, not from the cache
  const bool has_new = a.k_new != nullptr;
  const uint32_t t_new = has_new ? a.t_new : 0xFFFFFFFFu;
  float4 knew = make_float4(0.f, 0.f, 0.f, 0.f), vnew = knew;
  if (has_new && live) {
    const float *kn = a.k_new + (int64_t)b * a.kn_sb + (int64_t)kv * a.kn_skv;
    const uint32_t j = sub * 4;
    knew = *(const float4 *)(kn + j);
    if (a.kn_cos) {
      const uint32_t half = a.d / 2;
      const bool lo = j < half;
      float4 pv = *(const float4 *)(kn + (lo ? j + half : j - half));
      if (lo) { pv.x = -pv.x; pv.y = -pv.y; pv.z = -pv.z; pv.w = -pv.w; }
      const float4 c = *(const float4 *)(a.kn_cos + j), sn = *(const float4 *)(a.kn_sin + j);
      knew.x = c.x * knew.x + sn.x * pv.x; knew.y = c.y * knew.y + sn.y * pv.y;
      knew.z = c.z * knew.z + sn.z * pv.z; knew.w = c.w * knew.w + sn.w * pv.w;
    }
    vnew = *(const float4 *)(a.v_new + (int64_t)b * a.vn_sb + (int64_t)kv * a.vn_skv + j);
    if (rp == 0 && wave == 0 && kg == 0) {  // one writer per (batch, kv head)
      *(float4 *)(const_cast<float *>(K) + (int64_t)t_new * a.k_st + j) = knew;
      *(float4 *)(const_cast<float *>(V) + (int64_t)t_new * a.v_st + j) = vnew;
    }
  }
  const uint32_t first = wave * KPW + kg;
  // phase 1: scores and their maximum
  float mx = -3.40282347e+38f;
  for (uint32_t t0 = first; t0 < a.t; t0 += STRIDE * U) {
    float4 kr[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t t = t0 + u * STRIDE;
      kr[u] = (t == t_new) ? knew
              : (live && t < a.t) ? *(const float4 *)(K + (int64_t)t * a.k_st + sub * 4)
                                  : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t t = t0 + u * STRIDE;
      float s = qv.x * kr[u].x + qv.y * kr[u].y + qv.z * kr[u].z + qv.w * kr[u].w;
      s = group_sum<LPK>(s);
      if (a.has_scale) s = s / a.scale;
      if (a.has_mask_const) s = s + a.mask_const;
      if (t < a.t) {
        if (sub == 0) sc[t] = s;
        mx = fmaxf(mx, s);
      }
    }
  }
  mx = block_reduce<BLOCK, true>(mx, lds);  // its barrier also publishes sc[]
  // phase 2: exponentials and their sum
  float sum = 0.f;
  for (uint32_t t = tid; t < a.t; t += BLOCK) {
    const float e = expf(sc[t] - mx);
    sc[t] = e;
    sum += e;
  }
  sum = block_reduce<BLOCK, false>(sum, lds);
  // phase 3: weighted sum of V rows
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  for (uint32_t t0 = first; t0 < a.t; t0 += STRIDE * U) {
    float4 vr[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t t = t0 + u * STRIDE;
      vr[u] = (t == t_new) ? vnew
              : (live && t < a.t) ? *(const float4 *)(V + (int64_t)t * a.v_st + sub * 4)
                                  : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t t = t0 + u * STRIDE;
      if (t < a.t) {
        const float p = sc[t] / sum;
        acc.x += p * vr[u].x; acc.y += p * vr[u].y; acc.z += p * vr[u].z; acc.w += p * vr[u].w;
      }
    }
  }
  *(float4 *)(&red[wave * KPW + kg][sub * 4]) = acc;
  __syncthreads();
  if ((uint32_t)tid < a.d) {
    float o = 0.f;
#pragma unroll
    for (int g = 0; g < STRIDE; ++g) o += red[g][tid];
    a.out[((uint64_t)b * a.heads + h) * a.d + tid] = o;
  }
}

// The same attention with the keys of one (batch, head) divided over `splits` workgroups, for caches
// long enough that one compute unit's load path is the limit.  Every group of LPK lanes keeps a
// running maximum / sum / weighted value row over the rows it visits (all K and V rows of an
// iteration are requested before any is used); the groups of a workgroup are merged through LDS
// into one partial result (max, sum, d values) in `part`, and the workgroup that finds the counter
// of its (batch, head) at splits - 1 merges the partials and writes the output row.  The counters
// are zero between launches: the merging workgroup puts its counter back.
template <int LPK>
__global__ void __launch_bounds__(256) attn_decode_split_kernel(AttnDecodeDesc a) {
  constexpr int KPW = 64 / LPK, STRIDE = 4 * KPW, U = 8;
  constexpr float FMIN = -3.40282347e+38f;
  __shared__ float red[STRIDE][LPK * 4];
  __shared__ float red_m[STRIDE], red_l[STRIDE];
  __shared__ uint32_t last_flag;
  const uint32_t h = blockIdx.x, b = blockIdx.y, c = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int sub = lane % LPK, kg = lane / LPK, grp = wave * KPW + kg;
  const uint32_t kv = h / a.rep, rp = h % a.rep;
  const float *q = a.q + (int64_t)b * a.q_sb + (int64_t)h * a.q_sh;
  const float *K = a.k + (int64_t)b * a.k_sb + (int64_t)kv * a.k_skv + (int64_t)rp * a.k_srep;
  const float *V = a.v + (int64_t)b * a.v_sb + (int64_t)kv * a.v_skv + (int64_t)rp * a.v_srep;
  const bool live = (uint32_t)sub * 4 < a.d;
  const uint32_t t_begin = c * a.chunk, t_end = min(a.t, t_begin + a.chunk);
  // The cache rows of the first pass are asked for before anything else: the query, its rotation and
  // this step's own rows come back during the same trip to memory.
  float4 kn[U], vn[U];
  auto fetch_rows = [&](uint32_t t0) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t tc = min(t0 + u * STRIDE, t_end - 1);
      kn[u] = *(const float4 *)(K + (int64_t)tc * a.k_st + (live ? sub * 4 : 0));
      vn[u] = *(const float4 *)(V + (int64_t)tc * a.v_st + (live ? sub * 4 : 0));
    }
  };
  if (t_begin + grp < t_end) fetch_rows(t_begin + grp);
  float4 qv = make_float4(0.f, 0.f, 0.f, 0.f);
  if (live) {
    qv = *(const float4 *)(q + sub * 4);
    if (a.q_cos) {  // apply_rope_embedding on the fly, same arithmetic as rope_kernel
      const uint32_t j = sub * 4, half = a.d / 2;
      const bool lo = j < half;
      float4 pv = *(const float4 *)(q + (lo ? j + half : j - half));
      if (lo) { pv.x = -pv.x; pv.y = -pv.y; pv.z = -pv.z; pv.w = -pv.w; }
      const float4 cs = *(const float4 *)(a.q_cos + j), sn = *(const float4 *)(a.q_sin + j);
      qv.x = cs.x * qv.x + sn.x * pv.x; qv.y = cs.y * qv.y + sn.y * pv.y;
      qv.z = cs.z * qv.z + sn.z * pv.z; qv.w = cs.w * qv.w + sn.w * pv.w;
    }
  }
  // this step's own key / value row comes from the projections, not from the cache
  const bool has_new = a.k_new != nullptr && a.t_new >= t_begin && a.t_new < t_end;
  const uint32_t t_new = has_new ? a.t_new : 0xFFFFFFFFu;
  float4 knew = make_float4(0.f, 0.f, 0.f, 0.f), vnew = knew;
  if (has_new && live) {
    const float *kn = a.k_new + (int64_t)b * a.kn_sb + (int64_t)kv * a.kn_skv;
    const uint32_t j = sub * 4;
    knew = *(const float4 *)(kn + j);
    if (a.kn_cos) {
      const uint32_t half = a.d / 2;
      const bool lo = j < half;
      float4 pv = *(const float4 *)(kn + (lo ? j + half : j - half));
      if (lo) { pv.x = -pv.x; pv.y = -pv.y; pv.z = -pv.z; pv.w = -pv.w; }
      const float4 cs = *(const float4 *)(a.kn_cos + j), sn = *(const float4 *)(a.kn_sin + j);
      knew.x = cs.x * knew.x + sn.x * pv.x; knew.y = cs.y * knew.y + sn.y * pv.y;
      knew.z = cs.z * knew.z + sn.z * pv.z; knew.w = cs.w * knew.w + sn.w * pv.w;
    }
    vnew = *(const float4 *)(a.v_new + (int64_t)b * a.vn_sb + (int64_t)kv * a.vn_skv + j);
  }
  // A decode step is a chain of short dependent phases, so the arithmetic between two memory trips is
  // kept short: one reciprocal instead of a quotient per score, and the hardware exponential (2 ulp,
  // far inside the f32 bar for scores of this size).
  const float inv_scale = a.has_scale ? 1.0f / a.scale : 1.0f;
  float m_run = FMIN, l_run = 0.f;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  for (uint32_t t0 = t_begin + grp; t0 < t_end; t0 += STRIDE * U) {
    float4 kr[U], vr[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t t = t0 + u * STRIDE;
      const bool in = live && t < t_end && t != t_new;
      kr[u] = kn[u];
      vr[u] = vn[u];
      if (t == t_new) { kr[u] = knew; vr[u] = vnew; }
      else if (!in) { kr[u] = make_float4(0.f, 0.f, 0.f, 0.f); vr[u] = kr[u]; }
    }
    if (t0 + STRIDE * U < t_end) fetch_rows(t0 + STRIDE * U);  // the next pass, in flight during this one
    float sv[U], mx = FMIN;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float s = qv.x * kr[u].x + qv.y * kr[u].y + qv.z * kr[u].z + qv.w * kr[u].w;
      s = group_sum<LPK>(s);
      if (a.has_scale) s = s * inv_scale;
      if (a.has_mask_const) s = s + a.mask_const;
      sv[u] = s;
      if (t0 + u * STRIDE < t_end) mx = fmaxf(mx, s);
    }
    const float m_new = fmaxf(m_run, mx);
    const float alpha = __expf(m_run - m_new);
    l_run *= alpha;
    acc.x *= alpha; acc.y *= alpha; acc.z *= alpha; acc.w *= alpha;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (t0 + u * STRIDE < t_end) {
        const float p = __expf(sv[u] - m_new);
        l_run += p;
        acc.x += p * vr[u].x; acc.y += p * vr[u].y; acc.z += p * vr[u].z; acc.w += p * vr[u].w;
      }
    }
    m_run = m_new;
  }
  // The new row goes into the cache here, not where it was loaded: a store waits for its data, and
  // every cache row above was asked for without waiting for the projections' row first.  (The loop
  // never uses what memory holds at t_new.)
  if (has_new && live && rp == 0 && grp == 0) {  // one writer per (batch, kv head)
    const uint32_t j = sub * 4;
    *(float4 *)(const_cast<float *>(K) + (int64_t)t_new * a.k_st + j) = knew;
    *(float4 *)(const_cast<float *>(V) + (int64_t)t_new * a.v_st + j) = vnew;
  }
  // merge the lane groups of this workgroup
  *(float4 *)(&red[grp][sub * 4]) = acc;
  if (sub == 0) { red_m[grp] = m_run; red_l[grp] = l_run; }
  __syncthreads();
  const uint32_t pw = a.d + 2;  // floats per partial: max, sum, d values
  float *mine = a.part + (((uint64_t)b * a.heads + h) * a.splits + c) * pw;
  if ((uint32_t)tid < a.d) {
    float M = FMIN;
#pragma unroll
    for (int g = 0; g < STRIDE; ++g) M = fmaxf(M, red_m[g]);
    float L = 0.f, o = 0.f;
#pragma unroll
    for (int g = 0; g < STRIDE; ++g) {
      const float w = __expf(red_m[g] - M);
      L += w * red_l[g];
      o += w * red[g][tid];
    }
    if (a.splits == 1) {
      a.out[((uint64_t)b * a.heads + h) * a.d + tid] = o / L;
      return;
    }
    if (a.merge_later) {  // the reader of the result merges: plain stores, the kernel boundary orders them
      float *rec = a.part + (((uint64_t)b * a.heads + h) * a.splits + c) * (a.d + 4);
      rec[tid] = o;
      if (tid == 0) {
        rec[a.d] = M;
        rec[a.d + 1] = L;
      }
      return;
    }
    // The hand-over to the merging workgroup (another compute unit, usually another XCD).  A release
    // fence at agent scope would do it by the book, but it also writes back every dirty line of this
    // XCD's L2 (5 us per launch, measured); the partials need less.  They are agent-scope atomic
    // stores, which go through to the level every compute unit reads from, and a wave's vmcnt only
    // counts such a store down once it has been acknowledged from there.  So: every wave waits for its
    // own stores, then the barrier, and only then does thread 0 move the counter - no workgroup can
    // find the counter at splits - 1 before all the partials of the other splits have landed.
    __hip_atomic_store(mine + 2 + tid, o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (tid == 0) {
      __hip_atomic_store(mine, M, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(mine + 1, L, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  if (a.splits == 1 || a.merge_later) return;
  __syncthreads();
  uint32_t *counter = a.count + (uint64_t)b * a.heads + h;
  if (tid == 0)
    last_flag = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == a.splits - 1 ? 1u : 0u;
  __syncthreads();
  if (!last_flag) return;
  // The merging side: its loads of the partials are issued after the counter's value came back (the
  // branch above depends on it, and the compiler may not move atomic loads above the barrier), and
  // they are agent-scope atomic loads, which are served from the level the stores went through to,
  // never from this compute unit's own caches.
  // Every thread asks for all it needs at once - the maxima and sums of all partials (the same
  // addresses in every lane: one request) and its own column of values - so the merge costs one trip
  // to memory, not one for the statistics and another for the values.
  const float *base = a.part + ((uint64_t)b * a.heads + h) * a.splits * pw;
  if ((uint32_t)tid < a.d) {
    float M = FMIN, L = 0.f, o = 0.f;
    for (uint32_t s0 = 0; s0 < a.splits; s0 += 8) {
      float pm[8], pl[8], pv[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const uint32_t s = min(s0 + u, a.splits - 1);
        pm[u] = __hip_atomic_load(base + s * pw, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        pl[u] = __hip_atomic_load(base + s * pw + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        pv[u] = __hip_atomic_load(base + s * pw + 2 + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      float mx = M;
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (s0 + u < a.splits) mx = fmaxf(mx, pm[u]);
      const float keep = __expf(M - mx);  // rescale what the earlier groups of eight added up
      L *= keep;
      o *= keep;
      M = mx;
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (s0 + u < a.splits) {
          const float w = __expf(pm[u] - M);
          L += w * pl[u];
          o += w * pv[u];
        }
    }
    a.out[((uint64_t)b * a.heads + h) * a.d + tid] = o / L;
  }
  if (tid == 0) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

uint32_t attn_decode_rows_per_pass(uint32_t d) { return d <= 64 ? 128 : d <= 128 ? 64 : 32; }

hipError_t launch_attn_decode(const LaunchCtx &lc, const AttnDecodeDesc &d) {
  if (!d.b || !d.heads || !d.d) return hipSuccess;
  if (d.splits) {
    if (!d.part || !d.count || !d.chunk || (uint64_t)d.chunk * d.splits < d.t || d.splits > 64) return hipErrorInvalidValue;
    dim3 grid(d.heads, d.b, d.splits);
    if (d.d <= 64) CG_LAUNCH(lc, (attn_decode_split_kernel<16>), grid, 256, d);
    else if (d.d <= 128) CG_LAUNCH(lc, (attn_decode_split_kernel<32>), grid, 256, d);
    else CG_LAUNCH(lc, (attn_decode_split_kernel<64>), grid, 256, d);
    return hipGetLastError();
  }
  if (d.t > ATTN_DECODE_MAX_T) return hipErrorInvalidValue;
  dim3 grid(d.heads, d.b);
  // long caches: more rows in flight per workgroup
  if (d.t > 256) {
    if (d.d <= 64) CG_LAUNCH(lc, (attn_decode_kernel<16, 1024>), grid, 1024, d);
    else if (d.d <= 128) CG_LAUNCH(lc, (attn_decode_kernel<32, 1024>), grid, 1024, d);
    else CG_LAUNCH(lc, (attn_decode_kernel<64, 1024>), grid, 1024, d);
  } else {
    if (d.d <= 64) CG_LAUNCH(lc, (attn_decode_kernel<16, 512>), grid, 512, d);
    else if (d.d <= 128) CG_LAUNCH(lc, (attn_decode_kernel<32, 512>), grid, 512, d);
    else CG_LAUNCH(lc, (attn_decode_kernel<64, 512>), grid, 512, d);
  }
  return hipGetLastError();
}

// ---- rope -------------------------------------------------------------------------------------------
// out[b,h,s,j] = cos[s,j] * x[b,h,s,j] + sin[s,j] * rot, rot = j < half ? -x[..,j+half] : x[..,j-half]
// x is read through (b, h, s) strides with a unit stride along j, so the transposed view of the
// q/k projection is consumed in place; out is contiguous.  One thread per 4 consecutive j.
__device__ __forceinline__ void rope_rows(const RopeDesc &d, uint32_t block, uint32_t n_blocks) {
  const uint32_t q4 = d.dim / 4;
  const uint64_t total = (uint64_t)d.b * d.h * d.s * q4;
  for (uint64_t i = (uint64_t)block * 256 + threadIdx.x; i < total; i += (uint64_t)n_blocks * 256) {
    const uint32_t j = (uint32_t)(i % q4) * 4;
    uint64_t r = i / q4;
    const uint32_t s = (uint32_t)(r % d.s);
    r /= d.s;
    const uint32_t h = (uint32_t)(r % d.h), b = (uint32_t)(r / d.h);
    const float *xr = d.x + (int64_t)b * d.x_sb + (int64_t)h * d.x_sh + (int64_t)s * d.x_ss;
    const float4 xv = *(const float4 *)(xr + j);
    const bool lo = j < d.half;
    float4 pv = *(const float4 *)(xr + (lo ? j + d.half : j - d.half));
    if (lo) { pv.x = -pv.x; pv.y = -pv.y; pv.z = -pv.z; pv.w = -pv.w; }
    const float4 c = *(const float4 *)(d.cos + (int64_t)s * d.cs_ss + j);
    const float4 sn = *(const float4 *)(d.sin + (int64_t)s * d.cs_ss + j);
    float4 o;
    o.x = c.x * xv.x + sn.x * pv.x; o.y = c.y * xv.y + sn.y * pv.y;
    o.z = c.z * xv.z + sn.z * pv.z; o.w = c.w * xv.w + sn.w * pv.w;
    const int64_t oo = (int64_t)b * d.o_sb + (int64_t)h * d.o_sh + (int64_t)s * d.o_ss + j;
    *(float4 *)(d.out + oo) = o;
    if (d.out16) *(uint2 *)(d.out16 + oo) = bf16_pack4(o);
  }
}

// The same with every row normed on its way in (gemma3.rs:99-117: q and k are RMS-normed per head between the head
// transpose and the rotation): LPR = dim / 4 lanes hold a row, sum its squares among themselves, and a lane
// gets its partner half a row away from lane ^ (LPR / 2).  The normed rows are never stored.
template <int LPR>
__device__ __forceinline__ void rope_norm_rows(const RopeDesc &d, uint32_t block, uint32_t n_blocks) {
  const uint64_t total = (uint64_t)d.b * d.h * d.s * LPR;  // a multiple of LPR, as 256 is: a row's lanes stay together
  for (uint64_t i = (uint64_t)block * 256 + threadIdx.x; i < total; i += (uint64_t)n_blocks * 256) {
    const uint32_t j = (uint32_t)(i % LPR) * 4;
    uint64_t r = i / LPR;
    const uint32_t s = (uint32_t)(r % d.s);
    r /= d.s;
    const uint32_t h = (uint32_t)(r % d.h), b = (uint32_t)(r / d.h);
    const float4 xv = *(const float4 *)(d.x + (int64_t)b * d.x_sb + (int64_t)h * d.x_sh + (int64_t)s * d.x_ss + j);
    const float4 c = *(const float4 *)(d.cos + (int64_t)s * d.cs_ss + j);
    const float4 sn = *(const float4 *)(d.sin + (int64_t)s * d.cs_ss + j);
    float4 g = make_float4(0.f, 0.f, 0.f, 0.f);
    if (d.gamma) g = *(const float4 *)(d.gamma + j);
    float ss = xv.x * xv.x + xv.y * xv.y + xv.z * xv.z + xv.w * xv.w;
    ss = group_sum<LPR>(ss);
    const float rms = sqrtf(ss / d.n_as_float + d.eps);  // (a true square root and true divisions, as in rmsnorm_kernel)
    float4 y;
    y.x = xv.x / rms; y.y = xv.y / rms; y.z = xv.z / rms; y.w = xv.w / rms;
    if (d.gamma) {
      y.x *= d.gamma_offset + g.x; y.y *= d.gamma_offset + g.y;
      y.z *= d.gamma_offset + g.z; y.w *= d.gamma_offset + g.w;
    }
    float4 pv;
    pv.x = __shfl_xor(y.x, LPR / 2); pv.y = __shfl_xor(y.y, LPR / 2);
    pv.z = __shfl_xor(y.z, LPR / 2); pv.w = __shfl_xor(y.w, LPR / 2);
    if (j < d.half) { pv.x = -pv.x; pv.y = -pv.y; pv.z = -pv.z; pv.w = -pv.w; }
    float4 o;
    o.x = c.x * y.x + sn.x * pv.x; o.y = c.y * y.y + sn.y * pv.y;
    o.z = c.z * y.z + sn.z * pv.z; o.w = c.w * y.w + sn.w * pv.w;
    const int64_t oo = (int64_t)b * d.o_sb + (int64_t)h * d.o_sh + (int64_t)s * d.o_ss + j;
    *(float4 *)(d.out + oo) = o;
    if (d.out16) *(uint2 *)(d.out16 + oo) = bf16_pack4(o);
  }
}

__device__ __forceinline__ void rope_any_rows(const RopeDesc &d, uint32_t block, uint32_t n_blocks) {
  if (!d.norm) rope_rows(d, block, n_blocks);
  else if (d.dim == 256) rope_norm_rows<64>(d, block, n_blocks);
  else if (d.dim == 128) rope_norm_rows<32>(d, block, n_blocks);
  else rope_norm_rows<16>(d, block, n_blocks);
}

__global__ void __launch_bounds__(256) rope_kernel(RopeDesc d) {
  rope_any_rows(d, blockIdx.x, gridDim.x);
}

// queries and keys of one attention in one launch: the first blocks0 workgroups rotate d0, the rest d1
__global__ void __launch_bounds__(256) rope_pair_kernel(RopeDesc d0, RopeDesc d1, uint32_t blocks0) {
  if (blockIdx.x < blocks0) rope_any_rows(d0, blockIdx.x, blocks0);
  else rope_any_rows(d1, blockIdx.x - blocks0, gridDim.x - blocks0);
}

static unsigned rope_blocks(const LaunchCtx &lc, const RopeDesc &d) {
  const uint64_t total = (uint64_t)d.b * d.h * d.s * (d.dim / 4);
  const uint64_t blocks = (total + 255) / 256, cap = (uint64_t)lc.n_cus * 8;
  return (unsigned)(blocks < cap ? blocks : cap);
}

hipError_t launch_rope(const LaunchCtx &lc, const RopeDesc &d) {
  if (d.norm && d.dim != 64 && d.dim != 128 && d.dim != 256) return hipErrorInvalidValue;
  const unsigned blocks = rope_blocks(lc, d);
  if (!blocks) return hipSuccess;
  CG_LAUNCH(lc, (rope_kernel), blocks, 256, d);
  return hipGetLastError();
}

hipError_t launch_rope_pair(const LaunchCtx &lc, const RopeDesc &d0, const RopeDesc &d1) {
  for (const RopeDesc *d : {&d0, &d1})
    if (d->norm && d->dim != 64 && d->dim != 128 && d->dim != 256) return hipErrorInvalidValue;
  const unsigned b0 = rope_blocks(lc, d0), b1 = rope_blocks(lc, d1);
  if (!b0) return launch_rope(lc, d1);
  if (!b1) return launch_rope(lc, d0);
  CG_LAUNCH(lc, (rope_pair_kernel), b0 + b1, 256, d0, d1, (uint32_t)b0);
  return hipGetLastError();
}

// ---- gated activations --------------------------------------------------------------------------------
template <bool GELU>
__global__ void __launch_bounds__(256) glu_kernel(const float *gate, const float *up, float *out,
                                                  uint64_t n4, uint16_t *out16) {
  for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n4;
       i += (uint64_t)gridDim.x * 256) {
    const float4 g = ((const float4 *)gate)[i], u = ((const float4 *)up)[i];
    float4 o;
    if (GELU) {
      o.x = gelu_ref(g.x) * u.x; o.y = gelu_ref(g.y) * u.y;
      o.z = gelu_ref(g.z) * u.z; o.w = gelu_ref(g.w) * u.w;
    } else {
      o.x = g.x * sigmoid_ref(g.x) * u.x; o.y = g.y * sigmoid_ref(g.y) * u.y;
      o.z = g.z * sigmoid_ref(g.z) * u.z; o.w = g.w * sigmoid_ref(g.w) * u.w;
    }
    ((float4 *)out)[i] = o;
    if (out16) ((uint2 *)out16)[i] = bf16_pack4(o);
  }
}

// ---- a sum of rows, each scaled by a value of its own ------------------------------------------------
// One thread owns four consecutive columns of one row: it asks for its piece of every term and for every
// term's scale at once, then adds them up in the order given.
__global__ void __launch_bounds__(256) row_scaled_sum_kernel(RowSumDesc g) {
  const uint32_t per_row = g.d / 4, total = g.rows * per_row;
  for (uint32_t p = blockIdx.x * 256 + threadIdx.x; p < total; p += gridDim.x * 256) {
    const uint32_t row = p / per_row, c = (p - row * per_row) * 4;
    float4 xv[ROW_SUM_MAX_TERMS];
    float sv[ROW_SUM_MAX_TERMS];
#pragma unroll
    for (int j = 0; j < ROW_SUM_MAX_TERMS; ++j)
      if ((uint32_t)j < g.n_terms) {
        xv[j] = *(const float4 *)(g.t[j].x + (int64_t)row * g.t[j].x_rs + c);
        sv[j] = g.t[j].s ? g.t[j].s[(int64_t)row * g.t[j].s_rs] : 1.0f;
      }
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int j = 0; j < ROW_SUM_MAX_TERMS; ++j)
      if ((uint32_t)j < g.n_terms) {
        float4 t = xv[j];
        if (g.t[j].s) {
          const float w = g.t[j].sigmoid ? sigmoid_ref(sv[j]) : sv[j];
          t.x = __fmul_rn(t.x, w); t.y = __fmul_rn(t.y, w); t.z = __fmul_rn(t.z, w); t.w = __fmul_rn(t.w, w);
        }
        if (j == 0) {
          acc = t;
        } else {
          acc.x = __fadd_rn(acc.x, t.x); acc.y = __fadd_rn(acc.y, t.y);
          acc.z = __fadd_rn(acc.z, t.z); acc.w = __fadd_rn(acc.w, t.w);
        }
      }
    *(float4 *)(g.out + (int64_t)row * g.out_rs + c) = acc;
  }
}

hipError_t launch_row_scaled_sum(const LaunchCtx &lc, const RowSumDesc &g) {
  if (!g.rows || !g.d) return hipSuccess;
  if (g.n_terms < 1 || g.n_terms > ROW_SUM_MAX_TERMS || g.d % 4 || (uintptr_t)g.out % 16 || g.out_rs % 4 ||
      (uint64_t)g.rows * (g.d / 4) >= (1ull << 32))
    return hipErrorInvalidValue;
  for (uint32_t j = 0; j < g.n_terms; ++j)
    if (!g.t[j].x || (uintptr_t)g.t[j].x % 16 || g.t[j].x_rs % 4) return hipErrorInvalidValue;
  const uint64_t total = (uint64_t)g.rows * (g.d / 4);
  uint64_t blocks = (total + 255) / 256;
  const uint64_t cap = (uint64_t)lc.n_cus * 8;
  if (blocks > cap) blocks = cap;
  CG_LAUNCH(lc, row_scaled_sum_kernel, (unsigned)blocks, 256, g);
  return hipGetLastError();
}

hipError_t launch_glu(const LaunchCtx &lc, int gelu, const float *gate, const float *up, float *out,
                      uint64_t n, uint16_t *out16) {
  if (!n) return hipSuccess;
  const uint64_t n4 = n / 4;
  uint64_t blocks = (n4 + 255) / 256, cap = (uint64_t)lc.n_cus * 8;
  const unsigned grid = (unsigned)(blocks < cap ? blocks : cap);
  if (gelu) CG_LAUNCH(lc, (glu_kernel<true>), grid, 256, gate, up, out, n4, out16);
  else CG_LAUNCH(lc, (glu_kernel<false>), grid, 256, gate, up, out, n4, out16);
  return hipGetLastError();
}

// ---- one f32 binary op, a contiguous, b contiguous or a row vector repeated over rows ---------------
// A16: a is stored as bf16 (an uploaded matrix used directly in an elementwise op)
template <int OP, bool A16>
__global__ void __launch_bounds__(256) binary_kernel(const float *a, const float *b, float *out,
                                                     uint64_t n4, uint32_t b_period4) {
  for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n4;
       i += (uint64_t)gridDim.x * 256) {
    float4 x;
    if (A16) {
      const uint2 h = ((const uint2 *)a)[i];
      x = make_float4(__uint_as_float(h.x << 16), __uint_as_float(h.x & 0xFFFF0000u), __uint_as_float(h.y << 16),
                      __uint_as_float(h.y & 0xFFFF0000u));
    } else {
      x = ((const float4 *)a)[i];
    }
    const float4 y = ((const float4 *)b)[b_period4 ? i % b_period4 : i];
    float4 o;
    if (OP == 0) { o.x = x.x + y.x; o.y = x.y + y.y; o.z = x.z + y.z; o.w = x.w + y.w; }
    if (OP == 1) { o.x = x.x - y.x; o.y = x.y - y.y; o.z = x.z - y.z; o.w = x.w - y.w; }
    if (OP == 2) { o.x = x.x * y.x; o.y = x.y * y.y; o.z = x.z * y.z; o.w = x.w * y.w; }
    if (OP == 3) { o.x = x.x / y.x; o.y = x.y / y.y; o.z = x.z / y.z; o.w = x.w / y.w; }
    ((float4 *)out)[i] = o;
  }
}

hipError_t launch_binary_f32(const LaunchCtx &lc, int op, const float *a, const float *b, float *out,
                             uint64_t n, uint32_t b_period, bool a_bf16) {
  if (!n) return hipSuccess;
  const uint64_t n4 = n / 4;
  uint64_t blocks = (n4 + 255) / 256, cap = (uint64_t)lc.n_cus * 16;
  const unsigned grid = (unsigned)(blocks < cap ? blocks : cap);
  const uint32_t p4 = b_period / 4;
  if (a_bf16) {
    switch (op) {
      case 0: CG_LAUNCH(lc, (binary_kernel<0, true>), grid, 256, a, b, out, n4, p4); break;
      case 1: CG_LAUNCH(lc, (binary_kernel<1, true>), grid, 256, a, b, out, n4, p4); break;
      case 2: CG_LAUNCH(lc, (binary_kernel<2, true>), grid, 256, a, b, out, n4, p4); break;
      default: CG_LAUNCH(lc, (binary_kernel<3, true>), grid, 256, a, b, out, n4, p4); break;
    }
    return hipGetLastError();
  }
  switch (op) {
    case 0: CG_LAUNCH(lc, (binary_kernel<0, false>), grid, 256, a, b, out, n4, p4); break;
    case 1: CG_LAUNCH(lc, (binary_kernel<1, false>), grid, 256, a, b, out, n4, p4); break;
    case 2: CG_LAUNCH(lc, (binary_kernel<2, false>), grid, 256, a, b, out, n4, p4); break;
    default: CG_LAUNCH(lc, (binary_kernel<3, false>), grid, 256, a, b, out, n4, p4); break;
  }
  return hipGetLastError();
}

}  // namespace cgk
