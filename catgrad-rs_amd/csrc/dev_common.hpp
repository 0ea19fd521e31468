// dev_common.hpp — device helpers shared by the kernel files: wavefront / workgroup reductions and
// the activation formulas of the stdlib definitions.
#pragma once
#include <hip/hip_runtime.h>
#include <math.h>

namespace cgk {

// A kernel whose argument is a large descriptor reads it field by field as its control flow reaches
// each use: a chain of dependent scalar loads, each a trip of ~0.17 us to the argument segment in
// device memory when its 64-byte line is not in the scalar cache yet (eight of them, 1.2 us, stood in
// front of the first weight request of a one-row product in a stand-alone harness).  Touching every
// line of the descriptor at the top, all at once, turns the chain into cache hits: one trip, then the
// fields as they are needed.  Used by the one-row product kernels, where it measured faster inside a
// decode step as well (0.1 - 0.7 us per launch); kernels with short chains lose the up-front wait.
// (Reads only; the wait inside the statement means the scratch registers are dead when it ends.)
template <int OFF, int LINES>
__device__ __forceinline__ void warm_kernel_argument_lines() {
  const auto ka = __builtin_amdgcn_kernarg_segment_ptr();
  uint32_t t0, t1, t2, t3, t4, t5, t6, t7;
  constexpr int LAST = OFF + (LINES - 1) * 64;  // fewer than eight lines: the last one is touched again
#define CG_KA_LINE(i) (OFF + (i) * 64 < LAST ? OFF + (i) * 64 : LAST)
  asm volatile("s_load_dword %0, %8, %9\n\ts_load_dword %1, %8, %10\n\ts_load_dword %2, %8, %11\n\t"
               "s_load_dword %3, %8, %12\n\ts_load_dword %4, %8, %13\n\ts_load_dword %5, %8, %14\n\t"
               "s_load_dword %6, %8, %15\n\ts_load_dword %7, %8, %16\n\ts_waitcnt lgkmcnt(0)"
               : "=&s"(t0), "=&s"(t1), "=&s"(t2), "=&s"(t3), "=&s"(t4), "=&s"(t5), "=&s"(t6), "=&s"(t7)
               : "s"(ka), "i"(CG_KA_LINE(0)), "i"(CG_KA_LINE(1)), "i"(CG_KA_LINE(2)), "i"(CG_KA_LINE(3)),
                 "i"(CG_KA_LINE(4)), "i"(CG_KA_LINE(5)), "i"(CG_KA_LINE(6)), "i"(CG_KA_LINE(7))
               : "memory");
#undef CG_KA_LINE
}
// BYTES: size of the kernel's arguments (they start at offset 0 of the segment)
template <int BYTES>
__device__ __forceinline__ void warm_kernel_arguments() {
  constexpr int LINES = (BYTES + 63) / 64;
  static_assert(LINES >= 1 && LINES <= 24, "descriptor size");
  warm_kernel_argument_lines<0, (LINES < 8 ? LINES : 8)>();
  if constexpr (LINES > 8) warm_kernel_argument_lines<512, (LINES - 8 < 8 ? LINES - 8 : 8)>();
  if constexpr (LINES > 16) warm_kernel_argument_lines<1024, LINES - 16>();
}

// Sum over the 64 lanes of a wavefront (all active); every lane gets it.  The exchanges are DPP operands
// of the adds, not trips through the LDS crossbar: inside each row of 16 lanes quad permutes (distances
// 1 and 2) and the mirrors of 8 and 16 lanes - after which every lane of a row holds the row's sum -
// then lane 15 of rows 0 and 2 is added into rows 1 and 3 (row_bcast15), lane 31 into rows 2 and 3
// (row_bcast31), and lane 63 holds the total.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_add(float v) {
  return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xF, ROW_MASK == 0xF));
}
__device__ __forceinline__ float wave_sum(float v) {
  v = dpp_add<0xB1, 0xF>(v);   // quad_perm [1, 0, 3, 2]
  v = dpp_add<0x4E, 0xF>(v);   // quad_perm [2, 3, 0, 1]
  v = dpp_add<0x141, 0xF>(v);  // row_half_mirror
  v = dpp_add<0x140, 0xF>(v);  // row_mirror
  v = dpp_add<0x142, 0xA>(v);  // row_bcast15 into rows 1 and 3
  v = dpp_add<0x143, 0xC>(v);  // row_bcast31 into rows 2 and 3
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, 64));
  return v;
}

// The largest value over the 64 lanes of a wavefront (all active), in every lane: the exchanges of wave_sum
// with a maximum in place of the sum (lanes a step does not write keep their own value).
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int32_t dpp_max_i32(int32_t v) {
  const int32_t o = __builtin_amdgcn_update_dpp(v, v, CTRL, ROW_MASK, 0xF, false);
  return o > v ? o : v;
}
__device__ __forceinline__ int32_t wave_max_i32(int32_t v) {
  v = dpp_max_i32<0xB1, 0xF>(v);
  v = dpp_max_i32<0x4E, 0xF>(v);
  v = dpp_max_i32<0x141, 0xF>(v);
  v = dpp_max_i32<0x140, 0xF>(v);
  v = dpp_max_i32<0x142, 0xA>(v);
  v = dpp_max_i32<0x143, 0xC>(v);
  return __builtin_amdgcn_readlane(v, 63);
}

// f32::total_cmp as an integer order
__device__ __forceinline__ int32_t total_key_f(float v) {
  int32_t b = __float_as_int(v);
  return b ^ (int32_t)(((uint32_t)(b >> 31)) >> 1);
}

// topk(softmax(row)) by one wavefront (all 64 lanes active) over a row of n <= 64 * EPT values: the
// probabilities exactly as softmax_kernel<64, EPT> computes them (same folds, same order), then k selection
// rounds in the order of Backend::topk (ndarray.rs:495-520: descending, equal values by ascending index).
// emit(t, value, index) is called in every lane, with the same arguments, for t = 0 .. k - 1.
template <int EPT, typename Emit>
__device__ __forceinline__ void softmax_topk_row(const float *xr, uint32_t n, uint32_t k, uint32_t lane, Emit emit) {
  float v[EPT];
  float mx = -3.40282347e+38f;  // max folds from f32::MIN (ndarray.rs:455-460)
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const uint32_t c = lane + e * 64;
    if (c < n) {
      v[e] = xr[c];
      mx = fmaxf(mx, v[e]);
    }
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const uint32_t c = lane + e * 64;
    if (c < n) {
      v[e] = expf(v[e] - mx);
      sum += v[e];
    }
  }
  sum = wave_sum(sum);
#pragma unroll
  for (int e = 0; e < EPT; ++e) v[e] = v[e] / sum;
  int32_t prev_key = 0;
  uint32_t prev_idx = 0;
  if constexpr (EPT == 1) {
    // a lane holds one value and its column is its lane: the largest eligible key by a wavefront maximum, the
    // first lane that holds it by a ballot (no trips through the LDS crossbar)
    const int32_t key = lane < n ? total_key_f(v[0]) : INT32_MIN;
    for (uint32_t t = 0; t < k; ++t) {
      const bool eligible = lane < n && (t == 0 || key < prev_key || (key == prev_key && lane > prev_idx));
      const int32_t best = wave_max_i32(eligible ? key : INT32_MIN);
      const unsigned long long holders = __ballot(eligible && key == best);
      const uint32_t bi = holders ? (uint32_t)__builtin_ctzll(holders) : 0xFFFFFFFFu;
      const float bv = holders ? __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v[0]), (int)(bi & 63u))) : 0.f;
      prev_key = best;
      prev_idx = bi;
      emit(t, bv, bi);
    }
    return;
  }
  for (uint32_t t = 0; t < k; ++t) {
    int32_t bk = 0;
    uint32_t bi = 0xFFFFFFFFu;  // none
    float bv = 0.f;
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const uint32_t c = lane + e * 64;
      if (c < n) {
        const int32_t key = total_key_f(v[e]);
        const bool eligible = t == 0 || key < prev_key || (key == prev_key && c > prev_idx);
        if (eligible && (bi == 0xFFFFFFFFu || key > bk || (key == bk && c < bi))) {
          bk = key;
          bi = c;
          bv = v[e];
        }
      }
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
      const int32_t ok = __shfl_xor(bk, m, 64);
      const uint32_t oi = (uint32_t)__shfl_xor((int)bi, m, 64);
      const float ov = __shfl_xor(bv, m, 64);
      if (oi != 0xFFFFFFFFu && (bi == 0xFFFFFFFFu || ok > bk || (ok == bk && oi < bi))) {
        bk = ok;
        bi = oi;
        bv = ov;
      }
    }
    prev_key = bk;
    prev_idx = bi;
    emit(t, bv, bi);
  }
}

// Sum over aligned groups of LANES lanes (a power of two, 2 .. 64); every lane of a group gets the sum.
// The lanes of a group must be active together.
template <int LANES>
__device__ __forceinline__ float group_sum(float v) {
  if (LANES >= 64) return wave_sum(v);
  if (LANES >= 2) v = dpp_add<0xB1, 0xF>(v);
  if (LANES >= 4) v = dpp_add<0x4E, 0xF>(v);
  if (LANES >= 8) v = dpp_add<0x141, 0xF>(v);
  if (LANES >= 16) v = dpp_add<0x140, 0xF>(v);
  if (LANES >= 32) v += __shfl_xor(v, 16, 64);
  return v;
}

// Reduce across the workgroup (BLOCK threads, a multiple of 64); every thread gets the result.
template <int BLOCK, bool IS_MAX>
__device__ __forceinline__ float block_reduce(float v, float *lds) {
  v = IS_MAX ? wave_max(v) : wave_sum(v);
  if (BLOCK == 64) return v;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) lds[wave] = v;
  __syncthreads();
  float r = lds[0];
#pragma unroll
  for (int w = 1; w < BLOCK / 64; ++w) r = IS_MAX ? fmaxf(r, lds[w]) : r + lds[w];
  return r;
}

// f32 -> bf16, round to nearest even (NaN stays NaN); two values packed low / high
__device__ __forceinline__ uint32_t bf16_bits(float f) {
  const uint32_t u = __float_as_uint(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (u >> 16) | 0x40u;
  return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}
__device__ __forceinline__ uint2 bf16_pack4(float4 v) {
  return make_uint2(bf16_bits(v.x) | (bf16_bits(v.y) << 16), bf16_bits(v.z) | (bf16_bits(v.w) << 16));
}

__device__ __forceinline__ float sigmoid_ref(float x) { return 1.0f / (1.0f + expf(-x)); }
// nn::gelu: 0.5 x (1 + tanh(c (x + k x^3))), tanh(t) = 2 sigmoid(2 t) - 1 (nn/mod.rs:138-160)
__device__ __forceinline__ float gelu_ref(float x) {
  const float t = __uint_as_float(0x3F4C4229u) * (x + 0.044715f * (x * x * x));  // f32 sqrt(2/pi)
  const float th = 2.0f * sigmoid_ref(2.0f * t) - 1.0f;
  return 0.5f * x * (1.0f + th);
}

// The gated activations where the result leaves as bf16 only (the stacked gate / up GEMM of a bf16-mode prefill):
// the hardware's exp2 and reciprocal in place of expf and the division.  gelu(x) = x * sigmoid(2 t) and
// silu(x) = x * sigmoid(x) exactly; the approximations are good to a few units of the last place of an f32, far
// inside the rounding of the bf16 value that is stored, and cost a third of the instructions (a 256 x 128 tile
// spends 64 activations per lane between two main loops).
__device__ __forceinline__ float sigmoid_fast(float x) {
  return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.44269504f));
}
__device__ __forceinline__ float silu_fast(float x) { return x * sigmoid_fast(x); }
__device__ __forceinline__ float gelu_fast(float x) {
  const float t = __uint_as_float(0x3F4C4229u) * (x + 0.044715f * (x * x * x));
  return x * sigmoid_fast(2.0f * t);
}


}  // namespace cgk
