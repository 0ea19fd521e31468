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


}  // namespace cgk
