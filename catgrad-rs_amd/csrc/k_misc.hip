// k_misc.hip — index/gather, top-k, compare and fill kernels for gfx950.
//
// Backend::index  (mod.rs:66-71, ndarray.rs:373-381): select(Axis(dim), flattened indices)
// Backend::topk   (mod.rs:58,    ndarray.rs:495-520): stable sort by descending total_cmp
// Backend::compare(mod.rs:59,    ndarray.rs:337-343): shape and element equality
// All HBM- or latency-bound; index moves 16 bytes per lane along the innermost axis.
#include <hip/hip_runtime.h>
#include <algorithm>
#include <cstdlib>
#include "launch.hpp"
#include "dev_common.hpp"

namespace cgk {

template <int VEC>
__global__ void __launch_bounds__(256) gather_kernel(GatherDesc g, uint64_t n_groups,
                                                     uint32_t *err) {
  for (uint64_t t = (uint64_t)blockIdx.x * 256 + threadIdx.x; t < n_groups;
       t += (uint64_t)gridDim.x * 256) {
    uint64_t lin = t * VEC;
    uint64_t rem = lin;
    int64_t off = 0;
#pragma unroll
    for (int d = MAX_DIMS + 1; d >= 0; --d) {
      if (d < g.n_dims) {
        uint32_t c;
        if (d == 0) {
          c = (uint32_t)rem;
        } else {
          uint64_t q = rem / g.out_dims[d];
          c = (uint32_t)(rem - q * g.out_dims[d]);
          rem = q;
        }
        if (d == g.dim) {
          uint32_t ix = g.idx[c];
          if (ix >= g.x_dim_size) {  // the reference panics; flag it and stay in bounds
            atomicOr(err, ERRF_INDEX_OOB);
            ix = g.x_dim_size - 1;
          }
          c = ix;
        }
        off += (int64_t)c * g.x_stride[d];
      }
    }
    const int64_t inner = g.x_stride[g.n_dims - 1];
    uint32_t v[VEC];
    if (g.x_stype == ST_BF16) {
      const uint16_t *p = (const uint16_t *)g.x + off;
      if (VEC == 4 && g.vec) {
        uint2 q = *(const uint2 *)p;
        v[0] = q.x << 16; v[1 % VEC] = q.x & 0xFFFF0000u;
        v[2 % VEC] = q.y << 16; v[3 % VEC] = q.y & 0xFFFF0000u;
      } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = (uint32_t)p[j * inner] << 16;
      }
    } else {
      const uint32_t *p = (const uint32_t *)g.x + off;
      if (VEC == 4 && g.vec) {
        uint4 q = *(const uint4 *)p;
        v[0] = q.x; v[1 % VEC] = q.y; v[2 % VEC] = q.z; v[3 % VEC] = q.w;
      } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = p[j * inner];
      }
    }
    uint32_t *o = (uint32_t *)g.out + lin;
    if (VEC == 4) {
      *(uint4 *)o = make_uint4(v[0], v[1 % VEC], v[2 % VEC], v[3 % VEC]);
    } else {
      o[0] = v[0];
    }
  }
}

// Rows of a bf16 matrix by index (an embedding lookup in bf16 mode, helpers.rs:259-271: `index(0, ids, table)`),
// widened to f32: a wavefront owns an output row, reads its index once and streams the row - four values per lane
// and 8-byte load, U loads in flight, 16-byte stores - instead of decomposing every element's position with
// 64-bit divisions and keeping one short load in flight per lane.
template <typename T, int U>
__global__ void __launch_bounds__(256) gather_rows_kernel(const T *x, int64_t x_row_stride, const uint32_t *idx,
                                                          uint32_t x_rows, uint32_t *out, uint32_t rows, uint32_t n,
                                                          uint32_t *err) {
  const uint32_t lane = threadIdx.x & 63;
  for (uint32_t row = blockIdx.x * 4 + (threadIdx.x >> 6); row < rows; row += gridDim.x * 4) {  // (uniform per wave)
    uint32_t ix = idx[row];
    if (ix >= x_rows) {  // the reference panics; flag it and stay in bounds
      if (lane == 0) atomicOr(err, ERRF_INDEX_OOB);
      ix = x_rows - 1;
    }
    const T *src = x + (int64_t)ix * x_row_stride;
    uint32_t *dst = out + (uint64_t)row * n;
    for (uint32_t c0 = lane * 4; c0 < n; c0 += 64 * 4 * U) {
      uint4 v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t c = c0 + u * 256;
        if (c < n) {
          if (sizeof(T) == 4) {
            v[u] = *(const uint4 *)(src + c);
          } else {
            const uint2 q = *(const uint2 *)(src + c);
            v[u] = make_uint4(q.x << 16, q.x & 0xFFFF0000u, q.y << 16, q.y & 0xFFFF0000u);
          }
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t c = c0 + u * 256;
        if (c < n) *(uint4 *)(dst + c) = v[u];
      }
    }
  }
}

hipError_t launch_gather(const LaunchCtx &lc, const GatherDesc &g, uint64_t n_out) {
  if (!n_out) return hipSuccess;
  // (rows of 4-byte values stay on the generic kernel: the same row kernel moved them at 3.3 TB/s whatever its
  // grid, against 5 TB/s for the kernel below, whose consecutive waves take consecutive pieces of a row)
  if (g.vec && g.x_stype == ST_BF16 && g.n_dims == 2 && g.dim == 0 && g.x_stride[1] == 1 && g.out_dims[1] % 4 == 0 &&
      g.out_dims[1] >= 256 && g.out_dims[0] >= (uint32_t)lc.n_cus && (uintptr_t)g.out % 16 == 0) {  // (a wave per row: enough rows)
    const uint32_t rows = g.out_dims[0], n = g.out_dims[1];
    const uint32_t blocks = std::min((rows + 3) / 4, (uint32_t)lc.n_cus * 16u);
    CG_LAUNCH(lc, (gather_rows_kernel<uint16_t, 8>), blocks, 256, (const uint16_t *)g.x, g.x_stride[0], g.idx,
              g.x_dim_size, (uint32_t *)g.out, rows, n, lc.err_flag);
    return hipGetLastError();
  }
  const bool vec = g.vec && g.dim != g.n_dims - 1 && (g.out_dims[g.n_dims - 1] % 4 == 0);
  uint64_t groups = vec ? n_out / 4 : n_out;
  uint64_t blocks = (groups + 255) / 256, cap = (uint64_t)lc.n_cus * 8;
  unsigned grid = (unsigned)(blocks < cap ? blocks : cap);
  if (vec) CG_LAUNCH(lc, (gather_kernel<4>), grid, 256, g, groups, lc.err_flag);
  else CG_LAUNCH(lc, (gather_kernel<1>), grid, 256, g, groups, lc.err_flag);
  return hipGetLastError();
}


// One wavefront per row.  Round t selects the t-th element of the order
// (key descending, index ascending) = what a stable descending sort yields.
__global__ void __launch_bounds__(256) topk_kernel(const float *x, float *values, uint32_t *indices,
                                                   uint32_t rows, uint32_t n, uint32_t k) {
  const int lane = threadIdx.x & 63;
  const uint32_t row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const float *lane_x = x + (uint64_t)row * n;
  int32_t prev_key = 0;
  uint32_t prev_idx = 0;
  for (uint32_t t = 0; t < k; ++t) {
    int32_t bk = 0;
    uint32_t bi = 0xFFFFFFFFu;  // none
    for (uint32_t c = lane; c < n; c += 64) {
      int32_t key = total_key_f(lane_x[c]);
      bool eligible = t == 0 || key < prev_key || (key == prev_key && c > prev_idx);
      if (eligible && (bi == 0xFFFFFFFFu || key > bk || (key == bk && c < bi))) {
        bk = key;
        bi = c;
      }
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
      int32_t ok = __shfl_xor(bk, m, 64);
      uint32_t oi = (uint32_t)__shfl_xor((int)bi, m, 64);
      if (oi != 0xFFFFFFFFu && (bi == 0xFFFFFFFFu || ok > bk || (ok == bk && oi < bi))) {
        bk = ok;
        bi = oi;
      }
    }
    prev_key = bk;
    prev_idx = bi;
    if (lane == 0) {
      values[(uint64_t)row * k + t] = lane_x[bi];
      indices[(uint64_t)row * k + t] = bi;
    }
  }
}

// The router of a MoE layer (models/qwen3.rs:64-80): topk(softmax(x)) over rows of at most 256
// logits.  One wavefront per row keeps the row in registers: the probabilities are computed exactly
// as softmax_kernel<64, EPT> computes them (same folds, same order), then the selection rounds of
// topk_kernel run on the registers - no launch and no [rows, n] tensor in between.
template <int EPT>
__global__ void __launch_bounds__(256) softmax_topk_kernel(const float *x, int64_t x_row_stride, float *values, uint32_t *indices,
                                                           uint32_t rows, uint32_t n, uint32_t k) {
  const uint32_t lane = threadIdx.x, row = blockIdx.x * 4 + threadIdx.y;
  if (row >= rows) return;  // the whole wave exits together
  softmax_topk_row<EPT>(x + (int64_t)row * x_row_stride, n, k, lane, [&](uint32_t t, float bv, uint32_t bi) {
    if (lane == 0) {
      values[(uint64_t)row * k + t] = bv;
      indices[(uint64_t)row * k + t] = bi;
    }
  });
}

hipError_t launch_softmax_topk(const LaunchCtx &lc, const float *x, int64_t x_row_stride, float *values, uint32_t *indices,
                               uint32_t rows, uint32_t n, uint32_t k) {
  if (!rows || !k) return hipSuccess;
  if (n > 256 || k > n) return hipErrorInvalidValue;
  if (n <= 64) CG_LAUNCH(lc, (softmax_topk_kernel<1>), (rows + 3) / 4, dim3(64, 4), x, x_row_stride, values, indices, rows, n, k);
  else CG_LAUNCH(lc, (softmax_topk_kernel<4>), (rows + 3) / 4, dim3(64, 4), x, x_row_stride, values, indices, rows, n, k);
  return hipGetLastError();
}

hipError_t launch_topk(const LaunchCtx &lc, const float *x, float *values, uint32_t *indices,
                       uint32_t rows, uint32_t n, uint32_t k) {
  if (!rows || !k) return hipSuccess;
  CG_LAUNCH(lc, (topk_kernel), (rows + 3) / 4, 256, x, values, indices, rows, n, k);
  return hipGetLastError();
}

__global__ void __launch_bounds__(256) compare_kernel(const uint32_t *a, const uint32_t *b,
                                                      uint64_t n, int is_f32, uint32_t *flag) {
  bool diff = false;
  for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n;
       i += (uint64_t)gridDim.x * 256) {
    if (is_f32) diff |= !(__uint_as_float(a[i]) == __uint_as_float(b[i]));
    else diff |= a[i] != b[i];
  }
  if (diff) atomicOr(flag, 1u);
}

hipError_t launch_compare(const LaunchCtx &lc, const void *a, const void *b, uint64_t n,
                          int is_f32, uint32_t *flag) {
  if (!n) return hipSuccess;
  uint64_t blocks = (n + 255) / 256, cap = (uint64_t)lc.n_cus * 8;
  CG_LAUNCH(lc, (compare_kernel), (unsigned)(blocks < cap ? blocks : cap), 256, 
      (const uint32_t *)a, (const uint32_t *)b, n, is_f32, flag);
  return hipGetLastError();
}

__global__ void __launch_bounds__(256) fill_kernel(uint32_t *dst, uint32_t value, uint64_t n) {
  for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n;
       i += (uint64_t)gridDim.x * 256)
    dst[i] = value;
}

hipError_t launch_fill_u32(const LaunchCtx &lc, uint32_t *dst, uint32_t value, uint64_t n) {
  if (!n) return hipSuccess;
  uint64_t blocks = (n + 255) / 256, cap = (uint64_t)lc.n_cus * 8;
  CG_LAUNCH(lc, (fill_kernel), (unsigned)(blocks < cap ? blocks : cap), 256, dst, value, n);
  return hipGetLastError();
}

// ---- materialised transpose ------------------------------------------------------------------------------
// T: input element (uint16_t = bf16); OUT16: bf16 stays bf16, otherwise 4-byte output (bf16 widened)
template <typename T, bool OUT16>
__global__ void __launch_bounds__(256) transpose_copy_kernel(TransposeDesc d) {
  __shared__ uint32_t tile[64][65];
  // blockIdx.z enumerates the other axes
  uint32_t rem = blockIdx.z;
  int64_t xo = 0, oo = 0;
  for (int i = d.n_other - 1; i >= 0; --i) {
    const uint32_t c = rem % d.odims[i];
    rem /= d.odims[i];
    xo += (int64_t)c * d.x_so[i];
    oo += (int64_t)c * d.o_so[i];
  }
  const T *x = (const T *)d.x + xo;
  uint32_t *out = (uint32_t *)d.out + (OUT16 ? 0 : oo);
  uint16_t *out16 = (uint16_t *)d.out + oo;
  const uint32_t c0 = blockIdx.x * 64, j0 = blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const uint32_t c = c0 + ty + i * 4, j = j0 + tx;
    if (c < d.C && j < d.R) {
      const T v = x[(int64_t)c * d.x_sc + j];
      tile[ty + i * 4][tx] = (sizeof(T) == 2 && !OUT16) ? (uint32_t)v << 16 : (uint32_t)v;
    }
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const uint32_t j = j0 + ty + i * 4, c = c0 + tx;
    if (j < d.R && c < d.C) {
      if (OUT16) out16[(int64_t)j * d.o_sj + c] = (uint16_t)tile[tx][ty + i * 4];
      else out[(int64_t)j * d.o_sj + c] = tile[tx][ty + i * 4];
    }
  }
}

// The same for 4-byte elements whose rows allow 16-byte moves on both sides (R, C, the strides and the bases
// multiples of four elements): a lane loads four values of an input row and stores four values of an output
// row; the 64 x 64 tile turns around in LDS word by word (pitch 65: two lanes per bank at worst).  Four times
// the bytes per request of the kernel above, which left a transposed copy at 4.1 TB/s where a plain copy
// reaches 4.9.
__global__ void __launch_bounds__(256) transpose_copy_vec_kernel(TransposeDesc d) {
  __shared__ uint32_t tile[64][65];
  uint32_t rem = blockIdx.z;
  int64_t xo = 0, oo = 0;
  for (int i = d.n_other - 1; i >= 0; --i) {
    const uint32_t c = rem % d.odims[i];
    rem /= d.odims[i];
    xo += (int64_t)c * d.x_so[i];
    oo += (int64_t)c * d.o_so[i];
  }
  const uint32_t *x = (const uint32_t *)d.x + xo;
  uint32_t *out = (uint32_t *)d.out + oo;
  const uint32_t c0 = blockIdx.x * 64, j0 = blockIdx.y * 64;
  const uint32_t q4 = (threadIdx.x & 15) * 4, rr = threadIdx.x >> 4;
  uint4 v[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t c = c0 + rr + i * 16, j = j0 + q4;
    if (c < d.C && j < d.R) v[i] = *(const uint4 *)(x + (int64_t)c * d.x_sc + j);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t r = rr + i * 16;
    tile[r][q4] = v[i].x; tile[r][q4 + 1] = v[i].y; tile[r][q4 + 2] = v[i].z; tile[r][q4 + 3] = v[i].w;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t jr = rr + i * 16, j = j0 + jr, c = c0 + q4;
    if (j < d.R && c < d.C)
      *(uint4 *)(out + (int64_t)j * d.o_sj + c) = make_uint4(tile[q4][jr], tile[q4 + 1][jr], tile[q4 + 2][jr], tile[q4 + 3][jr]);
  }
}

hipError_t launch_transpose_copy(const LaunchCtx &lc, const TransposeDesc &d) {
  uint64_t other = 1;
  for (int i = 0; i < d.n_other; ++i) other *= d.odims[i];
  if (!d.R || !d.C || !other) return hipSuccess;
  dim3 grid((d.C + 63) / 64, (d.R + 63) / 64, (unsigned)other);
  if (d.x_stype != ST_BF16 && !d.out_bf16 && d.R % 4 == 0 && d.C % 4 == 0 && d.x_sc % 4 == 0 && d.o_sj % 4 == 0 &&
      (uintptr_t)d.x % 16 == 0 && (uintptr_t)d.out % 16 == 0) {
    bool ok = true;
    for (int i = 0; i < d.n_other; ++i) ok = ok && d.x_so[i] % 4 == 0 && d.o_so[i] % 4 == 0;
    if (ok) {
      CG_LAUNCH(lc, (transpose_copy_vec_kernel), grid, 256, d);
      return hipGetLastError();
    }
  }
  if (d.x_stype == ST_BF16 && d.out_bf16) CG_LAUNCH(lc, (transpose_copy_kernel<uint16_t, true>), grid, 256, d);
  else if (d.x_stype == ST_BF16) CG_LAUNCH(lc, (transpose_copy_kernel<uint16_t, false>), grid, 256, d);
  else CG_LAUNCH(lc, (transpose_copy_kernel<uint32_t, false>), grid, 256, d);
  return hipGetLastError();
}

// ---- peak probes --------------------------------------------------------------------------------------
// What the machine gives to the simplest possible code, as denominators next to the data-sheet
// numbers: a grid-stride 16-byte copy (HBM read + write) and a register-resident MFMA issue loop.
__global__ void __launch_bounds__(256) peak_copy_kernel(const uint4 *in, uint4 *out, uint64_t n) {
  for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256)
    out[i] = in[i];
}

hipError_t launch_peak_copy(const LaunchCtx &lc, const void *in, void *out, uint64_t bytes) {
  CG_LAUNCH(lc, (peak_copy_kernel), (unsigned)lc.n_cus * 8, 256, (const uint4 *)in, (uint4 *)out, bytes / 16);
  return hipGetLastError();
}

typedef __attribute__((ext_vector_type(8))) __bf16 pk_bf16x8;
typedef __attribute__((ext_vector_type(16))) float pk_f32x16;

template <bool BF16>
__global__ void __launch_bounds__(256) peak_mfma_kernel(float *out, int iters, unsigned long long *clock_ticks) {
  // (optional) shader-clock ticks and 100 MHz ticks of the loop, summed over the workgroups: the clock it ran at
  const unsigned long long tick0 = __builtin_amdgcn_s_memtime(), real0 = __builtin_amdgcn_s_memrealtime();
  pk_f32x16 acc[4];
  for (int i = 0; i < 4; ++i)
    for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
  pk_bf16x8 a, b;
  for (int e = 0; e < 8; ++e) {
    a[e] = (__bf16)(float)((threadIdx.x + e) & 3);
    b[e] = (__bf16)(float)(e & 1);
  }
  const float fa = (float)(threadIdx.x & 3), fb = 1.0f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (BF16) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[i], 0, 0, 0);
      else acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa, fb, acc[i], 0, 0, 0);
    }
  }
  float s = 0.f;
  for (int i = 0; i < 4; ++i)
    for (int e = 0; e < 16; ++e) s += acc[i][e];
  out[(uint64_t)blockIdx.x * 256 + threadIdx.x] = s;
  if (clock_ticks && threadIdx.x == 0) {
    atomicAdd(clock_ticks, __builtin_amdgcn_s_memtime() - tick0);
    atomicAdd(clock_ticks + 1, __builtin_amdgcn_s_memrealtime() - real0);
  }
}

// flops issued: grid * 4 waves * iters * 4 MFMAs * (2 * 32 * 32 * k), k = 16 (bf16) or 2 (f32)
hipError_t launch_peak_mfma(const LaunchCtx &lc, int bf16, float *out, unsigned grid, int iters, unsigned long long *clock_ticks) {
  if (bf16) CG_LAUNCH(lc, (peak_mfma_kernel<true>), grid, 256, out, iters, clock_ticks);
  else CG_LAUNCH(lc, (peak_mfma_kernel<false>), grid, 256, out, iters, clock_ticks);
  return hipGetLastError();
}

}  // namespace cgk
