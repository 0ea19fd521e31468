// k_ew.hip — fused elementwise programs and last-axis reductions for gfx950.
//
// Serves Backend::{add,sub,mul,div,pow,lt,eq,sin,cos,neg,cast,broadcast,zeros,arange} and the
// materialising forms of reshape/transpose/slice/concat (one strided pass), and
// Backend::{sum,max,argmax} with an optional elementwise prologue
// (catgrad/src/interpreter/backend/mod.rs:26-57; semantics: ndarray.rs:97-114, 164-246, 401-493).
//
// All of these are HBM-bound.  The kernels therefore (a) read each operand through its own
// strides so views are never materialised, (b) move 16 bytes per lane whenever the innermost
// stride allows it, (c) use grid-stride loops sized to the 256 CUs, and (d) evaluate a whole
// expression tree per element so intermediates never touch memory.
//
// The evaluator is a stack machine whose stack lives in VGPRs: every instruction carries the
// stack depth at which it runs, so register indices are compile-time constants inside a
// wave-uniform switch (no scratch memory, no divergence).
#include <hip/hip_runtime.h>
#include <math.h>
#include "program.hpp"
#include "launch.hpp"

namespace cgk {

__device__ __forceinline__ float as_f(uint32_t u) { return __uint_as_float(u); }
__device__ __forceinline__ uint32_t as_u(float f) { return __float_as_uint(f); }

// Rust `f32 as u32`: truncate toward zero, saturate, NaN -> 0 (ndarray.rs:101)
__device__ __forceinline__ uint32_t f2u_sat(float v) {
  if (!(v == v) || v <= 0.f) return 0u;
  if (v >= 4294967296.f) return 0xFFFFFFFFu;
  return (uint32_t)v;
}

__device__ __forceinline__ uint32_t upow(uint32_t a, uint32_t e) {
  uint32_t r = 1;
  while (e) {
    if (e & 1) r *= a;
    a *= a;
    e >>= 1;
  }
  return r;
}

__device__ __forceinline__ uint32_t f32_to_bf16_rne(uint32_t u) {
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (u >> 16) | 0x40u;  // quiet NaN
  return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

// pow(x, 0.5) with powf's answers at the points where sqrtf differs
__device__ __forceinline__ float sqrt_like_pow(float x) {
  if (x == 0.f) return 0.f;
  if (x == -INFINITY) return INFINITY;
  return sqrtf(x);
}

// powf / sinf / cosf expand to hundreds of instructions each; kept out of line so that the
// interpreter loop stays inside the instruction cache (they are rare in model graphs: exp,
// sqrt, cube and reciprocal have their own cheap opcodes)
__device__ __noinline__ float nf_pow(float a, float b) { return powf(a, b); }
__device__ __noinline__ float nf_sin(float a) { return sinf(a); }
__device__ __noinline__ float nf_cos(float a) { return cosf(a); }

__device__ __forceinline__ uint32_t apply_bin(uint8_t op, uint32_t a, uint32_t b, uint32_t *err) {
  switch (op) {
    case E_ADD_F: return as_u(as_f(a) + as_f(b));
    case E_SUB_F: return as_u(as_f(a) - as_f(b));
    case E_MUL_F: return as_u(as_f(a) * as_f(b));
    case E_DIV_F: return as_u(as_f(a) / as_f(b));
    case E_POW_F: return as_u(nf_pow(as_f(a), as_f(b)));
    case E_LT_F: return as_u(as_f(a) < as_f(b) ? 1.f : 0.f);
    case E_EQ_F: return as_u(as_f(a) == as_f(b) ? 1.f : 0.f);
    case E_ADD_U: return a + b;
    case E_SUB_U: return a - b;
    case E_MUL_U: return a * b;
    case E_DIV_U:
      if (b == 0u) {
        atomicOr(err, ERRF_DIV_ZERO);
        return 0xFFFFFFFFu;
      }
      return a / b;
    case E_POW_U: return upow(a, b);
    case E_LT_U: return a < b ? 1u : 0u;
    case E_EQ_U: return a == b ? 1u : 0u;
    default: return 0u;
  }
}

__device__ __forceinline__ uint32_t apply_un(uint8_t op, uint32_t a) {
  switch (op) {
    case E_NEG_F: return a ^ 0x80000000u;
    case E_NEG_U: return 0u - a;
    case E_SIN_F: return as_u(nf_sin(as_f(a)));
    case E_COS_F: return as_u(nf_cos(as_f(a)));
    case E_F2U: return f2u_sat(as_f(a));
    case E_U2F: return as_u((float)a);
    case E_EXP_F: return as_u(expf(as_f(a)));
    case E_SQRT_F: return as_u(sqrt_like_pow(as_f(a)));
    case E_CUBE_F: { float x = as_f(a); return as_u(x * x * x); }
    case E_RCP_F: return as_u(1.0f / as_f(a));
    default: return 0u;
  }
}

// A program staged in LDS (ST) is read with vector instructions; the values that steer control
// flow are the same in every lane and go back to scalar registers so that branches stay uniform.
template <bool ST>
__device__ __forceinline__ uint32_t uni(uint32_t v) {
  return ST ? (uint32_t)__builtin_amdgcn_readfirstlane((int)v) : v;
}

// Load VEC consecutive elements (along the innermost dim) of one operand at element offset off.
template <int VEC, bool ST = false>
__device__ __forceinline__ void load_vec(const Operand &in, int64_t off, int64_t inner,
                                         uint32_t *v) {
  const uint32_t stype = uni<ST>((uint32_t)in.stype), vec = uni<ST>((uint32_t)in.vec);
  if (stype == ST_BF16) {
    const uint16_t *p = (const uint16_t *)in.ptr + off;
    if (VEC == 4 && vec) {
      uint2 q = *(const uint2 *)p;
      v[0] = q.x << 16; v[1 % VEC] = q.x & 0xFFFF0000u;
      v[2 % VEC] = q.y << 16; v[3 % VEC] = q.y & 0xFFFF0000u;
    } else {
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[j] = (uint32_t)p[j * inner] << 16;
    }
  } else {
    const uint32_t *p = (const uint32_t *)in.ptr + off;
    if (VEC == 4 && vec) {
      uint4 q = *(const uint4 *)p;
      v[0] = q.x; v[1 % VEC] = q.y; v[2 % VEC] = q.z; v[3 % VEC] = q.w;
    } else if (uni<ST>((uint32_t)(inner == 0))) {
      uint32_t s = p[0];
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[j] = s;
    } else {
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[j] = p[j * inner];
    }
  }
}

#define CG_DEPTHS(M) \
  case 0: M(0) break; case 1: M(1) break; case 2: M(2) break; case 3: M(3) break; \
  case 4: M(4) break; case 5: M(5) break; case 6: M(6) break; case 7: M(7) break;

// Evaluate code[pc0, pc1) for K chunks of VEC consecutive elements.  Chunk k starts at inner
// coordinate c0 + k * cstride (idx[] holds the outer coordinates; its innermost entry is
// ignored); chunk k is skipped when bit k of `valid` is clear.  Running one instruction over
// K * VEC elements amortises the (wave-uniform) instruction decode.
// All K chunks of one operand for this thread.
template <int VEC, int K, bool ST = false>
__device__ __forceinline__ void load_chunks(const Program &p, int slot,
                                            const uint32_t (&idx)[MAX_DIMS], uint32_t c0,
                                            uint32_t cstride, uint32_t valid,
                                            uint32_t (&t)[K * VEC]) {
  const Operand &in = p.in[slot];
  const int n_dims = (int)uni<ST>((uint32_t)p.n_dims);
  int64_t off = 0;
#pragma unroll
  for (int d = 0; d < MAX_DIMS - 1; ++d)
    if (d < n_dims - 1) off += (int64_t)idx[d] * in.stride[d];
  const int64_t inner = in.stride[n_dims - 1];
#pragma unroll
  for (int k = 0; k < K; ++k) {
    if (valid & (1u << k)) {
      load_vec<VEC, ST>(in, off + (int64_t)(c0 + k * cstride) * inner, inner, &t[k * VEC]);
    } else {
#pragma unroll
      for (int j = 0; j < VEC; ++j) t[k * VEC + j] = 0u;
    }
  }
}

template <int VEC, int K, bool ST = false>
__device__ __forceinline__ void eval_program(const Program &p, int pc0, int pc1,
                                             const uint32_t (&idx)[MAX_DIMS], uint32_t c0,
                                             uint32_t cstride, uint32_t valid, uint32_t row0,
                                             uint32_t row1, uint32_t *err,
                                             uint32_t (&res)[K * VEC]) {
  constexpr int E = K * VEC;
  uint32_t r[MAX_STACK][E];
  for (int pc = pc0; pc < pc1; ++pc) {
    Instr ins;
    if (ST) {
      const uint32_t w = uni<ST>(*(const uint32_t *)&p.code[pc]);
      ins.op = (uint8_t)(w & 0xFFu);
      ins.depth = (uint8_t)((w >> 8) & 0xFFu);
      ins.arg = (uint16_t)(w >> 16);
    } else {
      ins = p.code[pc];
    }
    if (ins.op <= E_ROW1) {
      uint32_t t[E];
      if (ins.op == E_LOAD) {
        load_chunks<VEC, K, ST>(p, ins.arg, idx, c0, cstride, valid, t);
      } else if (ins.op == E_IOTA) {
#pragma unroll
        for (int k = 0; k < K; ++k)
#pragma unroll
          for (int j = 0; j < VEC; ++j) t[k * VEC + j] = c0 + k * cstride + j;
      } else {
        uint32_t c = ins.op == E_CONST ? uni<ST>(p.imm[ins.arg]) : (ins.op == E_ROW0 ? row0 : row1);
#pragma unroll
        for (int j = 0; j < E; ++j) t[j] = c;
      }
      switch (ins.depth) {
#define M(d) _Pragma("unroll") for (int j = 0; j < E; ++j) r[d][j] = t[j];
        CG_DEPTHS(M)
#undef M
      }
    } else if (ins.op <= E_EQ_U) {
      uint32_t a[E], b[E];
      switch (ins.depth) {
#define M(d) _Pragma("unroll") for (int j = 0; j < E; ++j) { \
    a[j] = r[(d) >= 2 ? (d)-2 : 0][j]; b[j] = r[(d) >= 1 ? (d)-1 : 0][j]; }
        CG_DEPTHS(M)
#undef M
        case 8:
#pragma unroll
          for (int j = 0; j < E; ++j) { a[j] = r[6][j]; b[j] = r[7][j]; }
          break;
      }
#pragma unroll
      for (int j = 0; j < E; ++j) a[j] = apply_bin(ins.op, a[j], b[j], err);
      switch (ins.depth) {
#define M(d) _Pragma("unroll") for (int j = 0; j < E; ++j) r[(d) >= 2 ? (d)-2 : 0][j] = a[j];
        CG_DEPTHS(M)
#undef M
        case 8:
#pragma unroll
          for (int j = 0; j < E; ++j) r[6][j] = a[j];
          break;
      }
    } else {
      uint32_t a[E];
      switch (ins.depth) {
#define M(d) _Pragma("unroll") for (int j = 0; j < E; ++j) a[j] = r[(d) >= 1 ? (d)-1 : 0][j];
        CG_DEPTHS(M)
#undef M
        case 8:
#pragma unroll
          for (int j = 0; j < E; ++j) a[j] = r[7][j];
          break;
      }
#pragma unroll
      for (int j = 0; j < E; ++j) a[j] = apply_un(ins.op, a[j]);
      switch (ins.depth) {
#define M(d) _Pragma("unroll") for (int j = 0; j < E; ++j) r[(d) >= 1 ? (d)-1 : 0][j] = a[j];
        CG_DEPTHS(M)
#undef M
        case 8:
#pragma unroll
          for (int j = 0; j < E; ++j) r[7][j] = a[j];
          break;
      }
    }
  }
#pragma unroll
  for (int j = 0; j < E; ++j) res[j] = r[0][j];
}

template <bool ST = false>
__device__ __forceinline__ void decompose(const Program &p, uint64_t lin,
                                          uint32_t (&idx)[MAX_DIMS]) {
  // all programs stay below 2^32 elements (checked on the host)
  uint32_t rem = (uint32_t)lin;
  const int n_dims = (int)uni<ST>((uint32_t)p.n_dims);
#pragma unroll
  for (int d = MAX_DIMS - 1; d >= 0; --d) {
    if (d < n_dims) {
      if (d == 0) {
        idx[d] = rem;
      } else {
        uint32_t q = rem / p.dims[d];
        idx[d] = rem - q * p.dims[d];
        rem = q;
      }
    } else {
      idx[d] = 0;
    }
  }
}

// The evaluator of a small launch.  Such a launch spends its time fetching instructions, not data: it
// starts with a cold instruction cache, and the register-file evaluator above is a few hundred
// cache lines of unrolled moves (one copy per stack depth) that a short program hops across.  Here
// the stack lives in LDS, indexed by the depth the instruction carries, so the code is one compact
// loop: a load path and one case per opcode, each written once for the VEC elements of a thread.
template <int VEC>
__device__ __forceinline__ void bin_vec(uint32_t op, const uint32_t *a, const uint32_t *b, uint32_t *r, uint32_t *err) {
#define CG_BIN(EXPR) _Pragma("unroll") for (int j = 0; j < VEC; ++j) { const uint32_t x = a[j * 256], y = b[j * 256]; r[j * 256] = (EXPR); } break;
  switch (op) {
    case E_ADD_F: CG_BIN(as_u(as_f(x) + as_f(y)))
    case E_SUB_F: CG_BIN(as_u(as_f(x) - as_f(y)))
    case E_MUL_F: CG_BIN(as_u(as_f(x) * as_f(y)))
    case E_DIV_F: CG_BIN(as_u(as_f(x) / as_f(y)))
    case E_POW_F: CG_BIN(as_u(nf_pow(as_f(x), as_f(y))))
    case E_LT_F: CG_BIN(as_u(as_f(x) < as_f(y) ? 1.f : 0.f))
    case E_EQ_F: CG_BIN(as_u(as_f(x) == as_f(y) ? 1.f : 0.f))
    case E_ADD_U: CG_BIN(x + y)
    case E_SUB_U: CG_BIN(x - y)
    case E_MUL_U: CG_BIN(x * y)
    case E_POW_U: CG_BIN(upow(x, y))
    case E_LT_U: CG_BIN(x < y ? 1u : 0u)
    case E_EQ_U: CG_BIN(x == y ? 1u : 0u)
    default: CG_BIN(apply_bin((uint8_t)op, x, y, err))  // E_DIV_U: flags a zero divisor
  }
#undef CG_BIN
}

template <int VEC>
__device__ __forceinline__ void un_vec(uint32_t op, uint32_t *a) {
#define CG_UN(EXPR) _Pragma("unroll") for (int j = 0; j < VEC; ++j) { const uint32_t x = a[j * 256]; a[j * 256] = (EXPR); } break;
  switch (op) {
    case E_NEG_F: CG_UN(x ^ 0x80000000u)
    case E_EXP_F: CG_UN(as_u(expf(as_f(x))))
    case E_RCP_F: CG_UN(as_u(1.0f / as_f(x)))
    case E_SQRT_F: CG_UN(as_u(sqrt_like_pow(as_f(x))))
    case E_CUBE_F: CG_UN(as_u(as_f(x) * as_f(x) * as_f(x)))
    default: CG_UN(apply_un((uint8_t)op, x))
  }
#undef CG_UN
}

// `stk` points at this thread's column of the LDS stack: element j of depth d is stk[(d * VEC + j) * 256]
template <int VEC>
__device__ __forceinline__ void eval_program_small(const Program &p, int n_instr, const uint32_t (&idx)[MAX_DIMS],
                                                   uint32_t c0, uint32_t *err, uint32_t *stk, uint32_t (&res)[VEC]) {
  for (int pc = 0; pc < n_instr; ++pc) {
    const uint32_t w = uni<true>(*(const uint32_t *)&p.code[pc]);
    const uint32_t op = w & 0xFFu, depth = (w >> 8) & 0xFFu, arg = w >> 16;
    uint32_t *top = stk + depth * VEC * 256;  // where a push lands
    if (op <= E_ROW1) {
      uint32_t t[VEC];
      if (op == E_LOAD) {
        load_chunks<VEC, 1, true>(p, (int)arg, idx, c0, 0u, 1u, t);
      } else if (op == E_IOTA) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) t[j] = c0 + j;
      } else {  // plain programs have no reduction stages: E_CONST
        const uint32_t c = uni<true>(p.imm[arg]);
#pragma unroll
        for (int j = 0; j < VEC; ++j) t[j] = c;
      }
#pragma unroll
      for (int j = 0; j < VEC; ++j) top[j * 256] = t[j];
    } else if (op <= E_EQ_U) {
      bin_vec<VEC>(op, top - 2 * VEC * 256, top - VEC * 256, top - 2 * VEC * 256, err);
    } else {
      un_vec<VEC>(op, top - VEC * 256);
    }
  }
#pragma unroll
  for (int j = 0; j < VEC; ++j) res[j] = stk[j * 256];
}

// ST: the launch is small (every thread runs the program once).  Walking the program through the
// kernel-argument segment costs one scalar-cache miss per operand descriptor and code line, one
// after the other, in memory the host has just written - most of such a launch's duration.  All
// threads copy the program into LDS in one round trip instead and the walk reads it from there.
template <int VEC, bool ST>
__global__ void __launch_bounds__(256) ew_kernel(const Program pk, OutDesc o, uint64_t n_groups,
                                                 uint32_t *err) {
  __shared__ __attribute__((aligned(16))) uint32_t staged[ST ? sizeof(Program) / 4 : 4];
  __shared__ uint32_t stack[ST ? MAX_STACK * VEC * 256 : 1];
  if (ST) {
    static_assert(sizeof(Program) % 16 == 0, "program copied in 16-byte pieces");
    const uint4 *src = (const uint4 *)&pk;
    for (uint32_t i = threadIdx.x; i < sizeof(Program) / 16; i += 256) ((uint4 *)staged)[i] = src[i];
    __syncthreads();
  }
  const Program &p = ST ? *(const Program *)staged : pk;
  const int n_dims = (int)uni<ST>((uint32_t)p.n_dims);
  const int n_instr = (int)uni<ST>((uint32_t)p.n_instr);
  for (uint64_t g = (uint64_t)blockIdx.x * 256 + threadIdx.x; g < n_groups;
       g += (uint64_t)gridDim.x * 256) {
    uint32_t idx[MAX_DIMS];
    const uint64_t lin = g * VEC;
    decompose<ST>(p, lin, idx);
    uint32_t v[VEC];
    uint32_t c0 = 0;
#pragma unroll
    for (int d = 0; d < MAX_DIMS; ++d)
      if (d == n_dims - 1) c0 = idx[d];
    // rank-1 programs (the only ones with E_IOTA) have c0 == lin
    if (ST) eval_program_small<VEC>(p, n_instr, idx, c0, err, stack + threadIdx.x, v);
    else eval_program<VEC, 1, false>(p, 0, n_instr, idx, c0, 0u, 1u, 0u, 0u, err, v);
    int64_t off = 0;
#pragma unroll
    for (int d = 0; d < MAX_DIMS; ++d)
      if (d < n_dims) off += (int64_t)idx[d] * o.stride[d];
    const int64_t inner = o.stride[n_dims - 1];
    if (o.stype == ST_BF16) {
      uint16_t *q = (uint16_t *)o.ptr + off;
#pragma unroll
      for (int j = 0; j < VEC; ++j) q[j * inner] = (uint16_t)f32_to_bf16_rne(v[j]);
    } else {
      uint32_t *q = (uint32_t *)o.ptr + off;
      if (VEC == 4 && o.vec) {
        *(uint4 *)q = make_uint4(v[0], v[1 % VEC], v[2 % VEC], v[3 % VEC]);
      } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) q[j * inner] = v[j];
      }
    }
  }
}

// ---- reductions over the innermost program dim -------------------------------------------------

// f32::total_cmp key (monotone signed integer)
__device__ __forceinline__ int32_t total_key(uint32_t bits) {
  int32_t b = (int32_t)bits;
  return b ^ (int32_t)(((uint32_t)(b >> 31)) >> 1);
}

template <int KIND> struct Acc;
// Every accumulator exposes its state as W 32-bit words (for shuffles and LDS), without
// type punning.
template <> struct Acc<R_SUM_F> {
  enum { W = 1 };
  float v = 0.f;
  __device__ void add(uint32_t x, uint32_t) { v += as_f(x); }
  __device__ void merge(const Acc &o) { v += o.v; }
  __device__ uint32_t result() const { return as_u(v); }
  __device__ void get(uint32_t *w) const { w[0] = as_u(v); }
  __device__ void set(const uint32_t *w) { v = as_f(w[0]); }
};
template <> struct Acc<R_SUM_U> {
  enum { W = 1 };
  uint32_t v = 0;
  __device__ void add(uint32_t x, uint32_t) { v += x; }
  __device__ void merge(const Acc &o) { v += o.v; }
  __device__ uint32_t result() const { return v; }
  __device__ void get(uint32_t *w) const { w[0] = v; }
  __device__ void set(const uint32_t *w) { v = w[0]; }
};
// fold(f32::MIN, f32::max): NaN ignored, floor at f32::MIN (ndarray.rs:455-460)
template <> struct Acc<R_MAX_F> {
  enum { W = 1 };
  float v = -3.40282347e+38f;
  __device__ void add(uint32_t x, uint32_t) { v = fmaxf(v, as_f(x)); }
  __device__ void merge(const Acc &o) { v = fmaxf(v, o.v); }
  __device__ uint32_t result() const { return as_u(v); }
  __device__ void get(uint32_t *w) const { w[0] = as_u(v); }
  __device__ void set(const uint32_t *w) { v = as_f(w[0]); }
};
template <> struct Acc<R_MAX_U> {
  enum { W = 1 };
  uint32_t v = 0;
  __device__ void add(uint32_t x, uint32_t) { v = x > v ? x : v; }
  __device__ void merge(const Acc &o) { v = o.v > v ? o.v : v; }
  __device__ uint32_t result() const { return v; }
  __device__ void get(uint32_t *w) const { w[0] = v; }
  __device__ void set(const uint32_t *w) { v = w[0]; }
};
// max_by(total_cmp): the LAST of equal maxima wins (ndarray.rs:469-480).  `any` = 0 marks an
// accumulator that has seen no element yet.
template <> struct Acc<R_ARGMAX_F> {
  enum { W = 3 };
  int32_t k = INT32_MIN;
  uint32_t i = 0, any = 0;
  __device__ void add(uint32_t x, uint32_t col) {
    int32_t kk = total_key(x);
    if (!any || kk > k || (kk == k && col > i)) { k = kk; i = col; any = 1; }
  }
  __device__ void merge(const Acc &o) {
    if (o.any && (!any || o.k > k || (o.k == k && o.i > i))) { k = o.k; i = o.i; any = 1; }
  }
  __device__ uint32_t result() const { return i; }
  __device__ void get(uint32_t *w) const { w[0] = (uint32_t)k; w[1] = i; w[2] = any; }
  __device__ void set(const uint32_t *w) { k = (int32_t)w[0]; i = w[1]; any = w[2]; }
};
template <> struct Acc<R_ARGMAX_U> {
  enum { W = 3 };
  uint32_t k = 0, i = 0, any = 0;
  __device__ void add(uint32_t x, uint32_t col) {
    if (!any || x > k || (x == k && col > i)) { k = x; i = col; any = 1; }
  }
  __device__ void merge(const Acc &o) {
    if (o.any && (!any || o.k > k || (o.k == k && o.i > i))) { k = o.k; i = o.i; any = 1; }
  }
  __device__ uint32_t result() const { return i; }
  __device__ void get(uint32_t *w) const { w[0] = k; w[1] = i; w[2] = any; }
  __device__ void set(const uint32_t *w) { k = w[0]; i = w[1]; any = w[2]; }
};

template <int KIND>
__device__ __forceinline__ Acc<KIND> shfl_xor_acc(const Acc<KIND> &a, int m) {
  uint32_t w[Acc<KIND>::W];
  a.get(w);
#pragma unroll
  for (int j = 0; j < Acc<KIND>::W; ++j) w[j] = (uint32_t)__shfl_xor((int)w[j], m, 64);
  Acc<KIND> r;
  r.set(w);
  return r;
}

// ---- reductions of a tensor that is already in memory ------------------------------------------------
// No program to interpret: rows of n unit-stride elements (f32 / u32 words, or bf16 widened to f32)
// streamed with 16-byte (8-byte for bf16) loads, four in flight per lane.  One row per workgroup
// (WPR = 4) or per wavefront (WPR = 1).
// W: values per load - 4, or 8 for bf16 rows whose pieces of 16 bytes are aligned (n, row stride % 8 == 0):
// with 8-byte requests a bf16 row has half the bytes in flight and - one short row per workgroup - the launch is
// paced by workgroup turnover, not by memory; short bf16 rows therefore also go a wave per row.
template <int KIND, typename T, int WPR, int W = 4>
__global__ void __launch_bounds__(256) reduce_plain_kernel(const T *x, int64_t row_stride, uint32_t *out,
                                                           uint32_t rows, uint32_t n) {
  __shared__ uint32_t part[4][Acc<KIND>::W];
  constexpr int U = 4;
  static_assert(W == 4 || (W == 8 && sizeof(T) == 2), "eight values per load: bf16 only");
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t row = WPR == 4 ? blockIdx.x : blockIdx.x * 4 + wave;
  const uint32_t t_in_row = WPR == 4 ? threadIdx.x : lane, tpr = WPR * 64;
  Acc<KIND> acc;
  // argmax over floats, the order of f32::total_cmp with the last of equal values winning (the Acc above), as one
  // 64-bit maximum: ordered bits of the value << 32 | column.  A thread meets its columns in increasing order,
  // so inside a thread "not smaller" replaces; 0 stands for "nothing seen" and loses to every element but
  // (smallest value, column 0), which is the same answer.  A third of the instructions of the three-word form,
  // which kept bf16 rows (half the bytes) from streaming at memory speed.
  uint32_t best_u = 0, best_c = 0;
  if (row < rows) {
    const T *r = x + (int64_t)row * row_stride;
    for (uint32_t c0 = t_in_row * W; c0 < n; c0 += tpr * W * U) {
      uint32_t v[U][W];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t c = c0 + u * tpr * W;
        if (c < n) {
          if (sizeof(T) == 4) {
            const uint4 q = *(const uint4 *)(r + c);
            v[u][0] = q.x; v[u][1] = q.y; v[u][2] = q.z; v[u][3] = q.w;
          } else if (W == 8) {
            const uint4 q = *(const uint4 *)(r + c);
            const uint32_t h[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              v[u][(2 * k) % W] = h[k] << 16;
              v[u][(2 * k + 1) % W] = h[k] & 0xFFFF0000u;
            }
          } else {
            const uint2 q = *(const uint2 *)(r + c);
            v[u][0] = q.x << 16; v[u][1] = q.x & 0xFFFF0000u; v[u][2] = q.y << 16; v[u][3] = q.y & 0xFFFF0000u;
          }
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t c = c0 + u * tpr * W;
        if (c < n) {
#pragma unroll
          for (int j = 0; j < W; ++j) {
            if constexpr (KIND == R_ARGMAX_F) {
              const uint32_t b = v[u][j], o = b ^ ((uint32_t)((int32_t)b >> 31) | 0x80000000u);  // total_cmp order, unsigned
              const bool take = o >= best_u;
              best_u = take ? o : best_u;
              best_c = take ? c + j : best_c;
            } else {
              acc.add(v[u][j], c + j);
            }
          }
        }
      }
    }
  }
  if constexpr (KIND == R_ARGMAX_F) {
    uint64_t best = (uint64_t)best_u << 32 | best_c;
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
      const uint64_t o = (uint64_t)(uint32_t)__shfl_xor((int)(best >> 32), m, 64) << 32 | (uint32_t)__shfl_xor((int)(uint32_t)best, m, 64);
      best = o > best ? o : best;
    }
    if (WPR == 4) {
      if (lane == 0) {
        part[wave][0] = (uint32_t)(best >> 32);
        part[wave][1] = (uint32_t)best;
      }
      __syncthreads();
      if (threadIdx.x == 0) {
        for (int w2 = 1; w2 < 4; ++w2) {
          const uint64_t o = (uint64_t)part[w2][0] << 32 | part[w2][1];
          best = o > best ? o : best;
        }
        out[row] = (uint32_t)best;
      }
    } else if (lane == 0 && row < rows) {
      out[row] = (uint32_t)best;
    }
    return;
  }
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) acc.merge(shfl_xor_acc<KIND>(acc, m));
  if (WPR == 4) {
    if (lane == 0) acc.get(part[wave]);
    __syncthreads();
    if (threadIdx.x == 0) {
      for (int w2 = 1; w2 < 4; ++w2) {
        Acc<KIND> o;
        o.set(part[w2]);
        acc.merge(o);
      }
      out[row] = acc.result();
    }
  } else if (lane == 0 && row < rows) {
    out[row] = acc.result();
  }
}

template <int KIND>
static void launch_reduce_plain_kind(const LaunchCtx &lc, const void *x, int bf16, int64_t row_stride, uint32_t *out,
                                     uint32_t rows, uint32_t n) {
  if (bf16 && n % 8 == 0 && row_stride % 8 == 0 && (uintptr_t)x % 16 == 0) {
    if (n > 8192) CG_LAUNCH(lc, (reduce_plain_kernel<KIND, uint16_t, 4, 8>), rows, 256, (const uint16_t *)x, row_stride, out, rows, n);
    else CG_LAUNCH(lc, (reduce_plain_kernel<KIND, uint16_t, 1, 8>), (rows + 3) / 4, 256, (const uint16_t *)x, row_stride, out, rows, n);
    return;
  }
  if (n >= 1024) {
    if (bf16) CG_LAUNCH(lc, (reduce_plain_kernel<KIND, uint16_t, 4>), rows, 256, (const uint16_t *)x, row_stride, out, rows, n);
    else CG_LAUNCH(lc, (reduce_plain_kernel<KIND, uint32_t, 4>), rows, 256, (const uint32_t *)x, row_stride, out, rows, n);
  } else {
    if (bf16) CG_LAUNCH(lc, (reduce_plain_kernel<KIND, uint16_t, 1>), (rows + 3) / 4, 256, (const uint16_t *)x, row_stride, out, rows, n);
    else CG_LAUNCH(lc, (reduce_plain_kernel<KIND, uint32_t, 1>), (rows + 3) / 4, 256, (const uint32_t *)x, row_stride, out, rows, n);
  }
}

hipError_t launch_reduce_plain(const LaunchCtx &lc, int kind, const void *x, int bf16, int64_t row_stride, void *out,
                               uint32_t rows, uint32_t n) {
  if (!rows) return hipSuccess;
  uint32_t *o = (uint32_t *)out;
  switch (kind) {
    case R_SUM_F: launch_reduce_plain_kind<R_SUM_F>(lc, x, bf16, row_stride, o, rows, n); break;
    case R_SUM_U: launch_reduce_plain_kind<R_SUM_U>(lc, x, bf16, row_stride, o, rows, n); break;
    case R_MAX_F: launch_reduce_plain_kind<R_MAX_F>(lc, x, bf16, row_stride, o, rows, n); break;
    case R_MAX_U: launch_reduce_plain_kind<R_MAX_U>(lc, x, bf16, row_stride, o, rows, n); break;
    case R_ARGMAX_F: launch_reduce_plain_kind<R_ARGMAX_F>(lc, x, bf16, row_stride, o, rows, n); break;
    case R_ARGMAX_U: launch_reduce_plain_kind<R_ARGMAX_U>(lc, x, bf16, row_stride, o, rows, n); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

// One row per workgroup (WAVES_PER_ROW = 4) or per wavefront (WAVES_PER_ROW = 1).
template <int KIND, int VEC, int WAVES_PER_ROW>
__global__ void __launch_bounds__(256) reduce_kernel(const Program p, uint32_t *out, uint32_t rows,
                                                     uint32_t n, uint32_t *err) {
  __shared__ uint32_t part[4][Acc<KIND>::W];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t rows_per_block = 4 / WAVES_PER_ROW;
  const uint32_t tid_in_row = WAVES_PER_ROW == 4 ? threadIdx.x : lane;
  const uint32_t threads_per_row = WAVES_PER_ROW * 64;
  for (uint32_t rb = blockIdx.x * rows_per_block; rb < rows; rb += gridDim.x * rows_per_block) {
    const uint32_t row = rb + (WAVES_PER_ROW == 4 ? 0 : wave);
    Acc<KIND> acc;
    if (row < rows) {
      uint32_t idx[MAX_DIMS];
      // outer coordinates: decompose the row number over dims[0 .. n_dims-2]
      uint32_t rem = row;
#pragma unroll
      for (int d = MAX_DIMS - 2; d >= 0; --d) {
        if (d < p.n_dims - 1) {
          if (d == 0) {
            idx[d] = rem;
          } else {
            uint32_t q = rem / p.dims[d];
            idx[d] = rem - q * p.dims[d];
            rem = q;
          }
        } else {
          idx[d] = 0;
        }
      }
      idx[MAX_DIMS - 1] = 0;
      for (uint32_t c = tid_in_row * VEC; c < n; c += threads_per_row * VEC) {
        // the innermost coordinate lives at position n_dims-1
#pragma unroll
        for (int d = 0; d < MAX_DIMS; ++d)
          if (d == p.n_dims - 1) idx[d] = c;
        uint32_t v[VEC];
        eval_program<VEC, 1>(p, 0, p.n_instr, idx, c, 0u, 1u, 0u, 0u, err, v);
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc.add(v[j], c + j);
      }
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) acc.merge(shfl_xor_acc<KIND>(acc, m));
    if (WAVES_PER_ROW == 4) {
      __syncthreads();
      if (lane == 0) acc.get(part[wave]);
      __syncthreads();
      if (threadIdx.x == 0) {
        for (int w2 = 1; w2 < 4; ++w2) {
          Acc<KIND> o;
          o.set(part[w2]);
          acc.merge(o);
        }
        out[row] = acc.result();
      }
    } else if (lane == 0 && row < rows) {
      out[row] = acc.result();
    }
  }
}

// ---- row programs: reduction stages + a final elementwise segment in one kernel --------------------
__device__ __forceinline__ uint32_t red_init(int kind) {
  switch (kind) {
    case R_MAX_F: return 0xFF7FFFFFu;  // f32::MIN
    default: return 0u;                // 0.0f and 0u share the bit pattern
  }
}
__device__ __forceinline__ uint32_t red_combine(int kind, uint32_t a, uint32_t b) {
  switch (kind) {
    case R_SUM_F: return as_u(as_f(a) + as_f(b));
    case R_SUM_U: return a + b;
    case R_MAX_F: return as_u(fmaxf(as_f(a), as_f(b)));
    default: return a > b ? a : b;
  }
}

// One row per workgroup (WPR = 4 waves) or per wavefront (WPR = 1).  A thread owns K chunks of
// VEC elements per pass, so a row of up to WPR * 64 * K * VEC elements is one pass per segment.
// Every stage re-reads the row through the program; rows come back from L2.
template <int VEC, int K, int WPR>
__global__ void __launch_bounds__(256) row_kernel(const Program p, OutDesc o, uint32_t rows,
                                                  uint32_t n, uint32_t *err) {
  __shared__ uint32_t part[4];
  constexpr int E = K * VEC;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t rows_per_block = 4 / WPR;
  const uint32_t tid_in_row = WPR == 4 ? threadIdx.x : lane;
  const uint32_t cstride = WPR * 64 * VEC;    // distance between a thread's chunks
  const uint32_t pass = cstride * K;          // elements per pass
  for (uint32_t rb = blockIdx.x * rows_per_block; rb < rows; rb += gridDim.x * rows_per_block) {
    const uint32_t row = rb + (WPR == 4 ? 0 : wave);
    const bool active = row < rows;
    uint32_t idx[MAX_DIMS];
    uint32_t rem = active ? row : 0;
#pragma unroll
    for (int d = MAX_DIMS - 2; d >= 0; --d) {
      if (d < p.n_dims - 1) {
        if (d == 0) {
          idx[d] = rem;
        } else {
          uint32_t q = rem / p.dims[d];
          idx[d] = rem - q * p.dims[d];
          rem = q;
        }
      } else {
        idx[d] = 0;
      }
    }
    idx[MAX_DIMS - 1] = 0;
    uint32_t rv0 = 0, rv1 = 0;
    int64_t obase = 0;
#pragma unroll
    for (int d = 0; d < MAX_DIMS - 1; ++d)
      if (d < p.n_dims - 1) obase += (int64_t)idx[d] * o.stride[d];
    const int64_t oinner = o.stride[p.n_dims - 1];
    int pc = 0;
    // segments 0 .. n_stages-1 feed a reduction, segment n_stages is stored
    for (int s = 0; s <= p.n_stages; ++s) {
      const bool final_seg = s == p.n_stages;
      const int kind = final_seg ? 0 : p.red_kind[s];
      const int pc_end = p.seg_end[s];
      uint32_t acc = red_init(kind);
      if (active) {
        for (uint32_t base = 0; base < n; base += pass) {
          const uint32_t c0 = base + tid_in_row * VEC;
          uint32_t valid = 0;
#pragma unroll
          for (int k = 0; k < K; ++k)
            if (c0 + k * cstride < n) valid |= 1u << k;
          if (!valid) continue;
          uint32_t v[E];
          eval_program<VEC, K>(p, pc, pc_end, idx, c0, cstride, valid, rv0, rv1, err, v);
          if (!final_seg) {
#pragma unroll
            for (int k = 0; k < K; ++k)
              if (valid & (1u << k))
#pragma unroll
                for (int j = 0; j < VEC; ++j) acc = red_combine(kind, acc, v[k * VEC + j]);
          } else {
#pragma unroll
            for (int k = 0; k < K; ++k) {
              if (valid & (1u << k)) {
                uint32_t *q = (uint32_t *)o.ptr + obase + (int64_t)(c0 + k * cstride) * oinner;
                if (VEC == 4 && o.vec) {
                  *(uint4 *)q = make_uint4(v[k * VEC], v[k * VEC + 1 % VEC], v[k * VEC + 2 % VEC],
                                           v[k * VEC + 3 % VEC]);
                } else {
#pragma unroll
                  for (int j = 0; j < VEC; ++j) q[j * oinner] = v[k * VEC + j];
                }
              }
            }
          }
        }
      }
      if (!final_seg) {
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1)
          acc = red_combine(kind, acc, (uint32_t)__shfl_xor((int)acc, m, 64));
        if (WPR == 4) {
          __syncthreads();
          if (lane == 0) part[wave] = acc;
          __syncthreads();
          acc = red_combine(kind, red_combine(kind, part[0], part[1]),
                            red_combine(kind, part[2], part[3]));
        }
        if (s == 0) rv0 = acc; else rv1 = acc;
      }
      pc = pc_end;
    }
  }
}

// ---- split-row reductions: few, very long rows (argmax over a vocabulary) ---------------------------
// Stage A: chunk c of row r -> accumulator words in scratch[(r * chunks + c) * W].
template <int KIND, int VEC>
__global__ void __launch_bounds__(256) reduce_split_kernel(const Program p, uint32_t *scratch,
                                                           uint32_t rows, uint32_t n,
                                                           uint32_t chunks, uint32_t chunk_len,
                                                           uint32_t *err) {
  __shared__ uint32_t part[4][Acc<KIND>::W];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t row = blockIdx.x / chunks, chunk = blockIdx.x - row * chunks;
  uint32_t idx[MAX_DIMS];
  uint32_t rem = row;
#pragma unroll
  for (int d = MAX_DIMS - 2; d >= 0; --d) {
    if (d < p.n_dims - 1) {
      if (d == 0) {
        idx[d] = rem;
      } else {
        uint32_t q = rem / p.dims[d];
        idx[d] = rem - q * p.dims[d];
        rem = q;
      }
    } else {
      idx[d] = 0;
    }
  }
  idx[MAX_DIMS - 1] = 0;
  Acc<KIND> acc;
  const uint32_t c0 = chunk * chunk_len, c1 = min(n, c0 + chunk_len);
  for (uint32_t c = c0 + threadIdx.x * VEC; c < c1; c += 256 * VEC) {
#pragma unroll
    for (int d = 0; d < MAX_DIMS; ++d)
      if (d == p.n_dims - 1) idx[d] = c;
    uint32_t v[VEC];
    eval_program<VEC, 1>(p, 0, p.n_instr, idx, c, 0u, 1u, 0u, 0u, err, v);
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc.add(v[j], c + j);
  }
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) acc.merge(shfl_xor_acc<KIND>(acc, m));
  if (lane == 0) acc.get(part[wave]);
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w2 = 1; w2 < 4; ++w2) {
      Acc<KIND> o;
      o.set(part[w2]);
      acc.merge(o);
    }
    acc.get(scratch + (uint64_t)blockIdx.x * Acc<KIND>::W);
  }
}

// Stage B: one wavefront per row merges the chunk accumulators.
template <int KIND>
__global__ void __launch_bounds__(64) reduce_merge_kernel(const uint32_t *scratch, uint32_t *out,
                                                          uint32_t rows, uint32_t chunks) {
  const uint32_t row = blockIdx.x;
  Acc<KIND> acc;
  for (uint32_t c = threadIdx.x; c < chunks; c += 64) {
    Acc<KIND> o;
    o.set(scratch + ((uint64_t)row * chunks + c) * Acc<KIND>::W);
    acc.merge(o);
  }
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) acc.merge(shfl_xor_acc<KIND>(acc, m));
  if (threadIdx.x == 0) out[row] = acc.result();
}

// ---- host launchers --------------------------------------------------------------------------

static inline unsigned grid_for(uint64_t blocks_needed, const LaunchCtx &lc) {
  uint64_t cap = (uint64_t)lc.n_cus * 8;
  uint64_t g = blocks_needed < cap ? blocks_needed : cap;
  return (unsigned)(g ? g : 1);
}

hipError_t launch_ew(const LaunchCtx &lc, const Program &p, const OutDesc &o, uint64_t n_elems,
                     bool vec4) {
  if (n_elems == 0) return hipSuccess;
  // up to one group per thread of the grid: the staged walk (see ew_kernel)
  const uint64_t one_pass = (uint64_t)lc.n_cus * 8 * 256;
  if (vec4) {
    uint64_t groups = n_elems / 4;
    if (groups <= one_pass)
      CG_LAUNCH(lc, (ew_kernel<4, true>), grid_for((groups + 255) / 256, lc), 256, p, o, groups, lc.err_flag);
    else
      CG_LAUNCH(lc, (ew_kernel<4, false>), grid_for((groups + 255) / 256, lc), 256, p, o, groups, lc.err_flag);
  } else {
    if (n_elems <= one_pass)
      CG_LAUNCH(lc, (ew_kernel<1, true>), grid_for((n_elems + 255) / 256, lc), 256, p, o, n_elems, lc.err_flag);
    else
      CG_LAUNCH(lc, (ew_kernel<1, false>), grid_for((n_elems + 255) / 256, lc), 256, p, o, n_elems, lc.err_flag);
  }
  return hipGetLastError();
}

// Thousands of argmax records (one per wave of the launch that stored the row): one workgroup of 1024 threads,
// a thread's records requested four at a time before any is merged, then wave shuffles and one exchange in LDS.
__global__ void __launch_bounds__(1024) argmax_records_kernel(const uint32_t *records, uint32_t *out, uint32_t n) {
  __shared__ uint32_t part[16][3];
  const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  Acc<R_ARGMAX_F> acc;
  for (uint32_t base = 0; base < n; base += 4096) {
    uint32_t w[4][3];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const uint32_t c = min(base + u * 1024 + tid, n - 1);  // (past the end: the last record again)
#pragma unroll
      for (int j = 0; j < 3; ++j) w[u][j] = records[(uint64_t)c * 3 + j];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      Acc<R_ARGMAX_F> o;
      o.set(w[u]);
      acc.merge(o);
    }
  }
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) acc.merge(shfl_xor_acc<R_ARGMAX_F>(acc, m));
  if (lane == 0) acc.get(part[wave]);
  __syncthreads();
  if (tid == 0) {
    for (int w2 = 1; w2 < 16; ++w2) {
      Acc<R_ARGMAX_F> o;
      o.set(part[w2]);
      acc.merge(o);
    }
    out[0] = acc.result();
  }
}

hipError_t launch_argmax_merge(const LaunchCtx &lc, const uint32_t *records, uint32_t *out, uint32_t n_records) {
  if (!n_records) return hipErrorInvalidValue;
  CG_LAUNCH(lc, (argmax_records_kernel), 1, 1024, records, out, n_records);
  return hipGetLastError();
}

template <int KIND>
static hipError_t launch_reduce_kind(const LaunchCtx &lc, const Program &p, uint32_t *out,
                                     uint32_t rows, uint32_t n, bool vec4, uint32_t *scratch,
                                     uint32_t chunks) {
  if (scratch && chunks > 1) {
    uint32_t chunk_len = (n + chunks - 1) / chunks;
    chunk_len = (chunk_len + 3) / 4 * 4;  // keep vector groups inside one chunk
    if (vec4)
      CG_LAUNCH(lc, (reduce_split_kernel<KIND, 4>), rows * chunks, 256, p, scratch, rows, n, chunks,
                                                                         chunk_len, lc.err_flag);
    else
      CG_LAUNCH(lc, (reduce_split_kernel<KIND, 1>), rows * chunks, 256, p, scratch, rows, n, chunks,
                                                                         chunk_len, lc.err_flag);
    LaunchCtx untimed = lc;  // the events stay with the (dominant) split pass
    untimed.ev_start = untimed.ev_stop = nullptr;
    CG_LAUNCH(untimed, (reduce_merge_kernel<KIND>), rows, 64, scratch, out, rows, chunks);
    return hipGetLastError();
  }
  const bool block_per_row = n >= 2048;
  if (block_per_row) {
    unsigned g = grid_for(rows, lc);
    if (vec4) CG_LAUNCH(lc, (reduce_kernel<KIND, 4, 4>), g, 256, p, out, rows, n, lc.err_flag);
    else CG_LAUNCH(lc, (reduce_kernel<KIND, 1, 4>), g, 256, p, out, rows, n, lc.err_flag);
  } else {
    unsigned g = grid_for((rows + 3) / 4, lc);
    if (vec4) CG_LAUNCH(lc, (reduce_kernel<KIND, 4, 1>), g, 256, p, out, rows, n, lc.err_flag);
    else CG_LAUNCH(lc, (reduce_kernel<KIND, 1, 1>), g, 256, p, out, rows, n, lc.err_flag);
  }
  return hipGetLastError();
}

uint32_t reduce_split_chunks(const LaunchCtx &lc, uint32_t rows, uint32_t n) {
  // worth splitting when the rows alone cannot fill the CUs and each row is long
  if (rows == 0 || n < 16384 || rows * 2 > (uint32_t)lc.n_cus) return 1;
  uint32_t chunks = (uint32_t)lc.n_cus * 2 / rows;
  uint32_t max_chunks = n / 2048;
  if (chunks > max_chunks) chunks = max_chunks;
  return chunks < 2 ? 1 : chunks;
}

hipError_t launch_reduce(const LaunchCtx &lc, int kind, const Program &p, void *out, uint32_t rows,
                         uint32_t n, bool vec4, uint32_t *scratch, uint32_t chunks) {
  if (rows == 0) return hipSuccess;
  uint32_t *o = (uint32_t *)out;
  switch (kind) {
    case R_SUM_F: return launch_reduce_kind<R_SUM_F>(lc, p, o, rows, n, vec4, scratch, chunks);
    case R_SUM_U: return launch_reduce_kind<R_SUM_U>(lc, p, o, rows, n, vec4, scratch, chunks);
    case R_MAX_F: return launch_reduce_kind<R_MAX_F>(lc, p, o, rows, n, vec4, scratch, chunks);
    case R_MAX_U: return launch_reduce_kind<R_MAX_U>(lc, p, o, rows, n, vec4, scratch, chunks);
    case R_ARGMAX_F: return launch_reduce_kind<R_ARGMAX_F>(lc, p, o, rows, n, vec4, scratch, chunks);
    case R_ARGMAX_U: return launch_reduce_kind<R_ARGMAX_U>(lc, p, o, rows, n, vec4, scratch, chunks);
  }
  return hipErrorInvalidValue;
}

hipError_t launch_row(const LaunchCtx &lc, const Program &p, const OutDesc &o, uint32_t rows,
                      uint32_t n, bool vec4) {
  if (rows == 0 || n == 0) return hipSuccess;
  // one pass per segment when the row fits: 64 lanes x K chunks x VEC per wave, x4 per workgroup
  if (vec4) {
    const bool block_per_row = n > 64 * 2 * 4 || rows * 8 <= (uint32_t)lc.n_cus;
    if (block_per_row) CG_LAUNCH(lc, (row_kernel<4, 2, 4>), grid_for(rows, lc), 256, p, o, rows, n, lc.err_flag);
    else CG_LAUNCH(lc, (row_kernel<4, 2, 1>), grid_for((rows + 3) / 4, lc), 256, p, o, rows, n, lc.err_flag);
  } else {
    const bool block_per_row = n > 64 * 4 || rows * 8 <= (uint32_t)lc.n_cus;
    if (block_per_row) CG_LAUNCH(lc, (row_kernel<1, 4, 4>), grid_for(rows, lc), 256, p, o, rows, n, lc.err_flag);
    else CG_LAUNCH(lc, (row_kernel<1, 4, 1>), grid_for((rows + 3) / 4, lc), 256, p, o, rows, n, lc.err_flag);
  }
  return hipGetLastError();
}

}  // namespace cgk
