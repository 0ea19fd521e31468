// ndarray_oracle.cpp — TEST INFRASTRUCTURE, NOT PRODUCT CODE.
//
// A single-threaded CPU restatement of catgrad's `NdArrayBackend`
// (catgrad/src/interpreter/backend/ndarray.rs) behind the same C ABI as the HIP backend
// (include/catgrad_hip.h).  It is the parity checker for tests/, for
// __graft_entry__.smoke() and the timed "cpu_baseline" leg of bench.py; nothing in the
// product library links, loads or calls it.
//
// Every function cites the reference lines it follows.  The arithmetic of the reference
// lives in two crates that are not vendored (ndarray 0.17.1, matrixmultiply 0.3.10); their
// published behaviour is restated: row-major logical order, IEEE-754 f32, Rust `as` casts,
// wrapping u32 arithmetic (release profile), libm powf/sinf/cosf.  f32 `sum` and `matmul`
// association order is unspecified in the reference, so those two are compared at a
// tolerance and never bit for bit.
//
// Like the reference every op materialises its result (broadcast, reshape, slice, transpose
// all copy), which keeps the reference's cost structure for the CPU baseline.
//
// What pins each function (tests/test_oracle_*.py): the reference's own unit and
// integration test vectors, closed forms, invariants and brute force on tiny inputs.
// Functions with no reference-held vector are pinned by IEEE/closed-form checks only:
// pow, div, mul, lt, eq, sin, cos, neg, cast, argmax, broadcast, reshape, transpose, concat,
// index, slice, arange are "parity unpinned by the reference's own ndarray tests" and pinned
// instead by the legacy evaluator's vectors for the same maths plus numpy closed forms.

#include "../include/catgrad_hip.h"

#include <atomic>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <algorithm>
#include <numeric>
#include <string>
#include <vector>

struct cg_backend {
  std::string err;
  uint32_t flags = 0;
};

struct cg_tensor {
  std::atomic<int> rc{1};
  cg_dtype dtype;
  std::vector<size_t> shape;
  std::vector<uint32_t> bits;  // row-major; f32 stored as its bit pattern
  float *f() { return reinterpret_cast<float *>(bits.data()); }
  const float *f() const { return reinterpret_cast<const float *>(bits.data()); }
  uint32_t *u() { return bits.data(); }
  const uint32_t *u() const { return bits.data(); }
  size_t size() const { return bits.size(); }
};

static size_t prod(const std::vector<size_t> &s) {
  size_t n = 1;
  for (size_t d : s) n *= d;
  return n;
}

static int fail(cg_backend *be, int code, const std::string &msg) {
  if (be) be->err = msg;
  return code;
}

static cg_tensor *make(cg_dtype dt, const std::vector<size_t> &shape) {
  cg_tensor *t = new cg_tensor();
  t->dtype = dt;
  t->shape = shape;
  t->bits.assign(prod(shape), 0u);
  return t;
}

static std::string shape_str(const std::vector<size_t> &s) {
  std::string r = "[";
  for (size_t i = 0; i < s.size(); ++i) r += (i ? ", " : "") + std::to_string(s[i]);
  return r + "]";
}

extern "C" {

int cg_backend_create(int, uint32_t flags, cg_backend **out) {
  if (!out) return CG_ERR_ARG;
  *out = new cg_backend();
  (*out)->flags = flags;
  return CG_OK;
}
void cg_backend_destroy(cg_backend *be) { delete be; }
const char *cg_last_error(const cg_backend *be) { return be ? be->err.c_str() : ""; }
int cg_sync(cg_backend *) { return CG_OK; }
// the oracle launches nothing
size_t cg_launch_counts(cg_backend *, int, char *buf, size_t cap) {
  if (buf && cap) buf[0] = 0;
  return 1;
}
int cg_tensor_realize(cg_backend *, cg_tensor *) { return CG_OK; }
int cg_tensor_prefetch(cg_backend *, cg_tensor *) { return CG_OK; }
// the probes measure a device; the oracle has none
int cg_peak_copy_gbs(cg_backend *, size_t, int, double *) { return CG_ERR_DEVICE; }
int cg_peak_mfma_tflops(cg_backend *, cg_dtype, int, double *) { return CG_ERR_DEVICE; }
int cg_peak_gemm_clock(cg_backend *, size_t, size_t, size_t, int, double *, double *) { return CG_ERR_DEVICE; }
const char *cg_backend_name(const cg_backend *) { return "ndarray-oracle"; }

cg_tensor *cg_tensor_retain(cg_tensor *t) {
  if (t) t->rc.fetch_add(1);
  return t;
}
void cg_tensor_release(cg_tensor *t) {
  if (t && t->rc.fetch_sub(1) == 1) delete t;
}
int cg_tensor_rank(const cg_tensor *t) { return (int)t->shape.size(); }
int cg_tensor_shape(const cg_tensor *t, size_t *dims) {
  for (size_t i = 0; i < t->shape.size(); ++i) dims[i] = t->shape[i];
  return CG_OK;
}
cg_dtype cg_tensor_dtype(const cg_tensor *t) { return t->dtype; }
size_t cg_tensor_size(const cg_tensor *t) { return t->size(); }

// ndarray.rs:53-65
int cg_zeros(cg_backend *be, const size_t *dims, int rank, cg_dtype dtype, cg_tensor **out) {
  if (rank < 0 || rank > CG_MAX_RANK) return fail(be, CG_ERR_ARG, "rank out of range");
  *out = make(dtype, std::vector<size_t>(dims, dims + rank));
  return CG_OK;
}

// ndarray.rs:67-89 and interpreter/mod.rs:21-31
static int from_bits(cg_backend *be, const void *data, size_t n, const size_t *dims, int rank,
                     cg_dtype dt, cg_tensor **out) {
  if (rank < 0 || rank > CG_MAX_RANK) return fail(be, CG_ERR_ARG, "rank out of range");
  std::vector<size_t> shape(dims, dims + rank);
  if (prod(shape) != n) return fail(be, CG_ERR_SHAPE, "ShapeError");
  cg_tensor *t = make(dt, shape);
  if (n) std::memcpy(t->bits.data(), data, n * 4);
  *out = t;
  return CG_OK;
}
int cg_from_f32(cg_backend *be, const float *d, size_t n, const size_t *dims, int rank,
                cg_tensor **out) {
  return from_bits(be, d, n, dims, rank, CG_F32, out);
}
int cg_from_u32(cg_backend *be, const uint32_t *d, size_t n, const size_t *dims, int rank,
                cg_tensor **out) {
  return from_bits(be, d, n, dims, rank, CG_U32, out);
}

// The weight loader's BF16 arm (catgrad-llm/examples/llama/main.rs:309-312): every bf16 widened to
// f32 on the host (half::bf16::to_f32 = the bits in the upper half of the word), then from_vec.
int cg_from_bf16(cg_backend *be, const uint16_t *bits, size_t n, const size_t *dims, int rank,
                 cg_tensor **out) {
  std::vector<uint32_t> wide(n);
  for (size_t i = 0; i < n; ++i) wide[i] = (uint32_t)bits[i] << 16;
  return from_bits(be, wide.data(), n, dims, rank, CG_F32, out);
}

// Rust `f32 as u32`: truncate toward zero, saturate, NaN -> 0 (ndarray.rs:101)
static inline uint32_t f32_as_u32(float v) {
  if (!(v == v)) return 0u;
  if (v <= 0.0f) return 0u;
  if (v >= 4294967296.0f) return 0xFFFFFFFFu;
  return (uint32_t)v;
}

// ndarray.rs:97-114
int cg_cast(cg_backend *, cg_tensor *x, cg_dtype target, cg_tensor **out) {
  if (x->dtype == target) {
    *out = cg_tensor_retain(x);
    return CG_OK;
  }
  cg_tensor *t = make(target, x->shape);
  size_t n = x->size();
  if (target == CG_U32)
    for (size_t i = 0; i < n; ++i) t->u()[i] = f32_as_u32(x->f()[i]);
  else
    for (size_t i = 0; i < n; ++i) t->f()[i] = (float)x->u()[i];  // round to nearest even
  *out = t;
  return CG_OK;
}

// ---- matmul ---------------------------------------------------------------------------
// Reference: Array2::dot -> matrixmultiply::sgemm (ndarray.rs:531-547).  Restated as a
// register-blocked GEBP kernel (6x16 accumulators, packed B panels) so that the CPU
// baseline is not handicapped by a naive triple loop.  f32 accumulation.
typedef float v8f __attribute__((vector_size(32)));

static void sgemm(const float *A, const float *B, float *C, size_t M, size_t K, size_t N) {
  std::memset(C, 0, M * N * sizeof(float));
  if (!M || !N || !K) return;
  const size_t KC = 256, NR = 16, MR = 6;
  std::vector<float> pack(KC * NR + 8);
  for (size_t j0 = 0; j0 < N; j0 += NR) {
    size_t nb = std::min(NR, N - j0);
    for (size_t k0 = 0; k0 < K; k0 += KC) {
      size_t kb = std::min(KC, K - k0);
      for (size_t k = 0; k < kb; ++k) {
        const float *src = B + (k0 + k) * N + j0;
        float *dst = pack.data() + k * NR;
        for (size_t j = 0; j < nb; ++j) dst[j] = src[j];
        for (size_t j = nb; j < NR; ++j) dst[j] = 0.f;
      }
      for (size_t i0 = 0; i0 < M; i0 += MR) {
        size_t mb = std::min(MR, M - i0);
        v8f acc[MR][2];
        for (size_t r = 0; r < MR; ++r) acc[r][0] = acc[r][1] = (v8f){0, 0, 0, 0, 0, 0, 0, 0};
        const float *a = A + i0 * K + k0;
        if (mb == MR) {
          for (size_t k = 0; k < kb; ++k) {
            v8f b0, b1;
            std::memcpy(&b0, pack.data() + k * NR, 32);
            std::memcpy(&b1, pack.data() + k * NR + 8, 32);
            for (size_t r = 0; r < MR; ++r) {
              float s = a[r * K + k];
              v8f sv = {s, s, s, s, s, s, s, s};
              acc[r][0] += sv * b0;
              acc[r][1] += sv * b1;
            }
          }
        } else {
          for (size_t k = 0; k < kb; ++k) {
            v8f b0, b1;
            std::memcpy(&b0, pack.data() + k * NR, 32);
            std::memcpy(&b1, pack.data() + k * NR + 8, 32);
            for (size_t r = 0; r < mb; ++r) {
              float s = a[r * K + k];
              v8f sv = {s, s, s, s, s, s, s, s};
              acc[r][0] += sv * b0;
              acc[r][1] += sv * b1;
            }
          }
        }
        for (size_t r = 0; r < mb; ++r) {
          float tmp[16];
          std::memcpy(tmp, &acc[r][0], 32);
          std::memcpy(tmp + 8, &acc[r][1], 32);
          float *c = C + (i0 + r) * N + j0;
          for (size_t j = 0; j < nb; ++j) c[j] += tmp[j];
        }
      }
    }
  }
}

// ndarray's generic (non-BLAS) dot for integer element types: wrapping u32
static void ugemm(const uint32_t *A, const uint32_t *B, uint32_t *C, size_t M, size_t K,
                  size_t N) {
  for (size_t i = 0; i < M; ++i)
    for (size_t j = 0; j < N; ++j) {
      uint32_t s = 0;
      for (size_t k = 0; k < K; ++k) s += A[i * K + k] * B[k * N + j];
      C[i * N + j] = s;
    }
}

// ndarray.rs:549-615
int cg_matmul(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **out) {
  if (a->dtype != b->dtype) return fail(be, CG_ERR_DTYPE, "matmul: dtype mismatch");
  size_t ra = a->shape.size(), rb = b->shape.size();
  if (ra < 2) return fail(be, CG_ERR_SHAPE, "batched_matmul: lhs must be at least rank 2");
  if (rb < 2) return fail(be, CG_ERR_SHAPE, "batched_matmul: rhs must be at least rank 2");
  size_t M = a->shape[ra - 2], K = a->shape[ra - 1], K2 = b->shape[rb - 2], N = b->shape[rb - 1];
  if (K != K2) return fail(be, CG_ERR_SHAPE, "batched_matmul: incompatible matrix dimensions");
  std::vector<size_t> ba(a->shape.begin(), a->shape.end() - 2);
  std::vector<size_t> bb(b->shape.begin(), b->shape.end() - 2);
  if (!(ra == 2 && rb == 2) && ba != bb)
    return fail(be, CG_ERR_SHAPE, "batched_matmul: batch dimensions must match");
  std::vector<size_t> os = ba;
  os.push_back(M);
  os.push_back(N);
  cg_tensor *t = make(a->dtype, os);
  size_t nb = prod(ba);
  for (size_t i = 0; i < nb; ++i) {
    if (a->dtype == CG_F32)
      sgemm(a->f() + i * M * K, b->f() + i * K * N, t->f() + i * M * N, M, K, N);
    else
      ugemm(a->u() + i * M * K, b->u() + i * K * N, t->u() + i * M * N, M, K, N);
  }
  *out = t;
  return CG_OK;
}

// ---- elementwise ------------------------------------------------------------------------
static uint32_t upow(uint32_t a, uint32_t e) {  // u32::pow, wrapping (release profile)
  uint32_t r = 1;
  while (e) {
    if (e & 1) r *= a;
    a *= a;
    e >>= 1;
  }
  return r;
}

enum BinOp { ADD, SUB, MUL, DIV, POW, LT, EQ };

// The reference's "Shape mismatch in operation" panic comes from ndarray's arithmetic
// operators / Zip on unequal shapes (ndarray.rs:401-453, 164-198).
static int binop(cg_backend *be, BinOp op, cg_tensor *a, cg_tensor *b, cg_tensor **out) {
  if (a->dtype != b->dtype) return fail(be, CG_ERR_DTYPE, "binary op: dtype mismatch");
  if (a->shape != b->shape)
    return fail(be, CG_ERR_SHAPE, "Shape mismatch in operation: " + shape_str(a->shape) +
                                      " vs " + shape_str(b->shape));
  size_t n = a->size();
  cg_tensor *t = make(a->dtype, a->shape);
  if (a->dtype == CG_F32) {
    const float *x = a->f(), *y = b->f();
    float *r = t->f();
    switch (op) {
      case ADD: for (size_t i = 0; i < n; ++i) r[i] = x[i] + y[i]; break;
      case SUB: for (size_t i = 0; i < n; ++i) r[i] = x[i] - y[i]; break;
      case MUL: for (size_t i = 0; i < n; ++i) r[i] = x[i] * y[i]; break;
      case DIV: for (size_t i = 0; i < n; ++i) r[i] = x[i] / y[i]; break;
      case POW: for (size_t i = 0; i < n; ++i) r[i] = powf(x[i], y[i]); break;
      case LT: for (size_t i = 0; i < n; ++i) r[i] = x[i] < y[i] ? 1.0f : 0.0f; break;
      case EQ: for (size_t i = 0; i < n; ++i) r[i] = x[i] == y[i] ? 1.0f : 0.0f; break;
    }
  } else {
    const uint32_t *x = a->u(), *y = b->u();
    uint32_t *r = t->u();
    switch (op) {
      case ADD: for (size_t i = 0; i < n; ++i) r[i] = x[i] + y[i]; break;
      case SUB: for (size_t i = 0; i < n; ++i) r[i] = x[i] - y[i]; break;
      case MUL: for (size_t i = 0; i < n; ++i) r[i] = x[i] * y[i]; break;
      case DIV:
        for (size_t i = 0; i < n; ++i) {
          if (y[i] == 0) {
            cg_tensor_release(t);
            return fail(be, CG_ERR_ARITH, "attempt to divide by zero");
          }
          r[i] = x[i] / y[i];
        }
        break;
      case POW: for (size_t i = 0; i < n; ++i) r[i] = upow(x[i], y[i]); break;
      case LT: for (size_t i = 0; i < n; ++i) r[i] = x[i] < y[i] ? 1u : 0u; break;
      case EQ: for (size_t i = 0; i < n; ++i) r[i] = x[i] == y[i] ? 1u : 0u; break;
    }
  }
  *out = t;
  return CG_OK;
}
int cg_add(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **o) { return binop(be, ADD, a, b, o); }
int cg_sub(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **o) { return binop(be, SUB, a, b, o); }
int cg_mul(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **o) { return binop(be, MUL, a, b, o); }
int cg_div(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **o) { return binop(be, DIV, a, b, o); }
int cg_pow(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **o) { return binop(be, POW, a, b, o); }
int cg_lt(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **o) { return binop(be, LT, a, b, o); }
int cg_eq(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **o) { return binop(be, EQ, a, b, o); }

// ndarray.rs:200-222
int cg_sin(cg_backend *be, cg_tensor *x, cg_tensor **out) {
  if (x->dtype != CG_F32) return fail(be, CG_ERR_DTYPE, "Invalid input types for sin");
  cg_tensor *t = make(CG_F32, x->shape);
  for (size_t i = 0; i < x->size(); ++i) t->f()[i] = sinf(x->f()[i]);
  *out = t;
  return CG_OK;
}
int cg_cos(cg_backend *be, cg_tensor *x, cg_tensor **out) {
  if (x->dtype != CG_F32) return fail(be, CG_ERR_DTYPE, "Invalid input types for cos");
  cg_tensor *t = make(CG_F32, x->shape);
  for (size_t i = 0; i < x->size(); ++i) t->f()[i] = cosf(x->f()[i]);
  *out = t;
  return CG_OK;
}
// ndarray.rs:433-441
int cg_neg(cg_backend *, cg_tensor *x, cg_tensor **out) {
  cg_tensor *t = make(x->dtype, x->shape);
  if (x->dtype == CG_F32)
    for (size_t i = 0; i < x->size(); ++i) t->f()[i] = -x->f()[i];
  else
    for (size_t i = 0; i < x->size(); ++i) t->u()[i] = 0u - x->u()[i];
  *out = t;
  return CG_OK;
}

// ---- shape ops ----------------------------------------------------------------------------
// ndarray.rs:355-361: ArrayBase::broadcast = numpy rules, right aligned, then to_owned
int cg_broadcast(cg_backend *be, cg_tensor *x, const size_t *dims, int rank, cg_tensor **out) {
  if (rank < 0 || rank > CG_MAX_RANK) return fail(be, CG_ERR_ARG, "rank out of range");
  std::vector<size_t> shape(dims, dims + rank);
  size_t rx = x->shape.size();
  if (rx > (size_t)rank) return fail(be, CG_ERR_SHAPE, "broadcast: rank of target too small");
  std::vector<size_t> stride(rank, 0);  // element strides of x seen from the target
  size_t s = 1;
  for (size_t i = 0; i < rx; ++i) {
    size_t xd = x->shape[rx - 1 - i], td = shape[rank - 1 - i];
    if (xd == td)
      stride[rank - 1 - i] = s;
    else if (xd == 1)
      stride[rank - 1 - i] = 0;
    else
      return fail(be, CG_ERR_SHAPE, "broadcast: " + shape_str(x->shape) + " to " + shape_str(shape));
    s *= xd;
  }
  cg_tensor *t = make(x->dtype, shape);
  size_t n = t->size();
  std::vector<size_t> idx(rank, 0);
  size_t off = 0;
  for (size_t i = 0; i < n; ++i) {
    t->bits[i] = x->bits[off];
    for (int d = rank - 1; d >= 0; --d) {
      idx[d]++;
      off += stride[d];
      if (idx[d] < shape[d]) break;
      off -= stride[d] * shape[d];
      idx[d] = 0;
    }
  }
  *out = t;
  return CG_OK;
}

// ndarray.rs:347-353
int cg_reshape(cg_backend *be, cg_tensor *x, const size_t *dims, int rank, cg_tensor **out) {
  if (rank < 0 || rank > CG_MAX_RANK) return fail(be, CG_ERR_ARG, "rank out of range");
  std::vector<size_t> shape(dims, dims + rank);
  if (prod(shape) != x->size())
    return fail(be, CG_ERR_SHAPE, "reshape: " + shape_str(x->shape) + " to " + shape_str(shape));
  cg_tensor *t = make(x->dtype, shape);
  t->bits = x->bits;
  *out = t;
  return CG_OK;
}

// ndarray.rs:363-371 (a lazy axis swap there; the logical result is the same)
int cg_transpose(cg_backend *be, cg_tensor *x, size_t d0, size_t d1, cg_tensor **out) {
  size_t r = x->shape.size();
  if (d0 >= r || d1 >= r) return fail(be, CG_ERR_ARG, "transpose: axis out of range");
  std::vector<size_t> shape = x->shape;
  std::swap(shape[d0], shape[d1]);
  std::vector<size_t> xs(r, 1);
  for (int i = (int)r - 2; i >= 0; --i) xs[i] = xs[i + 1] * x->shape[i + 1];
  std::swap(xs[d0], xs[d1]);
  cg_tensor *t = make(x->dtype, shape);
  size_t n = t->size();
  std::vector<size_t> idx(r, 0);
  size_t off = 0;
  for (size_t i = 0; i < n; ++i) {
    t->bits[i] = x->bits[off];
    for (int d = (int)r - 1; d >= 0; --d) {
      idx[d]++;
      off += xs[d];
      if (idx[d] < shape[d]) break;
      off -= xs[d] * shape[d];
      idx[d] = 0;
    }
  }
  *out = t;
  return CG_OK;
}

// ---- reductions ----------------------------------------------------------------------------
static int reduce_shape(cg_backend *be, cg_tensor *x, std::vector<size_t> &os, size_t &rows,
                        size_t &n) {
  if (x->shape.empty()) return fail(be, CG_ERR_SHAPE, "reduction of a rank-0 tensor");
  os = x->shape;
  n = os.back();
  os.back() = 1;
  rows = prod(os);
  return CG_OK;
}

// Rust f32::max: if one operand is NaN the other is returned
static inline float rust_fmax(float a, float b) {
  if (a != a) return b;
  if (b != b) return a;
  return a > b ? a : b;
}

// ndarray.rs:455-467
int cg_max(cg_backend *be, cg_tensor *x, cg_tensor **out) {
  std::vector<size_t> os;
  size_t rows, n;
  if (int e = reduce_shape(be, x, os, rows, n)) return e;
  cg_tensor *t = make(x->dtype, os);
  for (size_t r = 0; r < rows; ++r) {
    if (x->dtype == CG_F32) {
      float acc = -3.40282347e+38f;  // f32::MIN
      for (size_t i = 0; i < n; ++i) acc = rust_fmax(acc, x->f()[r * n + i]);
      t->f()[r] = acc;
    } else {
      uint32_t acc = 0;
      for (size_t i = 0; i < n; ++i) acc = std::max(acc, x->u()[r * n + i]);
      t->u()[r] = acc;
    }
  }
  *out = t;
  return CG_OK;
}

// ndarray.rs:522-529 (sum_axis: association order unspecified -> plain left-to-right here)
int cg_sum(cg_backend *be, cg_tensor *x, cg_tensor **out) {
  std::vector<size_t> os;
  size_t rows, n;
  if (int e = reduce_shape(be, x, os, rows, n)) return e;
  cg_tensor *t = make(x->dtype, os);
  for (size_t r = 0; r < rows; ++r) {
    if (x->dtype == CG_F32) {
      // eight interleaved partial sums, the shape of ndarray's unrolled_fold
      float p[8] = {0, 0, 0, 0, 0, 0, 0, 0};
      const float *row = x->f() + r * n;
      size_t i = 0;
      for (; i + 8 <= n; i += 8)
        for (int j = 0; j < 8; ++j) p[j] += row[i + j];
      float acc = ((p[0] + p[4]) + (p[1] + p[5])) + ((p[2] + p[6]) + (p[3] + p[7]));
      for (; i < n; ++i) acc += row[i];
      t->f()[r] = acc;
    } else {
      uint32_t acc = 0;
      for (size_t i = 0; i < n; ++i) acc += x->u()[r * n + i];
      t->u()[r] = acc;
    }
  }
  *out = t;
  return CG_OK;
}

// f32::total_cmp key: monotone map of the bit pattern to a signed integer
static inline int32_t total_key(float v) {
  int32_t b;
  std::memcpy(&b, &v, 4);
  b ^= (int32_t)(((uint32_t)(b >> 31)) >> 1);
  return b;
}

// ndarray.rs:469-493: Iterator::max_by returns the LAST of several equal maxima
int cg_argmax(cg_backend *be, cg_tensor *x, cg_tensor **out) {
  std::vector<size_t> os;
  size_t rows, n;
  if (int e = reduce_shape(be, x, os, rows, n)) return e;
  if (n == 0) return fail(be, CG_ERR_SHAPE, "argmax of an empty lane");
  cg_tensor *t = make(CG_U32, os);
  for (size_t r = 0; r < rows; ++r) {
    size_t best = 0;
    if (x->dtype == CG_F32) {
      int32_t bk = total_key(x->f()[r * n]);
      for (size_t i = 1; i < n; ++i) {
        int32_t k = total_key(x->f()[r * n + i]);
        if (k >= bk) { bk = k; best = i; }
      }
    } else {
      uint32_t bk = x->u()[r * n];
      for (size_t i = 1; i < n; ++i) {
        uint32_t k = x->u()[r * n + i];
        if (k >= bk) { bk = k; best = i; }
      }
    }
    t->u()[r] = (uint32_t)best;
  }
  *out = t;
  return CG_OK;
}

// cg_argmax into a tensor the caller brings (the product's entry point for callers that cannot allocate);
// here only so that both libraries export one ABI
int cg_argmax_into(cg_backend *be, cg_tensor *x, cg_tensor *out) {
  if (!x || !out) return fail(be, CG_ERR_ARG, "null argument");
  cg_tensor *t = nullptr;
  if (int e = cg_argmax(be, x, &t)) return e;
  int st = CG_OK;
  if (out->dtype != CG_U32 || out->shape != t->shape) st = fail(be, CG_ERR_SHAPE, "cg_argmax_into: out must be U32 and shaped like x with a last axis of 1");
  else out->bits = t->bits;
  cg_tensor_release(t);
  return st;
}

// ndarray.rs:495-520: stable sort of the indices by descending total_cmp, take k
int cg_topk(cg_backend *be, cg_tensor *x, size_t k, cg_tensor **values, cg_tensor **indices) {
  if (x->dtype != CG_F32) return fail(be, CG_ERR_DTYPE, "Unsupported type for topk");
  if (x->shape.empty()) return fail(be, CG_ERR_SHAPE, "topk of a rank-0 tensor");
  size_t n = x->shape.back();
  if (k > n) return fail(be, CG_ERR_SHAPE, "topk: k larger than the last dimension");
  std::vector<size_t> os = x->shape;
  os.back() = k;
  size_t rows = n ? x->size() / n : 0;
  cg_tensor *v = make(CG_F32, os), *ix = make(CG_U32, os);
  std::vector<size_t> idx(n);
  for (size_t r = 0; r < rows; ++r) {
    const float *lane = x->f() + r * n;
    std::iota(idx.begin(), idx.end(), 0);
    std::stable_sort(idx.begin(), idx.end(),
                     [&](size_t i, size_t j) { return total_key(lane[i]) > total_key(lane[j]); });
    for (size_t j = 0; j < k; ++j) {
      v->f()[r * k + j] = lane[idx[j]];
      ix->u()[r * k + j] = (uint32_t)idx[j];
    }
  }
  *values = v;
  *indices = ix;
  return CG_OK;
}

// ndarray.rs:337-343: ArcArray == : same shape and every element ==
int cg_compare(cg_backend *be, cg_tensor *a, cg_tensor *b, int *equal) {
  if (a->dtype != b->dtype) return fail(be, CG_ERR_DTYPE, "compare: dtype mismatch");
  *equal = 0;
  if (a->shape != b->shape) return CG_OK;
  size_t n = a->size();
  if (a->dtype == CG_F32) {
    for (size_t i = 0; i < n; ++i)
      if (!(a->f()[i] == b->f()[i])) return CG_OK;
  } else {
    for (size_t i = 0; i < n; ++i)
      if (a->u()[i] != b->u()[i]) return CG_OK;
  }
  *equal = 1;
  return CG_OK;
}

// ndarray.rs:393-399
int cg_concat(cg_backend *be, cg_tensor *x, cg_tensor *y, size_t dim, cg_tensor **out) {
  if (x->dtype != y->dtype) return fail(be, CG_ERR_DTYPE, "Incompatible types for concatenation");
  size_t r = x->shape.size();
  if (r != y->shape.size() || dim >= r) return fail(be, CG_ERR_SHAPE, "concat: rank/axis mismatch");
  for (size_t i = 0; i < r; ++i)
    if (i != dim && x->shape[i] != y->shape[i])
      return fail(be, CG_ERR_SHAPE, "concat: " + shape_str(x->shape) + " with " + shape_str(y->shape));
  std::vector<size_t> os = x->shape;
  os[dim] += y->shape[dim];
  size_t outer = 1, inner = 1;
  for (size_t i = 0; i < dim; ++i) outer *= os[i];
  for (size_t i = dim + 1; i < r; ++i) inner *= os[i];
  size_t xa = x->shape[dim] * inner, ya = y->shape[dim] * inner;
  cg_tensor *t = make(x->dtype, os);
  for (size_t o = 0; o < outer; ++o) {
    if (xa) std::memcpy(&t->bits[o * (xa + ya)], &x->bits[o * xa], xa * 4);
    if (ya) std::memcpy(&t->bits[o * (xa + ya) + xa], &y->bits[o * ya], ya * 4);
  }
  *out = t;
  return CG_OK;
}

// The expert stacking of catgrad-llm/examples/llama/main.rs:217-236 as written there: every part
// reshaped to [1, ...], then concatenated one by one along axis 0.
int cg_stack(cg_backend *be, cg_tensor *const *parts, size_t n, cg_tensor **out) {
  if (!parts || !out || n == 0) return fail(be, CG_ERR_ARG, "nothing to stack");
  std::vector<size_t> one{1};
  one.insert(one.end(), parts[0]->shape.begin(), parts[0]->shape.end());
  if (one.size() > CG_MAX_RANK) return fail(be, CG_ERR_SHAPE, "stack: rank too large");
  cg_tensor *acc = nullptr;
  for (size_t i = 0; i < n; ++i) {
    if (parts[i]->shape != parts[0]->shape) {
      if (acc) cg_tensor_release(acc);
      return fail(be, CG_ERR_SHAPE, "stack: Shape mismatch");
    }
    cg_tensor *r = nullptr;
    int st = cg_reshape(be, parts[i], one.data(), (int)one.size(), &r);
    if (st == CG_OK && acc) {
      cg_tensor *c = nullptr;
      st = cg_concat(be, acc, r, 0, &c);
      cg_tensor_release(acc);
      cg_tensor_release(r);
      acc = c;
    } else if (st == CG_OK) {
      acc = r;
    }
    if (st != CG_OK) {
      if (acc) cg_tensor_release(acc);
      return st;
    }
  }
  *out = acc;
  return CG_OK;
}

// ndarray.rs:373-381: select(Axis(dim), flattened indices)
int cg_index(cg_backend *be, cg_tensor *x, size_t dim, cg_tensor *indices, cg_tensor **out) {
  if (indices->dtype != CG_U32) return fail(be, CG_ERR_DTYPE, "Invalid input types for indexing");
  size_t r = x->shape.size();
  if (dim >= r) return fail(be, CG_ERR_ARG, "index: axis out of range");
  size_t ni = indices->size(), nd = x->shape[dim];
  for (size_t i = 0; i < ni; ++i)
    if (indices->u()[i] >= nd) return fail(be, CG_ERR_ARG, "index out of bounds");
  std::vector<size_t> os = x->shape;
  os[dim] = ni;
  size_t outer = 1, inner = 1;
  for (size_t i = 0; i < dim; ++i) outer *= os[i];
  for (size_t i = dim + 1; i < r; ++i) inner *= os[i];
  cg_tensor *t = make(x->dtype, os);
  for (size_t o = 0; o < outer; ++o)
    for (size_t i = 0; i < ni; ++i)
      if (inner)
        std::memcpy(&t->bits[(o * ni + i) * inner],
                    &x->bits[(o * nd + indices->u()[i]) * inner], inner * 4);
  *out = t;
  return CG_OK;
}

// ndarray.rs:383-391
int cg_slice(cg_backend *be, cg_tensor *x, size_t dim, size_t start, size_t len, cg_tensor **out) {
  size_t r = x->shape.size();
  if (dim >= r) return fail(be, CG_ERR_ARG, "slice: axis out of range");
  if (start + len > x->shape[dim]) return fail(be, CG_ERR_SHAPE, "slice: range out of bounds");
  std::vector<size_t> os = x->shape;
  os[dim] = len;
  size_t outer = 1, inner = 1, nd = x->shape[dim];
  for (size_t i = 0; i < dim; ++i) outer *= os[i];
  for (size_t i = dim + 1; i < r; ++i) inner *= os[i];
  cg_tensor *t = make(x->dtype, os);
  for (size_t o = 0; o < outer; ++o)
    if (len * inner != 0)
      std::memcpy(&t->bits[o * len * inner], &x->bits[(o * nd + start) * inner], len * inner * 4);
  *out = t;
  return CG_OK;
}

// ndarray.rs:91-95: f32 range cast to u32
int cg_arange(cg_backend *, size_t end, cg_tensor **out) {
  cg_tensor *t = make(CG_U32, {end});
  for (size_t i = 0; i < end; ++i) t->u()[i] = f32_as_u32((float)i);
  *out = t;
  return CG_OK;
}

// ndarray.rs:46-51
int cg_to_f32(cg_backend *be, cg_tensor *x, float *dst, size_t n) {
  if (x->dtype != CG_F32) return fail(be, CG_ERR_DTYPE, "to_vec: not an f32 tensor");
  if (n != x->size()) return fail(be, CG_ERR_SHAPE, "to_vec: size mismatch");
  if (n) std::memcpy(dst, x->bits.data(), n * 4);
  return CG_OK;
}
int cg_to_u32(cg_backend *be, cg_tensor *x, uint32_t *dst, size_t n) {
  if (x->dtype != CG_U32) return fail(be, CG_ERR_DTYPE, "to_vec: not a u32 tensor");
  if (n != x->size()) return fail(be, CG_ERR_SHAPE, "to_vec: size mismatch");
  if (n) std::memcpy(dst, x->bits.data(), n * 4);
  return CG_OK;
}

int cg_trace_enable(cg_backend *, int) { return CG_OK; }
int cg_trace_reset(cg_backend *) { return CG_OK; }
size_t cg_trace_report(cg_backend *, char *buf, size_t cap) {
  if (buf && cap) buf[0] = 0;
  return 1;
}
int cg_stats(cg_backend *, uint64_t *l, uint64_t *d, uint64_t *p) {
  if (l) *l = 0;
  if (d) *d = 0;
  if (p) *p = 0;
  return CG_OK;
}

}  // extern "C"
