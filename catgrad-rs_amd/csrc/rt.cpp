// rt.cpp — the HIP backend behind include/catgrad_hip.h (see rt.hpp for the design).
//
// Semantics follow catgrad/src/interpreter/backend/ndarray.rs method by method (cited at each
// entry point); shapes follow catgrad/src/interpreter/backend/shape_only.rs:255-327.
#include "rt.hpp"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>

using namespace cgrt;
using namespace cgk;

namespace {

int fail(cg_backend *be, int code, const std::string &msg) {
  if (be) be->err = msg;
  return code;
}

#define HIPCHK(be, call)                                                              \
  do {                                                                                \
    hipError_t e_ = (call);                                                           \
    if (e_ != hipSuccess)                                                             \
      return fail(be, CG_ERR_DEVICE, std::string(#call) + ": " + hipGetErrorString(e_)); \
  } while (0)

#define TRY(expr)            \
  do {                       \
    int st_ = (expr);        \
    if (st_) return st_;     \
  } while (0)

std::string shape_str(const int64_t *s, int r) {
  std::string o = "[";
  for (int i = 0; i < r; ++i) o += (i ? ", " : "") + std::to_string(s[i]);
  return o + "]";
}

int esize(int stype) { return stype == ST_BF16 ? 2 : 4; }

// ---- allocator -----------------------------------------------------------------------------
size_t size_class(size_t bytes) {
  if (bytes <= 256) return 256;
  if (bytes <= (1u << 20)) {
    size_t c = 256;
    while (c < bytes) c <<= 1;
    return c;
  }
  const size_t mb = 1u << 20;
  return (bytes + mb - 1) / mb * mb;
}

void trim_pool(cg_backend *be) {
  for (auto &kv : be->pool)
    for (void *p : kv.second) {
      (void)hipFree(p);
      be->device_bytes -= kv.first;
    }
  be->pool.clear();
  be->pool_bytes = 0;
}

int dev_alloc(cg_backend *be, size_t bytes, Storage **out) {
  const size_t cls = size_class(bytes);
  void *p = nullptr;
  auto it = be->pool.find(cls);
  if (it != be->pool.end() && !it->second.empty()) {
    p = it->second.back();
    it->second.pop_back();
    be->pool_bytes -= cls;
  } else {
    hipError_t e = hipMalloc(&p, cls);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      trim_pool(be);
      e = hipMalloc(&p, cls);
      if (e != hipSuccess) {
        (void)hipGetLastError();
        return fail(be, CG_ERR_OOM, "hipMalloc of " + std::to_string(cls) + " bytes failed");
      }
    }
    be->device_bytes += cls;
  }
  Storage *s = new Storage();
  s->ptr = p;
  s->bytes = cls;
  s->be = be;
  *out = s;
  return CG_OK;
}

void backend_release(cg_backend *be);

void storage_release(Storage *s) {
  if (!s || s->rc.fetch_sub(1) != 1) return;
  cg_backend *be = s->be;
  // Safe to recycle at once: every consumer was enqueued on the backend's only stream.
  be->pool[s->bytes].push_back(s->ptr);
  be->pool_bytes += s->bytes;
  delete s;
}

void backend_release(cg_backend *be) {
  if (!be || be->rc.fetch_sub(1) != 1) return;
  (void)hipSetDevice(be->device);
  (void)hipStreamSynchronize(be->stream);
  for (auto &pe : be->trace_pending) {
    (void)hipEventDestroy(pe.start);
    (void)hipEventDestroy(pe.stop);
  }
  trim_pool(be);
  if (be->d_words) (void)hipFree(be->d_words);
  if (be->h_words) (void)hipHostFree(be->h_words);
  if (be->stream) (void)hipStreamDestroy(be->stream);
  delete be;
}

// ---- nodes ---------------------------------------------------------------------------------
cg_tensor *new_node(cg_backend *be, cg_dtype dt, int rank, const int64_t *shape) {
  cg_tensor *t = new cg_tensor();
  t->be = be;
  be->rc.fetch_add(1);
  t->dtype = dt;
  t->rank = rank;
  for (int i = 0; i < rank; ++i) t->shape[i] = shape[i];
  t->stype = dt == CG_F32 ? ST_F32 : ST_U32;
  return t;
}

void node_release(cg_tensor *t) {
  if (!t) return;
  std::vector<cg_tensor *> stack{t};
  while (!stack.empty()) {
    cg_tensor *n = stack.back();
    stack.pop_back();
    if (n->rc.fetch_sub(1) != 1) continue;
    if (n->in[0]) stack.push_back(n->in[0]);
    if (n->in[1]) stack.push_back(n->in[1]);
    storage_release(n->st);
    cg_backend *be = n->be;
    delete n;
    backend_release(be);
  }
}

cg_tensor *retain(cg_tensor *t) {
  t->rc.fetch_add(1);
  return t;
}

void drop_inputs(cg_tensor *n) {
  cg_tensor *a = n->in[0], *b = n->in[1];
  n->in[0] = n->in[1] = nullptr;
  node_release(a);
  node_release(b);
}

void contiguous_strides(int rank, const int64_t *shape, int64_t *strides) {
  int64_t s = 1;
  for (int i = rank - 1; i >= 0; --i) {
    strides[i] = s;
    s *= shape[i];
  }
}

bool is_contiguous(const cg_tensor *t) {
  int64_t s = 1;
  for (int i = t->rank - 1; i >= 0; --i) {
    if (t->shape[i] != 1 && t->strides[i] != s) return false;
    s *= t->shape[i];
  }
  return true;
}

// numpy's no-copy reshape rule: succeeds iff the new shape can be laid over the old strides
bool try_reshape_view(int ornk, const int64_t *oshape, const int64_t *ostr, int nrnk,
                      const int64_t *nshape, int64_t *nstr) {
  int64_t od[CG_MAX_RANK], os[CG_MAX_RANK];
  int oldnd = 0;
  for (int i = 0; i < ornk; ++i)
    if (oshape[i] != 1) {
      od[oldnd] = oshape[i];
      os[oldnd] = ostr[i];
      oldnd++;
    }
  int oi = 0, oj = 1, ni = 0, nj = 1;
  while (ni < nrnk && oi < oldnd) {
    int64_t np = nshape[ni], op = od[oi];
    while (np != op) {
      if (np < op) {
        if (nj >= nrnk) return false;
        np *= nshape[nj++];
      } else {
        if (oj >= oldnd) return false;
        op *= od[oj++];
      }
    }
    for (int ok = oi; ok < oj - 1; ++ok)
      if (os[ok] != od[ok + 1] * os[ok + 1]) return false;
    nstr[nj - 1] = os[oj - 1];
    for (int nk = nj - 1; nk > ni; --nk) nstr[nk - 1] = nstr[nk] * nshape[nk];
    ni = nj++;
    oi = oj++;
  }
  int64_t last = ni >= 1 ? nstr[ni - 1] : 1;
  for (int nk = ni; nk < nrnk; ++nk) nstr[nk] = last;
  return true;
}

// ---- tracing -------------------------------------------------------------------------------
struct KernelScope {
  cg_backend *be;
  PendingEvent pe;
  bool on;
  KernelScope(cg_backend *b, const char *name, double bytes, double flops) : be(b), on(b->trace) {
    be->launches++;
    if (!on) return;
    pe.name = name;
    pe.bytes = bytes;
    pe.flops = flops;
    (void)hipEventCreate(&pe.start);
    (void)hipEventCreate(&pe.stop);
    (void)hipEventRecord(pe.start, be->stream);
  }
  void rename(const char *name) {
    if (on && name) pe.name = name;
  }
  ~KernelScope() {
    if (!on) return;
    (void)hipEventRecord(pe.stop, be->stream);
    be->trace_pending.push_back(pe);
  }
};

void trace_collect(cg_backend *be) {
  if (be->trace_pending.empty()) return;
  (void)hipStreamSynchronize(be->stream);
  for (auto &pe : be->trace_pending) {
    float ms = 0.f;
    (void)hipEventElapsedTime(&ms, pe.start, pe.stop);
    TraceRec &r = be->trace_recs[pe.name];
    r.launches++;
    r.ms += ms;
    r.bytes += pe.bytes;
    r.flops += pe.flops;
    (void)hipEventDestroy(pe.start);
    (void)hipEventDestroy(pe.stop);
  }
  be->trace_pending.clear();
}

// ---- realisation ---------------------------------------------------------------------------
int realize(cg_backend *be, cg_tensor *n);

int alloc_result(cg_backend *be, cg_tensor *n, int stype) {
  int64_t cnt = std::max<int64_t>(n->size(), 1);
  Storage *s = nullptr;
  TRY(dev_alloc(be, (size_t)cnt * esize(stype), &s));
  n->st = s;
  n->stype = stype;
  n->offset = 0;
  contiguous_strides(n->rank, n->shape, n->strides);
  return CG_OK;
}

void *data_ptr(const cg_tensor *t) { return (char *)t->st->ptr + t->offset * esize(t->stype); }

bool ew_inlineable(const cg_tensor *n) {
  return (n->op == N_BIN || n->op == N_UN) && n->rc.load() == 1;
}

struct Cost {
  int instr = 0, inputs = 0, depth = 0;
};

Cost measure(const cg_tensor *n) {
  Cost c;
  if (n->op == N_CONST || (n->op == N_ARANGE && n->rank == 1)) {
    c.instr = 1;
    c.depth = 1;
  } else if (n->op == N_BIN) {
    Cost a = ew_inlineable(n->in[0]) || n->in[0]->op == N_CONST ? measure(n->in[0]) : Cost{1, 1, 1};
    Cost b = ew_inlineable(n->in[1]) || n->in[1]->op == N_CONST ? measure(n->in[1]) : Cost{1, 1, 1};
    c.instr = a.instr + b.instr + 1;
    c.inputs = a.inputs + b.inputs;
    c.depth = std::max(a.depth, b.depth + 1);
  } else if (n->op == N_UN) {
    Cost a = ew_inlineable(n->in[0]) || n->in[0]->op == N_CONST ? measure(n->in[0]) : Cost{1, 1, 1};
    c.instr = a.instr + 1;
    c.inputs = a.inputs;
    c.depth = a.depth;
  } else {
    c = Cost{1, 1, 1};
  }
  return c;
}

struct EwCompiler {
  cg_backend *be;
  Program p;
  std::vector<cg_tensor *> ins;
  EwCompiler(cg_backend *b) : be(b) { std::memset(&p, 0, sizeof(p)); }

  int push(uint8_t op, int depth, uint16_t arg) {
    if (p.n_instr >= MAX_INSTR || depth > MAX_STACK)
      return fail(be, CG_ERR_INTERNAL, "elementwise program overflow");
    p.code[p.n_instr].op = op;
    p.code[p.n_instr].depth = (uint8_t)depth;
    p.code[p.n_instr].arg = arg;
    p.n_instr++;
    return CG_OK;
  }
  int push_const(uint32_t bits, int depth) {
    if (p.n_instr >= MAX_INSTR) return fail(be, CG_ERR_INTERNAL, "elementwise program overflow");
    p.imm[p.n_instr] = bits;
    return push(E_CONST, depth, (uint16_t)p.n_instr);
  }
  int load(cg_tensor *n, int depth) {
    if (n->op != N_REAL) TRY(realize(be, n));
    size_t slot = 0;
    for (; slot < ins.size(); ++slot)
      if (ins[slot] == n) break;
    if (slot == ins.size()) {
      if (ins.size() >= MAX_IN) return fail(be, CG_ERR_INTERNAL, "elementwise program: too many inputs");
      ins.push_back(n);
    }
    return push(E_LOAD, depth, (uint16_t)slot);
  }
  static bool is_const(const cg_tensor *n, uint32_t bits) { return n->op == N_CONST && n->cbits == bits; }

  // emit code leaving the value of `n` at stack slot `depth`
  int emit(cg_tensor *n, int depth, int pend_instr, int pend_in, bool root) {
    if (n->op == N_CONST) return push_const(n->cbits, depth);
    if (n->op == N_ARANGE && n->rank == 1) return push(E_IOTA, depth, 0);
    if (!(root || ew_inlineable(n)) || (n->op != N_BIN && n->op != N_UN)) return load(n, depth);
    if (!root) {
      Cost c = measure(n);
      if (p.n_instr + c.instr + pend_instr > MAX_INSTR ||
          (int)ins.size() + c.inputs + pend_in > MAX_IN || depth + c.depth > MAX_STACK)
        return load(n, depth);
    }
    if (n->op == N_UN) {
      TRY(emit(n->in[0], depth, pend_instr + 1, pend_in, false));
      return push(n->ew, depth + 1, 0);
    }
    cg_tensor *a = n->in[0], *b = n->in[1];
    if (n->ew == E_POW_F) {
      // nn::exp = pow(broadcast(E), x); nn::sqrt = pow(x, broadcast(0.5)); gelu: pow(x, 3)
      // (catgrad/src/stdlib/nn/mod.rs:117-128, 157)
      if (is_const(a, 0x402DF854u)) {
        TRY(emit(b, depth, pend_instr + 1, pend_in, false));
        return push(E_EXP_F, depth + 1, 0);
      }
      if (is_const(b, 0x3F000000u) || is_const(b, 0x40400000u)) {
        TRY(emit(a, depth, pend_instr + 1, pend_in, false));
        return push(is_const(b, 0x3F000000u) ? E_SQRT_F : E_CUBE_F, depth + 1, 0);
      }
    }
    if (n->ew == E_DIV_F && is_const(a, 0x3F800000u)) {
      TRY(emit(b, depth, pend_instr + 1, pend_in, false));
      return push(E_RCP_F, depth + 1, 0);
    }
    TRY(emit(a, depth, pend_instr + 2, pend_in + 1, false));
    TRY(emit(b, depth + 1, pend_instr + 1, pend_in, false));
    return push(n->ew, depth + 2, 0);
  }
};

// Collapse the logical dims shared by all operands: drop extent-1 dims, merge neighbours that
// every operand walks contiguously.  strides[o] are per-operand stride arrays of length rank.
int collapse_dims(int rank, const int64_t *shape, std::vector<const int64_t *> strides,
                  bool keep_last, uint32_t *dims, std::vector<std::vector<int64_t>> &out) {
  const size_t no = strides.size();
  out.assign(no, std::vector<int64_t>());
  std::vector<int64_t> dsz;
  for (int i = 0; i < rank; ++i) {
    if (shape[i] == 1 && !(keep_last && i == rank - 1)) continue;
    bool merge = !dsz.empty() && !(keep_last && i == rank - 1);
    if (merge)
      for (size_t o = 0; o < no; ++o)
        if (out[o].back() != strides[o][i] * shape[i]) {
          merge = false;
          break;
        }
    if (merge) {
      dsz.back() *= shape[i];
      for (size_t o = 0; o < no; ++o) out[o].back() = strides[o][i];
    } else {
      dsz.push_back(shape[i]);
      for (size_t o = 0; o < no; ++o) out[o].push_back(strides[o][i]);
    }
  }
  if (dsz.empty()) {
    dsz.push_back(1);
    for (size_t o = 0; o < no; ++o) out[o].push_back(0);
  }
  if ((int)dsz.size() > MAX_DIMS) return -1;
  for (size_t i = 0; i < dsz.size(); ++i) dims[i] = (uint32_t)dsz[i];
  return (int)dsz.size();
}

bool operand_vec_ok(const void *ptr, int stype, const std::vector<int64_t> &st) {
  if (st.back() != 1) return false;
  const int q = 4;  // four elements per vector access
  if (((uintptr_t)ptr) % (q * esize(stype))) return false;
  for (size_t i = 0; i + 1 < st.size(); ++i)
    if (st[i] % q) return false;
  return true;
}

// Fill Program operands/dims from the compiler's inputs.  `out_strides` (may be null) joins the
// collapse as one more operand; its collapsed strides are returned in `ostr`.
int finish_program(cg_backend *be, EwCompiler &c, int rank, const int64_t *shape,
                   const int64_t *out_strides, bool keep_last, std::vector<int64_t> &ostr,
                   double *bytes_in) {
  std::vector<const int64_t *> sv;
  for (cg_tensor *t : c.ins) sv.push_back(t->strides);
  if (out_strides) sv.push_back(out_strides);
  std::vector<std::vector<int64_t>> cs;
  int nd = collapse_dims(rank, shape, sv, keep_last, c.p.dims, cs);
  if (nd < 0) return fail(be, CG_ERR_INTERNAL, "elementwise program: more than 6 collapsed dims");
  c.p.n_dims = nd;
  c.p.n_in = (int)c.ins.size();
  double bytes = 0;
  for (size_t i = 0; i < c.ins.size(); ++i) {
    Operand &o = c.p.in[i];
    o.ptr = data_ptr(c.ins[i]);
    o.stype = c.ins[i]->stype;
    double uniq = 1;
    for (int d = 0; d < nd; ++d) {
      o.stride[d] = cs[i][d];
      if (cs[i][d] != 0) uniq *= c.p.dims[d];
    }
    bytes += uniq * esize(o.stype);
    o.vec = operand_vec_ok(o.ptr, o.stype, cs[i]) ? 1 : 0;
  }
  if (out_strides) ostr = cs.back();
  if (bytes_in) *bytes_in = bytes;
  return CG_OK;
}

// Evaluate the elementwise tree rooted at `root` into (dst storage, dst strides, dst stype).
int run_ew(cg_backend *be, cg_tensor *root, bool root_is_value, void *dst, const int64_t *dst_strides,
           int dst_stype, const char *name) {
  if (root->size() == 0) return CG_OK;
  EwCompiler c(be);
  if (root_is_value) TRY(c.load(root, 0));
  else TRY(c.emit(root, 0, 0, 0, true));
  std::vector<int64_t> ostr;
  double bytes_in = 0;
  TRY(finish_program(be, c, root->rank, root->shape, dst_strides, false, ostr, &bytes_in));
  const int64_t n = root->size();
  if (n >= (int64_t)1 << 32) return fail(be, CG_ERR_INTERNAL, "tensor above 2^32 elements");
  OutDesc o;
  std::memset(&o, 0, sizeof(o));
  o.ptr = dst;
  o.stype = dst_stype;
  for (int d = 0; d < c.p.n_dims; ++d) o.stride[d] = ostr[d];
  o.vec = dst_stype != ST_BF16 && operand_vec_ok(dst, dst_stype, ostr);
  const bool vec4 = c.p.dims[c.p.n_dims - 1] % 4 == 0;
  KernelScope ks(be, name, bytes_in + (double)n * esize(dst_stype), 0);
  HIPCHK(be, launch_ew(be->lc(), c.p, o, (uint64_t)n, vec4));
  return CG_OK;
}

// A fresh contiguous tensor holding the value of `src` (f32/u32 storage unless keep_bf16).
int materialize(cg_backend *be, cg_tensor *src, cg_tensor **out, bool keep_bf16 = false) {
  TRY(realize(be, src));
  cg_tensor *t = new_node(be, src->dtype, src->rank, src->shape);
  int stype = (keep_bf16 && src->stype == ST_BF16) ? ST_BF16 : (src->dtype == CG_F32 ? ST_F32 : ST_U32);
  int st = alloc_result(be, t, stype);
  if (!st) st = run_ew(be, src, true, data_ptr(t), t->strides, stype, "ew_copy");
  if (st) {
    node_release(t);
    return st;
  }
  *out = t;
  return CG_OK;
}

// src as a contiguous f32/u32 buffer: itself when it already is one
int contiguous(cg_backend *be, cg_tensor *src, cg_tensor **out) {
  TRY(realize(be, src));
  if (is_contiguous(src) && src->stype != ST_BF16) {
    *out = retain(src);
    return CG_OK;
  }
  return materialize(be, src, out);
}

int realize_const(cg_backend *be, cg_tensor *n) {
  TRY(alloc_result(be, n, n->dtype == CG_F32 ? ST_F32 : ST_U32));
  KernelScope ks(be, "fill", (double)n->size() * 4, 0);
  HIPCHK(be, launch_fill_u32(be->lc(), (uint32_t *)n->st->ptr, n->cbits, (uint64_t)n->size()));
  n->op = N_REAL;
  return CG_OK;
}

int realize_ew(cg_backend *be, cg_tensor *n) {
  int stype = n->dtype == CG_F32 ? ST_F32 : ST_U32;
  int64_t cnt = std::max<int64_t>(n->size(), 1);
  Storage *s = nullptr;
  TRY(dev_alloc(be, (size_t)cnt * 4, &s));
  int64_t strides[CG_MAX_RANK];
  contiguous_strides(n->rank, n->shape, strides);
  int st = run_ew(be, n, false, s->ptr, strides, stype, "ew_fused");
  if (st) {
    storage_release(s);
    return st;
  }
  n->st = s;
  n->stype = stype;
  n->offset = 0;
  std::memcpy(n->strides, strides, sizeof(strides));
  n->op = N_REAL;
  drop_inputs(n);
  return CG_OK;
}

int realize_view(cg_backend *be, cg_tensor *n) {
  cg_tensor *x = n->in[0];
  TRY(realize(be, x));
  switch (n->op) {
    case N_TRANSPOSE:
      std::memcpy(n->strides, x->strides, sizeof(n->strides));
      std::swap(n->strides[n->p0], n->strides[n->p1]);
      n->offset = x->offset;
      break;
    case N_SLICE:
      std::memcpy(n->strides, x->strides, sizeof(n->strides));
      n->offset = x->offset + n->p1 * x->strides[n->p0];
      break;
    case N_BROADCAST: {
      const int shift = n->rank - x->rank;
      for (int i = 0; i < n->rank; ++i) {
        const int xi = i - shift;
        n->strides[i] = (xi < 0 || (x->shape[xi] == 1 && n->shape[i] != 1)) ? 0 : x->strides[xi];
      }
      n->offset = x->offset;
      break;
    }
    case N_RESHAPE: {
      if (n->size() == 0) {
        contiguous_strides(n->rank, n->shape, n->strides);
        n->offset = x->offset;
        break;
      }
      if (try_reshape_view(x->rank, x->shape, x->strides, n->rank, n->shape, n->strides)) {
        n->offset = x->offset;
        break;
      }
      // strides cannot express it: one strided pass into logical row-major order
      // (what ndarray's to_shape().to_owned() does, ndarray.rs:347-353)
      cg_tensor *c = nullptr;
      TRY(materialize(be, x, &c, true));
      n->st = c->st;
      c->st->rc.fetch_add(1);
      n->stype = c->stype;
      n->offset = 0;
      contiguous_strides(n->rank, n->shape, n->strides);
      node_release(c);
      n->op = N_REAL;
      drop_inputs(n);
      return CG_OK;
    }
    default:
      return fail(be, CG_ERR_INTERNAL, "realize_view: not a view");
  }
  n->st = x->st;
  x->st->rc.fetch_add(1);
  n->stype = x->stype;
  n->op = N_REAL;
  drop_inputs(n);
  return CG_OK;
}

int realize_reduce(cg_backend *be, cg_tensor *n) {
  cg_tensor *x = n->in[0];
  const int kind = (int)n->p0;
  EwCompiler c(be);
  if (ew_inlineable(x)) TRY(c.emit(x, 0, 0, 0, true));
  else TRY(c.load(x, 0));
  std::vector<int64_t> ostr;
  double bytes_in = 0;
  TRY(finish_program(be, c, x->rank, x->shape, nullptr, true, ostr, &bytes_in));
  const int64_t cols = x->shape[x->rank - 1];
  const int64_t rows = cols ? x->size() / cols : n->size();
  if (x->size() >= (int64_t)1 << 32) return fail(be, CG_ERR_INTERNAL, "tensor above 2^32 elements");
  TRY(alloc_result(be, n, n->dtype == CG_F32 ? ST_F32 : ST_U32));
  const bool vec4 = cols % 4 == 0 && cols >= 4;
  const char *name = kind <= R_SUM_U ? "reduce_sum" : kind <= R_MAX_U ? "reduce_max" : "reduce_argmax";
  {
    KernelScope ks(be, name, bytes_in + (double)rows * 4, 0);
    HIPCHK(be, launch_reduce(be->lc(), kind, c.p, n->st->ptr, (uint32_t)rows, (uint32_t)cols, vec4));
  }
  n->op = N_REAL;
  drop_inputs(n);
  return CG_OK;
}

// Collapse the leading (batch) dims of a matmul operand pair into at most two.
bool collapse_batch(int nb, const int64_t *bshape, const int64_t *sa, const int64_t *sb,
                    uint32_t *nbo, int64_t *sao, int64_t *sbo) {
  std::vector<int64_t> sz, a, b;
  for (int i = 0; i < nb; ++i) {
    if (bshape[i] == 1) continue;
    if (!sz.empty() && a.back() == sa[i] * bshape[i] && b.back() == sb[i] * bshape[i]) {
      sz.back() *= bshape[i];
      a.back() = sa[i];
      b.back() = sb[i];
    } else {
      sz.push_back(bshape[i]);
      a.push_back(sa[i]);
      b.push_back(sb[i]);
    }
  }
  if (sz.size() > 2) return false;
  nbo[0] = nbo[1] = 1;
  sao[0] = sao[1] = sbo[0] = sbo[1] = 0;
  // right-align so that nb1 is the fastest batch dim
  for (size_t i = 0; i < sz.size(); ++i) {
    size_t d = 2 - sz.size() + i;
    nbo[d] = (uint32_t)sz[i];
    sao[d] = a[i];
    sbo[d] = b[i];
  }
  return true;
}

bool matrix_ok(const cg_tensor *t) {
  const int r = t->rank;
  const int64_t rows = t->shape[r - 2], cols = t->shape[r - 1];
  const int64_t sr = t->strides[r - 2], sc = t->strides[r - 1];
  return sc == 1 || cols == 1 || sr == 1 || rows == 1;
}

int realize_matmul(cg_backend *be, cg_tensor *n) {
  cg_tensor *a = nullptr, *b = nullptr;
  TRY(realize(be, n->in[0]));
  TRY(realize(be, n->in[1]));
  a = retain(n->in[0]);
  b = retain(n->in[1]);
  struct Guard {
    cg_tensor *&a, *&b;
    ~Guard() {
      node_release(a);
      node_release(b);
    }
  } guard{a, b};
  const int r = a->rank;
  const uint32_t M = (uint32_t)a->shape[r - 2], K = (uint32_t)a->shape[r - 1],
                 N = (uint32_t)b->shape[r - 1];
  TRY(alloc_result(be, n, n->dtype == CG_F32 ? ST_F32 : ST_U32));
  const int64_t batch = (int64_t)M * N ? n->size() / ((int64_t)M * N) : 0;
  if (n->size() == 0) {
    n->op = N_REAL;
    drop_inputs(n);
    return CG_OK;
  }
  if (n->dtype == CG_U32) {
    cg_tensor *ac = nullptr, *bc = nullptr;
    TRY(contiguous(be, a, &ac));
    node_release(a);
    a = ac;
    TRY(contiguous(be, b, &bc));
    node_release(b);
    b = bc;
    KernelScope ks(be, "matmul_u32", 0, 2.0 * batch * M * N * K);
    HIPCHK(be, launch_matmul_u32(be->lc(), (const uint32_t *)data_ptr(a), (const uint32_t *)data_ptr(b),
                                 (uint32_t *)n->st->ptr, (uint32_t)batch, M, N, K));
  } else {
    GemmDesc g;
    std::memset(&g, 0, sizeof(g));
    if (!matrix_ok(a)) {
      cg_tensor *c = nullptr;
      TRY(materialize(be, a, &c, true));
      node_release(a);
      a = c;
    }
    if (!matrix_ok(b)) {
      cg_tensor *c = nullptr;
      TRY(materialize(be, b, &c, true));
      node_release(b);
      b = c;
    }
    uint32_t nbo[2];
    int64_t sao[2], sbo[2];
    if (!collapse_batch(r - 2, a->shape, a->strides, b->strides, nbo, sao, sbo)) {
      cg_tensor *c = nullptr;
      TRY(materialize(be, a, &c, true));
      node_release(a);
      a = c;
      c = nullptr;
      TRY(materialize(be, b, &c, true));
      node_release(b);
      b = c;
      if (!collapse_batch(r - 2, a->shape, a->strides, b->strides, nbo, sao, sbo))
        return fail(be, CG_ERR_INTERNAL, "matmul: batch dims do not collapse");
    }
    g.a = data_ptr(a);
    g.b = data_ptr(b);
    g.c = (float *)n->st->ptr;
    g.a_stype = a->stype;
    g.b_stype = b->stype;
    g.M = M;
    g.N = N;
    g.K = K;
    g.sam = a->strides[r - 2];
    g.sak = a->strides[r - 1];
    g.sbk = b->strides[r - 2];
    g.sbn = b->strides[r - 1];
    // a unit extent makes its stride irrelevant: normalise so the kernels see a unit stride
    if (K == 1) g.sak = 1, g.sbk = 1;
    if (M == 1 && g.sak != 1) g.sam = 1;
    if (N == 1 && g.sbk != 1) g.sbn = 1;
    g.nb0 = nbo[0];
    g.nb1 = nbo[1];
    g.sa_b0 = sao[0];
    g.sa_b1 = sao[1];
    g.sb_b0 = sbo[0];
    g.sb_b1 = sbo[1];
    g.bf16_math = (be->flags & CG_FLAG_BF16) ? 1 : 0;
    if (!g.bf16_math && (a->stype == ST_BF16 || b->stype == ST_BF16))
      return fail(be, CG_ERR_INTERNAL, "matmul: bf16 storage without CG_FLAG_BF16");
    // bytes: each operand once (batch-broadcast operands once), output once
    auto uniq = [&](const cg_tensor *t, const int64_t *sb) {
      double e = (double)t->shape[r - 2] * t->shape[r - 1];
      if (sb[0]) e *= nbo[0];
      if (sb[1]) e *= nbo[1];
      return e * esize(t->stype);
    };
    const char *kname = "gemm";
    KernelScope ks(be, kname, uniq(a, sao) + uniq(b, sbo) + (double)n->size() * 4,
                   2.0 * batch * M * N * K);
    hipError_t e = launch_matmul(be->lc(), g, &kname);
    ks.rename(kname);
    HIPCHK(be, e);
  }
  n->op = N_REAL;
  drop_inputs(n);
  return CG_OK;
}

int realize_concat(cg_backend *be, cg_tensor *n) {
  cg_tensor *x = n->in[0], *y = n->in[1];
  TRY(realize(be, x));
  TRY(realize(be, y));
  const int keep = (x->stype == ST_BF16 && y->stype == ST_BF16) ? ST_BF16
                   : (n->dtype == CG_F32 ? ST_F32 : ST_U32);
  TRY(alloc_result(be, n, keep));
  const int dim = (int)n->p0;
  if (x->size())
    TRY(run_ew(be, x, true, n->st->ptr, n->strides, keep, "ew_concat"));
  if (y->size()) {
    char *dst = (char *)n->st->ptr + x->shape[dim] * n->strides[dim] * esize(keep);
    TRY(run_ew(be, y, true, dst, n->strides, keep, "ew_concat"));
  }
  n->op = N_REAL;
  drop_inputs(n);
  return CG_OK;
}

int realize_index(cg_backend *be, cg_tensor *n) {
  cg_tensor *x = n->in[0];
  TRY(realize(be, x));
  cg_tensor *idx = nullptr;
  TRY(contiguous(be, n->in[1], &idx));
  int st = alloc_result(be, n, n->dtype == CG_F32 ? ST_F32 : ST_U32);
  if (!st && n->size()) {
    GatherDesc g;
    std::memset(&g, 0, sizeof(g));
    g.x = data_ptr(x);
    g.idx = (const uint32_t *)data_ptr(idx);
    g.out = n->st->ptr;
    g.x_stype = x->stype;
    g.n_dims = n->rank;
    g.dim = (int)n->p0;
    g.x_dim_size = (uint32_t)x->shape[g.dim];
    bool vec = x->strides[x->rank - 1] == 1 && ((uintptr_t)g.x % (4 * esize(x->stype))) == 0;
    for (int i = 0; i < n->rank; ++i) {
      g.out_dims[i] = (uint32_t)n->shape[i];
      g.x_stride[i] = x->strides[i];
      if (i != x->rank - 1 && x->strides[i] % 4) vec = false;
    }
    g.vec = vec ? 1 : 0;
    KernelScope ks(be, "gather", (double)n->size() * (4 + esize(x->stype)) + (double)idx->size() * 4, 0);
    hipError_t e = launch_gather(be->lc(), g, (uint64_t)n->size());
    if (e != hipSuccess) st = fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
  }
  node_release(idx);
  if (st) return st;
  n->op = N_REAL;
  drop_inputs(n);
  return CG_OK;
}

int realize_arange(cg_backend *be, cg_tensor *n) {
  TRY(alloc_result(be, n, ST_U32));
  EwCompiler c(be);
  TRY(c.push(E_IOTA, 0, 0));
  c.p.n_dims = 1;
  c.p.dims[0] = (uint32_t)n->shape[0];
  OutDesc o;
  std::memset(&o, 0, sizeof(o));
  o.ptr = n->st->ptr;
  o.stype = ST_U32;
  o.stride[0] = 1;
  KernelScope ks(be, "ew_arange", (double)n->size() * 4, 0);
  HIPCHK(be, launch_ew(be->lc(), c.p, o, (uint64_t)n->size(), false));
  n->op = N_REAL;
  return CG_OK;
}

int realize(cg_backend *be, cg_tensor *n) {
  switch (n->op) {
    case N_REAL: return CG_OK;
    case N_CONST: return realize_const(be, n);
    case N_ARANGE: return realize_arange(be, n);
    case N_BIN:
    case N_UN: return realize_ew(be, n);
    case N_TRANSPOSE:
    case N_BROADCAST:
    case N_RESHAPE:
    case N_SLICE: return realize_view(be, n);
    case N_MATMUL: return realize_matmul(be, n);
    case N_REDUCE: return realize_reduce(be, n);
    case N_CONCAT: return realize_concat(be, n);
    case N_INDEX: return realize_index(be, n);
  }
  return fail(be, CG_ERR_INTERNAL, "realize: unknown node");
}

// wait for the stream and surface device-side error flags
int sync_and_check(cg_backend *be) {
  HIPCHK(be, hipMemcpyAsync(be->h_words, be->d_words, 8, hipMemcpyDeviceToHost, be->stream));
  HIPCHK(be, hipStreamSynchronize(be->stream));
  const uint32_t e = be->h_words[0];
  if (e) {
    HIPCHK(be, launch_fill_u32(be->lc(), be->d_words, 0u, 1));
    if (e & ERRF_DIV_ZERO) return fail(be, CG_ERR_ARITH, "attempt to divide by zero");
    if (e & ERRF_INDEX_OOB) return fail(be, CG_ERR_ARG, "index out of bounds");
  }
  return CG_OK;
}

int finish(cg_backend *be, cg_tensor *n, cg_tensor **out) {
  if (be->flags & CG_FLAG_EAGER) {
    int st = realize(be, n);
    if (st) {
      node_release(n);
      return st;
    }
  }
  *out = n;
  return CG_OK;
}

int check_args(cg_backend *be, cg_tensor *a, cg_tensor *b, void *out) {
  if (!be || !a || !out || (b && b->be != be) || a->be != be)
    return fail(be, CG_ERR_ARG, "null or foreign argument");
  return CG_OK;
}

int to_shape(cg_backend *be, const size_t *dims, int rank, int64_t *shape) {
  if (rank < 0 || rank > CG_MAX_RANK) return fail(be, CG_ERR_ARG, "rank out of range");
  for (int i = 0; i < rank; ++i) shape[i] = (int64_t)dims[i];
  return CG_OK;
}

int binary(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **out, EwOp f_op, EwOp u_op) {
  TRY(check_args(be, a, b, out));
  if (!b) return fail(be, CG_ERR_ARG, "null argument");
  if (a->dtype != b->dtype) return fail(be, CG_ERR_DTYPE, "binary op: dtype mismatch");
  if (a->rank != b->rank || !std::equal(a->shape, a->shape + a->rank, b->shape))
    return fail(be, CG_ERR_SHAPE, "Shape mismatch in operation: " + shape_str(a->shape, a->rank) +
                                      " vs " + shape_str(b->shape, b->rank));
  cg_tensor *n = new_node(be, a->dtype, a->rank, a->shape);
  n->op = N_BIN;
  n->ew = a->dtype == CG_F32 ? f_op : u_op;
  n->in[0] = retain(a);
  n->in[1] = retain(b);
  return finish(be, n, out);
}

int unary(cg_backend *be, cg_tensor *x, cg_tensor **out, EwOp op, cg_dtype out_dtype) {
  cg_tensor *n = new_node(be, out_dtype, x->rank, x->shape);
  n->op = N_UN;
  n->ew = op;
  n->in[0] = retain(x);
  return finish(be, n, out);
}

cg_tensor *const_node(cg_backend *be, cg_dtype dt, int rank, const int64_t *shape, uint32_t bits) {
  cg_tensor *n = new_node(be, dt, rank, shape);
  n->op = N_CONST;
  n->cbits = bits;
  return n;
}

uint32_t host_f2u(float v) {
  if (!(v == v) || v <= 0.f) return 0u;
  if (v >= 4294967296.f) return 0xFFFFFFFFu;
  return (uint32_t)v;
}

// upload `n` 32-bit words; in bf16 mode rank >= 2 f32 tensors are narrowed on the device
int upload(cg_backend *be, const void *data, size_t n, const int64_t *shape, int rank, cg_dtype dt,
           cg_tensor **out) {
  cg_tensor *t = new_node(be, dt, rank, shape);
  const bool narrow = dt == CG_F32 && rank >= 2 && (be->flags & CG_FLAG_BF16);
  int st = alloc_result(be, t, narrow ? ST_BF16 : (dt == CG_F32 ? ST_F32 : ST_U32));
  if (st) {
    node_release(t);
    return st;
  }
  if (n == 0) {
    *out = t;
    return CG_OK;
  }
  hipError_t e = hipSuccess;
  if (!narrow) {
    e = hipMemcpyAsync(t->st->ptr, data, n * 4, hipMemcpyHostToDevice, be->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(be->stream);
  } else {
    // stage through a bounded f32 buffer, narrow with the copy program (RNE)
    const size_t chunk = (size_t)16 << 20;  // elements
    Storage *stage = nullptr;
    st = dev_alloc(be, std::min(n, chunk) * 4, &stage);
    if (st) {
      node_release(t);
      return st;
    }
    for (size_t o = 0; o < n && e == hipSuccess; o += chunk) {
      const size_t c = std::min(chunk, n - o);
      e = hipMemcpyAsync(stage->ptr, (const char *)data + o * 4, c * 4, hipMemcpyHostToDevice, be->stream);
      if (e != hipSuccess) break;
      Program p;
      std::memset(&p, 0, sizeof(p));
      p.n_instr = 1;
      p.code[0].op = E_LOAD;
      p.n_in = 1;
      p.n_dims = 1;
      p.dims[0] = (uint32_t)c;
      p.in[0].ptr = stage->ptr;
      p.in[0].stride[0] = 1;
      p.in[0].stype = ST_F32;
      p.in[0].vec = 1;
      OutDesc od;
      std::memset(&od, 0, sizeof(od));
      od.ptr = (char *)t->st->ptr + o * 2;
      od.stype = ST_BF16;
      od.stride[0] = 1;
      KernelScope ks(be, "ew_to_bf16", (double)c * 6, 0);
      e = launch_ew(be->lc(), p, od, c, c % 4 == 0);
      if (e == hipSuccess) e = hipStreamSynchronize(be->stream);
    }
    storage_release(stage);
  }
  if (e != hipSuccess) {
    node_release(t);
    return fail(be, CG_ERR_DEVICE, std::string("upload: ") + hipGetErrorString(e));
  }
  *out = t;
  return CG_OK;
}

int download(cg_backend *be, cg_tensor *x, void *dst, size_t n, cg_dtype want) {
  if (!be || !x || (!dst && n)) return fail(be, CG_ERR_ARG, "null argument");
  if (x->dtype != want) return fail(be, CG_ERR_DTYPE, "to_vec: wrong dtype for this accessor");
  if ((int64_t)n != x->size()) return fail(be, CG_ERR_SHAPE, "to_vec: size mismatch");
  HIPCHK(be, hipSetDevice(be->device));
  cg_tensor *c = nullptr;
  TRY(contiguous(be, x, &c));
  int st = CG_OK;
  if (n) {
    hipError_t e = hipMemcpyAsync(dst, data_ptr(c), n * 4, hipMemcpyDeviceToHost, be->stream);
    if (e != hipSuccess) st = fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
  }
  if (!st) st = sync_and_check(be);
  node_release(c);
  return st;
}

}  // namespace

extern "C" {

int cg_backend_create(int device, uint32_t flags, cg_backend **out) {
  if (!out) return CG_ERR_ARG;
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || device < 0 || device >= count) {
    (void)hipGetLastError();
    return CG_ERR_DEVICE;
  }
  if (hipSetDevice(device) != hipSuccess) return CG_ERR_DEVICE;
  cg_backend *be = new cg_backend();
  be->device = device;
  be->flags = flags;
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, device) == hipSuccess) be->n_cus = prop.multiProcessorCount;
  if (hipStreamCreate(&be->stream) != hipSuccess || hipMalloc((void **)&be->d_words, 256) != hipSuccess ||
      hipHostMalloc((void **)&be->h_words, 256, hipHostMallocDefault) != hipSuccess ||
      hipMemsetAsync(be->d_words, 0, 256, be->stream) != hipSuccess ||
      hipStreamSynchronize(be->stream) != hipSuccess) {
    delete be;
    return CG_ERR_DEVICE;
  }
  *out = be;
  return CG_OK;
}

void cg_backend_destroy(cg_backend *be) { backend_release(be); }
const char *cg_last_error(const cg_backend *be) { return be ? be->err.c_str() : ""; }
const char *cg_backend_name(const cg_backend *) { return "hip-gfx950"; }

int cg_sync(cg_backend *be) {
  if (!be) return CG_ERR_ARG;
  HIPCHK(be, hipSetDevice(be->device));
  return sync_and_check(be);
}

cg_tensor *cg_tensor_retain(cg_tensor *t) { return t ? retain(t) : t; }
void cg_tensor_release(cg_tensor *t) { node_release(t); }
int cg_tensor_rank(const cg_tensor *t) { return t->rank; }
int cg_tensor_shape(const cg_tensor *t, size_t *dims) {
  for (int i = 0; i < t->rank; ++i) dims[i] = (size_t)t->shape[i];
  return CG_OK;
}
cg_dtype cg_tensor_dtype(const cg_tensor *t) { return t->dtype; }
size_t cg_tensor_size(const cg_tensor *t) { return (size_t)t->size(); }

// ndarray.rs:53-65
int cg_zeros(cg_backend *be, const size_t *dims, int rank, cg_dtype dtype, cg_tensor **out) {
  if (!be || !out) return CG_ERR_ARG;
  int64_t shape[CG_MAX_RANK];
  TRY(to_shape(be, dims, rank, shape));
  return finish(be, const_node(be, dtype, rank, shape, 0u), out);
}

// ndarray.rs:67-89; interpreter/mod.rs:21-31
static int from_host(cg_backend *be, const void *data, size_t n, const size_t *dims, int rank,
                     cg_dtype dt, cg_tensor **out) {
  if (!be || !out || (!data && n)) return fail(be, CG_ERR_ARG, "null argument");
  int64_t shape[CG_MAX_RANK];
  TRY(to_shape(be, dims, rank, shape));
  int64_t sz = 1;
  for (int i = 0; i < rank; ++i) sz *= shape[i];
  if ((int64_t)n != sz) return fail(be, CG_ERR_SHAPE, "ShapeError");
  if (n == 1) {  // scalars stay on the host until a kernel needs them (tensor_op.rs:55-78)
    uint32_t bits;
    std::memcpy(&bits, data, 4);
    return finish(be, const_node(be, dt, rank, shape, bits), out);
  }
  HIPCHK(be, hipSetDevice(be->device));
  return upload(be, data, n, shape, rank, dt, out);
}
int cg_from_f32(cg_backend *be, const float *d, size_t n, const size_t *dims, int rank, cg_tensor **out) {
  return from_host(be, d, n, dims, rank, CG_F32, out);
}
int cg_from_u32(cg_backend *be, const uint32_t *d, size_t n, const size_t *dims, int rank,
                cg_tensor **out) {
  return from_host(be, d, n, dims, rank, CG_U32, out);
}

// ndarray.rs:97-114
int cg_cast(cg_backend *be, cg_tensor *x, cg_dtype target, cg_tensor **out) {
  TRY(check_args(be, x, nullptr, out));
  if (x->dtype == target) {
    *out = retain(x);
    return CG_OK;
  }
  if (x->op == N_CONST) {
    uint32_t bits;
    if (target == CG_U32) {
      float f;
      std::memcpy(&f, &x->cbits, 4);
      bits = host_f2u(f);
    } else {
      float f = (float)x->cbits;
      std::memcpy(&bits, &f, 4);
    }
    return finish(be, const_node(be, target, x->rank, x->shape, bits), out);
  }
  return unary(be, x, out, target == CG_U32 ? E_F2U : E_U2F, target);
}

// ndarray.rs:549-615; shape_only.rs:255-285
int cg_matmul(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **out) {
  TRY(check_args(be, a, b, out));
  if (!b) return fail(be, CG_ERR_ARG, "null argument");
  if (a->dtype != b->dtype) return fail(be, CG_ERR_DTYPE, "matmul: dtype mismatch");
  if (a->rank < 2) return fail(be, CG_ERR_SHAPE, "batched_matmul: lhs must be at least rank 2");
  if (b->rank < 2) return fail(be, CG_ERR_SHAPE, "batched_matmul: rhs must be at least rank 2");
  if (a->shape[a->rank - 1] != b->shape[b->rank - 2])
    return fail(be, CG_ERR_SHAPE, "batched_matmul: incompatible matrix dimensions");
  if (a->rank != b->rank || !std::equal(a->shape, a->shape + a->rank - 2, b->shape))
    return fail(be, CG_ERR_SHAPE, "batched_matmul: batch dimensions must match");
  int64_t shape[CG_MAX_RANK];
  for (int i = 0; i < a->rank - 2; ++i) shape[i] = a->shape[i];
  shape[a->rank - 2] = a->shape[a->rank - 2];
  shape[a->rank - 1] = b->shape[b->rank - 1];
  cg_tensor *n = new_node(be, a->dtype, a->rank, shape);
  n->op = N_MATMUL;
  n->in[0] = retain(a);
  n->in[1] = retain(b);
  return finish(be, n, out);
}

// ndarray.rs:124-198, 401-453
int cg_add(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **o) { return binary(be, a, b, o, E_ADD_F, E_ADD_U); }
int cg_sub(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **o) { return binary(be, a, b, o, E_SUB_F, E_SUB_U); }
int cg_mul(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **o) { return binary(be, a, b, o, E_MUL_F, E_MUL_U); }
int cg_div(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **o) { return binary(be, a, b, o, E_DIV_F, E_DIV_U); }
int cg_pow(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **o) { return binary(be, a, b, o, E_POW_F, E_POW_U); }
int cg_lt(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **o) { return binary(be, a, b, o, E_LT_F, E_LT_U); }
int cg_eq(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **o) { return binary(be, a, b, o, E_EQ_F, E_EQ_U); }

// ndarray.rs:200-222, 433-441
int cg_sin(cg_backend *be, cg_tensor *x, cg_tensor **out) {
  TRY(check_args(be, x, nullptr, out));
  if (x->dtype != CG_F32) return fail(be, CG_ERR_DTYPE, "Invalid input types for sin");
  return unary(be, x, out, E_SIN_F, CG_F32);
}
int cg_cos(cg_backend *be, cg_tensor *x, cg_tensor **out) {
  TRY(check_args(be, x, nullptr, out));
  if (x->dtype != CG_F32) return fail(be, CG_ERR_DTYPE, "Invalid input types for cos");
  return unary(be, x, out, E_COS_F, CG_F32);
}
int cg_neg(cg_backend *be, cg_tensor *x, cg_tensor **out) {
  TRY(check_args(be, x, nullptr, out));
  return unary(be, x, out, x->dtype == CG_F32 ? E_NEG_F : E_NEG_U, x->dtype);
}

// ndarray.rs:355-361: numpy broadcasting, right aligned
int cg_broadcast(cg_backend *be, cg_tensor *x, const size_t *dims, int rank, cg_tensor **out) {
  TRY(check_args(be, x, nullptr, out));
  int64_t shape[CG_MAX_RANK];
  TRY(to_shape(be, dims, rank, shape));
  if (x->rank > rank) return fail(be, CG_ERR_SHAPE, "broadcast: rank of target too small");
  for (int i = 0; i < x->rank; ++i) {
    int64_t xd = x->shape[x->rank - 1 - i], td = shape[rank - 1 - i];
    if (xd != td && xd != 1)
      return fail(be, CG_ERR_SHAPE, "broadcast: " + shape_str(x->shape, x->rank) + " to " + shape_str(shape, rank));
  }
  if (x->op == N_CONST) return finish(be, const_node(be, x->dtype, rank, shape, x->cbits), out);
  cg_tensor *n = new_node(be, x->dtype, rank, shape);
  n->op = N_BROADCAST;
  n->in[0] = retain(x);
  if (x->op == N_REAL) TRY(realize_view(be, n));
  return finish(be, n, out);
}

// ndarray.rs:347-353
int cg_reshape(cg_backend *be, cg_tensor *x, const size_t *dims, int rank, cg_tensor **out) {
  TRY(check_args(be, x, nullptr, out));
  int64_t shape[CG_MAX_RANK];
  TRY(to_shape(be, dims, rank, shape));
  int64_t sz = 1;
  for (int i = 0; i < rank; ++i) sz *= shape[i];
  if (sz != x->size())
    return fail(be, CG_ERR_SHAPE, "reshape: " + shape_str(x->shape, x->rank) + " to " + shape_str(shape, rank));
  if (x->op == N_CONST) return finish(be, const_node(be, x->dtype, rank, shape, x->cbits), out);
  cg_tensor *n = new_node(be, x->dtype, rank, shape);
  n->op = N_RESHAPE;
  n->in[0] = retain(x);
  // a reshape that is a pure view of realised data costs nothing: do it now
  int64_t tmp[CG_MAX_RANK];
  if (x->op == N_REAL && (sz == 0 || try_reshape_view(x->rank, x->shape, x->strides, rank, shape, tmp)))
    TRY(realize_view(be, n));
  return finish(be, n, out);
}

// ndarray.rs:363-371
int cg_transpose(cg_backend *be, cg_tensor *x, size_t d0, size_t d1, cg_tensor **out) {
  TRY(check_args(be, x, nullptr, out));
  if (d0 >= (size_t)x->rank || d1 >= (size_t)x->rank) return fail(be, CG_ERR_ARG, "transpose: axis out of range");
  int64_t shape[CG_MAX_RANK];
  std::copy(x->shape, x->shape + x->rank, shape);
  std::swap(shape[d0], shape[d1]);
  if (x->op == N_CONST) return finish(be, const_node(be, x->dtype, x->rank, shape, x->cbits), out);
  cg_tensor *n = new_node(be, x->dtype, x->rank, shape);
  n->op = N_TRANSPOSE;
  n->p0 = (int64_t)d0;
  n->p1 = (int64_t)d1;
  n->in[0] = retain(x);
  if (x->op == N_REAL) TRY(realize_view(be, n));
  return finish(be, n, out);
}

static int reduce(cg_backend *be, cg_tensor *x, cg_tensor **out, int f_kind, int u_kind, cg_dtype odt) {
  TRY(check_args(be, x, nullptr, out));
  if (x->rank == 0) return fail(be, CG_ERR_SHAPE, "reduction of a rank-0 tensor");
  int64_t shape[CG_MAX_RANK];
  std::copy(x->shape, x->shape + x->rank, shape);
  shape[x->rank - 1] = 1;
  cg_tensor *n = new_node(be, odt, x->rank, shape);
  n->op = N_REDUCE;
  n->p0 = x->dtype == CG_F32 ? f_kind : u_kind;
  n->in[0] = retain(x);
  return finish(be, n, out);
}
// ndarray.rs:455-467, 522-529, 469-493
int cg_max(cg_backend *be, cg_tensor *x, cg_tensor **out) { return reduce(be, x, out, R_MAX_F, R_MAX_U, x ? x->dtype : CG_F32); }
int cg_sum(cg_backend *be, cg_tensor *x, cg_tensor **out) { return reduce(be, x, out, R_SUM_F, R_SUM_U, x ? x->dtype : CG_F32); }
int cg_argmax(cg_backend *be, cg_tensor *x, cg_tensor **out) {
  if (x && x->rank > 0 && x->shape[x->rank - 1] == 0) return fail(be, CG_ERR_SHAPE, "argmax of an empty lane");
  return reduce(be, x, out, R_ARGMAX_F, R_ARGMAX_U, CG_U32);
}

// ndarray.rs:495-520
int cg_topk(cg_backend *be, cg_tensor *x, size_t k, cg_tensor **values, cg_tensor **indices) {
  TRY(check_args(be, x, nullptr, values));
  if (!indices) return fail(be, CG_ERR_ARG, "null argument");
  if (x->dtype != CG_F32) return fail(be, CG_ERR_DTYPE, "Unsupported type for topk");
  if (x->rank == 0) return fail(be, CG_ERR_SHAPE, "topk of a rank-0 tensor");
  const int64_t n = x->shape[x->rank - 1];
  if ((int64_t)k > n) return fail(be, CG_ERR_SHAPE, "topk: k larger than the last dimension");
  HIPCHK(be, hipSetDevice(be->device));
  cg_tensor *c = nullptr;
  TRY(contiguous(be, x, &c));
  int64_t shape[CG_MAX_RANK];
  std::copy(x->shape, x->shape + x->rank, shape);
  shape[x->rank - 1] = (int64_t)k;
  cg_tensor *v = new_node(be, CG_F32, x->rank, shape), *ix = new_node(be, CG_U32, x->rank, shape);
  int st = alloc_result(be, v, ST_F32);
  if (!st) st = alloc_result(be, ix, ST_U32);
  if (!st) {
    const int64_t rows = n ? x->size() / n : 0;
    KernelScope ks(be, "topk", (double)x->size() * 4, 0);
    hipError_t e = launch_topk(be->lc(), (const float *)data_ptr(c), (float *)v->st->ptr,
                               (uint32_t *)ix->st->ptr, (uint32_t)rows, (uint32_t)n, (uint32_t)k);
    if (e != hipSuccess) st = fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
  }
  node_release(c);
  if (st) {
    node_release(v);
    node_release(ix);
    return st;
  }
  *values = v;
  *indices = ix;
  return CG_OK;
}

// ndarray.rs:337-343
int cg_compare(cg_backend *be, cg_tensor *a, cg_tensor *b, int *equal) {
  TRY(check_args(be, a, b, equal));
  if (!b) return fail(be, CG_ERR_ARG, "null argument");
  if (a->dtype != b->dtype) return fail(be, CG_ERR_DTYPE, "compare: dtype mismatch");
  *equal = 0;
  if (a->rank != b->rank || !std::equal(a->shape, a->shape + a->rank, b->shape)) return CG_OK;
  HIPCHK(be, hipSetDevice(be->device));
  cg_tensor *ac = nullptr, *bc = nullptr;
  TRY(contiguous(be, a, &ac));
  int st = contiguous(be, b, &bc);
  if (!st) {
    hipError_t e = launch_fill_u32(be->lc(), be->d_words + 1, 0u, 1);
    if (e == hipSuccess) {
      KernelScope ks(be, "compare", (double)a->size() * 8, 0);
      e = launch_compare(be->lc(), data_ptr(ac), data_ptr(bc), (uint64_t)a->size(), a->dtype == CG_F32,
                         be->d_words + 1);
    }
    if (e != hipSuccess) st = fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
    if (!st) st = sync_and_check(be);
    if (!st) *equal = be->h_words[1] == 0;
  }
  node_release(ac);
  node_release(bc);
  return st;
}

// ndarray.rs:393-399
int cg_concat(cg_backend *be, cg_tensor *x, cg_tensor *y, size_t dim, cg_tensor **out) {
  TRY(check_args(be, x, y, out));
  if (!y) return fail(be, CG_ERR_ARG, "null argument");
  if (x->dtype != y->dtype) return fail(be, CG_ERR_DTYPE, "Incompatible types for concatenation");
  if (x->rank != y->rank || dim >= (size_t)x->rank) return fail(be, CG_ERR_SHAPE, "concat: rank/axis mismatch");
  for (int i = 0; i < x->rank; ++i)
    if (i != (int)dim && x->shape[i] != y->shape[i])
      return fail(be, CG_ERR_SHAPE, "concat: " + shape_str(x->shape, x->rank) + " with " + shape_str(y->shape, y->rank));
  int64_t shape[CG_MAX_RANK];
  std::copy(x->shape, x->shape + x->rank, shape);
  shape[dim] += y->shape[dim];
  cg_tensor *n = new_node(be, x->dtype, x->rank, shape);
  n->op = N_CONCAT;
  n->p0 = (int64_t)dim;
  n->in[0] = retain(x);
  n->in[1] = retain(y);
  return finish(be, n, out);
}

// ndarray.rs:373-381
int cg_index(cg_backend *be, cg_tensor *x, size_t dim, cg_tensor *indices, cg_tensor **out) {
  TRY(check_args(be, x, indices, out));
  if (!indices) return fail(be, CG_ERR_ARG, "null argument");
  if (indices->dtype != CG_U32) return fail(be, CG_ERR_DTYPE, "Invalid input types for indexing");
  if (dim >= (size_t)x->rank) return fail(be, CG_ERR_ARG, "index: axis out of range");
  int64_t shape[CG_MAX_RANK];
  std::copy(x->shape, x->shape + x->rank, shape);
  shape[dim] = indices->size();
  cg_tensor *n = new_node(be, x->dtype, x->rank, shape);
  n->op = N_INDEX;
  n->p0 = (int64_t)dim;
  n->in[0] = retain(x);
  n->in[1] = retain(indices);
  return finish(be, n, out);
}

// ndarray.rs:383-391
int cg_slice(cg_backend *be, cg_tensor *x, size_t dim, size_t start, size_t len, cg_tensor **out) {
  TRY(check_args(be, x, nullptr, out));
  if (dim >= (size_t)x->rank) return fail(be, CG_ERR_ARG, "slice: axis out of range");
  if (start + len > (size_t)x->shape[dim]) return fail(be, CG_ERR_SHAPE, "slice: range out of bounds");
  int64_t shape[CG_MAX_RANK];
  std::copy(x->shape, x->shape + x->rank, shape);
  shape[dim] = (int64_t)len;
  if (x->op == N_CONST) return finish(be, const_node(be, x->dtype, x->rank, shape, x->cbits), out);
  cg_tensor *n = new_node(be, x->dtype, x->rank, shape);
  n->op = N_SLICE;
  n->p0 = (int64_t)dim;
  n->p1 = (int64_t)start;
  n->in[0] = retain(x);
  if (x->op == N_REAL) TRY(realize_view(be, n));
  return finish(be, n, out);
}

// ndarray.rs:91-95
int cg_arange(cg_backend *be, size_t end, cg_tensor **out) {
  if (!be || !out) return CG_ERR_ARG;
  int64_t shape[1] = {(int64_t)end};
  cg_tensor *n = new_node(be, CG_U32, 1, shape);
  n->op = N_ARANGE;
  return finish(be, n, out);
}

// ndarray.rs:46-51
int cg_to_f32(cg_backend *be, cg_tensor *x, float *dst, size_t n) { return download(be, x, dst, n, CG_F32); }
int cg_to_u32(cg_backend *be, cg_tensor *x, uint32_t *dst, size_t n) { return download(be, x, dst, n, CG_U32); }

int cg_trace_enable(cg_backend *be, int on) {
  if (!be) return CG_ERR_ARG;
  trace_collect(be);
  be->trace = on != 0;
  return CG_OK;
}
int cg_trace_reset(cg_backend *be) {
  if (!be) return CG_ERR_ARG;
  trace_collect(be);
  be->trace_recs.clear();
  return CG_OK;
}
size_t cg_trace_report(cg_backend *be, char *buf, size_t cap) {
  if (!be) return 0;
  trace_collect(be);
  std::string s;
  char line[256];
  for (auto &kv : be->trace_recs) {
    snprintf(line, sizeof(line), "%s %llu %.6f %.0f %.0f\n", kv.first.c_str(),
             (unsigned long long)kv.second.launches, kv.second.ms, kv.second.bytes, kv.second.flops);
    s += line;
  }
  if (buf && cap) {
    size_t n = std::min(cap - 1, s.size());
    std::memcpy(buf, s.data(), n);
    buf[n] = 0;
  }
  return s.size() + 1;
}
int cg_stats(cg_backend *be, uint64_t *l, uint64_t *d, uint64_t *p) {
  if (!be) return CG_ERR_ARG;
  if (l) *l = be->launches;
  if (d) *d = be->device_bytes;
  if (p) *p = be->pool_bytes;
  return CG_OK;
}

}  // extern "C"
