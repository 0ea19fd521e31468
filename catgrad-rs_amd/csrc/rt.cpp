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
  if (be->queue) be->queue->drain();  // a launch still in the queue may read what is about to be freed
  for (auto &kv : be->pool)
    for (void *p : kv.second) {
      (void)hipFree(p);
      be->device_bytes -= kv.first;
    }
  be->pool.clear();
  be->pool_bytes = 0;
}

// Called at synchronisation points (the stream is idle): a long run over changing sizes would otherwise
// keep every block it ever freed.  Above POOL_CAP of cached blocks the largest size classes go back to
// the driver until the pool is under half the cap; the working set of a steady loop (the same sizes
// every step) stays far below it and is never touched.
void cap_pool(cg_backend *be) {
  const uint64_t POOL_CAP = (uint64_t)32 << 30;
  if (be->pool_bytes <= POOL_CAP) return;
  for (auto it = be->pool.rbegin(); it != be->pool.rend() && be->pool_bytes > POOL_CAP / 2; ++it) {
    std::vector<void *> &blocks = it->second;
    while (!blocks.empty() && be->pool_bytes > POOL_CAP / 2) {
      (void)hipFree(blocks.back());
      blocks.pop_back();
      be->pool_bytes -= it->first;
      be->device_bytes -= it->first;
    }
  }
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
  storage_release(s->shadow);
  storage_release(s->tiles);
  cg_backend *be = s->be;
  // Safe to recycle at once: every consumer was enqueued on the backend's only stream.
  be->pool[s->bytes].push_back(s->ptr);
  be->pool_bytes += s->bytes;
  delete s;
}

void backend_release(cg_backend *be) {
  if (!be || be->rc.fetch_sub(1) != 1) return;
  (void)hipSetDevice(be->device);
  (void)hipStreamSynchronize(be->ordered_stream());
  for (auto &pe : be->trace_pending) {
    (void)hipEventDestroy(pe.start);
    (void)hipEventDestroy(pe.stop);
  }
  trim_pool(be);
  for (void *p : be->pinned_pool) (void)hipHostFree(p);
  for (hipEvent_t ev : be->event_pool) (void)hipEventDestroy(ev);
  if (be->d_words) (void)hipFree(be->d_words);
  if (be->attn_part) (void)hipFree(be->attn_part);
  if (be->attn_count) (void)hipFree(be->attn_count);
  if (be->h_words) (void)hipHostFree(be->h_words);
  delete be->queue;  // drains and joins its thread
  be->queue = nullptr;
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

void forget_gemv_candidate(cg_tensor *n) {
  auto &v = n->be->gemv_candidates;
  for (size_t i = 0; i < v.size(); ++i)
    if (v[i] == n) {
      v[i] = v.back();
      v.pop_back();
      break;
    }
  n->gemv_candidate = false;
}

void forget_gemm_candidate(cg_tensor *n) {
  auto &v = n->be->gemm_candidates;
  for (size_t i = 0; i < v.size(); ++i)
    if (v[i] == n) {
      v[i] = v.back();
      v.pop_back();
      break;
    }
  n->gemm_candidate = false;
}

enum { PREFETCH_BYTES = 4096 };  // pinned buffer of a prefetched tensor: data + 8 bytes of error words

void forget_shared(cg_tensor *n);

void node_release(cg_tensor *t) {
  if (!t || t->rc.fetch_sub(1) != 1) return;  // the common case takes no allocation
  std::vector<cg_tensor *> stack{t};
  while (!stack.empty()) {
    cg_tensor *n = stack.back();
    stack.pop_back();
    if (n != t && n->rc.fetch_sub(1) != 1) continue;
    if (n->gemv_candidate) forget_gemv_candidate(n);
    if (n->gemm_candidate) forget_gemm_candidate(n);
    forget_shared(n);
    if (n->bias_of && n->bias_of->bias_user == n) n->bias_of->bias_user = nullptr;  // its inputs are still alive here
    if (n->in[0]) stack.push_back(n->in[0]);
    if (n->in[1]) stack.push_back(n->in[1]);
    storage_release(n->st);
    cg_backend *be = n->be;
    if (n->host_copy) {
      // the copy may still be in flight: the buffer is only reused after its event has completed
      (void)hipEventSynchronize(n->host_ev);
      be->pinned_pool.push_back(n->host_copy);
      be->event_pool.push_back(n->host_ev);
    }
    delete n;
    backend_release(be);
  }
}

cg_tensor *retain(cg_tensor *t) {
  t->rc.fetch_add(1);
  return t;
}

// a deleted node leaves the table of shared nodes
void forget_shared(cg_tensor *n) {
  if (!n->cse_key) return;
  auto it = n->be->shared_nodes.find(*n->cse_key);
  if (it != n->be->shared_nodes.end() && it->second == n) n->be->shared_nodes.erase(it);
  delete n->cse_key;
  n->cse_key = nullptr;
}

void drop_inputs(cg_tensor *n) {
  if (n->bias_of) {
    if (n->bias_of->bias_user == n) n->bias_of->bias_user = nullptr;
    n->bias_of = nullptr;
  }
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
// Accounts one kernel launch.  When tracing, the launch (issued through CG_LAUNCH with the
// backend's current events) gets its own begin/end timestamps from the runtime.
struct KernelScope {
  cg_backend *be;
  PendingEvent pe;
  bool on;
  KernelScope(cg_backend *b, const char *name, double bytes, double flops) : be(b), on(b->trace) {
    be->launches++;
    count(name);
    if (!on) return;
    pe.name = name;
    pe.bytes = bytes;
    pe.flops = flops;
    (void)hipEventCreate(&pe.start);
    (void)hipEventCreate(&pe.stop);
    be->cur_start = pe.start;
    be->cur_stop = pe.stop;
  }
  // one cached slot per name pointer: the names are string literals
  void count(const char *name) {
    static thread_local const char *last_name = nullptr;
    static thread_local uint64_t last_be = 0;
    static thread_local uint64_t *last_slot = nullptr;
    if (name != last_name || be->uid != last_be) {
      last_slot = &be->launch_counts[name];
      last_name = name;
      last_be = be->uid;
    }
    ++*last_slot;
  }
  void rename(const std::string &name) {
    if (on && !name.empty()) pe.name = name;
  }
  ~KernelScope() {
    if (!on) return;
    be->cur_start = be->cur_stop = nullptr;
    be->trace_pending.push_back(pe);
  }
};

void trace_collect(cg_backend *be) {
  if (be->trace_pending.empty()) return;
  (void)hipStreamSynchronize(be->ordered_stream());
  for (auto &pe : be->trace_pending) {
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, pe.start, pe.stop) == hipSuccess) {  // fails if nothing was launched
      TraceRec &r = be->trace_recs[pe.name];
      r.launches++;
      r.ms += ms;
      r.bytes += pe.bytes;
      r.flops += pe.flops;
    } else {
      (void)hipGetLastError();
    }
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

// ---- fusion regions ------------------------------------------------------------------------
// A region is the set of deferred nodes that one kernel evaluates: the elementwise tree under a
// root and, when `rows` is on, the row values it reads through a last-axis broadcast:
//     root <- BIN/UN ... <- BROADCAST <- (BIN/UN on [.., 1])* <- REDUCE(sum|max) <- BIN/UN ...
// A node may be evaluated inside the region (instead of being materialised) iff every reference
// to it comes from inside the region; a node referenced k times is simply evaluated k times.
bool same_shape(const cg_tensor *a, const cg_tensor *b) {
  return a->rank == b->rank && std::equal(a->shape, a->shape + a->rank, b->shape);
}

// `b` broadcasts a [.., 1] tensor along the last axis only, to the shape of `root`
bool is_row_broadcast(const cg_tensor *b, const cg_tensor *root) {
  if (b->op != N_BROADCAST || !same_shape(b, root) || b->rank == 0) return false;
  const cg_tensor *r = b->in[0];
  if (r->rank != b->rank || r->shape[r->rank - 1] != 1) return false;
  for (int i = 0; i + 1 < r->rank; ++i)
    if (r->shape[i] != b->shape[i]) return false;
  return true;
}

// every leaf under the row value `r` is a constant or a fusable reduction of a root-shaped tensor
bool row_chain_ok(const cg_tensor *r, const cg_tensor *root, int depth = 0) {
  if (depth > 32) return false;
  if (r->op == N_CONST) return true;
  if (r->op == N_BIN) return row_chain_ok(r->in[0], root, depth + 1) && row_chain_ok(r->in[1], root, depth + 1);
  if (r->op == N_UN) return row_chain_ok(r->in[0], root, depth + 1);
  if (r->op == N_REDUCE && r->p0 <= R_MAX_U) return same_shape(r->in[0], root);
  return false;
}

struct Region {
  const cg_tensor *root = nullptr;
  bool rows = false;
  std::vector<std::pair<const cg_tensor *, int>> refs;  // internal reference counts
  std::vector<cg_tensor *> order;                        // children before parents

  int *count(const cg_tensor *n) {
    for (auto &kv : refs)
      if (kv.first == n) return &kv.second;
    return nullptr;
  }
  // true the first time `n` is seen
  bool edge(const cg_tensor *n) {
    if (int *c = count(n)) {
      ++*c;
      return false;
    }
    refs.emplace_back(n, 1);
    return true;
  }
  bool qualified(const cg_tensor *n) const {
    for (const cg_tensor *o : order)
      if (o == n) return true;
    return false;
  }
  // evaluated inside the kernel: a walked node all of whose readers are in the region
  bool inside(const cg_tensor *n) {
    if (n == root) return true;
    int *c = count(n);
    return c && n->op != N_REAL && n->rc.load() == *c && qualified(n);
  }

  void walk_full(cg_tensor *n) {
    if (n->op == N_BIN || n->op == N_UN) {
      for (int i = 0; i < 2; ++i)
        if (cg_tensor *c = n->in[i])
          if (edge(c)) walk_full(c);
      order.push_back(n);
    } else if (rows && is_row_broadcast(n, root) && row_chain_ok(n->in[0], root)) {
      if (edge(n->in[0])) walk_row(n->in[0]);
      order.push_back(n);
    }
  }
  void walk_row(cg_tensor *r) {
    if (r->op == N_BIN || r->op == N_UN) {
      for (int i = 0; i < 2; ++i)
        if (cg_tensor *c = r->in[i])
          if (edge(c)) walk_row(c);
      order.push_back(r);
    } else if (r->op == N_REDUCE) {
      if (edge(r->in[0])) walk_full(r->in[0]);
      order.push_back(r);
    }
  }
  void build(cg_tensor *root_, bool rows_) {
    root = root_;
    rows = rows_;
    refs.clear();
    order.clear();
    walk_full(root_);
  }
  // a deferred node of the region that somebody outside also reads: it has to exist in memory
  cg_tensor *shared_node() {
    for (cg_tensor *n : order)
      if (n != root && !inside(n)) return n;
    return nullptr;
  }
};

struct EwCompiler {
  cg_backend *be;
  Region *reg;
  Program p;
  std::vector<cg_tensor *> ins;
  std::vector<uint32_t> imms;
  struct Stage {
    const cg_tensor *reduce;
    std::vector<Instr> code;
  };
  std::vector<Stage> stages;
  std::vector<Instr> final_code;
  bool overflow = false;  // a limit was hit: the caller retries with a smaller region

  EwCompiler(cg_backend *b, Region *r) : be(b), reg(r) { std::memset(&p, 0, sizeof(p)); }

  int total_instr() const {
    size_t n = final_code.size();
    for (auto &s : stages) n += s.code.size();
    return (int)n;
  }
  int push(std::vector<Instr> &code, uint8_t op, int depth, uint16_t arg) {
    // a push writes slot `depth`; an operator reads the slots below `depth`
    const bool is_push = op <= E_ROW1;
    if (total_instr() >= MAX_INSTR || depth > MAX_STACK || (is_push && depth >= MAX_STACK)) {
      overflow = true;
      return fail(be, CG_ERR_INTERNAL, "elementwise program overflow");
    }
    Instr i;
    i.op = op;
    i.depth = (uint8_t)depth;
    i.arg = arg;
    code.push_back(i);
    return CG_OK;
  }
  int push_const(std::vector<Instr> &code, uint32_t bits, int depth) {
    size_t k = 0;
    for (; k < imms.size(); ++k)
      if (imms[k] == bits) break;
    if (k == imms.size()) imms.push_back(bits);
    return push(code, E_CONST, depth, (uint16_t)k);
  }
  int load(std::vector<Instr> &code, cg_tensor *n, int depth) {
    if (n->op != N_REAL) TRY(realize(be, n));
    size_t slot = 0;
    for (; slot < ins.size(); ++slot)
      if (ins[slot] == n) break;
    if (slot == ins.size()) {
      if (ins.size() >= MAX_IN) {
        overflow = true;
        return fail(be, CG_ERR_INTERNAL, "elementwise program: too many inputs");
      }
      ins.push_back(n);
    }
    return push(code, E_LOAD, depth, (uint16_t)slot);
  }
  static bool is_const(const cg_tensor *n, uint32_t bits) { return n->op == N_CONST && n->cbits == bits; }

  // stack slots needed to evaluate `n` (capped), mirroring emit/emit_op
  int need(cg_tensor *n, bool row, int budget = 64) {
    if (budget <= 0) return MAX_STACK + 1;
    if (n->op == N_CONST) return 1;
    if (!row) {
      if (!reg->inside(n)) return 1;
      if (n->op == N_BROADCAST) return need(n->in[0], true, budget - 1);
    } else if (n->op == N_REDUCE) {
      return 1;
    }
    if (n->op == N_UN) return need(n->in[0], row, budget - 1);
    if (n->op != N_BIN) return 1;
    cg_tensor *a = n->in[0], *b = n->in[1];
    if (n->ew == E_POW_F && is_const(a, 0x402DF854u)) return need(b, row, budget - 1);
    if (n->ew == E_POW_F && (is_const(b, 0x3F000000u) || is_const(b, 0x40400000u))) return need(a, row, budget - 1);
    if (n->ew == E_DIV_F && is_const(a, 0x3F800000u)) return need(b, row, budget - 1);
    const int na = need(a, row, budget / 2), nb = need(b, row, budget / 2);
    const int fwd = std::max(na, nb + 1), rev = std::max(nb, na + 1);
    return commutative(n->ew) ? std::min(fwd, rev) : fwd;
  }
  static bool commutative(uint8_t op) {
    return op == E_ADD_F || op == E_MUL_F || op == E_EQ_F || op == E_ADD_U || op == E_MUL_U || op == E_EQ_U;
  }

  int emit_op(std::vector<Instr> &code, cg_tensor *n, int depth, bool row) {
    auto sub = [&](cg_tensor *c, int d) { return row ? emit_row(code, c, d) : emit(code, c, d); };
    if (n->op == N_UN) {
      TRY(sub(n->in[0], depth));
      return push(code, n->ew, depth + 1, 0);
    }
    cg_tensor *a = n->in[0], *b = n->in[1];
    if (n->ew == E_POW_F) {
      // nn::exp = pow(broadcast(E), x); nn::sqrt = pow(x, broadcast(0.5)); gelu: pow(x, 3)
      // (catgrad/src/stdlib/nn/mod.rs:117-128, 157)
      if (is_const(a, 0x402DF854u)) {
        TRY(sub(b, depth));
        return push(code, E_EXP_F, depth + 1, 0);
      }
      if (is_const(b, 0x3F000000u) || is_const(b, 0x40400000u)) {
        TRY(sub(a, depth));
        return push(code, is_const(b, 0x3F000000u) ? E_SQRT_F : E_CUBE_F, depth + 1, 0);
      }
    }
    if (n->ew == E_DIV_F && is_const(a, 0x3F800000u)) {
      TRY(sub(b, depth));
      return push(code, E_RCP_F, depth + 1, 0);
    }
    // commutative ops evaluate the deeper operand first (fewer live stack slots)
    if (commutative(n->ew) && need(b, row) > need(a, row)) std::swap(a, b);
    TRY(sub(a, depth));
    TRY(sub(b, depth + 1));
    return push(code, n->ew, depth + 2, 0);
  }

  // value of the root-shaped node `n` at stack slot `depth`
  int emit(std::vector<Instr> &code, cg_tensor *n, int depth) {
    if (n->op == N_CONST) return push_const(code, n->cbits, depth);
    if (n->op == N_ARANGE && n->rank == 1) return push(code, E_IOTA, depth, 0);
    if (reg->inside(n)) {
      if (n->op == N_BIN || n->op == N_UN) return emit_op(code, n, depth, false);
      if (n->op == N_BROADCAST) return emit_row(code, n->in[0], depth);
    }
    return load(code, n, depth);
  }

  // value of the row-shaped node `r`
  int emit_row(std::vector<Instr> &code, cg_tensor *r, int depth) {
    if (r->op == N_CONST) return push_const(code, r->cbits, depth);
    if (!reg->inside(r)) {
      overflow = true;  // cannot happen in a prepared region
      return fail(be, CG_ERR_INTERNAL, "row value escaped its region");
    }
    if (r->op == N_BIN || r->op == N_UN) return emit_op(code, r, depth, true);
    // N_REDUCE: its input becomes (or already is) a reduction stage
    size_t sid = 0;
    for (; sid < stages.size(); ++sid)
      if (stages[sid].reduce == r) break;
    if (sid == stages.size()) {
      std::vector<Instr> sc;
      TRY(emit(sc, r->in[0], 0));  // may add earlier stages first
      if (stages.size() >= MAX_STAGES) {
        overflow = true;
        return fail(be, CG_ERR_INTERNAL, "row program: too many reduction stages");
      }
      sid = stages.size();
      stages.push_back(Stage{r, std::move(sc)});
    }
    return push(code, sid == 0 ? E_ROW0 : E_ROW1, depth, 0);
  }

  int compile_root(cg_tensor *root) { return emit(final_code, root, 0); }

  void flatten() {
    int k = 0;
    p.n_stages = (int)stages.size();
    for (size_t s = 0; s < stages.size(); ++s) {
      for (const Instr &i : stages[s].code) p.code[k++] = i;
      p.seg_end[s] = k;
      p.red_kind[s] = (int)stages[s].reduce->p0;
    }
    for (const Instr &i : final_code) p.code[k++] = i;
    p.seg_end[stages.size()] = k;
    p.n_instr = k;
    for (size_t i = 0; i < imms.size() && i < (size_t)MAX_INSTR; ++i) p.imm[i] = imms[i];
  }
};

// Realise every node of the region that is also read from outside it, until the region is
// closed.  Returns the prepared region.
int prepare_region(cg_backend *be, cg_tensor *root, bool rows, Region &reg) {
  for (int guard = 0; guard < 4096; ++guard) {
    reg.build(root, rows);
    cg_tensor *victim = reg.shared_node();
    if (!victim) return CG_OK;
    TRY(realize(be, victim));
  }
  return fail(be, CG_ERR_INTERNAL, "prepare_region did not converge");
}

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

// Launch the compiled program of `c` into (dst, dst_strides, dst_stype).
int launch_compiled(cg_backend *be, EwCompiler &c, cg_tensor *root, void *dst,
                    const int64_t *dst_strides, int dst_stype, const char *name) {
  c.flatten();
  const bool rowprog = c.p.n_stages > 0;
  std::vector<int64_t> ostr;
  double bytes_in = 0;
  TRY(finish_program(be, c, root->rank, root->shape, dst_strides, rowprog, ostr, &bytes_in));
  const int64_t n = root->size();
  if (n >= (int64_t)1 << 32) return fail(be, CG_ERR_INTERNAL, "tensor above 2^32 elements");
  OutDesc o;
  std::memset(&o, 0, sizeof(o));
  o.ptr = dst;
  o.stype = dst_stype;
  for (int d = 0; d < c.p.n_dims; ++d) o.stride[d] = ostr[d];
  o.vec = dst_stype != ST_BF16 && operand_vec_ok(dst, dst_stype, ostr);
  const uint32_t inner = c.p.dims[c.p.n_dims - 1];
  const bool vec4 = inner % 4 == 0;
  if (rowprog) {
    if (dst_stype == ST_BF16) return fail(be, CG_ERR_INTERNAL, "row program into bf16 storage");
    const int64_t cols = root->shape[root->rank - 1];
    KernelScope ks(be, "row_fused", bytes_in + (double)n * 4, 0);
    if (be->trace_shapes) {
      char buf[96];
      snprintf(buf, sizeof buf, "row_fused[%lldx%lld,i%d,in%d,st%d]", (long long)(n / cols), (long long)cols,
               (int)c.p.n_instr, (int)c.p.n_in, (int)c.p.n_stages);
      ks.rename(buf);
    }
    HIPCHK(be, launch_row(be->lc(), c.p, o, (uint32_t)(n / cols), (uint32_t)cols, vec4));
    return CG_OK;
  }
  KernelScope ks(be, name, bytes_in + (double)n * esize(dst_stype), 0);
  if (be->trace_shapes) {  // per-shape records: ew_fused[n8192,i7,in3]
    char buf[96];
    snprintf(buf, sizeof buf, "%s[n%lld,i%d,in%d]", name, (long long)n, (int)c.p.n_instr, (int)c.p.n_in);
    ks.rename(buf);
  }
  HIPCHK(be, launch_ew(be->lc(), c.p, o, (uint64_t)n, vec4));
  return CG_OK;
}

// Evaluate the elementwise tree rooted at `root` into (dst storage, dst strides, dst stype).
// root_is_value: just copy the (realised) value of root through its strides.
int run_ew(cg_backend *be, cg_tensor *root, bool root_is_value, void *dst, const int64_t *dst_strides,
           int dst_stype, const char *name) {
  if (root->size() == 0) return CG_OK;
  if (root_is_value) {
    Region reg;
    EwCompiler c(be, &reg);
    TRY(c.load(c.final_code, root, 0));
    return launch_compiled(be, c, root, dst, dst_strides, dst_stype, name);
  }
  // first with row values fused in, then without, then cutting the tree at its children
  for (int attempt = 0; attempt < 64; ++attempt) {
    const bool rows = attempt == 0 && root->rank > 0 && dst_stype != ST_BF16;
    Region reg;
    TRY(prepare_region(be, root, rows, reg));
    EwCompiler c(be, &reg);
    int st = c.compile_root(root);
    if (!st) return launch_compiled(be, c, root, dst, dst_strides, dst_stype, name);
    if (!c.overflow) return st;
    if (attempt >= 1) {
      // still too large: materialise the biggest deferred child and try again
      cg_tensor *victim = nullptr;
      for (cg_tensor *n : reg.order)
        if (n != root && (n->op == N_BIN || n->op == N_UN)) victim = n;  // last = closest to root
      if (!victim) return st;
      TRY(realize(be, victim));
    }
  }
  return fail(be, CG_ERR_INTERNAL, "elementwise program does not fit");
}

// A fresh contiguous tensor holding the value of `src` (f32/u32 storage unless keep_bf16).
// src (realised) -> dst (contiguous, 4-byte elements) when src's unit-stride axis is not its last
// one: the tiled transpose kernel instead of a strided elementwise pass.
int try_transpose_copy(cg_backend *be, const cg_tensor *src, cg_tensor *dst, bool *done) {
  const int r = src->rank;
  if (r < 2 || src->size() == 0 || (dst->stype == ST_BF16 && src->stype != ST_BF16)) return CG_OK;
  const int64_t C = src->shape[r - 1];
  if (C < 16 || src->strides[r - 1] == 1 || src->strides[r - 1] == 0) return CG_OK;
  int j = -1;
  for (int i = r - 2; i >= 0; --i)
    if (src->strides[i] == 1 && src->shape[i] >= 16) {
      j = i;
      break;
    }
  if (j < 0) return CG_OK;
  TransposeDesc d;
  std::memset(&d, 0, sizeof(d));
  d.x = data_ptr(src);
  d.out = data_ptr(dst);
  d.x_stype = src->stype;
  d.out_bf16 = dst->stype == ST_BF16;
  d.R = (uint32_t)src->shape[j];
  d.C = (uint32_t)C;
  d.x_sc = src->strides[r - 1];
  d.o_sj = dst->strides[j];
  uint64_t other = 1;
  for (int i = 0; i < r - 1; ++i) {
    if (i == j || src->shape[i] == 1) continue;
    d.odims[d.n_other] = (uint32_t)src->shape[i];
    d.x_so[d.n_other] = src->strides[i];
    d.o_so[d.n_other] = dst->strides[i];
    d.n_other++;
    other *= (uint64_t)src->shape[i];
  }
  if (other > 65535) return CG_OK;  // grid.z
  KernelScope ks(be, "transpose_copy", (double)src->size() * (esize(src->stype) + esize(dst->stype)), 0);
  HIPCHK(be, launch_transpose_copy(be->lc(), d));
  *done = true;
  return CG_OK;
}

int materialize(cg_backend *be, cg_tensor *src, cg_tensor **out, bool keep_bf16 = false) {
  TRY(realize(be, src));
  cg_tensor *t = new_node(be, src->dtype, src->rank, src->shape);
  int stype = (keep_bf16 && src->stype == ST_BF16) ? ST_BF16 : (src->dtype == CG_F32 ? ST_F32 : ST_U32);
  int st = alloc_result(be, t, stype);
  bool transposed = false;
  if (!st && !(be->flags & CG_FLAG_NO_PATTERNS)) st = try_transpose_copy(be, src, t, &transposed);
  if (!st && !transposed) st = run_ew(be, src, true, data_ptr(t), t->strides, stype, "ew_copy");
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

// ---- pattern kernels --------------------------------------------------------------------------
// The emitters of the reference produce fixed op sequences for softmax, RMSNorm, RoPE and the
// gated activations (cited in k_fused.hip).  When the deferred graph under a root is exactly one
// of those sequences, and nothing outside reads its interior, a hand-written kernel runs it.
// Everything else (and every near miss) goes to the generic program path below.
bool is_bin(const cg_tensor *n, uint8_t ew) { return n->op == N_BIN && n->ew == ew; }
bool is_un(const cg_tensor *n, uint8_t ew) { return n->op == N_UN && n->ew == ew; }
bool is_constf(const cg_tensor *n, uint32_t bits) { return n->op == N_CONST && n->cbits == bits; }
int refs(const cg_tensor *n) { return n->rc.load(); }
float bits_f(uint32_t b) {
  float f;
  std::memcpy(&f, &b, 4);
  return f;
}
enum : uint32_t { F_ONE = 0x3F800000u, F_HALF = 0x3F000000u, F_E = 0x402DF854u, F_TWO = 0x40000000u };

// t (realised, f32 storage) seen as rows of `n` unit-stride elements with one row stride
bool rows_view(const cg_tensor *t, int64_t *row_stride) {
  if (t->op != N_REAL || t->stype != ST_F32 || t->rank == 0) return false;
  const int r = t->rank;
  if (t->shape[r - 1] != 1 && t->strides[r - 1] != 1) return false;
  int64_t expect = -1;  // stride the next outer dim must have
  bool any = false;
  for (int i = r - 2; i >= 0; --i) {
    if (t->shape[i] == 1) continue;
    if (!any) {
      *row_stride = t->strides[i];
      expect = t->strides[i] * t->shape[i];
      any = true;
    } else {
      if (t->strides[i] != expect) return false;
      expect *= t->shape[i];
    }
  }
  if (!any) *row_stride = t->shape[r - 1];
  return true;
}

// Rows of a realised f32 tensor reached through up to three (extent, stride) pairs over the row
// index, outermost first (d0 is implied): [B, H, S, D] seen through a transpose of [B, S, H, D].
struct RowMap {
  uint32_t d1 = 1, d2 = 1;
  int64_t s0 = 0, s1 = 0, s2 = 0;
};
bool rows_map(const cg_tensor *t, RowMap *m) {
  if (t->op != N_REAL || t->stype != ST_F32 || t->rank == 0) return false;
  const int r = t->rank;
  if (t->shape[r - 1] != 1 && t->strides[r - 1] != 1) return false;
  int64_t ext[3], str[3];
  int g = 0;  // groups of dims that one stride walks, innermost first
  for (int i = r - 2; i >= 0; --i) {
    if (t->shape[i] == 1) continue;
    if (g && t->strides[i] == str[g - 1] * ext[g - 1]) {
      ext[g - 1] *= t->shape[i];
      continue;
    }
    if (g == 3) return false;
    ext[g] = t->shape[i];
    str[g] = t->strides[i];
    ++g;
  }
  for (int i = 0; i < g; ++i)
    if (str[i] % 4 || ext[i] > UINT32_MAX) return false;
  *m = RowMap();
  if (g == 0) return true;
  m->s0 = str[g - 1];
  if (g == 2) {
    m->d2 = (uint32_t)ext[0];
    m->s2 = str[0];
  } else if (g == 3) {
    m->d2 = (uint32_t)ext[0];
    m->s2 = str[0];
    m->d1 = (uint32_t)ext[1];
    m->s1 = str[1];
  }
  return true;
}

// Products still waiting that read n as their left operand, directly or through a reshape that only
// products hold.  all: every holder of n is one of them - n is needed in its bf16 form only.
int gemm_readers(cg_backend *be, const cg_tensor *n, bool *all) {
  int direct = 0, via = 0;
  const cg_tensor *seen[8];
  int readers[8], n_seen = 0;
  for (const cg_tensor *c : be->gemm_candidates) {
    if (c->op != N_MATMUL || !c->in[0]) continue;
    const cg_tensor *a = c->in[0];
    if (a == n) {
      ++direct;
    } else if (a->op == N_RESHAPE && a->in[0] == n) {
      int k = 0;
      while (k < n_seen && seen[k] != a) ++k;
      if (k == n_seen) {
        if (n_seen == 8) continue;
        seen[n_seen] = a;
        readers[n_seen++] = 0;
      }
      ++readers[k];
      ++via;
    }
  }
  int holders = direct;
  bool whole = true;
  for (int k = 0; k < n_seen; ++k) {
    ++holders;
    if (readers[k] != refs(seen[k])) whole = false;
  }
  *all = whole && holders > 0 && holders == refs(n);
  return direct + via;
}

// a realised f32 tensor usable as contiguous rows: itself or a contiguous copy
int as_rows(cg_backend *be, cg_tensor *t, cg_tensor **out, int64_t *row_stride) {
  TRY(realize(be, t));
  if (rows_view(t, row_stride) && (*row_stride % 4 == 0) &&
      ((uintptr_t)data_ptr(t) % 16 == 0)) {
    *out = retain(t);
    return CG_OK;
  }
  TRY(materialize(be, t, out));
  *row_stride = t->shape[t->rank - 1];
  return CG_OK;
}

void finish_fused(cg_tensor *n) {
  n->op = N_REAL;
  drop_inputs(n);
}

// In bf16 mode the results of the pattern kernels of a prefill (many rows) are the operands of
// the GEMMs that follow: the kernel writes the bf16 copy the GEMM would otherwise make with a
// pass of its own.  The copy becomes the twin of n's freshly allocated storage.
int twin_for_result(cg_backend *be, cg_tensor *n, uint16_t **out) {
  *out = nullptr;
  if (!(be->flags & CG_FLAG_BF16) || n->rank < 2 || n->stype != ST_F32 || n->offset != 0) return CG_OK;
  const int64_t cols = n->shape[n->rank - 1];
  if (cols % 8 || n->size() / std::max<int64_t>(cols, 1) < 32 || n->st->shadow || n->st->bytes % 32) return CG_OK;
  Storage *sh = nullptr;
  if (dev_alloc(be, n->st->bytes / 2, &sh) != CG_OK) return CG_OK;  // no room: the GEMM will narrow it later
  n->st->shadow = sh;
  *out = (uint16_t *)sh->ptr;
  return CG_OK;
}

// nn::softmax (stdlib/nn/mod.rs:162-171) with attention's `/ sqrt(d)` and `+ mask` in front:
// pure matching, nothing is realised.  src is the tensor the scale / mask / softmax apply to.
struct SoftmaxMatch {
  cg_tensor *src = nullptr, *mask = nullptr;
  cg_tensor *x = nullptr;  // what max / sub / exp are applied to (src after scale and mask)
  bool has_scale = false, has_mask_const = false;
  float scale = 1.f, mask_const = 0.f;
};

bool match_softmax(cg_tensor *root, SoftmaxMatch *m) {
  if (root->dtype != CG_F32 || root->rank == 0 || !is_bin(root, E_DIV_F)) return false;
  cg_tensor *ex = root->in[0], *bs = root->in[1];
  if (!is_bin(ex, E_POW_F) || refs(ex) != 2 || !is_constf(ex->in[0], F_E)) return false;
  if (bs->op != N_BROADCAST || refs(bs) != 1 || !is_row_broadcast(bs, root)) return false;
  cg_tensor *sm = bs->in[0];
  if (sm->op != N_REDUCE || sm->p0 != R_SUM_F || refs(sm) != 1 || sm->in[0] != ex) return false;
  cg_tensor *sb = ex->in[1];
  if (!is_bin(sb, E_SUB_F) || refs(sb) != 1) return false;
  cg_tensor *x = sb->in[0], *bm = sb->in[1];
  if (bm->op != N_BROADCAST || refs(bm) != 1 || !is_row_broadcast(bm, root)) return false;
  cg_tensor *mx = bm->in[0];
  if (mx->op != N_REDUCE || mx->p0 != R_MAX_F || refs(mx) != 1 || mx->in[0] != x) return false;
  const int64_t n = root->shape[root->rank - 1];
  if (n == 0 || n > 16384 || root->size() >= ((int64_t)1 << 31)) return false;
  m->src = x;
  m->x = x;
  if (x->op != N_REAL && refs(x) == 2) {
    cg_tensor *y = x;
    if (is_bin(x, E_ADD_F)) {  // attn + mask
      cg_tensor *mk = x->in[1];
      if (mk->op == N_CONST) {
        m->has_mask_const = true;
        m->mask_const = bits_f(mk->cbits);
      } else {
        m->mask = mk;
      }
      y = x->in[0];
      m->src = y;
    }
    if (is_bin(y, E_DIV_F) && y->in[1]->op == N_CONST && (y == x || refs(y) == 1)) {  // attn / sqrt(d)
      m->has_scale = true;
      m->scale = bits_f(y->in[1]->cbits);
      m->src = y->in[0];
    }
  }
  return true;
}

int try_softmax(cg_backend *be, cg_tensor *root, bool *done) {
  SoftmaxMatch sm_;
  if (!match_softmax(root, &sm_)) return CG_OK;
  const int64_t n = root->shape[root->rank - 1];
  SoftmaxDesc d;
  std::memset(&d, 0, sizeof(d));
  cg_tensor *src = sm_.src, *mask = sm_.mask;
  d.has_scale = sm_.has_scale;
  d.scale = sm_.scale;
  d.has_mask_const = sm_.has_mask_const;
  d.mask_const = sm_.mask_const;
  cg_tensor *xs = nullptr, *ms = nullptr;
  int64_t row_stride = 0;
  // rows stored as bf16 (an uploaded matrix) are read as they are by the 16-byte kernel
  TRY(realize(be, src));
  if (src->stype == ST_BF16 && !mask && is_contiguous(src) && n % 4 == 0 && n >= 256 && (uintptr_t)data_ptr(src) % 16 == 0) {
    xs = retain(src);
    row_stride = n;
    d.x_bf16 = 1;
  } else {
    TRY(as_rows(be, src, &xs, &row_stride));
  }
  int st = CG_OK;
  if (mask) {
    st = realize(be, mask);
    if (!st) {
      // rows of the mask: the leading dims must fold into (group, row)
      const int r = mask->rank;
      std::vector<int64_t> sz, sd;
      for (int i = 0; i + 1 < r; ++i) {
        if (mask->shape[i] == 1) continue;
        if (!sz.empty() && sd.back() == mask->strides[i] * mask->shape[i]) {
          sz.back() *= mask->shape[i];
          sd.back() = mask->strides[i];
        } else {
          sz.push_back(mask->shape[i]);
          sd.push_back(mask->strides[i]);
        }
      }
      if (mask->stype != ST_F32 || sz.size() > 2) {
        st = materialize(be, mask, &ms);
        if (!st) {
          d.mask = (const float *)data_ptr(ms);
          d.mask_rows = (uint32_t)(root->size() / n);
          d.mask_row_stride = n;
          d.mask_col_stride = 1;
        }
      } else {
        d.mask = (const float *)data_ptr(mask);
        d.mask_col_stride = mask->strides[r - 1];
        if (sz.size() == 2) {
          d.mask_rows = (uint32_t)sz[1];
          d.mask_row_stride = sd[1];
          d.mask_group_stride = sd[0];
        } else if (sz.size() == 1) {
          d.mask_rows = (uint32_t)sz[0];
          d.mask_row_stride = sd[0];
        } else {
          d.mask_rows = 1;
        }
      }
    }
  }
  if (!st) st = alloc_result(be, root, ST_F32);
  if (!st) {
    d.x = (const float *)data_ptr(xs);
    d.y = (float *)root->st->ptr;
    st = twin_for_result(be, root, &d.y16);
    d.x_row_stride = row_stride;
    d.rows = (uint32_t)(root->size() / n);
    d.n = (uint32_t)n;
    KernelScope ks(be, "softmax_fused", (double)root->size() * ((d.y16 ? 6 : 4) + (d.x_bf16 ? 2 : 4)), 0);
    hipError_t e = launch_softmax(be->lc(), d);
    if (e != hipSuccess) st = fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
  }
  node_release(xs);
  node_release(ms);
  if (st) return st;
  finish_fused(root);
  *done = true;
  return CG_OK;
}

// rmsnorm_raw / rmsnorm (catgrad-llm/src/helpers.rs:120-145; gemma3.rs:41-68)
struct RmsNormMatch {
  cg_tensor *x = nullptr, *gamma = nullptr;  // gamma: the broadcast node or null
  float eps = 0.f, n_as_float = 1.f, gamma_offset = 0.f;
};

// pure matching; nothing is realised
bool match_rmsnorm(cg_tensor *root, RmsNormMatch *m) {
  if (root->dtype != CG_F32 || root->rank == 0) return false;
  cg_tensor *dv = root, *gb = nullptr;
  float gamma_offset = 0.f;
  if (is_bin(root, E_MUL_F) && is_bin(root->in[0], E_DIV_F) && refs(root->in[0]) == 1) {
    dv = root->in[0];
    gb = root->in[1];
    if (is_bin(gb, E_ADD_F) && refs(gb) == 1 && is_constf(gb->in[0], F_ONE)) {  // (1 + gamma)
      gamma_offset = 1.f;
      gb = gb->in[1];
    }
  }
  if (!is_bin(dv, E_DIV_F)) return false;
  cg_tensor *x = dv->in[0], *br = dv->in[1];
  if (br->op != N_BROADCAST || refs(br) != 1 || !is_row_broadcast(br, root)) return false;
  cg_tensor *r = br->in[0];
  if (!is_bin(r, E_POW_F) || refs(r) != 1 || !is_constf(r->in[1], F_HALF)) return false;
  cg_tensor *a = r->in[0];
  if (!is_bin(a, E_ADD_F) || refs(a) != 1 || a->in[1]->op != N_CONST) return false;
  cg_tensor *mn = a->in[0];
  if (!is_bin(mn, E_DIV_F) || refs(mn) != 1 || mn->in[1]->op != N_CONST) return false;
  cg_tensor *sm = mn->in[0];
  if (sm->op != N_REDUCE || sm->p0 != R_SUM_F || refs(sm) != 1) return false;
  cg_tensor *sq = sm->in[0];
  if (!is_bin(sq, E_MUL_F) || refs(sq) != 1 || sq->in[0] != x || sq->in[1] != x) return false;
  const int64_t n = root->shape[root->rank - 1];
  if (n == 0 || n % 4 || n > 16384) return false;
  m->x = x;
  m->gamma = gb;
  m->eps = bits_f(a->in[1]->cbits);
  m->n_as_float = bits_f(mn->in[1]->cbits);
  m->gamma_offset = gamma_offset;
  return true;
}

// gamma as a row vector broadcast over the rows (realises it); false: some other layout
int gamma_row_vector(cg_backend *be, cg_tensor *gb, bool *ok) {
  TRY(realize(be, gb));
  bool vec = gb->stype == ST_F32 && (gb->shape[gb->rank - 1] == 1 || gb->strides[gb->rank - 1] == 1) &&
             ((uintptr_t)data_ptr(gb) % 16 == 0);
  for (int i = 0; i + 1 < gb->rank; ++i)
    if (gb->shape[i] != 1 && gb->strides[i] != 0) vec = false;
  *ok = vec;
  return CG_OK;
}

// gemma3.rs:198-240, many rows: `mid = res + rmsnorm(y)` followed by `rmsnorm(mid)` - the post-attention
// norm and the pre-feedforward one, the post-feedforward norm and the next layer's input norm.  One
// kernel writes mid (the residual stream, which later adds read) and norms it again from registers.
int try_rmsnorm_pair(cg_backend *be, cg_tensor *root, const RmsNormMatch &outer, bool *done) {
  cg_tensor *mid = outer.x;
  const int64_t n = root->shape[root->rank - 1];
  if (!mid || mid->op == N_REAL || mid->dtype != CG_F32 || !is_bin(mid, E_ADD_F) || !outer.gamma || mid->size() != root->size() ||
      root->size() / n < 32 || root->size() / n > UINT32_MAX)
    return CG_OK;
  RmsNormMatch inner;
  int side = -1;
  for (int i = 0; i < 2 && side < 0; ++i)
    if (mid->in[i]->op != N_REAL && refs(mid->in[i]) == 1 && match_rmsnorm(mid->in[i], &inner)) side = i;
  if (side < 0 || !inner.gamma || inner.n_as_float != outer.n_as_float) return CG_OK;
  cg_tensor *residual = mid->in[1 - side];
  if (residual->op == N_CONST || ((residual->op == N_BIN || residual->op == N_UN) && refs(residual) == 1)) return CG_OK;
  bool v1 = false, v2 = false;
  TRY(gamma_row_vector(be, inner.gamma, &v1));
  TRY(gamma_row_vector(be, outer.gamma, &v2));
  if (!v1 || !v2) return CG_OK;
  cg_tensor *rs = nullptr, *xs = nullptr;
  struct Rel {
    cg_tensor *&t;
    ~Rel() { node_release(t); }
  } rel_rs{rs}, rel_xs{xs};
  // the normed value first: what it is computed from (a layer's feed-forward) reads the norm of the
  // residual stream, and that norm pairs up with the one that produces the stream only while the
  // stream is still unwritten
  int64_t row_stride = 0;
  TRY(as_rows(be, inner.x, &xs, &row_stride));
  if (root->op == N_REAL) {  // (realised on the way: nothing left to do)
    *done = true;
    return CG_OK;
  }
  if (mid->op == N_REAL) return CG_OK;
  TRY(contiguous(be, residual, &rs));
  if ((uintptr_t)data_ptr(rs) % 16) return CG_OK;
  bool to_gemms = false, only_gemms = false;
  if ((be->flags & CG_FLAG_BF16) && root->rank >= 2 && n % 8 == 0) to_gemms = gemm_readers(be, root, &only_gemms) > 0;
  TRY(alloc_result(be, mid, ST_F32));
  TRY(alloc_result(be, root, only_gemms ? ST_BF16 : ST_F32));
  RmsNormDesc d;
  std::memset(&d, 0, sizeof(d));
  d.x = (const float *)data_ptr(xs);
  d.x_row_stride = row_stride;
  d.gamma = (const float *)data_ptr(inner.gamma);
  d.eps = inner.eps;
  d.gamma_offset = inner.gamma_offset;
  d.n_as_float = inner.n_as_float;
  d.residual = (const float *)data_ptr(rs);
  d.y_mid = (float *)mid->st->ptr;
  d.gamma2 = (const float *)data_ptr(outer.gamma);
  d.eps2 = outer.eps;
  d.gamma2_offset = outer.gamma_offset;
  d.rows = (uint32_t)(root->size() / n);
  d.n = (uint32_t)n;
  if (only_gemms) {
    d.y16 = (uint16_t *)root->st->ptr;
  } else {
    d.y = (float *)root->st->ptr;
    if (to_gemms) TRY(twin_for_result(be, root, &d.y16));
  }
  {
    KernelScope ks(be, "rmsnorm_fused", (double)root->size() * (12 + (d.y ? 4 : 0) + (d.y16 ? 2 : 0)) + n * 8, 0);
    if (be->trace_shapes) {  // rmsnorm_fused[16384x1152,+res,+norm,bf16]
      char buf[96];
      snprintf(buf, sizeof buf, "rmsnorm_fused[%ux%u,+res,+norm,%s]", d.rows, d.n, !d.y ? "bf16" : d.y16 ? "f32+bf16" : "f32");
      ks.rename(buf);
    }
    hipError_t e = launch_rmsnorm(be->lc(), d);
    if (e != hipSuccess) return fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
  }
  finish_fused(mid);
  finish_fused(root);
  *done = true;
  return CG_OK;
}

// also `res + rmsnorm(..)` / `rmsnorm(..) + res` (gemma3.rs:198-240 adds the residual right after the
// post-attention and post-feedforward norms): the addend rides along in the same kernel
int try_rmsnorm(cg_backend *be, cg_tensor *root, bool *done) {
  RmsNormMatch rm;
  cg_tensor *residual = nullptr;
  if (!match_rmsnorm(root, &rm)) {
    if (root->dtype != CG_F32 || !is_bin(root, E_ADD_F)) return CG_OK;
    int side = -1;
    for (int i = 0; i < 2 && side < 0; ++i)
      if (root->in[i]->op != N_REAL && refs(root->in[i]) == 1 && match_rmsnorm(root->in[i], &rm)) side = i;
    if (side < 0) return CG_OK;
    residual = root->in[1 - side];
    if (residual->op == N_CONST || ((residual->op == N_BIN || residual->op == N_UN) && refs(residual) == 1))
      return CG_OK;  // the addend is itself an unrealised expression: leave it to the generic fusion
  }
  if (!residual) {
    TRY(try_rmsnorm_pair(be, root, rm, done));
    if (*done) return CG_OK;
  }
  cg_tensor *x = rm.x, *gb = rm.gamma;
  const int64_t n = root->shape[root->rank - 1];
  cg_tensor *rs = nullptr;
  if (residual) {
    TRY(contiguous(be, residual, &rs));
    if ((uintptr_t)data_ptr(rs) % 16) {
      node_release(rs);
      return CG_OK;
    }
  }
  struct Rel {
    cg_tensor *t;
    ~Rel() { node_release(t); }
  } rel{rs};
  RmsNormDesc d;
  std::memset(&d, 0, sizeof(d));
  d.eps = rm.eps;
  d.n_as_float = rm.n_as_float;
  d.gamma_offset = rm.gamma_offset;
  cg_tensor *gs = nullptr;
  if (gb) {
    bool vec = false;
    TRY(gamma_row_vector(be, gb, &vec));
    if (!vec) return CG_OK;  // gamma is not a broadcast row vector: generic path
    gs = gb;
  }
  cg_tensor *xs = nullptr;
  int64_t row_stride = 0;
  RowMap rmap;
  // gemma3.rs:99-117 norms q and k after the head transpose, folded to [b * heads * s, head_dim]: a
  // reshape that strides cannot express.  The rows are read where they lie instead of from a copy.
  cg_tensor *view = x;
  while (view->op == N_RESHAPE && view->in[0] && view->in[0]->rank >= 1 && view->in[0]->shape[view->in[0]->rank - 1] == n)
    view = view->in[0];
  TRY(realize(be, view));
  if (rows_map(view, &rmap) && (rmap.d1 > 1 || rmap.d2 > 1) && (uintptr_t)data_ptr(view) % 16 == 0 &&
      root->size() / n <= UINT32_MAX) {
    xs = retain(view);
    row_stride = rmap.s0;
  } else {
    rmap = RowMap();
    TRY(as_rows(be, x, &xs, &row_stride));
  }
  // In bf16 mode with many rows: the GEMMs that wait for this value read it as bf16.  If nothing
  // else holds it, it is written in that form only; if something else does, in both.
  bool to_gemms = false, only_gemms = false;
  if (!residual && (be->flags & CG_FLAG_BF16) && root->rank >= 2 && n % 8 == 0 && root->size() / n >= 32)
    to_gemms = gemm_readers(be, root, &only_gemms) > 0;
  int st = alloc_result(be, root, only_gemms ? ST_BF16 : ST_F32);
  if (!st) {
    d.x = (const float *)data_ptr(xs);
    d.gamma = gs ? (const float *)data_ptr(gs) : nullptr;
    d.x_row_stride = row_stride;
    d.x_d1 = rmap.d1;
    d.x_d2 = rmap.d2;
    d.x_s1 = rmap.s1;
    d.x_s2 = rmap.s2;
    d.rows = (uint32_t)(root->size() / n);
    d.n = (uint32_t)n;
    d.residual = rs ? (const float *)data_ptr(rs) : nullptr;
    if (only_gemms) {
      d.y16 = (uint16_t *)root->st->ptr;
    } else {
      d.y = (float *)root->st->ptr;
      if (to_gemms) st = twin_for_result(be, root, &d.y16);
    }
    KernelScope ks(be, "rmsnorm_fused", (double)root->size() * ((rs ? 8 : 4) + (d.y ? 4 : 0) + (d.y16 ? 2 : 0)) + n * 4, 0);
    if (be->trace_shapes) {  // per-shape records: rmsnorm_fused[16384x1152,+res,f32+bf16]
      char buf[96];
      snprintf(buf, sizeof buf, "rmsnorm_fused[%ux%u%s%s,%s]", d.rows, d.n, rs ? ",+res" : "", rmap.d1 > 1 || rmap.d2 > 1 ? ",strided" : "",
               !d.y ? "bf16" : d.y16 ? "f32+bf16" : "f32");
      ks.rename(buf);
    }
    hipError_t e = launch_rmsnorm(be->lc(), d);
    if (e != hipSuccess) st = fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
  }
  node_release(xs);
  if (st) return st;
  finish_fused(root);
  *done = true;
  return CG_OK;
}

// apply_rope_embedding (catgrad-llm/src/helpers.rs:195-221): cos * x + sin * rotate_half(x)
struct RopeMatch {
  cg_tensor *cb = nullptr, *sb = nullptr, *x = nullptr;  // cos / sin broadcasts, the rotated tensor
};

// pure matching; nothing is realised
bool match_rope(cg_tensor *root, RopeMatch *m) {
  if (root->dtype != CG_F32 || root->rank != 4 || !is_bin(root, E_ADD_F)) return false;
  cg_tensor *m1 = root->in[0], *m2 = root->in[1];
  if (!is_bin(m1, E_MUL_F) || !is_bin(m2, E_MUL_F) || refs(m1) != 1 || refs(m2) != 1) return false;
  cg_tensor *cb = m1->in[0], *x = m1->in[1], *sb = m2->in[0], *rot = m2->in[1];
  if (rot->op != N_CONCAT || rot->p0 != 3 || refs(rot) != 1) return false;
  cg_tensor *ng = rot->in[0], *lo = rot->in[1];
  if (!is_un(ng, E_NEG_F) || refs(ng) != 1) return false;
  cg_tensor *hi = ng->in[0];
  const int64_t dim = root->shape[3], half = dim / 2;
  if (dim % 8 || hi->shape[3] != half || lo->shape[3] != half) return false;
  // the two halves are slices of x along the last axis: still deferred, or (x already in
  // memory) views created on the spot
  auto half_of = [&](const cg_tensor *t, int64_t start) {
    if (t->op == N_SLICE) return t->in[0] == x && t->p0 == 3 && t->p1 == start && refs(t) == 1;
    if (t->op != N_REAL || x->op != N_REAL || t->st != x->st) return false;
    for (int i = 0; i < 4; ++i)
      if (t->strides[i] != x->strides[i] && t->shape[i] != 1) return false;
    return t->offset == x->offset + start * x->strides[3];
  };
  if (!half_of(hi, half) || !half_of(lo, 0)) return false;
  if (root->size() >= ((int64_t)1 << 31)) return false;
  m->cb = cb;
  m->sb = sb;
  m->x = x;
  return true;
}

// realises the operands of a matched rope; *ok = the kernel's layout requirements hold
int rope_operands(cg_backend *be, const RopeMatch &m, bool *ok) {
  TRY(realize(be, m.cb));
  TRY(realize(be, m.sb));
  TRY(realize(be, m.x));
  auto table_ok = [&](const cg_tensor *t) {
    return t->stype == ST_F32 && t->strides[0] * (t->shape[0] != 1) == 0 &&
           t->strides[1] * (t->shape[1] != 1) == 0 && t->strides[3] == 1 && t->strides[2] % 4 == 0 &&
           (uintptr_t)data_ptr(t) % 16 == 0;
  };
  *ok = table_ok(m.cb) && table_ok(m.sb) && m.cb->strides[2] == m.sb->strides[2];
  return CG_OK;
}

// Launches the rope kernel for `root` (matched as m) into `out` with the given element strides.
// *done = false: layout requirements not met, nothing was launched.
int rope_into(cg_backend *be, cg_tensor *root, const RopeMatch &m, float *out, const int64_t *o_strides,
              const char *name, bool *done, uint16_t *out16 = nullptr) {
  bool tables = false;
  TRY(rope_operands(be, m, &tables));
  if (!tables) return CG_OK;
  cg_tensor *x = m.x, *cb = m.cb, *sb = m.sb;
  cg_tensor *xs = retain(x);
  bool ok = x->stype == ST_F32 && x->strides[3] == 1 && (uintptr_t)data_ptr(x) % 16 == 0;
  for (int i = 0; i < 3; ++i)
    if (x->strides[i] % 4) ok = false;
  if (!ok) {
    node_release(xs);
    xs = nullptr;
    TRY(materialize(be, x, &xs));
  }
  const int64_t dim = root->shape[3];
  RopeDesc d;
  std::memset(&d, 0, sizeof(d));
  d.x = (const float *)data_ptr(xs);
  d.cos = (const float *)data_ptr(cb);
  d.sin = (const float *)data_ptr(sb);
  d.out = out;
  d.out16 = out16;
  d.x_sb = xs->strides[0];
  d.x_sh = xs->strides[1];
  d.x_ss = xs->strides[2];
  d.o_sb = o_strides[0];
  d.o_sh = o_strides[1];
  d.o_ss = o_strides[2];
  d.cs_ss = root->shape[2] == 1 ? 0 : cb->strides[2];
  d.b = (uint32_t)root->shape[0];
  d.h = (uint32_t)root->shape[1];
  d.s = (uint32_t)root->shape[2];
  d.dim = (uint32_t)dim;
  d.half = (uint32_t)(dim / 2);
  int st = CG_OK;
  {
    KernelScope ks(be, name, (double)root->size() * 8, 0);
    hipError_t e = launch_rope(be->lc(), d);
    if (e != hipSuccess) st = fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
  }
  node_release(xs);
  if (st) return st;
  *done = true;
  return CG_OK;
}

// apply_rope_embedding (catgrad-llm/src/helpers.rs:195-221): cos * x + sin * rotate_half(x)
int try_rope(cg_backend *be, cg_tensor *root, bool *done) {
  RopeMatch m;
  if (!match_rope(root, &m)) return CG_OK;
  bool tables = false;
  TRY(rope_operands(be, m, &tables));
  if (!tables) return CG_OK;
  TRY(alloc_result(be, root, ST_F32));
  bool launched = false;
  uint16_t *y16 = nullptr;
  TRY(twin_for_result(be, root, &y16));
  int st = rope_into(be, root, m, (float *)root->st->ptr, root->strides, "rope_fused", &launched, y16);
  if (st || !launched) {
    storage_release(root->st);
    root->st = nullptr;
    return st;
  }
  finish_fused(root);
  *done = true;
  return CG_OK;
}

// nn::sigmoid as emitted: one / (one + exp(-g)) (stdlib/nn/mod.rs:130-136)
bool is_sigmoid_of(const cg_tensor *s, const cg_tensor **arg) {
  if (!is_bin(s, E_DIV_F) || refs(s) != 1 || !is_constf(s->in[0], F_ONE)) return false;
  const cg_tensor *ad = s->in[1];
  if (!is_bin(ad, E_ADD_F) || refs(ad) != 1 || !is_constf(ad->in[0], F_ONE)) return false;
  const cg_tensor *pw = ad->in[1];
  if (!is_bin(pw, E_POW_F) || refs(pw) != 1 || !is_constf(pw->in[0], F_E)) return false;
  const cg_tensor *ng = pw->in[1];
  if (!is_un(ng, E_NEG_F) || refs(ng) != 1) return false;
  *arg = ng->in[0];
  return true;
}

// nn::gelu as emitted (stdlib/nn/mod.rs:138-160):
//   half * x * (one + (two * sigmoid(two * (c * (x + k * pow(x, three)))) - one))
bool is_gelu_of(const cg_tensor *g, const cg_tensor **arg) {
  if (!is_bin(g, E_MUL_F) || refs(g) != 1) return false;
  const cg_tensor *hx = g->in[0], *op = g->in[1];
  if (!is_bin(hx, E_MUL_F) || refs(hx) != 1 || !is_constf(hx->in[0], F_HALF)) return false;
  const cg_tensor *x = hx->in[1];
  if (!is_bin(op, E_ADD_F) || refs(op) != 1 || !is_constf(op->in[0], F_ONE)) return false;
  const cg_tensor *th = op->in[1];
  if (!is_bin(th, E_SUB_F) || refs(th) != 1 || !is_constf(th->in[1], F_ONE)) return false;
  const cg_tensor *ts = th->in[0];
  if (!is_bin(ts, E_MUL_F) || refs(ts) != 1 || !is_constf(ts->in[0], F_TWO)) return false;
  const cg_tensor *sa = nullptr;
  if (!is_sigmoid_of(ts->in[1], &sa)) return false;
  if (!is_bin(sa, E_MUL_F) || refs(sa) != 1 || !is_constf(sa->in[0], F_TWO)) return false;
  const cg_tensor *ct = sa->in[1];
  if (!is_bin(ct, E_MUL_F) || refs(ct) != 1 || (!is_constf(ct->in[0], 0x3F4C4229u) && !is_constf(ct->in[0], 0x3F4C422Au))) return false;  // sqrt(2/pi)
  const cg_tensor *in = ct->in[1];
  if (!is_bin(in, E_ADD_F) || refs(in) != 1 || in->in[0] != x) return false;
  const cg_tensor *kx = in->in[1];
  if (!is_bin(kx, E_MUL_F) || refs(kx) != 1 || !is_constf(kx->in[0], 0x3D372713u)) return false;  // 0.044715
  const cg_tensor *pw = kx->in[1];
  if (!is_bin(pw, E_POW_F) || refs(pw) != 1 || pw->in[0] != x || !is_constf(pw->in[1], 0x40400000u)) return false;
  *arg = x;
  return true;
}

// silu(gate) * up (models/llama.rs:26) and gelu(gate) * up (models/gemma3.rs:28)
bool match_glu(cg_tensor *root, cg_tensor **gate, cg_tensor **up, int *gelu) {
  if (root->dtype != CG_F32 || !is_bin(root, E_MUL_F) || root->size() % 4) return false;
  cg_tensor *act = root->in[0];
  const cg_tensor *g = nullptr;
  if (is_bin(act, E_MUL_F) && refs(act) == 1 && is_sigmoid_of(act->in[1], &g) && g == act->in[0]) {
    *gelu = 0;
  } else if (is_gelu_of(act, &g)) {
    *gelu = 1;
  } else {
    return false;
  }
  *gate = const_cast<cg_tensor *>(g);
  *up = root->in[1];
  return true;
}

// What a GEMM may apply to its product before storing it: act(gate) * product (the gated activation
// of an MLP in up_proj's epilogue).  `applied` tells the caller whether the kernel that ran could.
struct MatmulEpilogue {
  const float *gate = nullptr;  // laid out like the product
  // or: the right operand of the gate product itself (realised, laid out like this product's); the
  // kernel then computes both products and stores act(A . dual_w) * (A . B)
  cg_tensor *dual_w = nullptr;
  int gelu = 0;
  bool applied = false;
};
int realize_matmul(cg_backend *be, cg_tensor *n, cg_tensor *addend, bool *added, MatmulEpilogue *ep);

// the same tensor, or two reshapes of one tensor to one shape (each linear folds the batch into its rows itself)
static bool same_rows(const cg_tensor *a, const cg_tensor *b) {
  if (a == b) return true;
  return a->op == N_RESHAPE && b->op == N_RESHAPE && a->in[0] == b->in[0] && a->rank == b->rank &&
         std::equal(a->shape, a->shape + a->rank, b->shape);
}

int try_gate_up_glu(cg_backend *be, cg_tensor *glu, cg_tensor *g, cg_tensor *u, int gelu, bool *done);
cg_tensor *bias_vector_of(cg_tensor *other, const cg_tensor *like);
bool bias_vector_ready(const cg_tensor *v);

int try_glu(cg_backend *be, cg_tensor *root, bool *done) {
  cg_tensor *gate = nullptr, *up = nullptr;
  int gelu = 0;
  if (!match_glu(root, &gate, &up, &gelu)) return CG_OK;
  cg_tensor *gc = nullptr, *uc = nullptr;
  if (!(be->flags & CG_FLAG_NO_PATTERNS)) {  // a few rows: both products and the activation in one launch
    TRY(try_gate_up_glu(be, root, gate, up, gelu, done));
    if (*done) return CG_OK;
  }
  // bf16 mode, many rows, gate and up both still deferred products of the same rows: one GEMM over the
  // two weight matrices stacked tile by tile, the activation applied where both products sit in
  // registers; the gate product never exists as a tensor.
  if ((be->flags & CG_FLAG_BF16) && root->dtype == CG_F32) {
    cg_tensor *gm = gate, *um = up;
    if (gm->op == N_RESHAPE && refs(gm->in[0]) == 1) gm = gm->in[0];
    if (um->op == N_RESHAPE && refs(um) == 1) um = um->in[0];
    const int r = um->rank;
    if (gm->op == N_MATMUL && um->op == N_MATMUL && gm != um && refs(gate) == (gelu ? 3 : 2) && refs(up) == 1 && refs(um) == 1 &&
        same_rows(gm->in[0], um->in[0]) && !gm->gemv_candidate && !um->gemv_candidate && gm->rank == r && r >= 2 &&
        std::equal(gm->shape, gm->shape + r, um->shape) && um->size() == um->shape[r - 2] * um->shape[r - 1] &&
        um->shape[r - 2] >= 64 && um->shape[r - 1] >= 64 && um->shape[r - 1] % 8 == 0 && um->in[0]->shape[r - 1] % 64 == 0) {
      cg_tensor *wg = gm->in[1], *wu = um->in[1];
      TRY(realize(be, wg));
      TRY(realize(be, wu));
      if (wg->stype == ST_BF16 && wu->stype == ST_BF16 && wg->rank == wu->rank && std::equal(wg->shape, wg->shape + wg->rank, wu->shape) &&
          std::equal(wg->strides, wg->strides + wg->rank, wu->strides) && wu->strides[wu->rank - 2] == 1 &&
          (uintptr_t)data_ptr(wg) % 16 == 0 && (uintptr_t)data_ptr(wu) % 16 == 0) {
        MatmulEpilogue ep;
        ep.dual_w = wg;
        ep.gelu = gelu;
        TRY(realize_matmul(be, um, nullptr, nullptr, &ep));
        if (ep.applied) {  // um holds the gated activations and nobody else can see it: root takes its storage
          root->st = um->st;
          root->st->rc.fetch_add(1);
          root->stype = um->stype;
          root->offset = um->offset;
          contiguous_strides(root->rank, root->shape, root->strides);
          finish_fused(root);  // releases the activation chain and with it the gate product
          *done = true;
          return CG_OK;
        }
      }
    }
  }
  TRY(contiguous(be, gate, &gc));
  // bf16 mode, many rows: up_proj's GEMM applies act(gate) to its product before storing it.  A
  // reshape between the product and the multiply (batch folded into the rows for the linear and
  // unfolded again) changes nothing in memory.
  cg_tensor *mm = up;
  if (mm->op == N_RESHAPE && refs(mm) == 1) mm = mm->in[0];
  if ((be->flags & CG_FLAG_BF16) && mm->op == N_MATMUL && refs(mm) == 1 && refs(up) == 1 && mm->dtype == CG_F32 &&
      !mm->gemv_candidate && gc->stype == ST_F32 && is_contiguous(gc)) {
    MatmulEpilogue ep;
    ep.gate = (const float *)data_ptr(gc);
    ep.gelu = gelu;
    int mst = realize_matmul(be, mm, nullptr, nullptr, &ep);
    if (mst) {
      node_release(gc);
      return mst;
    }
    if (ep.applied) {  // mm holds the gated activations and nobody else can see it: root takes its storage
      root->st = mm->st;
      root->st->rc.fetch_add(1);
      root->stype = mm->stype;
      root->offset = mm->offset;
      contiguous_strides(root->rank, root->shape, root->strides);  // mm is dense: same order, root's shape
      node_release(gc);
      finish_fused(root);
      *done = true;
      return CG_OK;
    }
  }
  int st = contiguous(be, up, &uc);
  if (!st) st = alloc_result(be, root, ST_F32);
  if (!st) {
    KernelScope ks(be, gelu ? "geglu_fused" : "swiglu_fused", (double)root->size() * 12, 0);
    uint16_t *y16 = nullptr;
    (void)twin_for_result(be, root, &y16);
    hipError_t e = launch_glu(be->lc(), gelu, (const float *)data_ptr(gc), (const float *)data_ptr(uc),
                              (float *)root->st->ptr, (uint64_t)root->size(), y16);
    if (e != hipSuccess) st = fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
  }
  node_release(gc);
  node_release(uc);
  if (st) return st;
  finish_fused(root);
  *done = true;
  return CG_OK;
}

int realize_matmul(cg_backend *be, cg_tensor *n, cg_tensor *addend, bool *added, MatmulEpilogue *ep);

// residual + linear(x) on a decode step (models/llama.rs:166-186: `res + attention`, `res + mlp`):
// the add rides in the epilogue of the one-row matmul kernel instead of a launch of its own.
int try_gemv_add(cg_backend *be, cg_tensor *root, bool *done) {
  if (root->dtype != CG_F32 || !is_bin(root, E_ADD_F)) return CG_OK;
  for (int side = 0; side < 2; ++side) {
    cg_tensor *mm = root->in[side], *other = root->in[1 - side];
    // a batch-folding linear hands its product back through a reshape: the same rows in the same order
    const bool folded = mm->op == N_RESHAPE && refs(mm) == 1 && mm->in[0]->op == N_MATMUL && mm->in[0]->size() == mm->size();
    if (folded) mm = mm->in[0];
    // one-row products add in their epilogue; so does the pass that sums the k-slices of a split GEMM
    if (mm->op != N_MATMUL || refs(mm) != 1 || mm->dtype != CG_F32) continue;
    if (!mm->gemv_candidate && mm->rank > 3) continue;  // attention products have fusions of their own
    if (other->op == N_CONST || ((other->op == N_BIN || other->op == N_UN) && refs(other) == 1)) continue;
    bool added = false;
    // (a single row in memory goes the residual's way below: every one-row kernel can add that)
    const bool plain_row = other->op == N_REAL && other->stype == ST_F32 && is_contiguous(other);
    if (cg_tensor *bv = (!folded && !plain_row && mm->gemv_candidate) ? bias_vector_of(other, root) : nullptr) {
      // linear(x) + bias on a few rows: the grouped product launch adds the vector to every row
      TRY(realize(be, bv));
      if (!bias_vector_ready(bv)) return CG_OK;
      be->addend_is_row = true;
      int st = realize_matmul(be, mm, bv, &added, nullptr);
      be->addend_is_row = false;
      if (st) return st;
    } else {
      TRY(realize(be, other));
      if (other->stype != ST_F32 || !is_contiguous(other)) return CG_OK;
      TRY(realize_matmul(be, mm, other, &added, nullptr));
    }
    if (!added) return CG_OK;  // the product is realised; the generic add takes it from here
    // mm now holds the sum and nobody else can see it: root takes over its storage
    root->st = mm->st;
    root->st->rc.fetch_add(1);
    root->stype = mm->stype;
    root->offset = mm->offset;
    if (folded) contiguous_strides(root->rank, root->shape, root->strides);  // products are dense
    else std::copy(mm->strides, mm->strides + mm->rank, root->strides);
    finish_fused(root);
    *done = true;
    return CG_OK;
  }
  return CG_OK;
}

int try_binary(cg_backend *be, cg_tensor *root, bool *done) {
  if (root->dtype != CG_F32 || root->op != N_BIN || root->size() % 4 || root->rank == 0) return CG_OK;
  int op;
  switch (root->ew) {
    case E_ADD_F: op = 0; break;
    case E_SUB_F: op = 1; break;
    case E_MUL_F: op = 2; break;
    case E_DIV_F: op = 3; break;
    default: return CG_OK;
  }
  cg_tensor *a = root->in[0], *b = root->in[1];
  auto leaf = [](const cg_tensor *t) {
    return t->op != N_CONST && !((t->op == N_BIN || t->op == N_UN) && t->rc.load() == 1);
  };
  if (!leaf(a) || !leaf(b)) return CG_OK;
  TRY(realize(be, a));
  TRY(realize(be, b));
  const bool a16 = a->stype == ST_BF16;  // an uploaded matrix used as it is stored
  if ((a->stype != ST_F32 && !a16) || b->stype != ST_F32 || !is_contiguous(a) || (uintptr_t)data_ptr(a) % 16 ||
      (uintptr_t)data_ptr(b) % 16)
    return CG_OK;
  uint32_t period = 0;
  if (!is_contiguous(b)) {
    // b = a trailing block repeated over the leading dims (a bias / row-vector broadcast)
    int k = b->rank;
    int64_t inner = 1;
    while (k > 0 && (b->shape[k - 1] == 1 || b->strides[k - 1] == inner)) {
      inner *= b->shape[k - 1];
      --k;
    }
    for (int i = 0; i < k; ++i)
      if (b->shape[i] != 1 && b->strides[i] != 0) return CG_OK;
    if (inner % 4 || inner >= ((int64_t)1 << 31)) return CG_OK;
    period = (uint32_t)inner;
  }
  TRY(alloc_result(be, root, ST_F32));
  {
    KernelScope ks(be, "binary_f32", (double)root->size() * ((period ? 4 : 8) + (a16 ? 2 : 4)) + period * 4.0, 0);
    HIPCHK(be, launch_binary_f32(be->lc(), op, (const float *)data_ptr(a), (const float *)data_ptr(b),
                                 (float *)root->st->ptr, (uint64_t)root->size(), period, a16));
  }
  finish_fused(root);
  *done = true;
  return CG_OK;
}

int try_patterns(cg_backend *be, cg_tensor *root, bool *done) {
  if (be->flags & CG_FLAG_NO_PATTERNS) return CG_OK;
  TRY(try_softmax(be, root, done));
  if (*done) return CG_OK;
  TRY(try_rmsnorm(be, root, done));
  if (*done) return CG_OK;
  TRY(try_rope(be, root, done));
  if (*done) return CG_OK;
  TRY(try_glu(be, root, done));
  if (*done) return CG_OK;
  TRY(try_gemv_add(be, root, done));
  if (*done) return CG_OK;
  return try_binary(be, root, done);
}

int realize_ew(cg_backend *be, cg_tensor *n) {
  bool done = false;
  TRY(try_patterns(be, n, &done));
  if (done) return CG_OK;
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

// t (realised) as rows of unit-stride elements with one stride between rows
bool rows_layout(const cg_tensor *t, int64_t *row_stride) {
  const int r = t->rank;
  if (r == 0 || (t->shape[r - 1] != 1 && t->strides[r - 1] != 1)) return false;
  int64_t rs = -1, expect = 0;
  for (int i = r - 2; i >= 0; --i) {
    if (t->shape[i] == 1) continue;
    if (rs < 0) {
      rs = t->strides[i];
      expect = rs * t->shape[i];
    } else {
      if (t->strides[i] != expect) return false;
      expect *= t->shape[i];
    }
  }
  *row_stride = rs < 0 ? t->shape[r - 1] : rs;
  return true;
}

int realize_reduce(cg_backend *be, cg_tensor *n) {
  cg_tensor *x = n->in[0];
  const int kind = (int)n->p0;
  // a tensor that is (or has to be) in memory anyway, with enough rows to fill the device: stream it
  if (!(be->flags & CG_FLAG_NO_PATTERNS) && !((x->op == N_BIN || x->op == N_UN) && x->rc.load() == 1) &&
      x->rank >= 1 && x->size() > 0 && x->size() < ((int64_t)1 << 32)) {
    const int64_t cols = x->shape[x->rank - 1], rows = x->size() / cols;
    if (cols % 4 == 0 && cols >= 64 && rows >= be->n_cus) {
      TRY(realize(be, x));
      int64_t rs = 0;
      const int es = esize(x->stype);
      if (rows_layout(x, &rs) && (uintptr_t)data_ptr(x) % (4 * es) == 0 && rs % 4 == 0 &&
          !(x->stype == ST_BF16 && (kind == R_SUM_U || kind == R_MAX_U || kind == R_ARGMAX_U))) {
        TRY(alloc_result(be, n, n->dtype == CG_F32 ? ST_F32 : ST_U32));
        const char *name = kind <= R_SUM_U ? "reduce_sum" : kind <= R_MAX_U ? "reduce_max" : "reduce_argmax";
        {
          KernelScope ks(be, name, (double)x->size() * es + (double)rows * 4, 0);
          HIPCHK(be, launch_reduce_plain(be->lc(), kind, data_ptr(x), x->stype == ST_BF16, rs, n->st->ptr,
                                         (uint32_t)rows, (uint32_t)cols));
        }
        n->op = N_REAL;
        drop_inputs(n);
        return CG_OK;
      }
    }
  }
  // the input tree is evaluated inside the reduction when nobody else reads it
  Region reg;
  EwCompiler c(be, &reg);
  bool fused = false;
  if ((x->op == N_BIN || x->op == N_UN) && x->rc.load() == 1) {
    TRY(prepare_region(be, x, false, reg));
    int st = c.compile_root(x);
    if (!st) fused = true;
    else if (!c.overflow) return st;
  }
  if (!fused) {
    c = EwCompiler(be, &reg);
    TRY(c.load(c.final_code, x, 0));
  }
  c.flatten();
  std::vector<int64_t> ostr;
  double bytes_in = 0;
  TRY(finish_program(be, c, x->rank, x->shape, nullptr, true, ostr, &bytes_in));
  const int64_t cols = x->shape[x->rank - 1];
  const int64_t rows = cols ? x->size() / cols : n->size();
  if (x->size() >= (int64_t)1 << 32) return fail(be, CG_ERR_INTERNAL, "tensor above 2^32 elements");
  TRY(alloc_result(be, n, n->dtype == CG_F32 ? ST_F32 : ST_U32));
  const bool vec4 = cols % 4 == 0 && cols >= 4;
  const char *name = kind <= R_SUM_U ? "reduce_sum" : kind <= R_MAX_U ? "reduce_max" : "reduce_argmax";
  const uint32_t chunks = reduce_split_chunks(be->lc(), (uint32_t)rows, (uint32_t)cols);
  Storage *scratch = nullptr;
  if (chunks > 1) TRY(dev_alloc(be, (size_t)rows * chunks * 3 * 4, &scratch));
  hipError_t e;
  {
    KernelScope ks(be, name, bytes_in + (double)rows * 4, 0);
    e = launch_reduce(be->lc(), kind, c.p, n->st->ptr, (uint32_t)rows, (uint32_t)cols, vec4,
                      scratch ? (uint32_t *)scratch->ptr : nullptr, chunks);
  }
  storage_release(scratch);
  HIPCHK(be, e);
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

// A matmul operand as the kernels see it: a realised tensor plus the shape/strides to read it
// with (which may differ from the tensor's own when a repeat_kv chain was peeled off).
struct MatOperand {
  cg_tensor *t = nullptr;  // retained
  int rank = 0;
  int64_t shape[CG_MAX_RANK + 1], strides[CG_MAX_RANK + 1];
  void set(cg_tensor *x) {
    node_release(t);
    t = x;
    rank = x->rank;
    std::copy(x->shape, x->shape + rank, shape);
    std::copy(x->strides, x->strides + rank, strides);
  }
  ~MatOperand() { node_release(t); }
};

// repeat_kv (catgrad-llm/src/helpers.rs:147-161) leaves K and V as
//   reshape([b, kv*rep, s, d]) <- broadcast([b, kv, rep, s, d]) <- reshape([b, kv, 1, s, d]) <- x
// optionally under transpose(2, 3).  Instead of materialising rep copies, the 5-d broadcast
// view (stride 0 along rep) is handed to the GEMM as three batch dims.
int peel_repeat_kv(cg_backend *be, cg_tensor *t, MatOperand *out, bool *peeled) {
  *peeled = false;
  bool tr = false;
  if (t->op == N_TRANSPOSE && refs(t) == 1 && t->rank == 4 &&
      ((t->p0 == 2 && t->p1 == 3) || (t->p0 == 3 && t->p1 == 2))) {
    tr = true;
    t = t->in[0];
  }
  if (t->op != N_RESHAPE || refs(t) != 1 || t->rank != 4) return CG_OK;
  cg_tensor *u = t->in[0];
  if (u->rank != 5 || u->shape[0] != t->shape[0] || u->shape[1] * u->shape[2] != t->shape[1] ||
      u->shape[3] != t->shape[2] || u->shape[4] != t->shape[3])
    return CG_OK;
  TRY(realize(be, u));
  out->set(retain(u));
  if (tr) {
    std::swap(out->shape[3], out->shape[4]);
    std::swap(out->strides[3], out->strides[4]);
  }
  *peeled = true;
  return CG_OK;
}

// view a rank-4 operand [b, h, r, c] as [b, h / rep, rep, r, c]
void split_heads(MatOperand *o, int64_t rep) {
  for (int i = 4; i >= 2; --i) {
    o->shape[i] = o->shape[i - 1];
    o->strides[i] = o->strides[i - 1];
  }
  o->shape[2] = rep;
  o->shape[1] = o->shape[1] / rep;
  o->strides[2] = o->strides[1];  // one head
  o->strides[1] = o->strides[2] * rep;
  o->rank = 5;
}

bool matrix_ok(const MatOperand &o) {
  const int r = o.rank;
  return o.strides[r - 1] == 1 || o.shape[r - 1] == 1 || o.strides[r - 2] == 1 || o.shape[r - 2] == 1;
}

// bf16 twin of an f32 storage (whole buffer, so any view of it maps onto the twin unchanged)
int bf16_shadow(cg_backend *be, Storage *st, Storage **out) {
  if (!st->shadow) {
    Storage *sh = nullptr;
    TRY(dev_alloc(be, st->bytes / 2, &sh));
    KernelScope ks(be, "cast_bf16", (double)st->bytes * 1.5, 0);
    hipError_t e = launch_cast_bf16(be->lc(), (const float *)st->ptr, sh->ptr, st->bytes / 4);
    if (e != hipSuccess) {
      storage_release(sh);
      return fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
    }
    st->shadow = sh;
  }
  *out = st->shadow;
  return CG_OK;
}

// Routed experts (catgrad-llm/src/models/qwen3.rs:104-123) multiply each token by the matrix of
// its expert:  matmul(x[S, 1, K], transpose(1, 2, index(0, idx[S], W[E, N, K]))).  Gathering S
// whole matrices first would move S*N*K elements twice; instead the one-row kernels are given
// the index vector and read W[idx[s]] in place.
struct ExpertPeel {
  cg_tensor *w = nullptr, *idx = nullptr;  // retained, realised
  int64_t idx_stride = 1;                  // elements between consecutive indices
  ~ExpertPeel() {
    node_release(w);
    node_release(idx);
  }
};

int peel_expert_index(cg_backend *be, cg_tensor *n, ExpertPeel *out) {
  if (be->flags & CG_FLAG_NO_PATTERNS) return CG_OK;
  cg_tensor *t = n->in[1];
  if (n->rank != 3 || n->shape[1] > 8 || n->size() == 0) return CG_OK;
  if (t->op != N_TRANSPOSE || refs(t) != 1 || !((t->p0 == 1 && t->p1 == 2) || (t->p0 == 2 && t->p1 == 1)))
    return CG_OK;
  cg_tensor *g = t->in[0];
  if (g->op != N_INDEX || refs(g) != 1 || g->p0 != 0 || g->rank != 3) return CG_OK;
  cg_tensor *w = g->in[0], *idx = g->in[1];
  if (idx->size() != n->shape[0] || w->shape[0] == 0) return CG_OK;
  TRY(realize(be, n->in[0]));
  if (n->in[0]->stype != ST_F32) return CG_OK;  // the one-row kernels take f32 activations
  TRY(realize(be, w));
  if (w->strides[2] != 1 && w->strides[1] != 1) return CG_OK;
  // indices of any rank are read flattened (ndarray.rs:373-381); a strided view needs one stride
  TRY(realize(be, idx));
  // one stride between consecutive (flattened) indices: a column of the [S, k] top-k result
  int64_t stride = 1, expect = -1;
  bool uniform = true;
  for (int i = idx->rank - 1; i >= 0; --i) {
    if (idx->shape[i] == 1) continue;
    if (expect < 0) stride = idx->strides[i];
    else if (idx->strides[i] != expect) uniform = false;
    expect = idx->strides[i] * idx->shape[i];
  }
  cg_tensor *flat = nullptr;
  if (uniform) {
    flat = retain(idx);
  } else {
    TRY(contiguous(be, idx, &flat));
    stride = 1;
  }
  out->w = retain(w);
  out->idx = flat;
  out->idx_stride = stride;
  return CG_OK;
}

// Attention of a decode step (models/llama.rs:77-112 with one query row):
//   matmul(softmax(matmul(q, K^T) / sqrt(d) + mask), V)
// in one launch that reads K and V rows in place from the cache; the [b, h, 1, T] scores and
// probabilities never exist in HBM.
// Attention over many query rows (prefill; models/llama.rs:95-107, gemma3.rs:153-186) in bf16 mode:
//   matmul(softmax(matmul(q, K^T) / sqrt(d) + mask), V)
// as one pass with online softmax (k_attn.hip); the [b, h, S, T] scores and probabilities are
// never written.  f32 mode keeps the generic path (the 1e-4 bar wants f32 products).
int try_attn_prefill(cg_backend *be, cg_tensor *n, bool *done) {
  if (!(be->flags & CG_FLAG_BF16)) return CG_OK;
  cg_tensor *P = n->in[0];
  if (P->op == N_REAL || refs(P) != 1 || P->rank != 4) return CG_OK;
  SoftmaxMatch m;
  if (!match_softmax(P, &m)) return CG_OK;
  cg_tensor *S = m.src;
  if (S->op != N_MATMUL || S->rank != 4 || refs(S) != (S == m.x ? 2 : 1)) return CG_OK;
  const int64_t Sq = S->shape[2], T = S->shape[3], d = n->shape[3], heads = n->shape[1], nb = n->shape[0];
  if (Sq < 16 || T < 1 || (d != 64 && d != 128 && d != 256) || n->in[1]->shape[2] != T || S->in[0]->shape[3] != d)
    return CG_OK;
  // Below this the three-launch path (GEMM, softmax, GEMM) is as fast and the scores are small;
  // above it the scores of one layer run to hundreds of MB.  CG_FLAG_ATTN_ONE_PASS lifts the threshold.
  if (T < 512 && !(be->flags & CG_FLAG_ATTN_ONE_PASS)) return CG_OK;
  if (nb > 65535 || heads > 65535) return CG_OK;
  MatOperand Kop, Vop;
  bool pk = false, pv = false;
  TRY(peel_repeat_kv(be, S->in[1], &Kop, &pk));
  TRY(peel_repeat_kv(be, n->in[1], &Vop, &pv));
  if (!pk || !pv) return CG_OK;  // operands get realised by the generic path below
  cg_tensor *q = S->in[0];
  TRY(realize(be, q));
  cg_tensor *mask = m.mask;
  if (mask) TRY(realize(be, mask));
  auto ok4 = [](const void *ptr, int64_t unit, std::initializer_list<int64_t> strides) {
    if (unit != 1 || (uintptr_t)ptr % 16) return false;
    for (int64_t st : strides)
      if (st % 4) return false;
    return true;
  };
  if (Kop.shape[2] != Vop.shape[2] || Kop.shape[1] != Vop.shape[1] || Kop.shape[1] * Kop.shape[2] != heads) return CG_OK;
  if (q->stype != ST_F32 || Kop.t->stype != ST_F32 || Vop.t->stype != ST_F32 || (mask && mask->stype != ST_F32)) return CG_OK;
  if (!ok4(data_ptr(q), q->strides[3], {q->strides[0], q->strides[1], q->strides[2]}) ||
      !ok4(data_ptr(Kop.t), Kop.strides[3], {Kop.strides[0], Kop.strides[1], Kop.strides[2], Kop.strides[4]}) ||
      !ok4(data_ptr(Vop.t), Vop.strides[4], {Vop.strides[0], Vop.strides[1], Vop.strides[2], Vop.strides[3]}))
    return CG_OK;
  // the bf16 keys are read eight at a time
  if (Kop.t->offset % 8 || Kop.strides[0] % 8 || Kop.strides[1] % 8 || Kop.strides[2] % 8 || Kop.strides[4] % 8) return CG_OK;
  TRY(alloc_result(be, n, ST_F32));
  // The models merge the heads next (`transpose(1, 2)` + `reshape [b, s, heads * d]`, llama.rs:107-109):
  // the result is laid out [b, s, heads, d] in memory and handed back as the [b, heads, s, d] view of
  // it, so that merge is a view and the bf16 twin is already the o_proj operand.
  n->strides[0] = Sq * heads * d;
  n->strides[1] = d;
  n->strides[2] = heads * d;
  n->strides[3] = 1;
  AttnPrefillDesc a;
  std::memset(&a, 0, sizeof(a));
  a.q = (const float *)data_ptr(q);
  a.v = (const float *)data_ptr(Vop.t);
  a.out = (float *)n->st->ptr;
  a.o_sb = n->strides[0]; a.o_sh = n->strides[1]; a.o_ss = n->strides[2];
  TRY(twin_for_result(be, n, &a.out16));
  a.q_sb = q->strides[0]; a.q_sh = q->strides[1]; a.q_ss = q->strides[2];
  a.k_sb = Kop.strides[0]; a.k_skv = Kop.strides[1]; a.k_srep = Kop.strides[2]; a.k_st = Kop.strides[4];
  a.v_sb = Vop.strides[0]; a.v_skv = Vop.strides[1]; a.v_srep = Vop.strides[2]; a.v_st = Vop.strides[3];
  if (mask) {
    a.mask = (const float *)data_ptr(mask);
    a.m_sb = mask->shape[0] == 1 ? 0 : mask->strides[0];
    a.m_sh = mask->shape[1] == 1 ? 0 : mask->strides[1];
    a.m_ss = mask->shape[2] == 1 ? 0 : mask->strides[2];
    a.m_st = mask->shape[3] == 1 ? 0 : mask->strides[3];
    a.m_vec = a.m_st == 1 && (uintptr_t)a.mask % 16 == 0 && a.m_sb % 4 == 0 && a.m_sh % 4 == 0 && a.m_ss % 4 == 0;
  }
  // the kernel reads mask rows and value columns 16 bytes at a time, and the keys from their bf16 twin
  Storage *ksh = nullptr;
  const bool twin_ok = Kop.t->st->grow_dim < 0 && Kop.t->st->bytes % 32 == 0;
  if ((mask && !a.m_vec) || T % 8 || !twin_ok) {
    storage_release(n->st);
    n->st = nullptr;
    return CG_OK;
  }
  TRY(bf16_shadow(be, Kop.t->st, &ksh));
  a.k16 = (const uint16_t *)ksh->ptr + Kop.t->offset;
  Storage *vt = nullptr;
  const int64_t kvh = Kop.shape[1];
  TRY(dev_alloc(be, (size_t)nb * kvh * d * T * 2, &vt));
  {
    KernelScope ks(be, "transpose_cast_bf16", (double)nb * kvh * d * T * 6, 0);
    hipError_t te = launch_transpose_cast_bf16(be->lc(), data_ptr(Vop.t), ST_F32, vt->ptr, (uint32_t)T, (uint32_t)d,
                                               Vop.strides[3], (uint32_t)nb, (uint32_t)kvh, Vop.strides[0], Vop.strides[1]);
    if (te != hipSuccess) {
      storage_release(vt);
      return fail(be, CG_ERR_DEVICE, hipGetErrorString(te));
    }
  }
  a.vt16 = (const uint16_t *)vt->ptr;
  a.b = (uint32_t)nb;
  a.heads = (uint32_t)heads;
  a.rep = (uint32_t)Kop.shape[2];
  a.s = (uint32_t)Sq;
  a.t = (uint32_t)T;
  a.d = (uint32_t)d;
  a.has_scale = m.has_scale;
  a.scale = m.scale;
  a.has_mask_const = m.has_mask_const;
  a.mask_const = m.mask_const;
  // One mask for every batch and head (the causal or sliding-window mask of a model): classify its
  // tiles once - the table stays with the mask's storage, so every layer of the run finds it - and let
  // the kernel skip the key tiles no query of a tile can see.
  if (mask && a.m_sb == 0 && a.m_sh == 0 && a.m_ss > 0 && mask->st->grow_dim < 0) {
    uint32_t q_rows = 0, keys = 0;
    attn_prefill_tiling(be->lc(), a, &q_rows, &keys);
    Storage *ms = mask->st;
    const int64_t key[5] = {mask->offset, Sq, T, q_rows, keys};
    const size_t rows = (size_t)(Sq + q_rows - 1) / q_rows, cols = (size_t)(T + keys - 1) / keys;
    if (!ms->tiles || !std::equal(key, key + 5, ms->tiles_key)) {
      storage_release(ms->tiles);
      ms->tiles = nullptr;
      int st = dev_alloc(be, rows * cols, &ms->tiles);
      if (st) {
        storage_release(vt);
        return st;
      }
      std::copy(key, key + 5, ms->tiles_key);
      KernelScope ks(be, "attn_mask_tiles", (double)Sq * T * 4, 0);
      hipError_t me = launch_mask_tiles(be->lc(), a.mask, a.m_ss, (uint32_t)Sq, (uint32_t)T, q_rows, keys, (uint8_t *)ms->tiles->ptr);
      if (me != hipSuccess) {
        storage_release(vt);
        return fail(be, CG_ERR_DEVICE, hipGetErrorString(me));
      }
    }
    a.tile_class = (const uint8_t *)ms->tiles->ptr;
    a.tile_cols = (uint32_t)cols;
  }
  {
    const double qo = 2.0 * nb * heads * Sq * d * 4, kvb = 2.0 * nb * Kop.shape[1] * T * d * 4;
    KernelScope ks(be, "attn_prefill", qo + kvb + (mask ? (double)Sq * T * 4 : 0.0), 4.0 * nb * heads * Sq * T * d);
    hipError_t ae = launch_attn_prefill(be->lc(), a);
    storage_release(vt);
    HIPCHK(be, ae);
  }
  n->op = N_REAL;
  drop_inputs(n);
  *done = true;
  return CG_OK;
}

// Scratch of the split decode attention, grown as needed (the stream is drained before the old
// buffers go, and new counters start at zero).
int attn_decode_scratch(cg_backend *be, size_t part_floats, size_t count_words) {
  if (part_floats > be->attn_part_floats) {
    size_t want = 1 << 16;
    while (want < part_floats) want <<= 1;
    HIPCHK(be, hipStreamSynchronize(be->ordered_stream()));
    if (be->attn_part) (void)hipFree(be->attn_part);
    be->attn_part = nullptr;
    be->attn_part_floats = 0;
    HIPCHK(be, hipMalloc((void **)&be->attn_part, want * sizeof(float)));
    be->attn_part_floats = want;
  }
  if (count_words > be->attn_count_words) {
    size_t want = 1 << 10;
    while (want < count_words) want <<= 1;
    HIPCHK(be, hipStreamSynchronize(be->ordered_stream()));
    if (be->attn_count) (void)hipFree(be->attn_count);
    be->attn_count = nullptr;
    be->attn_count_words = 0;
    HIPCHK(be, hipMalloc((void **)&be->attn_count, want * sizeof(uint32_t)));
    HIPCHK(be, hipMemsetAsync(be->attn_count, 0, want * sizeof(uint32_t), be->ordered_stream()));
    be->attn_count_words = want;
  }
  return CG_OK;
}

// The cache update of a decode step, `concat(2, cached, new)` (legacy/models/utils.rs:222-223), seen
// from the attention that reads it: the node under the repeat_kv chain of a K or V operand.
// `x` (realised) walks its storage exactly as the tensor the storage's spare room was laid out for
bool has_grow_layout(const cg_tensor *x) {
  const Storage *s = x->st;
  return s && x->rank == s->grow_rank && std::equal(x->strides, x->strides + x->rank, s->grow_strides);
}

cg_tensor *kv_concat_under(cg_tensor *t) {
  if (t->op == N_TRANSPOSE && refs(t) == 1 && t->rank == 4 &&
      ((t->p0 == 2 && t->p1 == 3) || (t->p0 == 3 && t->p1 == 2)))
    t = t->in[0];
  if (t->op != N_RESHAPE || refs(t) != 1 || t->rank != 4) return nullptr;
  cg_tensor *u = t->in[0];
  if (u->op != N_BROADCAST || refs(u) != 1 || u->rank != 5) return nullptr;
  cg_tensor *r5 = u->in[0];
  if (r5->op != N_RESHAPE || refs(r5) != 1 || r5->rank != 5 || r5->shape[2] != 1) return nullptr;
  cg_tensor *c = r5->in[0];
  if (c->op != N_CONCAT || c->p0 != 2 || c->rank != 4 || c->dtype != CG_F32) return nullptr;
  return c;
}

// One new row per (batch, kv head) to be appended in place by the attention kernel itself.
struct RowAppend {
  cg_tensor *concat = nullptr;
  cg_tensor *src = nullptr;  // retained: the tensor the rows are read from
  const float *cos = nullptr, *sin = nullptr;
  cg_tensor *cos_t = nullptr, *sin_t = nullptr;  // retained
  ~RowAppend() {
    node_release(src);
    node_release(cos_t);
    node_release(sin_t);
  }
};

// Checks that `c` can be appended to in place and that its new rows can be read by the kernel;
// realises what has to exist for that (the cache, the projection) but changes nothing.
int row_append_candidate(cg_backend *be, cg_tensor *c, bool allow_rope, RowAppend *out, bool *ok) {
  *ok = false;
  cg_tensor *x = c->in[0], *y = c->in[1];
  if (y->shape[2] != 1 || x->shape[2] < 1) return CG_OK;
  TRY(realize(be, x));
  const int64_t xd = x->shape[2];
  if (!(refs(x) == 1 && x->st->rc.load() == 1 && x->st->grow_dim == 2 && xd + 1 <= x->st->grow_cap &&
        x->offset == 0 && x->stype == ST_F32 && has_grow_layout(x)))
    return CG_OK;
  if (x->strides[3] != 1 || x->strides[0] % 4 || x->strides[1] % 4 || x->strides[2] % 4 ||
      (uintptr_t)data_ptr(x) % 16)
    return CG_OK;
  cg_tensor *src = y;
  RopeMatch rm;
  if (allow_rope && y->op != N_REAL && refs(y) == 1 && match_rope(y, &rm)) {
    bool tables = false;
    TRY(rope_operands(be, rm, &tables));
    if (!tables) return CG_OK;
    src = rm.x;
    out->cos_t = retain(rm.cb);
    out->sin_t = retain(rm.sb);
    out->cos = (const float *)data_ptr(rm.cb);
    out->sin = (const float *)data_ptr(rm.sb);
  } else {
    TRY(realize(be, y));
  }
  if (src->stype != ST_F32 || src->strides[3] != 1 || src->strides[0] % 4 || src->strides[1] % 4 ||
      (uintptr_t)data_ptr(src) % 16)
    return CG_OK;
  out->concat = c;
  out->src = retain(src);
  *ok = true;
  return CG_OK;
}

// The bookkeeping half of realize_concat's in-place append; the rows themselves are stored by
// the kernel launched right after.
void commit_row_append(cg_tensor *c) {
  cg_tensor *x = c->in[0];
  c->st = x->st;
  c->st->rc.fetch_add(1);
  storage_release(c->st->shadow);
  c->st->shadow = nullptr;
  c->stype = ST_F32;
  c->offset = 0;
  std::memcpy(c->strides, x->strides, sizeof(c->strides));
  c->op = N_REAL;
  drop_inputs(c);
}

// The rows of a committed append written by kernels of their own: what is left to do when the attention
// kernel that was to store them cannot be launched after all.
int write_row_append(cg_backend *be, const RowAppend &ra) {
  cg_tensor *c = ra.concat, *src = ra.src;
  float *dst = (float *)c->st->ptr + (c->shape[2] - 1) * c->strides[2];
  if (!ra.cos) return run_ew(be, src, true, dst, c->strides, ST_F32, "kv_append");
  RopeDesc d;
  std::memset(&d, 0, sizeof(d));
  d.x = (const float *)data_ptr(src);
  d.cos = ra.cos;
  d.sin = ra.sin;
  d.out = dst;
  d.x_sb = src->strides[0];
  d.x_sh = src->strides[1];
  d.x_ss = src->strides[2];
  d.o_sb = c->strides[0];
  d.o_sh = c->strides[1];
  d.o_ss = c->strides[2];
  d.cs_ss = 0;  // one position
  d.b = (uint32_t)c->shape[0];
  d.h = (uint32_t)c->shape[1];
  d.s = 1;
  d.dim = (uint32_t)c->shape[3];
  d.half = d.dim / 2;
  KernelScope ks(be, "rope_kv_append", (double)d.b * d.h * d.dim * 8, 0);
  HIPCHK(be, launch_rope(be->lc(), d));
  return CG_OK;
}

int try_attn_decode(cg_backend *be, cg_tensor *n, bool *done) {
  cg_tensor *P = n->in[0];
  if (P->op == N_REAL || refs(P) != 1 || P->rank != 4) return CG_OK;
  SoftmaxMatch m;
  if (!match_softmax(P, &m) || m.mask) return CG_OK;
  cg_tensor *S = m.src;
  if (S->op != N_MATMUL || S->rank != 4 || S->shape[2] != 1 || refs(S) != (S == m.x ? 2 : 1)) return CG_OK;
  const int64_t T = S->shape[3], d = n->shape[3], heads = n->shape[1], nb = n->shape[0];
  if (T < 1 || T > 0x7FFFFFFF || d > ATTN_DECODE_MAX_D || d % 4 || n->in[1]->shape[2] != T) return CG_OK;
  if (S->in[0]->shape[3] != d) return CG_OK;
  // This step's cache update, when both K and V are `concat(2, cached, new)` that can be done in
  // place: the kernel takes the new rows from the projections and stores them itself.
  RowAppend ka, va;
  bool fused_append = false;
  {
    cg_tensor *ck = kv_concat_under(S->in[1]), *cv = kv_concat_under(n->in[1]);
    if (ck && cv && ck != cv && ck->shape[2] == T && cv->shape[2] == T && T >= 2) {
      bool okk = false, okv = false;
      TRY(row_append_candidate(be, ck, true, &ka, &okk));
      if (okk) TRY(row_append_candidate(be, cv, false, &va, &okv));
      if (okk && okv) {
        commit_row_append(ck);
        commit_row_append(cv);
        fused_append = true;
      }
    }
  }
  // From here on the caches claim their new rows (the views above them must see realised values), and
  // the launch below is what stores them.  When a later check finds the kernel cannot take this graph,
  // the rows are written by kernels of their own and the unfused path goes on from two ordinary caches.
#define ATTN_BAIL()                               \
  do {                                            \
    if (fused_append) {                           \
      TRY(write_row_append(be, ka));              \
      TRY(write_row_append(be, va));              \
    }                                             \
    return CG_OK;                                 \
  } while (0)
  MatOperand Kop, Vop;
  bool pk = false, pv = false;
  TRY(peel_repeat_kv(be, S->in[1], &Kop, &pk));
  TRY(peel_repeat_kv(be, n->in[1], &Vop, &pv));
  auto unpeeled = [&](cg_tensor *t, MatOperand *o) -> int {  // [b, h, r, c] as [b, h, 1, r, c]
    TRY(realize(be, t));
    o->set(retain(t));
    for (int i = 4; i >= 3; --i) {
      o->shape[i] = o->shape[i - 1];
      o->strides[i] = o->strides[i - 1];
    }
    o->shape[2] = 1;
    o->strides[2] = 0;
    o->rank = 5;
    return CG_OK;
  };
  if (fused_append && (!pk || !pv)) ATTN_BAIL();
  if (!pk) TRY(unpeeled(S->in[1], &Kop));
  if (!pv) TRY(unpeeled(n->in[1], &Vop));
  cg_tensor *q = S->in[0];
  // q straight from apply_rope_embedding and read by nobody else: rotate it inside the kernel
  RopeMatch qrope;
  const float *q_cos = nullptr, *q_sin = nullptr;
  if (q->op != N_REAL && refs(q) == 1 && match_rope(q, &qrope)) {
    bool tables = false;
    TRY(rope_operands(be, qrope, &tables));
    cg_tensor *qx = qrope.x;
    if (tables && qx->stype == ST_F32 && qx->strides[3] == 1 && (uintptr_t)data_ptr(qx) % 16 == 0 &&
        qx->strides[0] % 4 == 0 && qx->strides[1] % 4 == 0) {
      q_cos = (const float *)data_ptr(qrope.cb);
      q_sin = (const float *)data_ptr(qrope.sb);
      q = qx;
    }
  }
  TRY(realize(be, q));
  auto rows_ok = [](const void *ptr, int64_t unit, std::initializer_list<int64_t> strides) {
    if (unit != 1 || (uintptr_t)ptr % 16) return false;
    for (int64_t st : strides)
      if (st % 4) return false;
    return true;
  };
  // K as [b, kv, rep, d, T] (the transposed view), V as [b, kv, rep, T, d]
  if (Kop.shape[2] != Vop.shape[2] || Kop.shape[1] != Vop.shape[1] || Kop.shape[1] * Kop.shape[2] != heads) ATTN_BAIL();
  if (q->stype != ST_F32 || Kop.t->stype != ST_F32 || Vop.t->stype != ST_F32) ATTN_BAIL();
  if (!rows_ok(data_ptr(q), q->strides[3], {q->strides[0], q->strides[1]}) ||
      !rows_ok(data_ptr(Kop.t), Kop.strides[3], {Kop.strides[0], Kop.strides[1], Kop.strides[2], Kop.strides[4]}) ||
      !rows_ok(data_ptr(Vop.t), Vop.strides[4], {Vop.strides[0], Vop.strides[1], Vop.strides[2], Vop.strides[3]}))
    ATTN_BAIL();
#undef ATTN_BAIL
  TRY(alloc_result(be, n, ST_F32));
  AttnDecodeDesc a;
  std::memset(&a, 0, sizeof(a));
  a.q = (const float *)data_ptr(q);
  a.k = (const float *)data_ptr(Kop.t);
  a.v = (const float *)data_ptr(Vop.t);
  a.out = (float *)n->st->ptr;
  a.q_sb = q->strides[0];
  a.q_sh = q->strides[1];
  a.k_sb = Kop.strides[0]; a.k_skv = Kop.strides[1]; a.k_srep = Kop.strides[2]; a.k_st = Kop.strides[4];
  a.v_sb = Vop.strides[0]; a.v_skv = Vop.strides[1]; a.v_srep = Vop.strides[2]; a.v_st = Vop.strides[3];
  a.b = (uint32_t)nb;
  a.heads = (uint32_t)heads;
  a.rep = (uint32_t)Kop.shape[2];
  a.t = (uint32_t)T;
  a.d = (uint32_t)d;
  a.has_scale = m.has_scale;
  a.scale = m.scale;
  a.has_mask_const = m.has_mask_const;
  a.mask_const = m.mask_const;
  a.q_cos = q_cos;
  a.q_sin = q_sin;
  if (fused_append) {
    a.k_new = (const float *)data_ptr(ka.src);
    a.v_new = (const float *)data_ptr(va.src);
    a.kn_cos = ka.cos;
    a.kn_sin = ka.sin;
    a.kn_sb = ka.src->strides[0];
    a.kn_skv = ka.src->strides[1];
    a.vn_sb = va.src->strides[0];
    a.vn_skv = va.src->strides[1];
    a.t_new = (uint32_t)(T - 1);
  }
  {
    // long caches: the keys of a (batch, head) go to several workgroups, enough of them to occupy
    // every compute unit, each with at most a few passes over its chunk
    const int64_t bh = nb * heads, rpp = attn_decode_rows_per_pass((uint32_t)d);
    int64_t ns = std::max((T + rpp - 1) / rpp, std::min((be->n_cus + bh - 1) / bh, (T + 31) / 32));
    ns = std::min<int64_t>(ns, 64);
    if (ns >= 2 || T > ATTN_DECODE_MAX_T) {
      const int64_t chunk = (T + ns - 1) / ns;
      a.chunk = (uint32_t)chunk;
      a.splits = (uint32_t)((T + chunk - 1) / chunk);
      TRY(attn_decode_scratch(be, (size_t)bh * a.splits * (d + 2), (size_t)bh));
      a.part = be->attn_part;
      a.count = be->attn_count;
    }
    const double kv_bytes = 2.0 * nb * Kop.shape[1] * T * d * 4;
    KernelScope ks(be, "attn_decode", kv_bytes + 2.0 * nb * heads * d * 4, 4.0 * nb * heads * T * d);
    HIPCHK(be, launch_attn_decode(be->lc(), a));
  }
  if (n->gemv_candidate) forget_gemv_candidate(n);
  n->op = N_REAL;
  drop_inputs(n);
  *done = true;
  return CG_OK;
}

// A batch-folding linear reshapes its input ([B, 1, K] -> [1, B, K]) and its product back; such a
// reshape only regroups rows.  The node under a reshape that nobody else holds and that keeps the
// last axis, else the node itself.
static cg_tensor *rows_base(cg_tensor *t) {
  if (t->op == N_RESHAPE && refs(t) == 1 && t->rank >= 1 && t->in[0]->rank >= 1 &&
      t->in[0]->shape[t->in[0]->rank - 1] == t->shape[t->rank - 1])
    return t->in[0];
  return t;
}

// h = act(gate_proj(x)) * up_proj(x) with one input row (models/llama.rs:11-35): both products and the
// activation in one launch, a wave computing column n of gate and of up (and x itself from its
// RMSNorm when nothing else reads the normed row).  `glu` is the deferred act(g) * u node; on
// success it becomes a realised tensor and g, u are never materialised.
int try_gate_up_glu(cg_backend *be, cg_tensor *glu, cg_tensor *g, cg_tensor *u, int gelu, bool *done) {
  // the activation reads the gate two (three) times, the product once; either may sit under a reshape
  if (refs(g) != (gelu ? 3 : 2) || refs(u) != 1) return CG_OK;
  if (g->op == N_RESHAPE && refs(g->in[0]) == 1 && g->in[0]->size() == g->size()) g = g->in[0];
  u = rows_base(u);
  if (g->op != N_MATMUL || u->op != N_MATMUL || !g->gemv_candidate || !u->gemv_candidate) return CG_OK;
  if (refs(u) != 1 || rows_base(g->in[0]) != rows_base(u->in[0]) || g->size() != u->size()) return CG_OK;
  cg_tensor *X = rows_base(g->in[0]);
  const int64_t K = X->shape[X->rank - 1], N = g->shape[g->rank - 1];
  // one row, or the few rows of a small batch: [B, 1, K] against weights repeated over the batch
  const int64_t rows = K > 0 ? X->size() / K : 0;
  if (rows < 1 || rows > 4 || X->size() != rows * K || rows * K > GEMV_PRO_MAX_K || g->size() != rows * N || K % 8 || K < 256 ||
      glu->size() != rows * N)
    return CG_OK;
  cg_tensor *ws[2] = {g->in[1], u->in[1]};
  for (cg_tensor *w : ws) {
    TRY(realize(be, w));
    if (rows > 1 && K > (int64_t)gemv_pro_multi_row_max_k(w->stype)) return CG_OK;
    if (w->rank < 2 || w->shape[w->rank - 2] != K || w->strides[w->rank - 2] != 1) return CG_OK;
    for (int i = 0; i + 2 < w->rank; ++i)
      if (w->shape[i] != 1 && w->strides[i] != 0) return CG_OK;
    if ((w->stype != ST_F32 && w->stype != ST_BF16) || w->stype != ws[0]->stype) return CG_OK;
    if ((uintptr_t)data_ptr(w) % 16 || w->strides[w->rank - 1] % (16 / esize(w->stype))) return CG_OK;
  }
  GemvProDesc d;
  std::memset(&d, 0, sizeof(d));
  RmsNormMatch rm;
  cg_tensor *a0 = nullptr, *a1 = nullptr;
  if (X->op != N_REAL && refs(X) == 2 && match_rmsnorm(X, &rm)) {
    bool vec = true;
    if (rm.gamma) TRY(gamma_row_vector(be, rm.gamma, &vec));
    TRY(realize(be, rm.x));
    if (vec && rm.x->stype == ST_F32 && is_contiguous(rm.x) && (uintptr_t)data_ptr(rm.x) % 16 == 0) {
      d.pro = PRO_RMSNORM;
      a0 = retain(rm.x);
      if (rm.gamma) a1 = retain(rm.gamma);
      d.n_as_float = rm.n_as_float;
      d.eps = rm.eps;
      d.gamma_offset = rm.gamma_offset;
    }
  }
  if (!a0) {
    TRY(contiguous(be, X, &a0));
    if (a0->stype != ST_F32 || (uintptr_t)data_ptr(a0) % 16) {
      node_release(a0);
      return CG_OK;
    }
    d.pro = PRO_NONE;
  }
  int st = alloc_result(be, glu, ST_F32);
  if (!st) {
    d.a = (const float *)data_ptr(a0);
    d.aux = a1 ? (const float *)data_ptr(a1) : nullptr;
    d.glu_epilogue = gelu ? PRO_GEGLU : PRO_SWIGLU;
    d.rows = (uint32_t)rows;
    d.a_rstride = d.aux_rstride = K;
    d.m.K = (uint32_t)K;
    d.m.b_stype = ws[0]->stype;
    d.m.n_prob = 2;
    for (int i = 0; i < 2; ++i) {
      d.m.p[i].b = data_ptr(ws[i]);
      d.m.p[i].c = (float *)glu->st->ptr;
      d.m.p[i].sbn = ws[i]->strides[ws[i]->rank - 1];
      d.m.p[i].N = (uint32_t)N;
    }
    const char *base = ws[0]->stype == ST_BF16 ? "gemv_rowdot_bf16" : "gemv_rowdot_f32";
    KernelScope ks(be, base, 2.0 * N * K * esize(ws[0]->stype) + (double)rows * (K * 8 + N * 4), 4.0 * rows * N * K);
    if (be->trace_shapes) {
      char buf[96];
      snprintf(buf, sizeof buf, "%s[%sgate*up,M%lld,K%lld,N%lld]", base, d.pro == PRO_RMSNORM ? "rmsnorm+" : "", (long long)rows,
               (long long)K, (long long)(2 * N));
      ks.rename(buf);
    }
    hipError_t e = launch_gemv_pro(be->lc(), d);
    if (e != hipSuccess) st = fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
  }
  node_release(a0);
  node_release(a1);
  if (st) return st;
  finish_fused(glu);  // releases the activation chain and with it g and u
  *done = true;
  return CG_OK;
}

// q/k/v, gate/up and down_proj of a decode step: one-row products whose input row is an RMSNorm
// or a SwiGLU/GeGLU of earlier values.  When every consumer of that row is such a product, the
// row is computed inside the product kernel (launch_gemv_pro) and its node is never realised.
int try_gemv_prologue(cg_backend *be, cg_tensor *n, cg_tensor *addend, bool *added, bool *done) {
  cg_tensor *A = rows_base(n->in[0]);
  if (A->op == N_REAL || A->dtype != CG_F32 || !n->gemv_candidate || A->rank < 1) return CG_OK;
  const int64_t K = A->shape[A->rank - 1];
  const int64_t rows = K > 0 ? A->size() / K : 0;  // one row, or the few rows of a small batch
  if (rows < 1 || rows > 4 || A->size() != rows * K || K % 8 || K < 256 || rows * K > GEMV_PRO_MAX_K) return CG_OK;
  RmsNormMatch rm;
  cg_tensor *gate = nullptr, *up = nullptr;
  int gelu = 0, pro = 0;
  if (match_rmsnorm(A, &rm)) pro = PRO_RMSNORM;
  else if (match_glu(A, &gate, &up, &gelu)) pro = gelu ? PRO_GEGLU : PRO_SWIGLU;
  else return CG_OK;
  if (pro != PRO_RMSNORM) {
    // better still: the activation in the epilogue of the gate / up products themselves; A is
    // then a row in memory and this product runs without a prologue
    bool fused = false;
    TRY(try_gate_up_glu(be, A, gate, up, gelu, &fused));
    if (fused) return CG_OK;
  }
  // the group: every deferred one-row product reading A (n first)
  std::vector<cg_tensor *> members{n};
  for (cg_tensor *c : be->gemv_candidates)
    if (c != n && c->op == N_MATMUL && rows_base(c->in[0]) == A) members.push_back(c);
  if ((int)members.size() != refs(A) || members.size() > 4) return CG_OK;
  GemvProDesc d;
  std::memset(&d, 0, sizeof(d));
  int b_stype = -1;
  for (cg_tensor *c : members) {
    cg_tensor *w = c->in[1];
    if (c->size() != rows * c->shape[c->rank - 1]) return CG_OK;
    TRY(realize(be, w));
    if (w->rank < 2 || w->shape[w->rank - 2] != K || w->strides[w->rank - 2] != 1) return CG_OK;
    for (int i = 0; i + 2 < w->rank; ++i)
      if (w->shape[i] != 1 && w->strides[i] != 0) return CG_OK;
    if (w->stype != ST_F32 && w->stype != ST_BF16) return CG_OK;
    if (b_stype >= 0 && w->stype != b_stype) return CG_OK;
    if (rows > 1 && K > (int64_t)gemv_pro_multi_row_max_k(w->stype)) return CG_OK;
    b_stype = w->stype;
    if ((uintptr_t)data_ptr(w) % 16 || w->strides[w->rank - 1] % (16 / esize(w->stype))) return CG_OK;
  }
  // operands of the row
  cg_tensor *a0 = nullptr, *a1 = nullptr;
  if (pro == PRO_RMSNORM) {
    if (rm.gamma) {
      bool vec = false;
      TRY(gamma_row_vector(be, rm.gamma, &vec));
      if (!vec) return CG_OK;
    }
    TRY(realize(be, rm.x));
    if (rm.x->stype != ST_F32 || !is_contiguous(rm.x) || (uintptr_t)data_ptr(rm.x) % 16) return CG_OK;
    a0 = retain(rm.x);
    if (rm.gamma) a1 = retain(rm.gamma);
  } else {
    TRY(contiguous(be, gate, &a0));
    int st = contiguous(be, up, &a1);
    if (st) {
      node_release(a0);
      return st;
    }
    if (a0->stype != ST_F32 || a1->stype != ST_F32 || (uintptr_t)data_ptr(a0) % 16 || (uintptr_t)data_ptr(a1) % 16) {
      node_release(a0);
      node_release(a1);
      return CG_OK;
    }
  }
  d.pro = pro;
  d.a = (const float *)data_ptr(a0);
  d.aux = a1 ? (const float *)data_ptr(a1) : nullptr;
  d.n_as_float = rm.n_as_float;
  d.eps = rm.eps;
  d.gamma_offset = rm.gamma_offset;
  d.rows = (uint32_t)rows;
  d.a_rstride = d.aux_rstride = K;
  d.m.K = (uint32_t)K;
  d.m.b_stype = b_stype;
  double bytes = (double)rows * K * 8, flops = 0;
  int st = CG_OK;
  // A sibling whose only reader adds a bias vector to it: the launch stores the sum, as that add's value
  // (the root's own bias arrives as `addend`).
  std::vector<cg_tensor *> bias_add(members.size(), nullptr), bias_vec(members.size(), nullptr);
  for (size_t i = 0; i < members.size(); ++i) {
    cg_tensor *c = members[i], *add = c->bias_user;
    if (c == n || !add || refs(c) != 1 || add->op != N_BIN || add->bias_of != c || add->size() != c->size()) continue;
    cg_tensor *bv = bias_vector_of(add->in[add->in[0] == c ? 1 : 0], add);
    if (!bv) continue;
    st = realize(be, bv);
    if (st) break;
    if (!bias_vector_ready(bv)) continue;
    bias_add[i] = add;
    bias_vec[i] = bv;
  }
  for (size_t i = 0; i < members.size() && !st; ++i) {
    cg_tensor *c = members[i];
    cg_tensor *w = c->in[1];
    cg_tensor *dest = bias_add[i] ? bias_add[i] : c;
    st = alloc_result(be, dest, ST_F32);
    if (st) break;
    auto &pr = d.m.p[d.m.n_prob++];
    pr.b = data_ptr(w);
    pr.c = (float *)dest->st->ptr;
    pr.c_add = (c == n && addend) ? (const float *)data_ptr(addend) : bias_vec[i] ? (const float *)data_ptr(bias_vec[i]) : nullptr;
    pr.c_add_is_row = (c == n && addend) ? (be->addend_is_row ? 1 : 0) : bias_vec[i] ? 1 : 0;
    pr.sbn = w->strides[w->rank - 1];
    pr.N = (uint32_t)w->shape[w->rank - 1];
    bytes += (double)pr.N * K * esize(w->stype) + (double)rows * pr.N * 4;
    flops += 2.0 * rows * pr.N * K;
  }
  if (!st) {
    const char *base = b_stype == ST_BF16 ? "gemv_rowdot_bf16" : "gemv_rowdot_f32";
    KernelScope ks(be, base, bytes, flops);
    if (be->trace_shapes) {
      char buf[96];
      snprintf(buf, sizeof buf, "%s[%s%d,M%lld,K%lld,N%.0f]", base, pro == PRO_RMSNORM ? "rmsnorm+multi" : "glu+multi",
               d.m.n_prob, (long long)rows, (long long)K, flops / (2.0 * rows * K));
      ks.rename(buf);
    }
    hipError_t e = launch_gemv_pro(be->lc(), d);
    if (e != hipSuccess) st = fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
  }
  node_release(a0);
  node_release(a1);
  if (st) return st;
  if (addend) *added = true;
  for (size_t i = 0; i < members.size(); ++i) {
    if (bias_add[i]) {  // the add holds the value; letting go of its inputs deletes the product node
      finish_fused(bias_add[i]);
      continue;
    }
    cg_tensor *c = members[i];
    forget_gemv_candidate(c);
    c->op = N_REAL;
    drop_inputs(c);
  }
  *done = true;
  return CG_OK;
}

// The routed experts of a MoE layer as the reference emits them (models/qwen3.rs:104-123), per slot:
//   g = matmul(x[S,1,H], T(index(0, idx, Wg)));  u = matmul(x, T(index(0, idx, Wu)))
//   y = matmul(silu(g) * u, T(index(0, idx, Wd)))
// g and u go out as one launch (two problems sharing the staged input rows); the SwiGLU runs in the
// prologue of the down product.  Every workgroup stages the row of its token in LDS once and
// reads the weight rows of that token's expert in place (no gather of expert matrices).
struct ExpertOperand {
  cg_tensor *w = nullptr, *idx = nullptr;  // the stacked matrices [E, N, K] and the index tensor
};

bool match_expert_operand(const cg_tensor *t, int64_t S, ExpertOperand *o) {
  if (t->op != N_TRANSPOSE || refs(t) != 1 || t->rank != 3 ||
      !((t->p0 == 1 && t->p1 == 2) || (t->p0 == 2 && t->p1 == 1)))
    return false;
  const cg_tensor *g = t->in[0];
  if (g->op != N_INDEX || refs(g) != 1 || g->p0 != 0 || g->rank != 3) return false;
  if (g->in[1]->size() != S || g->in[0]->shape[0] == 0) return false;
  o->w = g->in[0];
  o->idx = g->in[1];
  return true;
}

// The same products over many tokens (a prefill, bf16 mode): expert by expert instead of token by
// token, and all k slots of the layer in one launch - every deferred expert product on the same
// stacked weights joins, with its own indices, input rows and output (launch_moe_gemm).
int try_moe_gemm(cg_backend *be, cg_tensor *n, bool *done) {
  const int64_t S = n->shape[0];
  if (S < 64 || S > 65535 || !(be->flags & CG_FLAG_BF16)) return CG_OK;
  ExpertOperand eo;
  if (!match_expert_operand(n->in[1], S, &eo)) return CG_OK;
  const int64_t K = n->in[0]->shape[2];
  if (n->in[0]->rank != 3 || K % 8 || K < 8) return CG_OK;
  cg_tensor *gate = nullptr, *up = nullptr;
  int gelu = 0;
  const bool glu = n->in[0]->op != N_REAL && refs(n->in[0]) == 1 && match_glu(n->in[0], &gate, &up, &gelu);
  struct Member {
    cg_tensor *c, *w, *idx;
    int slot, prob;
  };
  std::vector<Member> members;
  std::vector<cg_tensor *> slot_idx, prob_w, slot_a;
  auto find_or_add = [](std::vector<cg_tensor *> &v, cg_tensor *t) {
    for (size_t i = 0; i < v.size(); ++i)
      if (v[i] == t) return (int)i;
    v.push_back(t);
    return (int)v.size() - 1;
  };
  // n first, then every other deferred expert product that fits: same rows and any of the same
  // weight tensors (gate / up), or - for down_proj - the same weights and its own gated rows
  std::vector<cg_tensor *> cands{n};
  for (cg_tensor *c : be->gemv_candidates)
    if (c != n) cands.push_back(c);
  for (cg_tensor *c : cands) {
    if (c->op != N_MATMUL || c->rank != 3 || c->shape[0] != S || c->shape[1] != 1 || c->in[0]->rank != 3 || c->in[0]->shape[2] != K)
      continue;
    ExpertOperand co;
    if (!match_expert_operand(c->in[1], S, &co)) continue;
    if (glu) {
      cg_tensor *g2 = nullptr, *u2 = nullptr;
      int ge2 = 0;
      if (co.w != eo.w || c->in[0]->op == N_REAL || refs(c->in[0]) != 1 || !match_glu(c->in[0], &g2, &u2, &ge2) || ge2 != gelu)
        continue;
      if (slot_idx.size() >= 8 && c != n) continue;
      members.push_back(Member{c, co.w, co.idx, (int)slot_idx.size(), 0});
      slot_idx.push_back(co.idx);
      slot_a.push_back(c->in[0]);
      if (prob_w.empty()) prob_w.push_back(co.w);
    } else {
      if (c->in[0] != n->in[0]) continue;
      // a third weight tensor or a ninth slot stays outside
      bool known_w = false, known_i = false;
      for (cg_tensor *w : prob_w) known_w = known_w || w == co.w;
      for (cg_tensor *i : slot_idx) known_i = known_i || i == co.idx;
      if ((!known_w && prob_w.size() >= 2) || (!known_i && slot_idx.size() >= 8)) continue;
      members.push_back(Member{c, co.w, co.idx, find_or_add(slot_idx, co.idx), find_or_add(prob_w, co.w)});
    }
  }
  // every (slot, problem) pair exactly once, or only n's own slot
  auto complete = [&]() {
    if (members.size() != slot_idx.size() * prob_w.size()) return false;
    std::vector<int> seen(slot_idx.size() * prob_w.size(), 0);
    for (const Member &m : members)
      if (seen[m.slot * prob_w.size() + m.prob]++) return false;
    return true;
  };
  if (!complete()) {
    std::vector<Member> own;
    for (const Member &m : members)
      if (m.idx == eo.idx && (glu ? m.c == n : true)) own.push_back(m);
    members.swap(own);
    slot_idx.assign(1, eo.idx);
    if (glu) slot_a.assign(1, n->in[0]);
    prob_w.clear();
    for (Member &m : members) {
      m.slot = 0;
      m.prob = find_or_add(prob_w, m.w);
    }
    if (!complete()) return CG_OK;
  }
  MoeGemmDesc d;
  std::memset(&d, 0, sizeof(d));
  d.S = (uint32_t)S;
  d.K = (uint32_t)K;
  d.n_slot = (uint32_t)slot_idx.size();
  d.n_prob = (uint32_t)prob_w.size();
  d.pro = glu ? (gelu ? PRO_GEGLU : PRO_SWIGLU) : PRO_NONE;
  d.err = be->d_words;
  // weights: bf16, unit stride along k, one expert stride for every problem
  for (size_t p = 0; p < prob_w.size(); ++p) {
    cg_tensor *w = prob_w[p];
    TRY(realize(be, w));
    if (w->rank != 3 || w->stype != ST_BF16 || w->shape[2] != K || w->strides[2] != 1 || w->shape[0] != prob_w[0]->shape[0] ||
        w->strides[0] != prob_w[0]->strides[0] || (uintptr_t)data_ptr(w) % 16 || w->strides[1] % 8 || w->strides[0] % 8)
      return CG_OK;
    d.prob[p].w = data_ptr(w);
    d.prob[p].sbn = w->strides[1];
    d.prob[p].N = (uint32_t)w->shape[1];
  }
  d.n_expert = (uint32_t)prob_w[0]->shape[0];
  d.sb_index = prob_w[0]->strides[0];
  if (d.n_expert > 65535) return CG_OK;
  // indices: u32, one stride between consecutive tokens
  for (size_t sl = 0; sl < slot_idx.size(); ++sl) {
    cg_tensor *idx = slot_idx[sl];
    TRY(realize(be, idx));
    if (idx->dtype != CG_U32) return CG_OK;
    int64_t istride = 1, expect = -1;
    for (int i = idx->rank - 1; i >= 0; --i) {
      if (idx->shape[i] == 1) continue;
      if (expect < 0) istride = idx->strides[i];
      else if (idx->strides[i] != expect) return CG_OK;
      expect = idx->strides[i] * idx->shape[i];
    }
    d.slot[sl].idx = (const uint32_t *)data_ptr(idx);
    d.slot[sl].idx_stride = istride;
  }
  // The whole expert MLP of every slot in two launches: when the gated rows of down_proj come from
  // expert products of one input x that nobody else reads, gate and up are never stored - one
  // workgroup computes both for its tokens and keeps act(gate) * up as bf16 rows, which the second
  // launch multiplies with down_proj's matrices.
  if (glu) {
    bool fits = true;
    cg_tensor *x = nullptr, *wg = nullptr, *wu = nullptr;
    for (size_t sl = 0; sl < slot_a.size() && fits; ++sl) {
      cg_tensor *g2 = nullptr, *u2 = nullptr;
      int ge2 = 0;
      ExpertOperand og, ou;
      fits = match_glu(slot_a[sl], &g2, &u2, &ge2) && g2->op == N_MATMUL && u2->op == N_MATMUL && refs(g2) == (ge2 ? 3 : 2) &&
             refs(u2) == 1 && g2->rank == 3 && u2->rank == 3 && g2->in[0] == u2->in[0] &&
             match_expert_operand(g2->in[1], S, &og) && match_expert_operand(u2->in[1], S, &ou) && og.idx == slot_idx[sl] &&
             ou.idx == slot_idx[sl];
      if (!fits) break;
      if (!x) {
        x = g2->in[0];
        wg = og.w;
        wu = ou.w;
      }
      fits = g2->in[0] == x && og.w == wg && ou.w == wu;
    }
    if (fits && x && x->rank == 3 && x->shape[0] == S && x->shape[1] == 1) {
      const int64_t H = x->shape[2], F = K;
      TRY(realize(be, x));
      TRY(realize(be, wg));
      TRY(realize(be, wu));
      auto w_ok = [&](const cg_tensor *w, int64_t n_rows, int64_t k) {
        return w->rank == 3 && w->stype == ST_BF16 && w->shape[0] == d.n_expert && w->shape[1] == n_rows && w->shape[2] == k &&
               w->strides[2] == 1 && (uintptr_t)data_ptr(w) % 16 == 0 && w->strides[1] % 8 == 0 && w->strides[0] % 8 == 0;
      };
      if (H % 8 == 0 && x->stype == ST_F32 && x->strides[2] == 1 && x->strides[0] % 8 == 0 && x->offset % 8 == 0 &&
          x->st->bytes % 32 == 0 && x->st->grow_dim < 0 && w_ok(wg, F, H) && w_ok(wu, F, H) && wg->strides[0] == wu->strides[0]) {
        Storage *xsh = nullptr;
        TRY(bf16_shadow(be, x->st, &xsh));
        std::vector<Storage *> hbuf(slot_a.size(), nullptr);
        auto drop_h = [&]() {
          for (Storage *h : hbuf) storage_release(h);
        };
        int st = CG_OK;
        for (size_t sl = 0; sl < hbuf.size() && !st; ++sl) st = dev_alloc(be, (size_t)S * F * 2, &hbuf[sl]);
        for (const Member &m : members)
          if (!st) st = alloc_result(be, m.c, ST_F32);
        if (st) {
          drop_h();
          return st;
        }
        MoeGemmDesc f = d;  // same slots' indices and experts; products gate and up over x
        f.K = (uint32_t)H;
        f.n_prob = 2;
        f.pro = PRO_NONE;
        f.fuse_glu = gelu ? PRO_GEGLU : PRO_SWIGLU;
        f.sb_index = wg->strides[0];
        f.prob[0].w = data_ptr(wg); f.prob[0].sbn = wg->strides[1]; f.prob[0].N = (uint32_t)F;
        f.prob[1].w = data_ptr(wu); f.prob[1].sbn = wu->strides[1]; f.prob[1].N = (uint32_t)F;
        for (size_t sl = 0; sl < hbuf.size(); ++sl) {
          f.slot[sl].a16 = (const uint16_t *)xsh->ptr + x->offset;
          f.slot[sl].a_bs = x->strides[0];
          f.slot[sl].h16 = (uint16_t *)hbuf[sl]->ptr;
          d.slot[sl].a16 = (const uint16_t *)hbuf[sl]->ptr;
          d.slot[sl].a_bs = F;
        }
        d.pro = PRO_NONE;
        for (const Member &m : members) d.slot[m.slot].c[0] = (float *)m.c->st->ptr;
        hipError_t e = hipSuccess;
        // the pairs sorted by expert once, for both launches: count, offset (one word per expert), list
        Storage *route = nullptr;
        if (d.n_expert <= MOE_ROUTE_MAX_EXPERTS && H % 64 == 0 && F % 64 == 0) {
          const size_t words = 2 * (size_t)d.n_expert + (size_t)S * d.n_slot;
          st = dev_alloc(be, words * 4, &route);
          if (st) {
            drop_h();
            return st;
          }
          uint32_t *rc = (uint32_t *)route->ptr, *ro = rc + d.n_expert, *rl = ro + d.n_expert;
          {
            KernelScope ks(be, "experts_route", (double)S * d.n_slot * 8, 0);
            e = launch_moe_route(be->lc(), d, rc, ro, rl);
          }
          f.route_count = d.route_count = rc;
          f.route_offset = d.route_offset = ro;
          f.route_list = d.route_list = rl;
        }
        if (e == hipSuccess) {
          KernelScope ks(be, "gemm_experts_bf16", 2.0 * d.n_expert * F * H * 2 + (double)S * H * 2 + (double)d.n_slot * S * F * 2,
                         4.0 * d.n_slot * S * F * H);
          if (be->trace_shapes) ks.rename("gemm_experts_bf16[gate*up]");
          e = launch_moe_gemm(be->lc(), f);
        }
        if (e == hipSuccess) {
          KernelScope ks(be, "gemm_experts_bf16",
                         (double)d.n_expert * d.prob[0].N * F * 2 + (double)d.n_slot * S * (F * 2 + d.prob[0].N * 4),
                         2.0 * d.n_slot * S * d.prob[0].N * F);
          if (be->trace_shapes) ks.rename("gemm_experts_bf16[down]");
          e = launch_moe_gemm(be->lc(), d);
        }
        drop_h();
        storage_release(route);
        if (e != hipSuccess) return fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
        for (const Member &m : members) {
          forget_gemv_candidate(m.c);
          m.c->op = N_REAL;
          drop_inputs(m.c);  // the gate and up products under it were never needed as tensors
        }
        *done = true;
        return CG_OK;
      }
    }
  }
  // input rows
  std::vector<cg_tensor *> held;
  auto drop_held = [&]() {
    for (cg_tensor *t : held) node_release(t);
  };
  if (!glu) {
    cg_tensor *A = n->in[0];
    TRY(realize(be, A));
    if (A->stype != ST_F32 || A->strides[2] != 1 || A->strides[0] % 4 || (uintptr_t)data_ptr(A) % 16) return CG_OK;
    for (size_t sl = 0; sl < slot_idx.size(); ++sl) {
      d.slot[sl].a = (const float *)data_ptr(A);
      d.slot[sl].a_bs = A->strides[0];
    }
  } else {
    for (size_t sl = 0; sl < slot_a.size(); ++sl) {
      cg_tensor *g2 = nullptr, *u2 = nullptr, *gc = nullptr, *uc = nullptr;
      int ge2 = 0;
      if (!match_glu(slot_a[sl], &g2, &u2, &ge2)) {
        drop_held();
        return CG_OK;
      }
      int st = contiguous(be, g2, &gc);
      if (!st) {
        held.push_back(gc);
        st = contiguous(be, u2, &uc);
      }
      if (st) {
        drop_held();
        return st;
      }
      held.push_back(uc);
      if (gc->stype != ST_F32 || uc->stype != ST_F32 || (uintptr_t)data_ptr(gc) % 16 || (uintptr_t)data_ptr(uc) % 16 || K % 4) {
        drop_held();
        return CG_OK;
      }
      d.slot[sl].a = (const float *)data_ptr(gc);
      d.slot[sl].aux = (const float *)data_ptr(uc);
      d.slot[sl].a_bs = d.slot[sl].aux_bs = K;
    }
    // realising gate and up may have run this very function for them; n itself is still deferred
    if (n->op != N_MATMUL) {
      drop_held();
      *done = true;
      return CG_OK;
    }
  }
  double bytes = 0, flops = 0;
  int st = CG_OK;
  for (const Member &m : members) {
    if (m.c->op != N_MATMUL) {  // realised on the way (cannot happen for a complete set; be safe)
      drop_held();
      return CG_OK;
    }
  }
  for (const Member &m : members) {
    st = alloc_result(be, m.c, ST_F32);
    if (st) break;
    d.slot[m.slot].c[m.prob] = (float *)m.c->st->ptr;
    bytes += (double)S * d.prob[m.prob].N * 4;
    flops += 2.0 * S * d.prob[m.prob].N * K;
  }
  if (!st) {
    for (uint32_t p = 0; p < d.n_prob; ++p) bytes += (double)d.n_expert * d.prob[p].N * K * 2;
    bytes += (double)S * K * 4 * (glu ? 2.0 * d.n_slot : 1.0);
    KernelScope ks(be, "gemm_experts_bf16", bytes, flops);
    hipError_t e = launch_moe_gemm(be->lc(), d);
    if (e != hipSuccess) st = fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
  }
  drop_held();
  if (st) return st;
  for (const Member &m : members) {
    forget_gemv_candidate(m.c);
    m.c->op = N_REAL;
    drop_inputs(m.c);
  }
  *done = true;
  return CG_OK;
}

// A decode step's routed experts, all k slots of the layer in one batched launch per stage instead of
// one per slot: gate_proj and up_proj of every (slot, token) pair, then down_proj of every pair with
// the gated activation in its prologue.  The products of a stage share one storage laid out
// [slot][token][N] (each product tensor is a view of its slot's part), which is what lets the second
// stage address its inputs by pair.  Anything that does not fit leaves the slot-by-slot path below.
int try_moe_gemv_slots(cg_backend *be, cg_tensor *n, bool *done) {
  const int64_t S = n->shape[0];
  ExpertOperand eo;
  if (!match_expert_operand(n->in[1], S, &eo)) return CG_OK;
  cg_tensor *A = n->in[0];
  const int64_t K = A->shape[2];
  if (A->rank != 3 || A->shape[0] != S || A->shape[1] != 1 || K % 8 || K < 64 || K > GEMV_PRO_MAX_K || S > 4096) return CG_OK;
  cg_tensor *gate = nullptr, *up = nullptr;
  int gelu = 0;
  const bool glu = A->op != N_REAL && refs(A) == 1 && match_glu(A, &gate, &up, &gelu);
  if (glu) {  // the first stage (this function again, for gate's product) puts every slot's rows in place
    TRY(realize(be, gate));
    TRY(realize(be, up));
    if (n->op != N_MATMUL) return CG_OK;
  }
  struct Member {
    cg_tensor *c, *idx;
    int slot, prob;
  };
  std::vector<Member> members;
  std::vector<cg_tensor *> slot_idx, prob_w;
  auto find_or_add = [](std::vector<cg_tensor *> &v, cg_tensor *t) {
    for (size_t i = 0; i < v.size(); ++i)
      if (v[i] == t) return (int)i;
    v.push_back(t);
    return (int)v.size() - 1;
  };
  std::vector<cg_tensor *> cands{n};
  for (cg_tensor *c : be->gemv_candidates)
    if (c != n) cands.push_back(c);
  Storage *gs = nullptr, *us = nullptr;  // second stage: the storages every slot's gate / up rows live in
  for (cg_tensor *c : cands) {
    if (c->op != N_MATMUL || c->rank != 3 || c->shape[0] != S || c->shape[1] != 1 || c->in[0]->rank != 3 || c->in[0]->shape[2] != K)
      continue;
    ExpertOperand co;
    if (!match_expert_operand(c->in[1], S, &co)) continue;
    if (!glu) {
      if (c->in[0] != A) continue;
      bool known_w = false, known_i = false;
      for (cg_tensor *w : prob_w) known_w = known_w || w == co.w;
      for (cg_tensor *i : slot_idx) known_i = known_i || i == co.idx;
      if ((!known_w && prob_w.size() >= 2) || (!known_i && slot_idx.size() >= 8)) continue;
      members.push_back(Member{c, co.idx, find_or_add(slot_idx, co.idx), find_or_add(prob_w, co.w)});
    } else {
      cg_tensor *g2 = nullptr, *u2 = nullptr;
      int ge2 = 0;
      if (co.w != eo.w || c->in[0]->op == N_REAL || refs(c->in[0]) != 1 || !match_glu(c->in[0], &g2, &u2, &ge2) || ge2 != gelu) continue;
      // rows written by the first stage: dense views of two shared storages, the same slot in both
      if (g2->op != N_REAL || u2->op != N_REAL || g2->stype != ST_F32 || u2->stype != ST_F32 || !is_contiguous(g2) ||
          !is_contiguous(u2) || g2->offset != u2->offset || g2->offset % (S * K))
        continue;
      if (!gs) gs = g2->st, us = u2->st;
      if (g2->st != gs || u2->st != us || gs == us) continue;
      const int slot = (int)(g2->offset / (S * K));
      if (slot >= 8 || members.size() >= 8) continue;
      members.push_back(Member{c, co.idx, slot, 0});
      if (prob_w.empty()) prob_w.push_back(co.w);
    }
  }
  const size_t n_slot = glu ? members.size() : slot_idx.size();
  if (n_slot < 2 || members.size() != n_slot * prob_w.size()) return CG_OK;
  {
    std::vector<int> seen(n_slot * prob_w.size(), 0);
    for (const Member &m : members)
      if (m.slot >= (int)n_slot || seen[m.slot * prob_w.size() + m.prob]++) return CG_OK;
  }
  if (glu && ((size_t)gs->bytes < n_slot * S * K * 4 || (size_t)us->bytes < n_slot * S * K * 4)) return CG_OK;
  bool has_n = false;
  for (const Member &m : members) has_n = has_n || m.c == n;
  if (!has_n) return CG_OK;
  GemvProDesc d;
  std::memset(&d, 0, sizeof(d));
  // indices: u32, one stride between consecutive tokens, the same stride in every slot
  int64_t istride0 = -1;
  for (const Member &m : members) {
    cg_tensor *idx = m.idx;
    TRY(realize(be, idx));
    if (idx->dtype != CG_U32) return CG_OK;
    int64_t istride = 1, expect = -1;
    for (int i = idx->rank - 1; i >= 0; --i) {
      if (idx->shape[i] == 1) continue;
      if (expect < 0) istride = idx->strides[i];
      else if (idx->strides[i] != expect) return CG_OK;
      expect = idx->strides[i] * idx->shape[i];
    }
    if (istride0 >= 0 && istride != istride0) return CG_OK;
    istride0 = istride;
    d.b_index_slot[m.slot] = (const uint32_t *)data_ptr(idx);
  }
  int b_stype = -1;
  for (cg_tensor *w : prob_w) {
    TRY(realize(be, w));
    if (w->rank != 3 || w->shape[2] != K || w->strides[2] != 1 || (w->stype != ST_F32 && w->stype != ST_BF16)) return CG_OK;
    if (b_stype >= 0 && (w->stype != b_stype || w->shape[0] != prob_w[0]->shape[0] || w->strides[0] != prob_w[0]->strides[0]))
      return CG_OK;
    b_stype = w->stype;
    const int q = 16 / esize(w->stype);
    if ((uintptr_t)data_ptr(w) % 16 || w->strides[1] % q || w->strides[0] % q) return CG_OK;
  }
  if (!glu) {
    TRY(realize(be, A));
    if (A->stype != ST_F32 || A->strides[2] != 1 || A->strides[0] % 4 || (uintptr_t)data_ptr(A) % 16) return CG_OK;
    d.pro = PRO_NONE;
    d.a = (const float *)data_ptr(A);
    d.a_bstride = A->strides[0];
    d.a_by_token = 1;
  } else {
    if ((uintptr_t)gs->ptr % 16 || (uintptr_t)us->ptr % 16) return CG_OK;
    d.pro = gelu ? PRO_GEGLU : PRO_SWIGLU;
    d.a = (const float *)gs->ptr;
    d.aux = (const float *)us->ptr;
    d.a_bstride = d.aux_bstride = K;
  }
  d.batch = (uint32_t)(n_slot * S);
  d.slot_tokens = (uint32_t)S;
  d.b_index_stride = istride0;
  d.sb_index = prob_w[0]->strides[0];
  d.b_index_limit = (uint32_t)prob_w[0]->shape[0];
  d.err = be->d_words;
  d.m.K = (uint32_t)K;
  d.m.b_stype = b_stype;
  // one storage per problem, [slot][token][N]
  std::vector<Storage *> outs(prob_w.size(), nullptr);
  auto drop_outs = [&]() {
    for (Storage *o : outs) storage_release(o);
  };
  double bytes = (double)(glu ? 2 * n_slot : 1) * S * K * 4, flops = 0;
  for (size_t p2 = 0; p2 < prob_w.size(); ++p2) {
    cg_tensor *w = prob_w[p2];
    const int64_t N = w->shape[1];
    int st = dev_alloc(be, (size_t)n_slot * S * N * 4, &outs[p2]);
    if (st) {
      drop_outs();
      return st;
    }
    auto &pr = d.m.p[d.m.n_prob++];
    pr.b = data_ptr(w);
    pr.c = (float *)outs[p2]->ptr;
    pr.sbn = w->strides[1];
    pr.N = (uint32_t)N;
    bytes += (double)n_slot * S * N * (K * esize(w->stype) + 4);
    flops += 2.0 * n_slot * S * N * K;
  }
  hipError_t e;
  {
    KernelScope ks(be, b_stype == ST_BF16 ? "gemv_experts_bf16" : "gemv_experts_f32", bytes, flops);
    e = launch_gemv_pro(be->lc(), d);
  }
  if (e != hipSuccess) {
    drop_outs();
    return fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
  }
  for (const Member &m : members) {
    cg_tensor *c = m.c;
    const int64_t N = prob_w[m.prob]->shape[1];
    c->st = outs[m.prob];
    c->st->rc.fetch_add(1);
    c->stype = ST_F32;
    c->offset = (int64_t)m.slot * S * N;
    contiguous_strides(c->rank, c->shape, c->strides);
    forget_gemv_candidate(c);
    c->op = N_REAL;
    drop_inputs(c);
  }
  drop_outs();
  *done = true;
  return CG_OK;
}

int try_moe_gemv(cg_backend *be, cg_tensor *n, bool *done) {
  if (n->rank != 3 || n->shape[1] != 1 || !n->gemv_candidate || n->size() == 0) return CG_OK;
  TRY(try_moe_gemm(be, n, done));
  if (*done) return CG_OK;
  TRY(try_moe_gemv_slots(be, n, done));
  if (*done) return CG_OK;
  const int64_t S = n->shape[0];
  ExpertOperand eo;
  if (!match_expert_operand(n->in[1], S, &eo)) return CG_OK;
  cg_tensor *A = n->in[0];
  const int64_t K = A->shape[2];
  if (A->rank != 3 || K % 8 || K < 64 || K > GEMV_PRO_MAX_K || S > 65535) return CG_OK;
  cg_tensor *gate = nullptr, *up = nullptr;
  int gelu = 0, pro = PRO_NONE;
  if (A->op != N_REAL && refs(A) == 1 && match_glu(A, &gate, &up, &gelu)) pro = gelu ? PRO_GEGLU : PRO_SWIGLU;
  // siblings: other deferred expert products of the same rows by the same indices (gate and up)
  std::vector<cg_tensor *> members{n};
  std::vector<ExpertOperand> ops{eo};
  if (pro == PRO_NONE)
    for (cg_tensor *c : be->gemv_candidates) {
      if (c == n || c->op != N_MATMUL || c->in[0] != A || c->rank != 3 || c->shape[0] != S || members.size() >= 4) continue;
      ExpertOperand co;
      if (!match_expert_operand(c->in[1], S, &co) || co.idx != eo.idx) continue;
      members.push_back(c);
      ops.push_back(co);
    }
  // index vector: one stride between consecutive indices
  cg_tensor *idx = eo.idx;
  TRY(realize(be, idx));
  int64_t istride = 1, expect = -1;
  for (int i = idx->rank - 1; i >= 0; --i) {
    if (idx->shape[i] == 1) continue;
    if (expect < 0) istride = idx->strides[i];
    else if (idx->strides[i] != expect) return CG_OK;
    expect = idx->strides[i] * idx->shape[i];
  }
  if (idx->dtype != CG_U32) return CG_OK;
  int b_stype = -1;
  for (auto &o : ops) {
    cg_tensor *w = o.w;
    TRY(realize(be, w));
    if (w->shape[2] != K || w->strides[2] != 1 || (w->stype != ST_F32 && w->stype != ST_BF16)) return CG_OK;
    if (b_stype >= 0 && (w->stype != b_stype || w->shape[0] != ops[0].w->shape[0] || w->strides[0] != ops[0].w->strides[0]))
      return CG_OK;
    b_stype = w->stype;
    const int q = 16 / esize(w->stype);
    if ((uintptr_t)data_ptr(w) % 16 || w->strides[1] % q || w->strides[0] % q) return CG_OK;
  }
  // input rows
  cg_tensor *a0 = nullptr, *a1 = nullptr;
  int64_t a_bs = 0, aux_bs = 0;
  if (pro == PRO_NONE) {
    TRY(realize(be, A));
    if (A->stype != ST_F32 || A->strides[2] != 1 || A->strides[0] % 4 || (uintptr_t)data_ptr(A) % 16) return CG_OK;
    a0 = retain(A);
    a_bs = A->strides[0];
  } else {
    TRY(contiguous(be, gate, &a0));
    int st = contiguous(be, up, &a1);
    if (st) {
      node_release(a0);
      return st;
    }
    if (a0->stype != ST_F32 || a1->stype != ST_F32 || (uintptr_t)data_ptr(a0) % 16 || (uintptr_t)data_ptr(a1) % 16) {
      node_release(a0);
      node_release(a1);
      return CG_OK;
    }
    a_bs = aux_bs = K;
  }
  GemvProDesc d;
  std::memset(&d, 0, sizeof(d));
  d.pro = pro;
  d.a = (const float *)data_ptr(a0);
  d.aux = a1 ? (const float *)data_ptr(a1) : nullptr;
  d.batch = (uint32_t)S;
  d.a_bstride = a_bs;
  d.aux_bstride = aux_bs;
  d.b_index = (const uint32_t *)data_ptr(idx);
  d.b_index_stride = istride;
  d.sb_index = ops[0].w->strides[0];
  d.b_index_limit = (uint32_t)ops[0].w->shape[0];
  d.err = be->d_words;
  d.m.K = (uint32_t)K;
  d.m.b_stype = b_stype;
  double bytes = (double)S * K * 4 * (pro == PRO_NONE ? 1 : 2), flops = 0;
  int st = CG_OK;
  for (size_t i = 0; i < members.size() && !st; ++i) {
    cg_tensor *w = ops[i].w, *c = members[i];
    st = alloc_result(be, c, ST_F32);
    if (st) break;
    auto &pr = d.m.p[d.m.n_prob++];
    pr.b = data_ptr(w);
    pr.c = (float *)c->st->ptr;
    pr.c_add = nullptr;
    pr.sbn = w->strides[1];
    pr.N = (uint32_t)w->shape[1];
    bytes += (double)S * pr.N * K * esize(w->stype) + (double)S * pr.N * 4;
    flops += 2.0 * S * pr.N * K;
  }
  if (!st) {
    const char *base = b_stype == ST_BF16 ? "gemv_experts_bf16" : "gemv_experts_f32";
    KernelScope ks(be, base, bytes, flops);
    hipError_t e = launch_gemv_pro(be->lc(), d);
    if (e != hipSuccess) st = fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
  }
  node_release(a0);
  node_release(a1);
  if (st) return st;
  for (cg_tensor *c : members) {
    forget_gemv_candidate(c);
    c->op = N_REAL;
    drop_inputs(c);
  }
  *done = true;
  return CG_OK;
}

// `addend` (optional; realised, f32, contiguous, shaped like n) is added in the epilogue when a
// one-row kernel runs the product; *added tells the caller whether that happened.
int realize_matmul(cg_backend *be, cg_tensor *n, cg_tensor *addend, bool *added, MatmulEpilogue *ep) {
  if (!addend && n->dtype == CG_F32 && n->rank == 4 && n->shape[2] == 1 && !(be->flags & CG_FLAG_NO_PATTERNS)) {
    bool done = false;
    TRY(try_attn_decode(be, n, &done));
    if (done) return CG_OK;
  }
  if (!addend && n->dtype == CG_F32 && n->rank == 4 && n->shape[2] >= 16 && !(be->flags & CG_FLAG_NO_PATTERNS)) {
    bool done = false;
    TRY(try_attn_prefill(be, n, &done));
    if (done) return CG_OK;
  }
  if (n->dtype == CG_F32 && n->gemv_candidate && !(be->flags & CG_FLAG_NO_PATTERNS)) {
    bool done = false;
    if (!addend) TRY(try_moe_gemv(be, n, &done));
    if (done) return CG_OK;
    TRY(try_gemv_prologue(be, n, addend, added, &done));
    if (done) return CG_OK;
  }
  MatOperand A, B;
  bool pa = false, pb = false;
  ExpertPeel ex;
  if (n->dtype == CG_F32) TRY(peel_expert_index(be, n, &ex));
  if (ex.w) {
    // B as the kernels see it: [S, K, N] = W[.]^T with the expert axis resolved per batch
    B.set(retain(ex.w));
    B.shape[0] = n->shape[0];
    B.strides[0] = 0;
    B.shape[1] = ex.w->shape[2];
    B.shape[2] = ex.w->shape[1];
    B.strides[1] = ex.w->strides[2];
    B.strides[2] = ex.w->strides[1];
    pb = true;
  } else if (n->dtype == CG_F32 && n->rank == 4) {
    TRY(peel_repeat_kv(be, n->in[1], &B, &pb));
    if (!pb) TRY(peel_repeat_kv(be, n->in[0], &A, &pa));
  }
  if (!pa) {
    TRY(realize(be, n->in[0]));
    A.set(retain(n->in[0]));
  }
  if (!pb) {
    TRY(realize(be, n->in[1]));
    B.set(retain(n->in[1]));
  }
  if (pb && !ex.w) split_heads(&A, B.shape[2]);
  if (pa) split_heads(&B, A.shape[2]);
  const int r = n->rank;
  const uint32_t M = (uint32_t)n->shape[r - 2], N = (uint32_t)n->shape[r - 1],
                 K = (uint32_t)A.shape[A.rank - 1];
  TRY(alloc_result(be, n, n->dtype == CG_F32 ? ST_F32 : ST_U32));
  const int64_t batch = (int64_t)M * N ? n->size() / ((int64_t)M * N) : 0;
  if (n->size() == 0) {
    n->op = N_REAL;
    drop_inputs(n);
    return CG_OK;
  }
  if (n->dtype == CG_U32) {
    cg_tensor *ac = nullptr, *bc = nullptr;
    TRY(contiguous(be, A.t, &ac));
    A.set(ac);
    TRY(contiguous(be, B.t, &bc));
    B.set(bc);
    KernelScope ks(be, "matmul_u32", 0, 2.0 * batch * M * N * K);
    HIPCHK(be, launch_matmul_u32(be->lc(), (const uint32_t *)data_ptr(A.t), (const uint32_t *)data_ptr(B.t),
                                 (uint32_t *)n->st->ptr, (uint32_t)batch, M, N, K));
  } else {
    GemmDesc g;
    std::memset(&g, 0, sizeof(g));
    // an operand with no unit stride in its matrix dims is laid out once (a peeled operand
    // always has one: it is a view of the cache)
    if (!matrix_ok(A) && !pa && !pb) {
      cg_tensor *c = nullptr;
      TRY(materialize(be, A.t, &c, true));
      A.set(c);
    }
    if (!matrix_ok(B) && !pa && !pb) {
      cg_tensor *c = nullptr;
      TRY(materialize(be, B.t, &c, true));
      B.set(c);
    }
    uint32_t nbo[2];
    int64_t sao[2], sbo[2];
    bool ok = matrix_ok(A) && matrix_ok(B) &&
              collapse_batch(A.rank - 2, A.shape, A.strides, B.strides, nbo, sao, sbo);
    if (!ok) {
      // fall back to plain contiguous operands of the logical shapes
      node_release(ex.w);
      ex.w = nullptr;
      cg_tensor *c = nullptr;
      TRY(materialize(be, n->in[0], &c, true));
      A.set(c);
      c = nullptr;
      TRY(materialize(be, n->in[1], &c, true));
      B.set(c);
      if (!collapse_batch(A.rank - 2, A.shape, A.strides, B.strides, nbo, sao, sbo))
        return fail(be, CG_ERR_INTERNAL, "matmul: batch dims do not collapse");
    }
    const int ra = A.rank;
    g.a = data_ptr(A.t);
    g.b = data_ptr(B.t);
    g.c = (float *)n->st->ptr;
    g.a_stype = A.t->stype;
    g.b_stype = B.t->stype;
    // MFMA path in bf16 mode: f32 operands with a unit k stride are read from the bf16 twin of
    // their storage (narrowed once, shared by every GEMM on the same activations)
    if ((be->flags & CG_FLAG_BF16) && M >= 32 && K % 8 == 0) {
      auto twin = [&](MatOperand &o, bool unit_k, const void **ptr, int32_t *stype) -> int {
        Storage *st = o.t->st;
        if (o.t->stype != ST_F32 || !unit_k || st->grow_dim >= 0 || st->bytes % 32) return CG_OK;
        Storage *sh = nullptr;
        TRY(bf16_shadow(be, st, &sh));
        *ptr = (const char *)sh->ptr + o.t->offset * 2;
        *stype = ST_BF16;
        return CG_OK;
      };
      TRY(twin(A, A.strides[ra - 1] == 1, &g.a, &g.a_stype));
      TRY(twin(B, B.strides[ra - 2] == 1 || B.strides[ra - 1] == 1, &g.b, &g.b_stype));
    }
    g.M = M;
    g.N = N;
    g.K = K;
    g.sam = A.strides[ra - 2];
    g.sak = A.strides[ra - 1];
    g.sbk = B.strides[ra - 2];
    g.sbn = B.strides[ra - 1];
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
    // B with unit stride along n (bmm of row-major matrices, p . V): re-laid out once as bf16 [N, K]
    // so that the product takes the direct-to-LDS kernel (one pass over B against K/64 strided ones)
    Storage *bt = nullptr;
    if (g.bf16_math && M >= 64 && N >= 64 && K % 64 == 0 && g.a_stype == ST_BF16 && g.sak == 1 && g.sbn == 1 &&
        g.sbk != 1 && !ex.w && (g.b_stype == ST_F32 || g.b_stype == ST_BF16)) {
      // batches that only repeat (stride 0) are transposed once
      const uint32_t tb0 = g.sb_b0 ? g.nb0 : 1, tb1 = g.sb_b1 ? g.nb1 : 1;
      TRY(dev_alloc(be, (size_t)tb0 * tb1 * N * K * 2, &bt));
      hipError_t te;
      {
        KernelScope ks(be, "transpose_cast_bf16", (double)tb0 * tb1 * N * K * (esize(g.b_stype) + 2), 0);
        te = launch_transpose_cast_bf16(be->lc(), g.b, g.b_stype, bt->ptr, K, N, g.sbk, tb0, tb1, g.sb_b0, g.sb_b1);
      }
      if (te != hipSuccess) {
        storage_release(bt);
        return fail(be, CG_ERR_DEVICE, hipGetErrorString(te));
      }
      g.b = bt->ptr;
      g.b_stype = ST_BF16;
      g.sbk = 1;
      g.sbn = K;
      g.sb_b1 = g.sb_b1 ? (int64_t)N * K : 0;
      g.sb_b0 = g.sb_b0 ? (int64_t)tb1 * N * K : 0;
    }
    if (addend && !be->addend_is_row && M <= 8 && g.a_stype == ST_F32 && K > 0 && (g.sbk == 1 || g.sbn == 1 || K == 1 || N == 1)) {
      g.c_add = (const float *)data_ptr(addend);
      *added = true;
    }
    if (ex.w) {
      g.b_index = (const uint32_t *)data_ptr(ex.idx);
      g.b_index_stride = ex.idx_stride;
      g.sb_index = ex.w->strides[0];
      g.b_index_limit = (uint32_t)ex.w->shape[0];
      g.err = be->d_words;
    }
    if (!g.bf16_math && (g.a_stype == ST_BF16 || g.b_stype == ST_BF16))
      return fail(be, CG_ERR_INTERNAL, "matmul: bf16 storage without CG_FLAG_BF16");
    // bytes: each operand once (batch-broadcast operands once), output once
    auto uniq = [&](const MatOperand &o, const int64_t *sb) {
      double e = (double)o.shape[ra - 2] * o.shape[ra - 1];
      if (sb[0]) e *= nbo[0];
      if (sb[1]) e *= nbo[1];
      return e * esize(o.t->stype);
    };
    // q/k/v and gate/up: other deferred one-row matmuls on the same left operand go out in the
    // same launch (weights are read once either way; the launch ramp is paid once)
    if (M == 1 && batch == 1 && !g.b_index && n->gemv_candidate && g.a_stype == ST_F32 && g.sak == 1 && g.sbk == 1 &&
        K % 8 == 0 && K >= 512 && (uintptr_t)g.a % 16 == 0) {
      auto weight_ok = [&](const void *ptr, int stype, int64_t sbn) {
        return (uintptr_t)ptr % 16 == 0 && sbn % (16 / esize(stype)) == 0;
      };
      GemvMultiDesc md;
      std::memset(&md, 0, sizeof(md));
      std::vector<cg_tensor *> members;
      if (weight_ok(g.b, g.b_stype, g.sbn)) {
        for (cg_tensor *c : std::vector<cg_tensor *>(be->gemv_candidates)) {
          if (c == n || members.size() >= 3 || c->op != N_MATMUL || c->in[0] != n->in[0]) continue;
          cg_tensor *w = c->in[1];
          if (w->op != N_REAL || w->rank != n->rank || w->stype != g.b_stype) continue;
          if (w->shape[w->rank - 2] != (int64_t)K || w->strides[w->rank - 2] != 1) continue;
          bool one_batch = true;
          for (int i = 0; i + 2 < w->rank; ++i) one_batch = one_batch && w->shape[i] == 1;
          if (!one_batch || !weight_ok(data_ptr(w), w->stype, w->strides[w->rank - 1])) continue;
          members.push_back(c);
        }
      }
      if (!members.empty()) {
        md.x = (const float *)g.a;
        md.K = K;
        md.b_stype = g.b_stype;
        md.p[0].b = g.b;
        md.p[0].c = g.c;
        md.p[0].c_add = g.c_add;
        md.p[0].sbn = g.sbn;
        md.p[0].N = N;
        md.n_prob = 1;
        double bytes = uniq(A, sao) + uniq(B, sbo) + (double)n->size() * 4, flops = 2.0 * N * K;
        for (cg_tensor *c : members) {
          cg_tensor *w = c->in[1];
          TRY(alloc_result(be, c, ST_F32));
          auto &pr = md.p[md.n_prob++];
          pr.c_add = nullptr;
          pr.b = data_ptr(w);
          pr.c = (float *)c->st->ptr;
          pr.sbn = w->strides[w->rank - 1];
          pr.N = (uint32_t)w->shape[w->rank - 1];
          bytes += (double)pr.N * K * esize(w->stype) + (double)pr.N * 4;
          flops += 2.0 * pr.N * K;
        }
        {
          KernelScope ks(be, g.b_stype == ST_BF16 ? "gemv_rowdot_bf16" : "gemv_rowdot_f32", bytes, flops);
          if (be->trace_shapes) {
            char buf[96];
            snprintf(buf, sizeof buf, "%s[multi%d,K%u,N%.0f]", g.b_stype == ST_BF16 ? "gemv_rowdot_bf16" : "gemv_rowdot_f32",
                     md.n_prob, K, flops / (2.0 * K));
            ks.rename(buf);
          }
          HIPCHK(be, launch_gemv_multi(be->lc(), md));
        }
        for (cg_tensor *c : members) {
          forget_gemv_candidate(c);
          c->op = N_REAL;
          drop_inputs(c);
        }
        forget_gemv_candidate(n);
        n->op = N_REAL;
        drop_inputs(n);
        return CG_OK;
      }
    }
    // q/k/v of a prefill: the other deferred many-row products on the same left operand join this
    // launch as further column ranges (their own weights, their own outputs)
    std::vector<cg_tensor *> group;
    if (n->gemm_candidate && !addend && !ep && !ex.w && batch == 1 && g.bf16_math && g.a_stype == ST_BF16 &&
        g.b_stype == ST_BF16 && g.sbk == 1 && N % 128 == 0 && gemm_epilogue_ok(g)) {
      // the same rows: one node, or - each linear folding the batch itself - dense reshapes of one value
      auto dense_view = [](const cg_tensor *t, const Storage **st, int64_t *off) {
        const cg_tensor *base = t->op == N_RESHAPE && t->in[0] ? t->in[0] : t;
        if (base->op != N_REAL || !is_contiguous(base) || (t != base && t->size() != base->size())) return false;
        *st = base->st;
        *off = base->offset;
        return true;
      };
      auto same_matrix = [&](const cg_tensor *a, const cg_tensor *b) {
        if (a == b) return true;
        const Storage *sa = nullptr, *sb = nullptr;
        int64_t oa = 0, ob = 0;
        return a->rank == b->rank && std::equal(a->shape, a->shape + a->rank, b->shape) && dense_view(a, &sa, &oa) &&
               dense_view(b, &sb, &ob) && sa == sb && oa == ob;
      };
      for (cg_tensor *c : std::vector<cg_tensor *>(be->gemm_candidates)) {
        if (c == n || group.size() >= 2 || c->op != N_MATMUL || !same_matrix(c->in[0], n->in[0]) || c->rank != n->rank) continue;
        cg_tensor *w = c->in[1];
        if (w->op != N_REAL || w->rank != 3 || w->stype != ST_BF16 || w->shape[0] != 1) continue;
        if (w->shape[1] != (int64_t)K || w->strides[1] != 1 || w->strides[2] != g.sbn) continue;
        if (w->shape[2] % 128 || (uintptr_t)data_ptr(w) % 16) continue;
        group.push_back(c);
      }
      if (group.size() < 2) group.clear();  // pairs (gate / up) keep their own launches and epilogues
    }
    if (!group.empty()) {
      g.n_group = 1;
      g.grp_b[0] = g.b;
      g.grp_c[0] = g.c;
      g.grp_n[0] = N;
      for (cg_tensor *c : group) {
        TRY(alloc_result(be, c, ST_F32));
        g.grp_b[g.n_group] = data_ptr(c->in[1]);
        g.grp_c[g.n_group] = (float *)c->st->ptr;
        g.grp_n[g.n_group] = (uint32_t)c->in[1]->shape[2];
        g.N += g.grp_n[g.n_group];
        ++g.n_group;
      }
    }
    Storage *ws = nullptr;
    const bool dual = ep && ep->dual_w;  // twice the work per tile: no k-slices on top
    const uint32_t splits = group.empty() && !dual ? gemm_split_k(be->lc(), g) : 1;
    if (splits > 1) {
      TRY(dev_alloc(be, (size_t)splits * n->size() * 4, &ws));
      g.workspace = (float *)ws->ptr;
      g.splits = splits;
      g.k_per_split = ((K + splits - 1) / splits + 63) / 64 * 64;
      if (addend && !be->addend_is_row && !g.c_add && !g.b_index) {  // the pass that sums the k-slices adds the residual too
        g.c_add = (const float *)data_ptr(addend);
        *added = true;
      }
    }
    if (dual) {
      if (!g.c_add && batch == 1 && !ex.w && g.sbk == 1 && g.b_stype == ST_BF16 && gemm_epilogue_ok(g)) {
        g.dual_b = g.b;  // this product is up_proj's; the activation goes on the other one
        g.b = data_ptr(ep->dual_w);
        g.glu_kind = ep->gelu;
        // The gated activations are down_proj's operand, which reads them as bf16: store them as bf16
        // only (a later reader of another kind widens them, like a matrix uploaded in this mode).
        storage_release(n->st);
        n->st = nullptr;
        TRY(alloc_result(be, n, ST_BF16));
        g.c = nullptr;
        g.c16 = (uint16_t *)n->st->ptr;
        ep->applied = true;
      }
    } else if (ep && !g.c_add && gemm_epilogue_ok(g)) {
      g.glu_gate = ep->gate;
      g.glu_kind = ep->gelu;
      (void)twin_for_result(be, n, &g.c16);  // the gated activations are down_proj's operand
      ep->applied = true;
    }
    const char *kname = "gemm";
    hipError_t e;
    {
      // grouped: g.N counts every member's columns; B and C bytes scale with it
      // stacked gate / up: two weight matrices read, two products computed
      const double nb = g.dual_b ? 2.0 : 1.0;
      KernelScope ks(be, kname,
                     uniq(A, sao) + (uniq(B, sbo) * nb * (ex.w ? (double)batch : 1.0) + (double)n->size() * 4) * ((double)g.N / N),
                     2.0 * nb * batch * M * g.N * K);
      e = launch_matmul(be->lc(), g, &kname);
      ks.rename(kname);
      if (be->trace_shapes) {  // per-shape records: gemm_mfma_bf16[b32,512x512x64,s1]
        char buf[96];
        snprintf(buf, sizeof buf, "%s[b%lld,%ux%ux%u,s%u%s]", kname, (long long)batch, M, g.N, K, splits,
                 g.dual_b ? ",gate*up" : group.empty() ? "" : ",grouped");
        ks.rename(buf);
      }
    }
    for (cg_tensor *c : group) {
      forget_gemm_candidate(c);
      c->op = N_REAL;
      drop_inputs(c);
    }
    storage_release(ws);
    storage_release(bt);
    HIPCHK(be, e);
  }
  if (n->gemv_candidate) forget_gemv_candidate(n);
  if (n->gemm_candidate) forget_gemm_candidate(n);
  n->op = N_REAL;
  drop_inputs(n);
  return CG_OK;
}

// concat(x, y, dim).  The KV cache grows by `concat(2, cached, new)` once per decode step
// (catgrad-llm/src/legacy/models/utils.rs:210-228): copying the whole cache every step would cost
// O(T) traffic per layer, so a small y appended to a large x gets storage with room to grow along
// `dim`, and when the next concat finds that x is owned by nobody else it writes y in place.
int realize_concat(cg_backend *be, cg_tensor *n) {
  cg_tensor *x = n->in[0], *y = n->in[1];
  TRY(realize(be, x));
  const int dim = (int)n->p0;
  const int64_t xd = x->shape[dim], yd = y->shape[dim];
  const int plain = n->dtype == CG_F32 ? ST_F32 : ST_U32;
  const bool in_place = xd > 0 && yd > 0 && refs(x) == 1 && x->st->rc.load() == 1 && x->st->grow_dim == dim &&
                        xd + yd <= x->st->grow_cap && x->offset == 0 && x->stype == plain && has_grow_layout(x);
  // the new key rows arrive through apply_rope_embedding: rotate them straight into the cache slot
  RopeMatch rope;
  const bool rope_y = in_place && !(be->flags & CG_FLAG_NO_PATTERNS) && y->op != N_REAL && refs(y) == 1 &&
                      n->rank == 4 && dim == 2 && match_rope(y, &rope);
  if (!rope_y) TRY(realize(be, y));
  // (1) append in place
  if (in_place) {
    n->st = x->st;
    n->st->rc.fetch_add(1);
    storage_release(n->st->shadow);  // contents change: any bf16 twin is stale
    n->st->shadow = nullptr;
    n->stype = plain;
    n->offset = 0;
    std::memcpy(n->strides, x->strides, sizeof(n->strides));
    char *dst = (char *)n->st->ptr + xd * n->strides[dim] * 4;
    bool roped = false;
    int st = CG_OK;
    if (rope_y) {
      st = rope_into(be, y, rope, (float *)dst, n->strides, "rope_kv_append", &roped);
      if (!st && !roped) st = realize(be, y);
    }
    if (!st && !roped) st = run_ew(be, y, true, dst, n->strides, plain, "kv_append");
    if (st) {  // still a deferred concat: give the storage reference back
      storage_release(n->st);
      n->st = nullptr;
      return st;
    }
    n->op = N_REAL;
    drop_inputs(n);
    return CG_OK;
  }
  // (2) an append-shaped concat: allocate with capacity along dim
  if (xd > 0 && yd > 0 && yd * 4 <= xd && x->stype != ST_BF16 && y->stype != ST_BF16 &&
      n->size() < ((int64_t)1 << 30)) {
    int64_t cap = 64;
    while (cap < 2 * (xd + yd)) cap <<= 1;
    int64_t cshape[CG_MAX_RANK];
    std::copy(n->shape, n->shape + n->rank, cshape);
    cshape[dim] = cap;
    int64_t total = 1;
    for (int i = 0; i < n->rank; ++i) total *= cshape[i];
    Storage *s = nullptr;
    TRY(dev_alloc(be, (size_t)total * 4, &s));
    s->grow_dim = dim;
    s->grow_cap = cap;
    n->st = s;
    n->stype = plain;
    n->offset = 0;
    contiguous_strides(n->rank, cshape, n->strides);
    s->grow_rank = n->rank;
    std::copy(n->strides, n->strides + n->rank, s->grow_strides);
    TRY(run_ew(be, x, true, s->ptr, n->strides, plain, "ew_concat"));
    char *dst = (char *)s->ptr + xd * n->strides[dim] * 4;
    TRY(run_ew(be, y, true, dst, n->strides, plain, "ew_concat"));
    n->op = N_REAL;
    drop_inputs(n);
    return CG_OK;
  }
  const int keep = (x->stype == ST_BF16 && y->stype == ST_BF16) ? ST_BF16 : plain;
  TRY(alloc_result(be, n, keep));
  if (x->size())
    TRY(run_ew(be, x, true, n->st->ptr, n->strides, keep, "ew_concat"));
  if (y->size()) {
    char *dst = (char *)n->st->ptr + xd * n->strides[dim] * esize(keep);
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
  Program p;
  std::memset(&p, 0, sizeof(p));
  p.n_instr = 1;
  p.seg_end[0] = 1;
  p.code[0].op = E_IOTA;
  p.n_dims = 1;
  p.dims[0] = (uint32_t)n->shape[0];
  OutDesc o;
  std::memset(&o, 0, sizeof(o));
  o.ptr = n->st->ptr;
  o.stype = ST_U32;
  o.stride[0] = 1;
  KernelScope ks(be, "ew_arange", (double)n->size() * 4, 0);
  HIPCHK(be, launch_ew(be->lc(), p, o, (uint64_t)n->size(), false));
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
    case N_MATMUL: return realize_matmul(be, n, nullptr, nullptr, nullptr);
    case N_REDUCE: return realize_reduce(be, n);
    case N_CONCAT: return realize_concat(be, n);
    case N_INDEX: return realize_index(be, n);
  }
  return fail(be, CG_ERR_INTERNAL, "realize: unknown node");
}

// wait for the stream and surface device-side error flags
int sync_and_check(cg_backend *be) {
  HIPCHK(be, hipMemcpyAsync(be->h_words, be->d_words, 8, hipMemcpyDeviceToHost, be->ordered_stream()));
  if (be->queue) HIPCHK(be, be->queue->take_error());  // a launch the queue's thread could not make
  HIPCHK(be, hipStreamSynchronize(be->ordered_stream()));
  cap_pool(be);
  const uint32_t e = be->h_words[0];
  if (e) {
    HIPCHK(be, launch_fill_u32(be->lc(), be->d_words, 0u, 1));
    if (e & ERRF_DIV_ZERO) return fail(be, CG_ERR_ARITH, "attempt to divide by zero");
    if (e & ERRF_INDEX_OOB) return fail(be, CG_ERR_ARG, "index out of bounds");
  }
  return CG_OK;
}

// Structural sharing of values built from constants and aranges only (masks).  Such a node carries
// a key that spells out how it is computed - the op with its parameters and shape, constants by
// value, other inputs by their own keys - so the key stays true after the node is realised and
// after its inputs are gone.  A second request for the same computation gets the same node.
bool share_node(cg_backend *be, cg_tensor *n, cg_tensor **out) {
  if (n->cse_key) return false;
  switch (n->op) {
    case N_BIN: case N_UN: case N_TRANSPOSE: case N_BROADCAST: case N_RESHAPE: case N_SLICE: break;
    case N_CONCAT: break;  // the two halves of a RoPE table
    default: return false;
  }
  std::string key;
  auto put = [&key](const void *p, size_t len) { key.append((const char *)p, len); };
  put(&n->op, 1); put(&n->ew, 1); put(&n->dtype, sizeof n->dtype); put(&n->rank, sizeof n->rank);
  put(n->shape, sizeof(int64_t) * n->rank); put(&n->p0, 8); put(&n->p1, 8); put(&n->cbits, 4);
  for (cg_tensor *in : n->in) {
    if (!in) { key += 'n'; continue; }
    if (in->op == N_CONST) {
      key += 'c';
      put(&in->dtype, sizeof in->dtype); put(&in->cbits, 4); put(&in->rank, sizeof in->rank);
      put(in->shape, sizeof(int64_t) * in->rank);
    } else if (in->cse_key && in->cse_key->size() < 2048) {
      key += '(';
      key += *in->cse_key;
      key += ')';
    } else {
      return false;
    }
  }
  auto it = be->shared_nodes.find(key);
  if (it != be->shared_nodes.end()) {
    *out = retain(it->second);
    node_release(n);
    return true;
  }
  n->const_like = true;
  n->cse_key = new std::string(key);
  if (be->shared_nodes.size() < 4096) {
    be->shared_nodes.emplace(std::move(key), n);
    be->shared_keep.push_back(retain(n));
    if (be->shared_keep.size() > 64) {  // a handful of masks: each may hold S x S floats once realised
      cg_tensor *old = be->shared_keep.front();
      be->shared_keep.pop_front();
      node_release(old);
    }
  }
  return false;
}

int finish(cg_backend *be, cg_tensor *n, cg_tensor **out) {
  if (!(be->flags & CG_FLAG_EAGER) && share_node(be, n, out)) return CG_OK;
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

// the block-closing value noted by the previous call (see `binary`), if any, is realised now
int run_pending_flush(cg_backend *be) {
  cg_tensor *f = be->flush_node;
  if (!f) return CG_OK;
  be->flush_node = nullptr;
  int st = CG_OK;
  if (f->rc.load() > 1 && f->op != N_REAL) {  // somebody still wants it
    hipError_t e = hipSetDevice(be->device);
    st = e == hipSuccess ? realize(be, f) : fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
  }
  node_release(f);
  return st;
}

// realize_view for a node its creator has not handed out yet: on failure the node goes
int realize_view_or_release(cg_backend *be, cg_tensor *n) {
  const int st = realize_view(be, n);
  if (st) node_release(n);
  return st;
}

int check_args(cg_backend *be, cg_tensor *a, cg_tensor *b, void *out) {
  if (!be || !a || !out || (b && b->be != be) || a->be != be)
    return fail(be, CG_ERR_ARG, "null or foreign argument");
  return run_pending_flush(be);
}

int to_shape(cg_backend *be, const size_t *dims, int rank, int64_t *shape) {
  if (rank < 0 || rank > CG_MAX_RANK) return fail(be, CG_ERR_ARG, "rank out of range");
  for (int i = 0; i < rank; ++i) shape[i] = (int64_t)dims[i];
  return CG_OK;
}

uint32_t host_upow(uint32_t a, uint32_t e) {
  uint32_t r = 1;
  while (e) {
    if (e & 1) r *= a;
    a *= a;
    e >>= 1;
  }
  return r;
}

// Exactly specified scalar ops on two host-known constants (IEEE-754 basic operations and
// comparisons, wrapping integer arithmetic).  pow/sin/cos are left to the device.
bool fold_binary(EwOp op, uint32_t a, uint32_t b, uint32_t *out) {
  float x, y, r;
  std::memcpy(&x, &a, 4);
  std::memcpy(&y, &b, 4);
  switch (op) {
    case E_ADD_F: r = x + y; break;
    case E_SUB_F: r = x - y; break;
    case E_MUL_F: r = x * y; break;
    case E_DIV_F: r = x / y; break;
    case E_LT_F: r = x < y ? 1.f : 0.f; break;
    case E_EQ_F: r = x == y ? 1.f : 0.f; break;
    case E_ADD_U: *out = a + b; return true;
    case E_SUB_U: *out = a - b; return true;
    case E_MUL_U: *out = a * b; return true;
    case E_DIV_U: if (!b) return false; *out = a / b; return true;
    case E_POW_U: *out = host_upow(a, b); return true;
    case E_LT_U: *out = a < b ? 1u : 0u; return true;
    case E_EQ_U: *out = a == b ? 1u : 0u; return true;
    default: return false;
  }
  std::memcpy(out, &r, 4);
  return true;
}

cg_tensor *const_node(cg_backend *be, cg_dtype dt, int rank, const int64_t *shape, uint32_t bits);

static cg_tensor *rows_base(cg_tensor *t);

// `other` adds one f32 row vector to every row of `like`'s shape: a deferred broadcast of a rank-1
// tensor (the vector is returned), or - what a broadcast of a value already in memory is - a view
// whose every stride but the last is zero (the view itself is returned: its first row is the
// vector).  Null otherwise.
cg_tensor *bias_vector_of(cg_tensor *other, const cg_tensor *like) {
  if (other->dtype != CG_F32 || other->rank != like->rank || like->rank < 1 ||
      !std::equal(other->shape, other->shape + other->rank, like->shape))
    return nullptr;
  const int r = other->rank;
  if (other->op == N_BROADCAST) {
    cg_tensor *v = other->in[0];
    return v && v->rank == 1 && v->shape[0] == like->shape[r - 1] ? v : nullptr;
  }
  if (other->op != N_REAL || other->stype != ST_F32 || (other->shape[r - 1] != 1 && other->strides[r - 1] != 1)) return nullptr;
  for (int i = 0; i + 1 < r; ++i)
    if (other->shape[i] != 1 && other->strides[i] != 0) return nullptr;
  return other;  // (with a single row, a bias and a residual are the same thing)
}

// the vector bias_vector_of returned, once realised: N contiguous f32 values at data_ptr
bool bias_vector_ready(const cg_tensor *v) {
  if (v->op != N_REAL || v->stype != ST_F32) return false;
  return v->rank == 1 ? is_contiguous(v) : true;  // the view form was checked when it was recognised
}

int binary(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **out, EwOp f_op, EwOp u_op) {
  TRY(check_args(be, a, b, out));
  if (!b) return fail(be, CG_ERR_ARG, "null argument");
  if (a->dtype != b->dtype) return fail(be, CG_ERR_DTYPE, "binary op: dtype mismatch");
  if (a->rank != b->rank || !std::equal(a->shape, a->shape + a->rank, b->shape))
    return fail(be, CG_ERR_SHAPE, "Shape mismatch in operation: " + shape_str(a->shape, a->rank) +
                                      " vs " + shape_str(b->shape, b->rank));
  uint32_t folded;
  if (a->op == N_CONST && b->op == N_CONST &&
      fold_binary(a->dtype == CG_F32 ? f_op : u_op, a->cbits, b->cbits, &folded))
    return finish(be, const_node(be, a->dtype, a->rank, a->shape, folded), out);
  cg_tensor *n = new_node(be, a->dtype, a->rank, a->shape);
  n->op = N_BIN;
  n->ew = a->dtype == CG_F32 ? f_op : u_op;
  n->in[0] = retain(a);
  n->in[1] = retain(b);
  // `residual + linear(...)` over many rows (models/llama.rs:166-186 at prefill sizes) closes a block:
  // everything the block computes has been recorded, nothing fuses across this add, and the next block
  // takes a millisecond to record.  Realising it now starts the device on this block while the
  // caller records the next one.  One-row steps (decode) stay deferred: there the caller overlaps
  // whole steps.  A broadcast operand (a bias) is not a residual, nor is a value that is still deferred.
  // With a launch thread the same holds for the few rows of a decode step: the block's kernels are
  // handed over now and reach the runtime while this thread records the next block.
  bool block_end = false;
  if (n->ew == E_ADD_F && n->rank == 3 && (n->shape[1] >= 64 || be->queue) && !(be->flags & (CG_FLAG_EAGER | CG_FLAG_NO_PATTERNS))) {
    for (int side = 0; side < 2 && !block_end; ++side) {
      const cg_tensor *mm = n->in[side], *other = n->in[1 - side];
      if (mm->op == N_RESHAPE) mm = mm->in[0];  // batch folded into the rows for the linear and unfolded again
      // the residual stream is a value in memory (the previous block end); anything still deferred
      // on the other side may be part of a pattern around the product (gelu's x + c x^3)
      if (mm->op != N_MATMUL || other->op != N_REAL) continue;
      bool dense = true;
      for (int i = 0; i < other->rank; ++i) dense = dense && (other->shape[i] == 1 || other->strides[i] != 0);
      // a few-row product with siblings on the same rows (q/k/v, each about to get its bias) is the
      // middle of a block: the siblings' adds are not recorded yet
      if (dense && mm->gemv_candidate)
        for (const cg_tensor *c : be->gemv_candidates)
          if (c != mm && c->op == N_MATMUL && rows_base(c->in[0]) == rows_base(mm->in[0])) dense = false;
      block_end = dense;
    }
  }
  // `linear(x) + bias` on a few rows: the product's launch can add the bias itself (try_gemv_prologue)
  if (n->ew == E_ADD_F && !(be->flags & (CG_FLAG_EAGER | CG_FLAG_NO_PATTERNS))) {
    for (int side = 0; side < 2; ++side) {
      cg_tensor *mm = n->in[side], *other = n->in[1 - side];
      if (mm->op == N_MATMUL && mm->gemv_candidate && !mm->bias_user && bias_vector_of(other, n) != nullptr) {
        mm->bias_user = n;
        n->bias_of = mm;
        break;
      }
    }
  }
  TRY(finish(be, n, out));
  if (*out != n) return CG_OK;  // folded or shared: n is gone
  if (block_end && !be->flush_node) be->flush_node = retain(n);
  return CG_OK;
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
    e = hipMemcpyAsync(t->st->ptr, data, n * 4, hipMemcpyHostToDevice, be->ordered_stream());
    if (e == hipSuccess) e = hipStreamSynchronize(be->ordered_stream());
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
      e = hipMemcpyAsync(stage->ptr, (const char *)data + o * 4, c * 4, hipMemcpyHostToDevice, be->ordered_stream());
      if (e != hipSuccess) break;
      Program p;
      std::memset(&p, 0, sizeof(p));
      p.n_instr = 1;
      p.seg_end[0] = 1;
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
      if (e == hipSuccess) e = hipStreamSynchronize(be->ordered_stream());
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
  if (x->host_copy) {  // prefetched: wait for that copy only, not for work queued behind it
    HIPCHK(be, hipEventSynchronize(x->host_ev));
    const uint32_t *words = (const uint32_t *)((const char *)x->host_copy + PREFETCH_BYTES - 8);
    if (words[0] == 0) {
      std::memcpy(dst, x->host_copy, n * 4);
      return CG_OK;
    }
    // a kernel flagged an error: take the synchronising path, which reports it
  }
  cg_tensor *c = nullptr;
  TRY(contiguous(be, x, &c));
  int st = CG_OK;
  if (n) {
    hipError_t e = hipMemcpyAsync(dst, data_ptr(c), n * 4, hipMemcpyDeviceToHost, be->ordered_stream());
    if (e != hipSuccess) st = fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
  }
  if (!st) st = sync_and_check(be);
  node_release(c);
  return st;
}

}  // namespace

namespace cgrt {

// The generic (program-prologue) path of realize_reduce on memory the caller brings: `x` and `out` are
// realised tensors, `scratch` receives the per-chunk accumulators when the rows are split over several
// workgroups (3 words per chunk).  Calls no allocator; traced launches are not recorded.
int reduce_into(cg_backend *be, int kind, cg_tensor *x, cg_tensor *out, uint32_t *scratch, size_t scratch_bytes) {
  Region reg;
  EwCompiler c(be, &reg);
  TRY(c.load(c.final_code, x, 0));
  c.flatten();
  std::vector<int64_t> ostr;
  TRY(finish_program(be, c, x->rank, x->shape, nullptr, true, ostr, nullptr));
  const int64_t cols = x->shape[x->rank - 1];
  const int64_t rows = x->size() / cols;
  const uint32_t chunks = reduce_split_chunks(be->lc(), (uint32_t)rows, (uint32_t)cols);
  if (chunks > 1 && (size_t)rows * chunks * 3 * 4 > scratch_bytes)
    return fail(be, CG_ERR_ARG, "reduction of " + std::to_string(rows) + " rows in " + std::to_string(chunks) +
                                    " chunks needs " + std::to_string((size_t)rows * chunks * 12) +
                                    " bytes of scratch, above the fixed " + std::to_string(scratch_bytes));
  be->launches++;
  LaunchCtx lc = be->lc();
  lc.ev_start = lc.ev_stop = nullptr;
  HIPCHK(be, launch_reduce(lc, kind, c.p, data_ptr(out), (uint32_t)rows, (uint32_t)cols, cols % 4 == 0 && cols >= 4,
                           chunks > 1 ? scratch : nullptr, chunks));
  return CG_OK;
}

int fail_with(cg_backend *be, int code, const std::string &msg) { return fail(be, code, msg); }
bool tensor_is_contiguous(const cg_tensor *t) { return is_contiguous(t); }

}  // namespace cgrt

extern "C" {

int cg_backend_create(int device, uint32_t flags, cg_backend **out) {
  if (!out) return CG_ERR_ARG;
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || device < 0 || device >= count) {
    (void)hipGetLastError();
    return CG_ERR_DEVICE;
  }
  if (hipSetDevice(device) != hipSuccess) return CG_ERR_DEVICE;
  if (cgrt::noalloc_init_device(device) != CG_OK) return CG_ERR_DEVICE;
  cg_backend *be = new cg_backend();
  static std::atomic<uint64_t> next_uid{1};
  be->uid = next_uid.fetch_add(1);
  be->device = device;
  be->flags = flags;
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, device) == hipSuccess) be->n_cus = prop.multiProcessorCount;
  if (hipStreamCreate(&be->stream) != hipSuccess || hipMalloc((void **)&be->d_words, 256) != hipSuccess ||
      hipHostMalloc((void **)&be->h_words, 256, hipHostMallocDefault) != hipSuccess ||
      hipMemsetAsync(be->d_words, 0, 256, be->ordered_stream()) != hipSuccess ||
      hipStreamSynchronize(be->ordered_stream()) != hipSuccess) {
    delete be;
    return CG_ERR_DEVICE;
  }
  // deferred evaluation issues kernels in bursts: a second thread makes the runtime calls
  if (!(flags & CG_FLAG_EAGER)) be->queue = new cgk::LaunchQueue(device);
  *out = be;
  return CG_OK;
}

void cg_backend_destroy(cg_backend *be) {
  if (!be) return;
  // cached nodes hold references to the backend: drop them first
  std::map<int64_t, cg_tensor *> cache;
  cache.swap(be->arange_cache);
  for (auto &kv : cache) node_release(kv.second);
  std::deque<cg_tensor *> keep;
  keep.swap(be->shared_keep);
  for (cg_tensor *t : keep) node_release(t);
  if (be->flush_node) {
    cg_tensor *f = be->flush_node;
    be->flush_node = nullptr;
    node_release(f);
  }
  backend_release(be);
}
const char *cg_last_error(const cg_backend *be) { return be ? be->err.c_str() : ""; }
const char *cg_backend_name(const cg_backend *) { return "hip-gfx950"; }

int cg_sync(cg_backend *be) {
  if (!be) return CG_ERR_ARG;
  HIPCHK(be, hipSetDevice(be->device));
  return sync_and_check(be);
}

int cg_tensor_prefetch(cg_backend *be, cg_tensor *t) {
  if (!be || !t || t->be != be) return CG_ERR_ARG;
  HIPCHK(be, hipSetDevice(be->device));
  TRY(realize(be, t));
  const size_t bytes = (size_t)t->size() * 4;
  if (t->host_copy || bytes == 0 || bytes > PREFETCH_BYTES - 8 || esize(t->stype) != 4 || !is_contiguous(t))
    return CG_OK;  // the read will take the synchronising path
  void *buf = nullptr;
  hipEvent_t ev = nullptr;
  if (!be->pinned_pool.empty()) {
    buf = be->pinned_pool.back();
    be->pinned_pool.pop_back();
  } else {
    HIPCHK(be, hipHostMalloc(&buf, PREFETCH_BYTES, hipHostMallocDefault));
  }
  if (!be->event_pool.empty()) {
    ev = be->event_pool.back();
    be->event_pool.pop_back();
  } else if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) {
    be->pinned_pool.push_back(buf);
    return fail(be, CG_ERR_DEVICE, "hipEventCreate failed");
  }
  hipError_t e = hipMemcpyAsync(buf, data_ptr(t), bytes, hipMemcpyDeviceToHost, be->ordered_stream());
  if (e == hipSuccess)
    e = hipMemcpyAsync((char *)buf + PREFETCH_BYTES - 8, be->d_words, 8, hipMemcpyDeviceToHost, be->ordered_stream());
  if (e == hipSuccess) e = hipEventRecord(ev, be->ordered_stream());
  if (e != hipSuccess) {
    be->pinned_pool.push_back(buf);
    be->event_pool.push_back(ev);
    return fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
  }
  t->host_copy = buf;
  t->host_ev = ev;
  return CG_OK;
}

int cg_tensor_realize(cg_backend *be, cg_tensor *t) {
  if (!be || !t || t->be != be) return CG_ERR_ARG;
  HIPCHK(be, hipSetDevice(be->device));
  return realize(be, t);
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

// An F32 tensor from bf16 bit patterns (the widening of examples/llama/main.rs:309-312 done on the
// device).  In bf16 mode a tensor of rank >= 2 keeps the bits as its storage.
int cg_from_bf16(cg_backend *be, const uint16_t *bits, size_t n, const size_t *dims, int rank, cg_tensor **out) {
  if (!be || !out || (!bits && n)) return fail(be, CG_ERR_ARG, "null argument");
  int64_t shape[CG_MAX_RANK];
  TRY(to_shape(be, dims, rank, shape));
  int64_t sz = 1;
  for (int i = 0; i < rank; ++i) sz *= shape[i];
  if ((int64_t)n != sz) return fail(be, CG_ERR_SHAPE, "ShapeError");
  if (n == 1) return finish(be, const_node(be, CG_F32, rank, shape, (uint32_t)bits[0] << 16), out);
  HIPCHK(be, hipSetDevice(be->device));
  cg_tensor *t = new_node(be, CG_F32, rank, shape);
  const bool keep = rank >= 2 && (be->flags & CG_FLAG_BF16);
  int st = alloc_result(be, t, keep ? ST_BF16 : ST_F32);
  if (st) {
    node_release(t);
    return st;
  }
  hipError_t e = hipSuccess;
  if (n == 0) {
  } else if (keep) {
    e = hipMemcpyAsync(t->st->ptr, bits, n * 2, hipMemcpyHostToDevice, be->ordered_stream());
    if (e == hipSuccess) e = hipStreamSynchronize(be->ordered_stream());
  } else {
    const size_t chunk = (size_t)16 << 20;  // elements per staged piece
    Storage *stage = nullptr;
    st = dev_alloc(be, std::min(n, chunk) * 2, &stage);
    if (st) {
      node_release(t);
      return st;
    }
    for (size_t o = 0; o < n && e == hipSuccess; o += chunk) {
      const size_t c = std::min(chunk, n - o);
      e = hipMemcpyAsync(stage->ptr, bits + o, c * 2, hipMemcpyHostToDevice, be->ordered_stream());
      if (e != hipSuccess) break;
      Program p;
      std::memset(&p, 0, sizeof(p));
      p.n_instr = 1;
      p.seg_end[0] = 1;
      p.code[0].op = E_LOAD;
      p.n_in = 1;
      p.n_dims = 1;
      p.dims[0] = (uint32_t)c;
      p.in[0].ptr = stage->ptr;
      p.in[0].stride[0] = 1;
      p.in[0].stype = ST_BF16;
      p.in[0].vec = 1;
      OutDesc od;
      std::memset(&od, 0, sizeof(od));
      od.ptr = (char *)t->st->ptr + o * 4;
      od.stype = ST_F32;
      od.stride[0] = 1;
      KernelScope ks(be, "ew_from_bf16", (double)c * 6, 0);
      e = launch_ew(be->lc(), p, od, c, c % 4 == 0);
      if (e == hipSuccess) e = hipStreamSynchronize(be->ordered_stream());
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

// [n, ...] from n tensors of one shape (the stacked experts of examples/llama/main.rs:217-236): one
// allocation, n device copies.  Parts that are all dense in one storage type keep it (bf16 weights
// stay bf16); otherwise every part is first written out as plain f32 / u32.
int cg_stack(cg_backend *be, cg_tensor *const *parts, size_t n, cg_tensor **out) {
  if (!be || !parts || !out || n == 0) return fail(be, CG_ERR_ARG, "null argument or nothing to stack");
  for (size_t i = 0; i < n; ++i) {
    if (!parts[i] || parts[i]->be != be) return fail(be, CG_ERR_ARG, "null tensor or tensor of another backend");
    if (parts[i]->dtype != parts[0]->dtype) return fail(be, CG_ERR_DTYPE, "stack: mixed dtypes");
    if (parts[i]->rank != parts[0]->rank) return fail(be, CG_ERR_SHAPE, "stack: Shape mismatch");
    for (int d = 0; d < parts[0]->rank; ++d)
      if (parts[i]->shape[d] != parts[0]->shape[d]) return fail(be, CG_ERR_SHAPE, "stack: Shape mismatch");
  }
  if (parts[0]->rank + 1 > CG_MAX_RANK) return fail(be, CG_ERR_SHAPE, "stack: rank too large");
  HIPCHK(be, hipSetDevice(be->device));
  std::vector<cg_tensor *> dense(n, nullptr);
  auto drop = [&]() {
    for (cg_tensor *t : dense)
      if (t) node_release(t);
  };
  bool same = true;
  for (size_t i = 0; i < n; ++i) {
    int st = realize(be, parts[i]);
    if (st) return st;
    same = same && is_contiguous(parts[i]) && parts[i]->stype == parts[0]->stype;
  }
  for (size_t i = 0; i < n; ++i) {
    if (same) {
      dense[i] = retain(parts[i]);
    } else {
      int st = contiguous(be, parts[i], &dense[i]);
      if (st) {
        drop();
        return st;
      }
    }
  }
  int64_t shape[CG_MAX_RANK];
  shape[0] = (int64_t)n;
  for (int d = 0; d < parts[0]->rank; ++d) shape[d + 1] = parts[0]->shape[d];
  cg_tensor *t = new_node(be, parts[0]->dtype, parts[0]->rank + 1, shape);
  int st = alloc_result(be, t, dense[0]->stype);
  if (st) {
    node_release(t);
    drop();
    return st;
  }
  const size_t each = (size_t)parts[0]->size() * esize(dense[0]->stype);
  hipError_t e = hipSuccess;
  for (size_t i = 0; i < n && e == hipSuccess && each; ++i)
    e = hipMemcpyAsync((char *)t->st->ptr + i * each, data_ptr(dense[i]), each, hipMemcpyDeviceToDevice, be->ordered_stream());
  drop();
  if (e != hipSuccess) {
    node_release(t);
    return fail(be, CG_ERR_DEVICE, std::string("stack: ") + hipGetErrorString(e));
  }
  *out = t;
  return CG_OK;
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
  // one input row per batch, or the rows of a small batch folded into one matrix ([1, B, K])
  const bool few_rows = shape[a->rank - 2] == 1 || (a->rank == 3 && shape[0] == 1 && shape[1] <= 4);
  if (a->dtype == CG_F32 && few_rows && !(be->flags & CG_FLAG_EAGER)) {
    if (be->gemv_candidates.size() >= 4096) forget_gemv_candidate(be->gemv_candidates.front());
    be->gemv_candidates.push_back(n);
    n->gemv_candidate = true;
  }
  if (a->dtype == CG_F32 && a->rank == 3 && shape[0] == 1 && shape[1] >= 64 && (be->flags & CG_FLAG_BF16) &&
      !(be->flags & (CG_FLAG_EAGER | CG_FLAG_NO_PATTERNS))) {
    if (be->gemm_candidates.size() >= 1024) forget_gemm_candidate(be->gemm_candidates.front());
    be->gemm_candidates.push_back(n);
    n->gemm_candidate = true;
  }
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
  if (x->op == N_CONST)
    return finish(be, const_node(be, x->dtype, x->rank, x->shape,
                                 x->dtype == CG_F32 ? x->cbits ^ 0x80000000u : 0u - x->cbits), out);
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
  if (!(be->flags & CG_FLAG_EAGER) && share_node(be, n, out)) return CG_OK;
  if (x->op == N_REAL) TRY(realize_view_or_release(be, n));
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
  if (!(be->flags & CG_FLAG_EAGER) && share_node(be, n, out)) return CG_OK;
  // a reshape that is a pure view of realised data costs nothing: do it now
  int64_t tmp[CG_MAX_RANK];
  if (x->op == N_REAL && (sz == 0 || try_reshape_view(x->rank, x->shape, x->strides, rank, shape, tmp)))
    TRY(realize_view_or_release(be, n));
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
  if (!(be->flags & CG_FLAG_EAGER) && share_node(be, n, out)) return CG_OK;
  if (x->op == N_REAL) TRY(realize_view_or_release(be, n));
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
  // The router of a MoE layer: topk(softmax(logits)) where nobody else reads the probabilities (the
  // caller's handle is the only reference) - both in one launch, the probabilities never stored.
  cg_tensor *c = nullptr;
  bool router = false;
  SoftmaxMatch sm;
  if (x->op != N_REAL && !(be->flags & (CG_FLAG_EAGER | CG_FLAG_NO_PATTERNS)) && refs(x) == 1 && n <= 256 && n > 0 &&
      match_softmax(x, &sm) && !sm.has_scale && !sm.has_mask_const && !sm.mask && sm.src == sm.x) {
    TRY(contiguous(be, sm.src, &c));
    router = c->stype == ST_F32;
    if (!router) {
      node_release(c);
      c = nullptr;
    }
  }
  if (!router) TRY(contiguous(be, x, &c));
  int64_t shape[CG_MAX_RANK];
  std::copy(x->shape, x->shape + x->rank, shape);
  shape[x->rank - 1] = (int64_t)k;
  cg_tensor *v = new_node(be, CG_F32, x->rank, shape), *ix = new_node(be, CG_U32, x->rank, shape);
  int st = alloc_result(be, v, ST_F32);
  if (!st) st = alloc_result(be, ix, ST_U32);
  if (!st) {
    const int64_t rows = n ? x->size() / n : 0;
    KernelScope ks(be, router ? "softmax_topk" : "topk", (double)x->size() * 4, 0);
    hipError_t e = router ? launch_softmax_topk(be->lc(), (const float *)data_ptr(c), n, (float *)v->st->ptr,
                                                (uint32_t *)ix->st->ptr, (uint32_t)rows, (uint32_t)n, (uint32_t)k)
                          : launch_topk(be->lc(), (const float *)data_ptr(c), (float *)v->st->ptr, (uint32_t *)ix->st->ptr,
                                        (uint32_t)rows, (uint32_t)n, (uint32_t)k);
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
  if (!(be->flags & CG_FLAG_EAGER) && share_node(be, n, out)) return CG_OK;
  if (x->op == N_REAL) TRY(realize_view_or_release(be, n));
  return finish(be, n, out);
}

// ndarray.rs:91-95
int cg_arange(cg_backend *be, size_t end, cg_tensor **out) {
  if (!be || !out) return CG_ERR_ARG;
  int64_t shape[1] = {(int64_t)end};
  if (end == 1) return finish(be, const_node(be, CG_U32, 1, shape, 0u), out);
  if (!(be->flags & CG_FLAG_EAGER) && end <= ((size_t)1 << 20)) {
    auto it = be->arange_cache.find((int64_t)end);
    if (it != be->arange_cache.end()) {
      *out = retain(it->second);
      return CG_OK;
    }
    if (be->arange_cache.size() < 32) {
      cg_tensor *n = new_node(be, CG_U32, 1, shape);
      n->op = N_ARANGE;
      n->const_like = true;
      n->cse_key = new std::string("arange" + std::to_string(end));
      be->arange_cache[(int64_t)end] = retain(n);
      return finish(be, n, out);
    }
  }
  cg_tensor *n = new_node(be, CG_U32, 1, shape);
  n->op = N_ARANGE;
  return finish(be, n, out);
}

// ndarray.rs:46-51
int cg_to_f32(cg_backend *be, cg_tensor *x, float *dst, size_t n) { return download(be, x, dst, n, CG_F32); }
int cg_to_u32(cg_backend *be, cg_tensor *x, uint32_t *dst, size_t n) { return download(be, x, dst, n, CG_U32); }

// ---- peak probes (measured denominators; nothing in the product depends on them) ------------------
int cg_peak_copy_gbs(cg_backend *be, size_t bytes, int iters, double *gbs) {
  if (!be || !gbs || bytes < 4096 || iters < 1) return CG_ERR_ARG;
  HIPCHK(be, hipSetDevice(be->device));
  bytes &= ~(size_t)4095;
  Storage *a = nullptr, *b = nullptr;
  TRY(dev_alloc(be, bytes, &a));
  int st = dev_alloc(be, bytes, &b);
  if (st) {
    storage_release(a);
    return st;
  }
  hipEvent_t e0 = nullptr, e1 = nullptr;
  hipError_t e = hipEventCreate(&e0);
  if (e == hipSuccess) e = hipEventCreate(&e1);
  LaunchCtx lc = be->lc();
  lc.ev_start = lc.ev_stop = nullptr;
  if (e == hipSuccess) e = launch_fill_u32(lc, (uint32_t *)a->ptr, 0x3F800000u, bytes / 4);
  if (e == hipSuccess) e = launch_peak_copy(lc, a->ptr, b->ptr, bytes);  // warm-up
  if (e == hipSuccess) e = hipEventRecord(e0, be->ordered_stream());
  for (int i = 0; i < iters && e == hipSuccess; ++i) e = launch_peak_copy(lc, a->ptr, b->ptr, bytes);
  if (e == hipSuccess) e = hipEventRecord(e1, be->ordered_stream());
  if (e == hipSuccess) e = hipStreamSynchronize(be->ordered_stream());
  float ms = 0.f;
  if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  storage_release(a);
  storage_release(b);
  if (e != hipSuccess) return fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
  *gbs = 2.0 * (double)bytes * iters / (ms * 1e-3) / 1e9;  // read + write
  return CG_OK;
}

int cg_peak_mfma_tflops(cg_backend *be, cg_dtype operand, int iters, double *tflops) {
  if (!be || !tflops || iters < 1) return CG_ERR_ARG;
  HIPCHK(be, hipSetDevice(be->device));
  const int bf16 = operand != CG_F32;  // CG_F32: v_mfma_f32_32x32x2_f32; otherwise bf16 32x32x16
  const unsigned grid = (unsigned)be->n_cus * 8;
  Storage *o = nullptr;
  TRY(dev_alloc(be, (size_t)grid * 256 * 4, &o));
  hipEvent_t e0 = nullptr, e1 = nullptr;
  hipError_t e = hipEventCreate(&e0);
  if (e == hipSuccess) e = hipEventCreate(&e1);
  LaunchCtx lc = be->lc();
  lc.ev_start = lc.ev_stop = nullptr;
  if (e == hipSuccess) e = launch_peak_mfma(lc, bf16, (float *)o->ptr, grid, 64);
  if (e == hipSuccess) e = hipEventRecord(e0, be->ordered_stream());
  if (e == hipSuccess) e = launch_peak_mfma(lc, bf16, (float *)o->ptr, grid, iters);
  if (e == hipSuccess) e = hipEventRecord(e1, be->ordered_stream());
  if (e == hipSuccess) e = hipStreamSynchronize(be->ordered_stream());
  float ms = 0.f;
  if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  storage_release(o);
  if (e != hipSuccess) return fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
  const double k = bf16 ? 16.0 : 2.0;
  *tflops = (double)grid * 4 * iters * 4 * (2.0 * 32 * 32 * k) / (ms * 1e-3) / 1e12;
  return CG_OK;
}

int cg_trace_enable(cg_backend *be, int on) {
  if (!be) return CG_ERR_ARG;
  trace_collect(be);
  be->trace = on != 0;
  be->trace_shapes = on == 2;
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
size_t cg_launch_counts(cg_backend *be, int reset, char *buf, size_t cap) {
  if (!be) return 0;
  std::string out;
  for (auto &kv : be->launch_counts) out += kv.first + " " + std::to_string(kv.second) + "\n";
  if (buf && cap) {
    const size_t n = std::min(cap - 1, out.size());
    std::memcpy(buf, out.data(), n);
    buf[n] = 0;
  }
  if (reset) {
    // the slots stay (KernelScope caches a pointer to the last one): zero them
    for (auto &kv : be->launch_counts) kv.second = 0;
  }
  return out.size() + 1;
}

int cg_stats(cg_backend *be, uint64_t *l, uint64_t *d, uint64_t *p) {
  if (!be) return CG_ERR_ARG;
  if (l) *l = be->launches;
  if (d) *d = be->device_bytes;
  if (p) *p = be->pool_bytes;
  return CG_OK;
}

}  // extern "C"
