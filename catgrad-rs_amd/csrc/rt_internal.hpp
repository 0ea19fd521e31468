// rt_internal.hpp — what the translation units of the host runtime share: error macros, the
// structures of the fusion compiler and of the pattern matchers, and the prototypes of every runtime
// function.  Layout of the runtime:
//   rt_core.cpp      errors, device allocator, node lifetime, stride helpers, launch accounting
//   rt_ew.cpp        fusion regions, the elementwise / row program compiler, views, reductions
//   rt_patterns.cpp  matchers for the op sequences the reference's emitters produce (softmax, RMSNorm,
//                    RoPE, gated activations, residual adds) and their hand-written kernels
//   rt_matmul.cpp    matmul operands (weights read in place, repeat_kv peeled), GEMM / GEMV dispatch,
//                    the fusions around one-row products
//   rt_attention.cpp one-pass attention over many rows and over one query row, the cache append inside it
//   rt_moe.cpp       expert-indirect products: routed experts of a few tokens and of many
//   rt_graph.cpp     concat / index / arange, realisation, shared constant nodes, host transfers
//   rt_abi.cpp       the extern "C" entry points of include/catgrad_hip.h
#pragma once
#include "rt.hpp"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>

namespace cgrt {
using namespace cgk;


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


enum { PREFETCH_BYTES = 4096 };  // pinned buffer of a prefetched tensor: data + 8 bytes of error words
enum : uint32_t { F_ONE = 0x3F800000u, F_HALF = 0x3F000000u, F_E = 0x402DF854u, F_TWO = 0x40000000u };

struct KernelScope;
struct Region;
struct EwCompiler;
struct RowMap;
struct SoftmaxMatch;
struct RmsNormMatch;
struct RopeMatch;
struct RopeNormed;
struct MatmulEpilogue;
struct MatOperand;
struct ExpertPeel;
struct RowAppend;
struct ExpertOperand;

// ---- functions (defined in the file named above their group in the layout)
int fail(cg_backend *be, int code, const std::string &msg);
std::string shape_str(const int64_t *s, int r);
int esize(int stype);
size_t size_class(size_t bytes);
void trim_pool(cg_backend *be);
void cap_pool(cg_backend *be);
int dev_alloc(cg_backend *be, size_t bytes, Storage **out);
void storage_release(Storage *s);
void backend_release(cg_backend *be);
cg_tensor *new_node(cg_backend *be, cg_dtype dt, int rank, const int64_t *shape);
void forget_gemv_candidate(cg_tensor *n);
void forget_gemm_candidate(cg_tensor *n);
void node_release(cg_tensor *t);
cg_tensor *retain(cg_tensor *t);
void forget_shared(cg_tensor *n);
void drop_inputs(cg_tensor *n);
void contiguous_strides(int rank, const int64_t *shape, int64_t *strides);
bool is_contiguous(const cg_tensor *t);
bool try_reshape_view(int ornk, const int64_t *oshape, const int64_t *ostr, int nrnk,
                      const int64_t *nshape, int64_t *nstr);
void trace_collect(cg_backend *be);
int alloc_result(cg_backend *be, cg_tensor *n, int stype);
void *data_ptr(const cg_tensor *t);
bool same_shape(const cg_tensor *a, const cg_tensor *b);
bool is_row_broadcast(const cg_tensor *b, const cg_tensor *root);
bool row_chain_ok(const cg_tensor *r, const cg_tensor *root, int depth = 0);
int prepare_region(cg_backend *be, cg_tensor *root, bool rows, Region &reg);
int collapse_dims(int rank, const int64_t *shape, std::vector<const int64_t *> strides,
                  bool keep_last, uint32_t *dims, std::vector<std::vector<int64_t>> &out);
bool operand_vec_ok(const void *ptr, int stype, const std::vector<int64_t> &st);
int finish_program(cg_backend *be, EwCompiler &c, int rank, const int64_t *shape,
                   const int64_t *out_strides, bool keep_last, std::vector<int64_t> &ostr,
                   double *bytes_in);
int launch_compiled(cg_backend *be, EwCompiler &c, cg_tensor *root, void *dst,
                    const int64_t *dst_strides, int dst_stype, const char *name);
int run_ew(cg_backend *be, cg_tensor *root, bool root_is_value, void *dst, const int64_t *dst_strides,
           int dst_stype, const char *name);
int try_transpose_copy(cg_backend *be, const cg_tensor *src, cg_tensor *dst, bool *done);
int materialize(cg_backend *be, cg_tensor *src, cg_tensor **out, bool keep_bf16 = false);
int contiguous(cg_backend *be, cg_tensor *src, cg_tensor **out);
int realize_const(cg_backend *be, cg_tensor *n);
bool is_bin(const cg_tensor *n, uint8_t ew);
bool is_un(const cg_tensor *n, uint8_t ew);
bool is_constf(const cg_tensor *n, uint32_t bits);
int refs(const cg_tensor *n);
float bits_f(uint32_t b);
bool rows_view(const cg_tensor *t, int64_t *row_stride);
bool rows_map(const cg_tensor *t, RowMap *m);
int gemm_readers(cg_backend *be, const cg_tensor *n, bool *all);
int as_rows(cg_backend *be, cg_tensor *t, cg_tensor **out, int64_t *row_stride);
void finish_fused(cg_tensor *n);
int twin_for_result(cg_backend *be, cg_tensor *n, uint16_t **out);
bool match_softmax(cg_tensor *root, SoftmaxMatch *m);
int try_softmax(cg_backend *be, cg_tensor *root, bool *done);
bool match_rmsnorm(cg_tensor *root, RmsNormMatch *m);
int gamma_row_vector(cg_backend *be, cg_tensor *gb, bool *ok);
int try_rmsnorm_pair(cg_backend *be, cg_tensor *root, const RmsNormMatch &outer, bool *done);
int try_rmsnorm(cg_backend *be, cg_tensor *root, bool *done);
int try_row_scaled_sum(cg_backend *be, cg_tensor *root, bool *done);
bool match_rope(cg_tensor *root, RopeMatch *m);
int rope_tables(cg_backend *be, const RopeMatch &m, bool *ok);
int rope_operands(cg_backend *be, const RopeMatch &m, bool *ok);
int rope_into(cg_backend *be, cg_tensor *root, const RopeMatch &m, float *out, const int64_t *o_strides,
              const char *name, bool *done, uint16_t *out16 = nullptr);
int try_rope(cg_backend *be, cg_tensor *root, bool *done);
int rope_describe(cg_backend *be, cg_tensor *root, const RopeMatch &m, float *out, const int64_t *o_strides,
                  uint16_t *out16, RopeDesc *dsc, cg_tensor **xs_out, bool *ok, const RopeNormed *normed = nullptr);
int try_rope_pair(cg_backend *be, cg_tensor *rq, cg_tensor *rk, bool *done);
int try_qkv_rope_gemm(cg_backend *be, cg_tensor *rq, cg_tensor *rk, cg_tensor *v, Storage **vt, const Storage **v_st,
                      bool *done);
cg_tensor *node_under_repeat_kv(cg_tensor *t);
bool is_sigmoid_of(const cg_tensor *s, const cg_tensor **arg);
bool is_gelu_of(const cg_tensor *g, const cg_tensor **arg);
bool match_glu(cg_tensor *root, cg_tensor **gate, cg_tensor **up, int *gelu);
cg_tensor *glu_gate_of(const cg_tensor *root);
bool same_rows(const cg_tensor *a, const cg_tensor *b);
int try_glu(cg_backend *be, cg_tensor *root, bool *done);
int try_gemv_add(cg_backend *be, cg_tensor *root, bool *done);
int try_binary(cg_backend *be, cg_tensor *root, bool *done);
int try_patterns(cg_backend *be, cg_tensor *root, bool *done);
int realize_ew(cg_backend *be, cg_tensor *n);
int realize_view(cg_backend *be, cg_tensor *n);
bool rows_layout(const cg_tensor *t, int64_t *row_stride);
int realize_reduce(cg_backend *be, cg_tensor *n);
bool collapse_batch(int nb, const int64_t *bshape, const int64_t *sa, const int64_t *sb,
                    uint32_t *nbo, int64_t *sao, int64_t *sbo);
int peel_repeat_kv(cg_backend *be, cg_tensor *t, MatOperand *out, bool *peeled);
void split_heads(MatOperand *o, int64_t rep);
bool matrix_ok(const MatOperand &o);
int bf16_shadow(cg_backend *be, Storage *st, Storage **out);
int peel_expert_index(cg_backend *be, cg_tensor *n, ExpertPeel *out);
int try_attn_prefill(cg_backend *be, cg_tensor *n, bool *done);
int attn_decode_scratch(cg_backend *be, size_t part_floats, size_t count_words);
bool has_grow_layout(const cg_tensor *x);
cg_tensor *kv_concat_under(cg_tensor *t);
int row_append_candidate(cg_backend *be, cg_tensor *c, bool allow_rope, RowAppend *out, bool *ok);
void commit_row_append(cg_tensor *c);
int write_row_append(cg_backend *be, const RowAppend &ra);
// later (optional): when the launch divides the keys over workgroups and the caller can merge the
// partials itself (launch_gemv_pro with PRO_ATTN_MERGE), the attention stops at its partials, *later
// describes them and n's own storage is left unwritten.
struct AttnMergeLater {
  const float *part = nullptr;
  uint32_t splits = 0, heads = 0, d = 0;
  bool deferred = false;
};
int try_attn_decode(cg_backend *be, cg_tensor *n, bool *done, AttnMergeLater *later = nullptr);
int try_gemv_attn_merge(cg_backend *be, cg_tensor *n, cg_tensor *addend, bool *added, bool *done);
cg_tensor *rows_base(cg_tensor *t);
int try_gate_up_glu(cg_backend *be, cg_tensor *glu, cg_tensor *g, cg_tensor *u, int gelu, bool *done);
bool norm_row_readers_ok(cg_backend *be, cg_tensor *base, cg_tensor *view, RmsNormMatch *rm);
int try_gemv_prologue(cg_backend *be, cg_tensor *n, cg_tensor *addend, bool *added, bool *done);
bool match_expert_operand(const cg_tensor *t, int64_t S, ExpertOperand *o);
int try_moe_gemm(cg_backend *be, cg_tensor *n, bool *done);
int try_moe_gemv_slots(cg_backend *be, cg_tensor *n, bool *done);
int try_moe_gemv(cg_backend *be, cg_tensor *n, bool *done);
int realize_matmul(cg_backend *be, cg_tensor *n, cg_tensor *addend, bool *added, MatmulEpilogue *ep);
int realize_concat(cg_backend *be, cg_tensor *n);
int realize_index(cg_backend *be, cg_tensor *n);
int realize_arange(cg_backend *be, cg_tensor *n);
int realize(cg_backend *be, cg_tensor *n);
int sync_and_check(cg_backend *be);
bool share_node(cg_backend *be, cg_tensor *n, cg_tensor **out);
int finish(cg_backend *be, cg_tensor *n, cg_tensor **out);
int run_pending_flush(cg_backend *be);
int realize_view_or_release(cg_backend *be, cg_tensor *n);
int check_args(cg_backend *be, cg_tensor *a, cg_tensor *b, void *out);
int to_shape(cg_backend *be, const size_t *dims, int rank, int64_t *shape);
uint32_t host_upow(uint32_t a, uint32_t e);
bool fold_binary(EwOp op, uint32_t a, uint32_t b, uint32_t *out);
cg_tensor *bias_vector_of(cg_tensor *other, const cg_tensor *like);
bool bias_vector_ready(const cg_tensor *v);
int binary(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **out, EwOp f_op, EwOp u_op);
int unary(cg_backend *be, cg_tensor *x, cg_tensor **out, EwOp op, cg_dtype out_dtype);
cg_tensor *const_node(cg_backend *be, cg_dtype dt, int rank, const int64_t *shape, uint32_t bits);
uint32_t host_f2u(float v);
int upload(cg_backend *be, const void *data, size_t n, const int64_t *shape, int rank, cg_dtype dt,
           cg_tensor **out);
int download(cg_backend *be, cg_tensor *x, void *dst, size_t n, cg_dtype want);


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


// Rows of a realised f32 tensor reached through up to three (extent, stride) pairs over the row
// index, outermost first (d0 is implied): [B, H, S, D] seen through a transpose of [B, S, H, D].
struct RowMap {
  uint32_t d1 = 1, d2 = 1;
  int64_t s0 = 0, s1 = 0, s2 = 0;
};


// nn::softmax (stdlib/nn/mod.rs:162-171) with attention's `/ sqrt(d)` and `+ mask` in front:
// pure matching, nothing is realised.  src is the tensor the scale / mask / softmax apply to.
struct SoftmaxMatch {
  cg_tensor *src = nullptr, *mask = nullptr;
  cg_tensor *x = nullptr;  // what max / sub / exp are applied to (src after scale and mask)
  bool has_scale = false, has_mask_const = false;
  float scale = 1.f, mask_const = 0.f;
};


// rmsnorm_raw / rmsnorm (catgrad-llm/src/helpers.rs:120-145; gemma3.rs:41-68)
struct RmsNormMatch {
  cg_tensor *x = nullptr, *gamma = nullptr;  // gamma: the broadcast node or null
  float eps = 0.f, n_as_float = 1.f, gamma_offset = 0.f;
};


// apply_rope_embedding (catgrad-llm/src/helpers.rs:195-221): cos * x + sin * rotate_half(x)
struct RopeMatch {
  cg_tensor *cb = nullptr, *sb = nullptr, *x = nullptr;  // cos / sin broadcasts, the rotated tensor
};

// The rotated tensor of a RopeMatch as the RMS norm of `view` ([b, h, s, d], realised), read by nothing but the
// rotation: the rotation's kernel norms each row on its way in (rope_normed_input).
struct RopeNormed {
  bool on = false;
  RmsNormMatch rm;
  cg_tensor *view = nullptr;  // not retained: the graph under the rotation holds it
  const float *gamma = nullptr;
};

// What the q / k / v projections of a prefill are asked to do in the epilogue of their grouped launch: leave the
// queries and keys rotated, head-major, and a transposed bf16 copy of the values (GemmDesc::rope_role).  The
// launch sets `applied` when it did.
struct RopeGemmRequest {
  cg_tensor *mm[3] = {nullptr, nullptr, nullptr};  // the products: q, k, v
  float *out[2] = {nullptr, nullptr};              // rotated q, k: [sequences][heads][positions][head_dim]
  uint16_t *out16[3] = {nullptr, nullptr, nullptr};  // their bf16 copies (optional); [2]: v as [sequences][heads][head_dim][positions]
  const float *cos[2] = {nullptr, nullptr}, *sin[2] = {nullptr, nullptr};
  int64_t cs_ss[2] = {0, 0};
  uint32_t positions = 0, head_dim = 0;
  bool applied = false;
};


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


// The routed experts of a MoE layer as the reference emits them (models/qwen3.rs:104-123), per slot:
//   g = matmul(x[S,1,H], T(index(0, idx, Wg)));  u = matmul(x, T(index(0, idx, Wu)))
//   y = matmul(silu(g) * u, T(index(0, idx, Wd)))
// g and u go out as one launch (two problems sharing the staged input rows); the SwiGLU runs in the
// prologue of the down product.  Every workgroup stages the row of its token in LDS once and
// reads the weight rows of that token's expert in place (no gather of expert matrices).
struct ExpertOperand {
  cg_tensor *w = nullptr, *idx = nullptr;  // the stacked matrices [E, N, K] and the index tensor
};

}  // namespace cgrt
