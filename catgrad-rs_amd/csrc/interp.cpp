// interp.cpp — evaluator of core terms over the C ABI of include/catgrad_hip.h.
//
// Restates, for a host without a Rust toolchain, the part of catgrad that drives a
// `Backend`:
//   - core::Term / Operation            catgrad/src/category/core.rs:12-241
//   - parallel_ssa (layered order)      catgrad/src/ssa/mod.rs:24-76
//   - eval_with, apply_* handlers       catgrad/src/abstract_interpreter/eval.rs:18-184
//   - tensor_op and argument orders     catgrad/src/interpreter/tensor_op.rs:9-226
//   - handle_load / handle_definition   catgrad/src/interpreter/interpreter.rs:56-74
// It is written against the C ABI only, so the same translation unit is linked with the HIP
// backend (the product) and with the CPU oracle (the checker).
//
// Differences from the reference, all host-side and result-neutral: the layered order of a
// term is computed once and cached on the term (the reference recomputes `to_core` and
// `parallel_ssa` on every run, interpreter.rs:33-36, eval.rs:38); the state map is a
// vector indexed by node id instead of a HashMap.

#include "../../include/catgrad_hip.h"

#include <cstring>
#include <map>
#include <iterator>
#include <string>
#include <unordered_map>
#include <vector>

namespace {

struct Op {
  cg_opcode op;
  std::string path;
  uint64_t scalar;
  std::vector<uint32_t> src, tgt;
};

struct Value {
  int kind = -1;  // -1 = absent
  size_t nat = 0;
  int dtype = 0;
  int rank = 0;
  size_t dims[CG_MAX_RANK] = {};
  cg_tensor *tensor = nullptr;
};

thread_local std::string g_err;
thread_local uint64_t g_calls = 0;

int ierr(int code, const std::string &m) {
  g_err = m;
  return code;
}

}  // namespace

struct cg_term {
  std::vector<cg_object> nodes;
  std::vector<Op> ops;
  std::vector<uint32_t> sources, targets;
  bool ordered = false;
  bool cyclic = false;
  std::vector<uint32_t> order;  // edge ids, layer by layer
  size_t n_layers = 0;
};

struct cg_env {
  std::unordered_map<std::string, cg_term *> definitions;
};

struct cg_params {
  std::unordered_map<std::string, cg_tensor *> values;
  ~cg_params() {
    for (auto &kv : values) cg_tensor_release(kv.second);
  }
};

namespace {

// Layered topological order of the hyperedges: an edge sits one layer above the deepest edge
// that produces one of its sources (ssa/mod.rs:38-76 via layered_operations).
void order_term(cg_term *t) {
  if (t->ordered) return;
  const size_t nn = t->nodes.size(), ne = t->ops.size();
  std::vector<int32_t> producer(nn, -1);
  for (size_t e = 0; e < ne; ++e)
    for (uint32_t n : t->ops[e].tgt)
      if (n < nn) producer[n] = (int32_t)e;
  std::vector<uint32_t> indeg(ne, 0);
  std::vector<std::vector<uint32_t>> consumers(ne);
  for (size_t e = 0; e < ne; ++e)
    for (uint32_t n : t->ops[e].src)
      if (n < nn && producer[n] >= 0) {
        indeg[e]++;
        consumers[producer[n]].push_back((uint32_t)e);
      }
  std::vector<uint32_t> frontier, next;
  for (size_t e = 0; e < ne; ++e)
    if (!indeg[e]) frontier.push_back((uint32_t)e);
  t->order.clear();
  t->n_layers = 0;
  while (!frontier.empty()) {
    t->n_layers++;
    next.clear();
    for (uint32_t e : frontier) {
      t->order.push_back(e);
      for (uint32_t c : consumers[e])
        if (--indeg[c] == 0) next.push_back(c);
    }
    frontier.swap(next);
  }
  t->cyclic = t->order.size() != ne;
  t->ordered = true;
}

void drop(Value &v) {
  if (v.kind == CG_VAL_TENSOR && v.tensor) cg_tensor_release(v.tensor);
  v.kind = -1;
  v.tensor = nullptr;
}

Value clone(const Value &v) {
  Value r = v;
  if (v.kind == CG_VAL_TENSOR) cg_tensor_retain(v.tensor);
  return r;
}

struct Ctx {
  cg_backend *be;
  const cg_env *env;
  const cg_params *params;
  uint32_t err_id = 0;
};

int eval_term(Ctx &cx, cg_term *term, std::vector<Value> &args, std::vector<Value> &results);

// get_exact_arity / to_nat / to_shape / to_tensor / to_dtype (abstract_interpreter/util.rs)
#define ARITY(n)                                                               \
  if (args.size() != (n)) {                                                    \
    cx.err_id = edge;                                                          \
    return ierr(CG_ERR_ARITY, "ArityError(EdgeId(" + std::to_string(edge) + "))"); \
  }
#define WANT(i, k)                                                             \
  if (args[i].kind != (k)) {                                                   \
    cx.err_id = edge;                                                          \
    return ierr(CG_ERR_TYPE, "TypeError(EdgeId(" + std::to_string(edge) + "))");  \
  }

int backend_failed(Ctx &cx, uint32_t edge, int st) {
  cx.err_id = edge;
  g_err = std::string(cg_last_error(cx.be));
  return st;
}

Value tensor_value(cg_tensor *t) {
  Value v;
  v.kind = CG_VAL_TENSOR;
  v.tensor = t;
  return v;
}

typedef int (*binfn)(cg_backend *, cg_tensor *, cg_tensor *, cg_tensor **);
typedef int (*unfn)(cg_backend *, cg_tensor *, cg_tensor **);

int apply_op(Ctx &cx, const Op &op, uint32_t edge, std::vector<Value> &args,
             std::vector<Value> &out) {
  cg_backend *be = cx.be;
  cg_tensor *r = nullptr;
  int st = CG_OK;
  switch (op.op) {
    // eval.rs:104-113
    case CG_OP_COPY: {
      ARITY(1);
      size_t n = op.tgt.size();
      for (size_t i = 1; i < n; ++i) out.push_back(clone(args[0]));
      if (n) {
        out.insert(out.begin(), args[0]);
        args[0].kind = -1;  // moved
      }
      return CG_OK;
    }
    // interpreter.rs:56-59
    case CG_OP_LOAD: {
      cg_tensor *p = nullptr;
      if (cx.params) {
        auto it = cx.params->values.find(op.path);
        if (it != cx.params->values.end()) p = it->second;
      }
      if (!p) {
        cx.err_id = edge;
        return ierr(CG_ERR_LOAD, "Load(EdgeId(" + std::to_string(edge) + "), " + op.path + ")");
      }
      out.push_back(tensor_value(cg_tensor_retain(p)));
      return CG_OK;
    }
    // interpreter.rs:61-74
    case CG_OP_DEF: {
      cg_term *def = nullptr;
      if (cx.env) {
        auto it = cx.env->definitions.find(op.path);
        if (it != cx.env->definitions.end()) def = it->second;
      }
      if (!def) {
        cx.err_id = edge;
        return ierr(CG_ERR_APPLY, "Definition not found for path: " + op.path);
      }
      return eval_term(cx, def, args, out);
    }
    // eval.rs:119-162
    case CG_OP_PACK: {
      Value v;
      v.kind = CG_VAL_SHAPE;
      if (args.size() > CG_MAX_RANK) {
        cx.err_id = edge;
        return ierr(CG_ERR_APPLY, "pack: rank above CG_MAX_RANK");
      }
      v.rank = (int)args.size();
      for (size_t i = 0; i < args.size(); ++i) {
        WANT(i, CG_VAL_NAT);
        v.dims[i] = args[i].nat;
      }
      out.push_back(v);
      return CG_OK;
    }
    case CG_OP_UNPACK: {
      ARITY(1);
      WANT(0, CG_VAL_SHAPE);
      for (int i = 0; i < args[0].rank; ++i) {
        Value v;
        v.kind = CG_VAL_NAT;
        v.nat = args[0].dims[i];
        out.push_back(v);
      }
      return CG_OK;
    }
    case CG_OP_SHAPE: {
      ARITY(1);
      WANT(0, CG_VAL_TENSOR);
      Value v;
      v.kind = CG_VAL_SHAPE;
      v.rank = cg_tensor_rank(args[0].tensor);
      cg_tensor_shape(args[0].tensor, v.dims);
      out.push_back(v);
      return CG_OK;
    }
    case CG_OP_DTYPE: {
      ARITY(1);
      WANT(0, CG_VAL_TENSOR);
      Value v;
      v.kind = CG_VAL_DTYPE;
      v.dtype = cg_tensor_dtype(args[0].tensor);
      out.push_back(v);
      return CG_OK;
    }
    // eval.rs:167-184
    case CG_OP_NAT_CONST: {
      ARITY(0);
      Value v;
      v.kind = CG_VAL_NAT;
      v.nat = (size_t)op.scalar;
      out.push_back(v);
      return CG_OK;
    }
    case CG_OP_NAT_MUL:
    case CG_OP_NAT_ADD: {
      for (size_t i = 0; i < args.size(); ++i) WANT(i, CG_VAL_NAT);
      ARITY(2);
      Value v;
      v.kind = CG_VAL_NAT;
      v.nat = op.op == CG_OP_NAT_MUL ? args[0].nat * args[1].nat : args[0].nat + args[1].nat;
      out.push_back(v);
      return CG_OK;
    }
    case CG_OP_DTYPE_CONST: {
      Value v;
      v.kind = CG_VAL_DTYPE;
      v.dtype = (int)op.scalar;
      out.push_back(v);
      return CG_OK;
    }
    // tensor_op.rs:16-26, 174-226: binop over a same-dtype pair
    case CG_OP_ADD: case CG_OP_SUB: case CG_OP_MUL: case CG_OP_DIV: case CG_OP_POW:
    case CG_OP_LT: case CG_OP_EQ: case CG_OP_MATMUL: {
      ARITY(2);
      WANT(0, CG_VAL_TENSOR);
      WANT(1, CG_VAL_TENSOR);
      if (cg_tensor_dtype(args[0].tensor) != cg_tensor_dtype(args[1].tensor)) {
        cx.err_id = edge;
        return ierr(CG_ERR_TYPE, "TypeError(EdgeId(" + std::to_string(edge) + "))");
      }
      binfn f = op.op == CG_OP_ADD ? cg_add : op.op == CG_OP_SUB ? cg_sub
              : op.op == CG_OP_MUL ? cg_mul : op.op == CG_OP_DIV ? cg_div
              : op.op == CG_OP_POW ? cg_pow : op.op == CG_OP_LT ? cg_lt
              : op.op == CG_OP_EQ ? cg_eq : cg_matmul;
      g_calls++;
      st = f(be, args[0].tensor, args[1].tensor, &r);
      break;
    }
    case CG_OP_NEG: case CG_OP_COS: case CG_OP_SIN:
    case CG_OP_SUM: case CG_OP_MAX: case CG_OP_ARGMAX: {
      ARITY(1);
      WANT(0, CG_VAL_TENSOR);
      unfn f = op.op == CG_OP_NEG ? cg_neg : op.op == CG_OP_COS ? cg_cos
             : op.op == CG_OP_SIN ? cg_sin : op.op == CG_OP_SUM ? cg_sum
             : op.op == CG_OP_MAX ? cg_max : cg_argmax;
      g_calls++;
      st = f(be, args[0].tensor, &r);
      break;
    }
    // tensor_op.rs:68-78
    case CG_OP_NAT_TO_U32: {
      ARITY(1);
      WANT(0, CG_VAL_NAT);
      if (args[0].nat > 0xFFFFFFFFull) {
        cx.err_id = edge;
        return ierr(CG_ERR_APPLY, "ApplyError(EdgeId(" + std::to_string(edge) + "))");
      }
      uint32_t v = (uint32_t)args[0].nat;
      g_calls++;
      st = cg_from_u32(be, &v, 1, nullptr, 0, &r);
      break;
    }
    // tensor_op.rs:55-66
    case CG_OP_SCALAR_F32: {
      ARITY(0);
      uint32_t bits = (uint32_t)op.scalar;
      float v;
      std::memcpy(&v, &bits, 4);
      g_calls++;
      st = cg_from_f32(be, &v, 1, nullptr, 0, &r);
      break;
    }
    case CG_OP_SCALAR_U32: {
      ARITY(0);
      uint32_t v = (uint32_t)op.scalar;
      g_calls++;
      st = cg_from_u32(be, &v, 1, nullptr, 0, &r);
      break;
    }
    // tensor_op.rs:80-84: [tensor, dtype]
    case CG_OP_CAST: {
      ARITY(2);
      WANT(0, CG_VAL_TENSOR);
      WANT(1, CG_VAL_DTYPE);
      g_calls++;
      st = cg_cast(be, args[0].tensor, (cg_dtype)args[1].dtype, &r);
      break;
    }
    // tensor_op.rs:104-109: [x, k] -> [values, indices]
    case CG_OP_TOPK: {
      ARITY(2);
      WANT(0, CG_VAL_TENSOR);
      WANT(1, CG_VAL_NAT);
      cg_tensor *vals = nullptr, *idx = nullptr;
      g_calls++;
      st = cg_topk(be, args[0].tensor, args[1].nat, &vals, &idx);
      if (st) return backend_failed(cx, edge, st);
      out.push_back(tensor_value(vals));
      out.push_back(tensor_value(idx));
      return CG_OK;
    }
    // tensor_op.rs:111-119: [x, shape]
    case CG_OP_BROADCAST: {
      ARITY(2);
      WANT(0, CG_VAL_TENSOR);
      WANT(1, CG_VAL_SHAPE);
      g_calls++;
      st = cg_broadcast(be, args[0].tensor, args[1].dims, args[1].rank, &r);
      break;
    }
    // tensor_op.rs:121-125: [shape, x]
    case CG_OP_RESHAPE: {
      ARITY(2);
      WANT(0, CG_VAL_SHAPE);
      WANT(1, CG_VAL_TENSOR);
      g_calls++;
      st = cg_reshape(be, args[1].tensor, args[0].dims, args[0].rank, &r);
      break;
    }
    // tensor_op.rs:127-135: [x, dim0, dim1]
    case CG_OP_TRANSPOSE: {
      ARITY(3);
      WANT(0, CG_VAL_TENSOR);
      WANT(1, CG_VAL_NAT);
      WANT(2, CG_VAL_NAT);
      g_calls++;
      st = cg_transpose(be, args[0].tensor, args[1].nat, args[2].nat, &r);
      break;
    }
    // tensor_op.rs:137-142: [x, dim, start, len]
    case CG_OP_SLICE: {
      ARITY(4);
      WANT(0, CG_VAL_TENSOR);
      WANT(1, CG_VAL_NAT);
      WANT(2, CG_VAL_NAT);
      WANT(3, CG_VAL_NAT);
      g_calls++;
      st = cg_slice(be, args[0].tensor, args[1].nat, args[2].nat, args[3].nat, &r);
      break;
    }
    // tensor_op.rs:144-148: [a, b, dim]
    case CG_OP_CONCAT: {
      ARITY(3);
      WANT(0, CG_VAL_TENSOR);
      WANT(1, CG_VAL_TENSOR);
      WANT(2, CG_VAL_NAT);
      g_calls++;
      st = cg_concat(be, args[0].tensor, args[1].tensor, args[2].nat, &r);
      break;
    }
    // tensor_op.rs:150-153
    case CG_OP_ARANGE: {
      ARITY(1);
      WANT(0, CG_VAL_NAT);
      g_calls++;
      st = cg_arange(be, args[0].nat, &r);
      break;
    }
    // tensor_op.rs:155-159: [x, dim, indices]
    case CG_OP_INDEX: {
      ARITY(3);
      WANT(0, CG_VAL_TENSOR);
      WANT(1, CG_VAL_NAT);
      WANT(2, CG_VAL_TENSOR);
      g_calls++;
      st = cg_index(be, args[0].tensor, args[1].nat, args[2].tensor, &r);
      break;
    }
    default:
      cx.err_id = edge;
      return ierr(CG_ERR_APPLY, "unknown operation");
  }
  if (st) return backend_failed(cx, edge, st);
  out.push_back(tensor_value(r));
  return CG_OK;
}

// eval.rs:18-77.  args are consumed (moved into the state); on success results own their
// tensors; on failure everything still held is released.
int eval_term(Ctx &cx, cg_term *term, std::vector<Value> &args, std::vector<Value> &results) {
  if (args.size() != term->sources.size())
    return ierr(CG_ERR_ARITY, "eval: " + std::to_string(args.size()) + " values for " +
                                  std::to_string(term->sources.size()) + " sources");
  order_term(term);
  if (term->cyclic) return ierr(CG_ERR_CYCLE, "SSAError(Cycle)");

  std::vector<Value> state(term->nodes.size());
  int st = CG_OK;
  auto cleanup = [&]() {
    for (Value &v : state) drop(v);
    for (Value &v : args) drop(v);
  };
  for (size_t i = 0; i < args.size(); ++i) {
    uint32_t n = term->sources[i];
    if (state[n].kind != -1) {
      cx.err_id = n;
      cleanup();
      return ierr(CG_ERR_MULTIPLE_WRITE, "MultipleWrite(NodeId(" + std::to_string(n) + "))");
    }
    state[n] = args[i];
    args[i].kind = -1;
  }

  std::vector<Value> a, out;
  for (uint32_t e : term->order) {
    const Op &op = term->ops[e];
    a.clear();
    out.clear();
    for (uint32_t n : op.src) {
      if (state[n].kind == -1) {
        cx.err_id = n;
        st = ierr(CG_ERR_MULTIPLE_READ, "MultipleRead(NodeId(" + std::to_string(n) + "))");
        break;
      }
      a.push_back(state[n]);
      state[n].kind = -1;
    }
    if (!st) st = apply_op(cx, op, e, a, out);
    for (Value &v : a) drop(v);  // arguments were passed by value: dropped after the call
    if (st) {
      for (Value &v : out) drop(v);
      cleanup();
      return st;
    }
    // zip(targets, results): surplus results are dropped, like the reference's zip
    for (size_t i = 0; i < out.size(); ++i) {
      if (i >= op.tgt.size()) {
        drop(out[i]);
        continue;
      }
      uint32_t n = op.tgt[i];
      if (state[n].kind != -1) {
        cx.err_id = n;
        for (size_t j = i; j < out.size(); ++j) drop(out[j]);
        cleanup();
        return ierr(CG_ERR_MULTIPLE_WRITE, "MultipleWrite(NodeId(" + std::to_string(n) + "))");
      }
      state[n] = out[i];
    }
  }

  results.clear();
  for (uint32_t n : term->targets) {
    if (state[n].kind == -1) {
      cx.err_id = n;
      for (Value &v : results) drop(v);
      results.clear();
      cleanup();
      return ierr(CG_ERR_MULTIPLE_READ, "MultipleRead(NodeId(" + std::to_string(n) + "))");
    }
    results.push_back(state[n]);
    state[n].kind = -1;
  }
  cleanup();
  return CG_OK;
}

}  // namespace

extern "C" {

int cg_term_create(cg_term **out) {
  if (!out) return CG_ERR_ARG;
  *out = new cg_term();
  return CG_OK;
}
void cg_term_destroy(cg_term *t) { delete t; }

int cg_term_add_node(cg_term *t, cg_object label, uint32_t *node_id) {
  if (!t) return CG_ERR_ARG;
  t->nodes.push_back(label);
  t->ordered = false;
  if (node_id) *node_id = (uint32_t)t->nodes.size() - 1;
  return CG_OK;
}

int cg_term_add_op(cg_term *t, cg_opcode op, const char *path, uint64_t scalar,
                   const uint32_t *sources, size_t n_sources, const uint32_t *targets,
                   size_t n_targets, uint32_t *edge_id) {
  if (!t || op < 0 || op >= CG_OP__COUNT) return ierr(CG_ERR_ARG, "add_op: bad argument");
  Op o;
  o.op = op;
  if (path) o.path = path;
  o.scalar = scalar;
  o.src.assign(sources, sources + n_sources);
  o.tgt.assign(targets, targets + n_targets);
  for (uint32_t n : o.src)
    if (n >= t->nodes.size()) return ierr(CG_ERR_ARG, "add_op: unknown source node");
  for (uint32_t n : o.tgt)
    if (n >= t->nodes.size()) return ierr(CG_ERR_ARG, "add_op: unknown target node");
  t->ops.push_back(std::move(o));
  t->ordered = false;
  if (edge_id) *edge_id = (uint32_t)t->ops.size() - 1;
  return CG_OK;
}

int cg_term_set_boundary(cg_term *t, const uint32_t *sources, size_t n_sources,
                         const uint32_t *targets, size_t n_targets) {
  if (!t) return CG_ERR_ARG;
  for (size_t i = 0; i < n_sources; ++i)
    if (sources[i] >= t->nodes.size()) return ierr(CG_ERR_ARG, "boundary: unknown node");
  for (size_t i = 0; i < n_targets; ++i)
    if (targets[i] >= t->nodes.size()) return ierr(CG_ERR_ARG, "boundary: unknown node");
  t->sources.assign(sources, sources + n_sources);
  t->targets.assign(targets, targets + n_targets);
  return CG_OK;
}

int cg_term_stats(cg_term *t, size_t *n_ops, size_t *n_layers) {
  if (!t) return CG_ERR_ARG;
  order_term(t);
  if (n_ops) *n_ops = t->ops.size();
  if (n_layers) *n_layers = t->n_layers;
  return t->cyclic ? ierr(CG_ERR_CYCLE, "SSAError(Cycle)") : CG_OK;
}

int cg_env_create(cg_env **out) {
  if (!out) return CG_ERR_ARG;
  *out = new cg_env();
  return CG_OK;
}
void cg_env_destroy(cg_env *e) { delete e; }
int cg_env_define(cg_env *e, const char *path, cg_term *term) {
  if (!e || !path || !term) return CG_ERR_ARG;
  e->definitions[path] = term;
  return CG_OK;
}

int cg_params_create(cg_params **out) {
  if (!out) return CG_ERR_ARG;
  *out = new cg_params();
  return CG_OK;
}
void cg_params_destroy(cg_params *p) { delete p; }
int cg_params_set(cg_params *p, const char *path, cg_tensor *t) {
  if (!p || !path || !t) return CG_ERR_ARG;
  auto it = p->values.find(path);
  cg_tensor_retain(t);
  if (it != p->values.end()) {
    cg_tensor_release(it->second);
    it->second = t;
  } else {
    p->values.emplace(path, t);
  }
  return CG_OK;
}

size_t cg_params_len(const cg_params *p) { return p ? p->values.size() : 0; }
const char *cg_params_key(const cg_params *p, size_t i) {
  if (!p || i >= p->values.size()) return nullptr;
  auto it = p->values.begin();
  std::advance(it, (std::ptrdiff_t)i);
  return it->first.c_str();
}
int cg_params_get(const cg_params *p, const char *path, cg_tensor **out) {
  if (!p || !path || !out) return CG_ERR_ARG;
  auto it = p->values.find(path);
  if (it == p->values.end()) return CG_ERR_LOAD;
  *out = cg_tensor_retain(it->second);
  return CG_OK;
}
int cg_params_remove(cg_params *p, const char *path) {
  if (!p || !path) return CG_ERR_ARG;
  auto it = p->values.find(path);
  if (it == p->values.end()) return CG_OK;
  cg_tensor_release(it->second);
  p->values.erase(it);
  return CG_OK;
}

static int eval_entry(cg_backend *be, const cg_env *env, const cg_params *params, cg_term *term,
                      const cg_value *args, size_t n_args, cg_value *results, size_t n_results,
                      uint32_t *err_id, bool owned) {
  auto give_back = [&]() {  // an owned call consumes its tensor arguments on every path
    if (owned)
      for (size_t i = 0; i < n_args; ++i)
        if (args[i].kind == CG_VAL_TENSOR && args[i].tensor) cg_tensor_release(args[i].tensor);
  };
  if (!be || !term) {
    give_back();
    return ierr(CG_ERR_ARG, "eval: null backend or term");
  }
  if (n_results != term->targets.size()) {
    give_back();
    return ierr(CG_ERR_ARITY, "eval: result buffer does not match the term's targets");
  }
  std::vector<Value> a(n_args), r;
  for (size_t i = 0; i < n_args; ++i) {
    a[i].kind = args[i].kind;
    a[i].nat = args[i].nat;
    a[i].dtype = args[i].dtype;
    a[i].rank = args[i].rank;
    std::memcpy(a[i].dims, args[i].dims, sizeof(a[i].dims));
    a[i].tensor = args[i].kind != CG_VAL_TENSOR ? nullptr
                  : owned                       ? args[i].tensor
                                                : cg_tensor_retain(args[i].tensor);
  }
  Ctx cx{be, env, params};
  int st = eval_term(cx, term, a, r);
  if (err_id) *err_id = cx.err_id;
  if (st) {
    for (Value &v : a) drop(v);  // whatever the failed run did not consume
    return st;
  }
  for (size_t i = 0; i < n_results; ++i) {
    std::memset(&results[i], 0, sizeof(cg_value));
    results[i].kind = r[i].kind;
    results[i].nat = r[i].nat;
    results[i].dtype = r[i].dtype;
    results[i].rank = r[i].rank;
    std::memcpy(results[i].dims, r[i].dims, sizeof(r[i].dims));
    results[i].tensor = r[i].tensor;
  }
  return CG_OK;
}

int cg_interp_eval(cg_backend *be, const cg_env *env, const cg_params *params, cg_term *term,
                   const cg_value *args, size_t n_args, cg_value *results, size_t n_results,
                   uint32_t *err_id) {
  return eval_entry(be, env, params, term, args, n_args, results, n_results, err_id, false);
}

int cg_interp_eval_owned(cg_backend *be, const cg_env *env, const cg_params *params, cg_term *term,
                         const cg_value *args, size_t n_args, cg_value *results, size_t n_results,
                         uint32_t *err_id) {
  return eval_entry(be, env, params, term, args, n_args, results, n_results, err_id, true);
}

const char *cg_interp_last_error(void) { return g_err.c_str(); }

uint64_t cg_interp_backend_calls(int reset) {
  uint64_t c = g_calls;
  if (reset) g_calls = 0;
  return c;
}

}  // extern "C"
