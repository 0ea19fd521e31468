// rt_graph.cpp — part of the host runtime behind include/catgrad_hip.h (layout: rt_internal.hpp).
#include "rt_internal.hpp"

namespace cgrt {


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


// the k-slices of a split product (N_KSUM) that no norm took on its way in: summed by a pass of their own
int realize_ksum(cg_backend *be, cg_tensor *n) {
  const cg_tensor *slices = n->in[0], *add = n->in[1];
  {
    KernelScope ks(be, "splitk_sum", (double)n->size() * 4 * (n->p0 + (add ? 2 : 1)), 0);
    HIPCHK(be, launch_splitk_sum(be->lc(), (const float *)data_ptr(slices), (float *)data_ptr(n), (uint64_t)n->size(), (uint32_t)n->p0,
                                 add ? (const float *)data_ptr(add) : nullptr));
  }
  n->op = N_REAL;
  drop_inputs(n);
  return CG_OK;
}


// ndarray.rs:495-520.  The values node computes both results; the index node is filled with it.
int realize_topk(cg_backend *be, cg_tensor *v) {
  if (v->op == N_TOPK_INDEX) {
    cg_tensor *vals = retain(v->in[0]);  // (letting go of the inputs below must not delete it mid-way)
    int st = vals->op == N_TOPK ? realize_topk(be, vals) : CG_OK;
    node_release(vals);
    if (st) return st;
    return v->op == N_REAL ? CG_OK : fail(be, CG_ERR_INTERNAL, "topk: indices without their values");
  }
  cg_tensor *x = v->in[0], *ix = v->pair;
  const int64_t n = x->shape[x->rank - 1], k = v->p0;
  HIPCHK(be, hipSetDevice(be->device));
  // The router of a MoE layer: topk(softmax(logits)) where nobody else reads the probabilities - both in one
  // launch, the probabilities never stored.
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
  Storage *spare = nullptr;  // nobody holds the indices any more
  int st = alloc_result(be, v, ST_F32);
  if (!st) st = ix ? alloc_result(be, ix, ST_U32) : dev_alloc(be, (size_t)std::max<int64_t>(v->size(), 1) * 4, &spare);
  if (!st && v->size()) {
    const int64_t rows = n ? x->size() / n : 0;
    KernelScope ks(be, router ? "softmax_topk" : "topk", (double)x->size() * 4, 0);
    uint32_t *ip = (uint32_t *)(ix ? ix->st->ptr : spare->ptr);
    hipError_t e = router ? launch_softmax_topk(be->lc(), (const float *)data_ptr(c), n, (float *)v->st->ptr, ip, (uint32_t)rows,
                                                (uint32_t)n, (uint32_t)k)
                          : launch_topk(be->lc(), (const float *)data_ptr(c), (float *)v->st->ptr, ip, (uint32_t)rows, (uint32_t)n,
                                        (uint32_t)k);
    if (e != hipSuccess) st = fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
  }
  node_release(c);
  storage_release(spare);
  if (st) return st;
  v->op = N_REAL;
  v->pair = nullptr;
  drop_inputs(v);
  if (ix) {
    ix->op = N_REAL;
    drop_inputs(ix);
  }
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
    case N_KSUM: return realize_ksum(be, n);
    case N_TOPK:
    case N_TOPK_INDEX: return realize_topk(be, n);
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
    // (a norm reads this value next: if its product is split along k, the norm sums the slices itself)
    be->ksum_flush_node = f;
    st = e == hipSuccess ? realize(be, f) : fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
    be->ksum_flush_node = nullptr;
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
      // (or the previous block end still as the k-slices of its product: its strides are those of the sum;
      // or, in the first block, the embedding rows not yet gathered, behind reshapes at most)
      const cg_tensor *src = other;
      while (src->op == N_RESHAPE && src->in[0]) src = src->in[0];
      const bool in_memory = other->op == N_REAL || other->op == N_KSUM;
      // (or a sum with other readers besides this add - the norm before the product reads it twice: the residual
      // stream where the previous block ended in something else than a product, a MoE block's weighted sum; a
      // value with several readers is computed on its own whatever follows)
      const bool stream_sum = other->op == N_BIN && other->ew == E_ADD_F && other->rc.load() >= 3;
      if (mm->op != N_MATMUL || !(in_memory || src->op == N_INDEX || stream_sum)) continue;
      bool dense = true;
      for (int i = 0; in_memory && i < other->rank; ++i) dense = dense && (other->shape[i] == 1 || other->strides[i] != 0);
      // a few-row product with siblings on the same rows (q/k/v, each about to get its bias) is the
      // middle of a block: the siblings' adds are not recorded yet
      if (dense && mm->gemv_candidate)
        for (const cg_tensor *c : be->gemv_candidates)
          if (c != mm && c->op == N_MATMUL && rows_base(c->in[0]) == rows_base(mm->in[0])) dense = false;
      block_end = dense;
    }
  }
  // `linear(x) + bias`: the product's launch can add the bias itself (a few rows: try_gemv_prologue; many rows
  // in bf16 mode: the grouped q / k / v launch of realize_matmul)
  if (n->ew == E_ADD_F && !(be->flags & (CG_FLAG_EAGER | CG_FLAG_NO_PATTERNS))) {
    for (int side = 0; side < 2; ++side) {
      cg_tensor *mm = n->in[side], *other = n->in[1 - side];
      if (mm->op == N_MATMUL && (mm->gemv_candidate || mm->gemm_candidate) && !mm->bias_user && bias_vector_of(other, n) != nullptr) {
        mm->bias_user = n;
        n->bias_of = mm;
        break;
      }
    }
  }
  // `act(gate_proj(x)) * up_proj(x)` on a few rows: the gate's product can be asked which multiplication it
  // gates (the launch of a sibling product on the same rows may take the pair along)
  if (n->ew == E_MUL_F && !(be->flags & (CG_FLAG_EAGER | CG_FLAG_NO_PATTERNS))) {
    cg_tensor *g = glu_gate_of(n);
    if (g && g->op == N_RESHAPE && g->in[0]) g = g->in[0];
    if (g && g->op == N_MATMUL && g->gemv_candidate && !g->glu_user) {
      g->glu_user = n;
      n->glu_of = g;
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

}  // namespace cgrt
