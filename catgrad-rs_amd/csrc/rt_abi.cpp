// rt_abi.cpp — the extern "C" entry points of include/catgrad_hip.h (semantics follow
// catgrad/src/interpreter/backend/ndarray.rs method by method, cited at each entry point; shapes follow
// catgrad/src/interpreter/backend/shape_only.rs:255-327).
#include "rt_internal.hpp"

using namespace cgrt;
using namespace cgk;


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
  be->arange_order.clear();
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
  // (up to 4 rows on the vector ALUs, up to 16 against bf16 weights on the matrix cores)
  const bool few_rows = shape[a->rank - 2] == 1 ||
                        (a->rank == 3 && shape[0] == 1 && shape[1] <= ((be->flags & CG_FLAG_BF16) ? GEMV_PRO_MAX_ROWS : 4));
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
  // Both results stay deferred (realize_topk) like any other value: what feeds the router - and what reads the
  // chosen indices - is then realised with the whole block recorded.
  int64_t shape[CG_MAX_RANK];
  std::copy(x->shape, x->shape + x->rank, shape);
  shape[x->rank - 1] = (int64_t)k;
  cg_tensor *v = new_node(be, CG_F32, x->rank, shape), *ix = new_node(be, CG_U32, x->rank, shape);
  v->op = N_TOPK;
  v->p0 = (int64_t)k;
  v->in[0] = retain(x);
  ix->op = N_TOPK_INDEX;
  ix->in[0] = retain(v);
  v->pair = ix;
  if (be->flags & CG_FLAG_EAGER) {
    int st = realize(be, v);
    if (st) {
      node_release(ix);
      node_release(v);
      return st;
    }
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
    // A backend lives through many sequence lengths: when the cache is full its oldest extent leaves (whoever
    // still holds that node keeps it alive), so that the lengths in use now are always the cached ones.
    if (be->arange_cache.size() >= 32 && !be->arange_order.empty()) {
      auto old = be->arange_cache.find(be->arange_order.front());
      be->arange_order.pop_front();
      if (old != be->arange_cache.end()) {
        cg_tensor *t = old->second;
        be->arange_cache.erase(old);
        node_release(t);
      }
    }
    cg_tensor *n = new_node(be, CG_U32, 1, shape);
    n->op = N_ARANGE;
    n->const_like = true;
    n->cse_key = new std::string("arange" + std::to_string(end));
    be->arange_cache[(int64_t)end] = retain(n);
    be->arange_order.push_back((int64_t)end);
    return finish(be, n, out);
  }
  cg_tensor *n = new_node(be, CG_U32, 1, shape);
  n->op = N_ARANGE;
  if (!(be->flags & CG_FLAG_EAGER)) {  // not cached, but still a value any mask built from it can be shared by
    n->const_like = true;
    n->cse_key = new std::string("arange" + std::to_string(end));
  }
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

int cg_peak_gemm_clock(cg_backend *be, size_t m, size_t n, size_t k, int iters, double *tflops, double *clock_mhz) {
  if (!be || !tflops || !clock_mhz || iters < 1) return CG_ERR_ARG;
  if (m && (m % 128 || n % 128 || k % 64 || !n || !k || m * k >= ((size_t)1 << 31) || n * k >= ((size_t)1 << 31)))
    return fail(be, CG_ERR_ARG, "cg_peak_gemm_clock: m, n multiples of 128, k of 64");
  HIPCHK(be, hipSetDevice(be->device));
  LaunchCtx lc = be->lc();
  lc.ev_start = lc.ev_stop = nullptr;
  Storage *a = nullptr, *b = nullptr, *c = nullptr, *ticks = nullptr;
  const unsigned grid = (unsigned)be->n_cus * 8;
  int st = dev_alloc(be, 16, &ticks);
  if (!st) st = dev_alloc(be, m ? m * n * 4 : (size_t)grid * 256 * 4, &c);
  if (!st && m) st = dev_alloc(be, m * k * 2, &a);
  if (!st && m) st = dev_alloc(be, n * k * 2, &b);
  hipEvent_t e0 = nullptr, e1 = nullptr;
  hipError_t e = hipSuccess;
  GemmDesc g;
  std::memset(&g, 0, sizeof(g));
  if (!st) {
    if (m) {
      // operands that toggle like real data (a constant operand draws less power and clocks higher)
      std::vector<uint16_t> h(std::max(m, n) * k);
      uint32_t r = 12345u;
      for (auto &v : h) {
        r = r * 1664525u + 1013904223u;
        const float f = (float)((r >> 8) & 0xffff) / 65536.f - 0.5f;
        uint32_t u;
        std::memcpy(&u, &f, 4);
        v = (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
      }
      e = hipStreamSynchronize(be->ordered_stream());
      if (e == hipSuccess) e = hipMemcpy(a->ptr, h.data(), m * k * 2, hipMemcpyHostToDevice);
      if (e == hipSuccess) e = hipMemcpy(b->ptr, h.data(), n * k * 2, hipMemcpyHostToDevice);
      g.a = a->ptr; g.b = b->ptr; g.c = (float *)c->ptr;
      g.a_stype = g.b_stype = ST_BF16;
      g.bf16_math = 1;
      g.M = (uint32_t)m; g.N = (uint32_t)n; g.K = (uint32_t)k;
      g.nb0 = g.nb1 = 1;
      g.sam = (int64_t)k; g.sak = 1; g.sbn = (int64_t)k; g.sbk = 1;
      g.splits = 1; g.k_per_split = (uint32_t)k;
    }
    auto once = [&](unsigned long long *t) -> hipError_t {
      if (!m) return launch_peak_mfma(lc, 1, (float *)c->ptr, grid, 20000, t);
      g.clock_ticks = t;
      return launch_matmul(lc, g, nullptr);
    };
    if (e == hipSuccess) e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    if (e == hipSuccess) e = once(nullptr);  // warm-up
    if (e == hipSuccess) e = launch_fill_u32(lc, (uint32_t *)ticks->ptr, 0u, 4);
    if (e == hipSuccess) e = hipEventRecord(e0, be->ordered_stream());
    for (int i = 0; i < iters && e == hipSuccess; ++i) e = once((unsigned long long *)ticks->ptr);
    if (e == hipSuccess) e = hipEventRecord(e1, be->ordered_stream());
    if (e == hipSuccess) e = hipStreamSynchronize(be->ordered_stream());
    float ms = 0.f;
    unsigned long long t[2] = {0, 0};
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    if (e == hipSuccess) e = hipMemcpy(t, ticks->ptr, 16, hipMemcpyDeviceToHost);
    if (e == hipSuccess) {
      const double flops = m ? 2.0 * (double)m * (double)n * (double)k : (double)grid * 4 * 20000.0 * 4 * (2.0 * 32 * 32 * 16);
      *tflops = flops * iters / (ms * 1e-3) / 1e12;
      *clock_mhz = t[1] ? (double)t[0] / (double)t[1] * 100.0 : 0.0;
    }
  }
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  storage_release(a);
  storage_release(b);
  storage_release(c);
  storage_release(ticks);
  if (st) return st;
  if (e != hipSuccess) return fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
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
