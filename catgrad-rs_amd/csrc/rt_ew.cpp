// rt_ew.cpp — part of the host runtime behind include/catgrad_hip.h (layout: rt_internal.hpp).
#include "rt_internal.hpp"

namespace cgrt {


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
bool row_chain_ok(const cg_tensor *r, const cg_tensor *root, int depth) {
  if (depth > 32) return false;
  if (r->op == N_CONST) return true;
  if (r->op == N_BIN) return row_chain_ok(r->in[0], root, depth + 1) && row_chain_ok(r->in[1], root, depth + 1);
  if (r->op == N_UN) return row_chain_ok(r->in[0], root, depth + 1);
  if (r->op == N_REDUCE && r->p0 <= R_MAX_U) return same_shape(r->in[0], root);
  return false;
}


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


int materialize(cg_backend *be, cg_tensor *src, cg_tensor **out, bool keep_bf16) {
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
  // Greedy decoding (llm/utils.rs: argmax of the last position's logits): the row is a one-row product that is
  // still deferred.  Its launch keeps, per wave, the largest value it stores; the argmax merges those records
  // instead of reading 128 K logits back with two launches of its own.
  if (kind == R_ARGMAX_F && !(be->flags & CG_FLAG_NO_PATTERNS) && x->rank >= 1 && x->size() == x->shape[x->rank - 1] &&
      x->size() >= 4096) {
    cg_tensor *mm = x;
    while (mm->op == N_RESHAPE && mm->in[0] && mm->in[0]->size() == mm->size()) mm = mm->in[0];
    if (mm->op == N_MATMUL && mm->gemv_candidate && mm->dtype == CG_F32) {
      be->amax_want = mm;
      be->amax_records = nullptr;
      const int st = realize(be, mm);
      be->amax_want = nullptr;
      Storage *records = be->amax_records;
      be->amax_records = nullptr;
      if (st) {
        storage_release(records);
        return st;
      }
      if (records) {
        int st2 = alloc_result(be, n, ST_U32);
        hipError_t e = hipSuccess;
        if (!st2) {
          KernelScope ks(be, "reduce_argmax", (double)be->amax_n_records * 12 + 4, 0);
          if (be->trace_shapes) ks.rename("reduce_argmax[records]");
          e = launch_argmax_merge(be->lc(), (const uint32_t *)records->ptr, (uint32_t *)n->st->ptr, be->amax_n_records);
        }
        storage_release(records);
        if (st2) return st2;
        HIPCHK(be, e);
        n->op = N_REAL;
        drop_inputs(n);
        return CG_OK;
      }
    }
  }
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

}  // namespace cgrt
