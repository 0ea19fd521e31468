// rt_matmul.cpp — part of the host runtime behind include/catgrad_hip.h (layout: rt_internal.hpp).
#include "rt_internal.hpp"

namespace cgrt {


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


// A batch-folding linear reshapes its input ([B, 1, K] -> [1, B, K]) and its product back; such a
// reshape only regroups rows.  The node under a reshape that nobody else holds and that keeps the
// last axis, else the node itself.
cg_tensor *rows_base(cg_tensor *t) {
  if (t->op == N_RESHAPE && refs(t) == 1 && t->rank >= 1 && t->in[0]->rank >= 1 &&
      t->in[0]->shape[t->in[0]->rank - 1] == t->shape[t->rank - 1])
    return t->in[0];
  return t;
}


// A deferred RMSNorm row A (or a reshape of one that regroups its rows) whose every reader can compute the norm
// on its own way in, so that the norm needs no launch and its value is never stored: few-row products reading
// A directly - at most one gated pair (`glu`, with its gate and up products) and narrow plain ones - and
// expert-indexed products reading it through one view (a MoE block's post-attention norm: router, shared
// expert, routed experts; models/qwen3.rs:64-133, models/deepseek.rs:163-165).  A reader that does not take
// the prologue after all realises A like any other value; the others still compute the same numbers.
struct NormReaders {
  cg_tensor *norm = nullptr;
  RmsNormMatch rm;
  std::vector<cg_tensor *> plain;
  cg_tensor *glu = nullptr, *gate = nullptr, *up = nullptr;
  int gelu = 0;
  cg_tensor *view = nullptr;
};
static bool keeps_rows(const cg_tensor *v, const cg_tensor *of) {
  if (!v->in[0] || v->in[0] != of || v->rank < 1 || of->rank < 1 || v->size() != of->size() ||
      v->shape[v->rank - 1] != of->shape[of->rank - 1])
    return false;
  if (v->op == N_RESHAPE) return true;
  // a transpose that moves an axis of extent 1 among the leading axes
  if (v->op != N_TRANSPOSE || v->p0 == v->rank - 1 || v->p1 == v->rank - 1) return false;
  return of->shape[v->p0] == 1 || of->shape[v->p1] == 1;
}
static bool norm_readers(cg_backend *be, cg_tensor *A, NormReaders *o) {
  if (A->op == N_REAL || A->dtype != CG_F32 || A->rank < 1) return false;
  cg_tensor *norm = A;
  if (A->op == N_RESHAPE && A->in[0] && A->in[0]->op != N_REAL && refs(A->in[0]) == 1 && keeps_rows(A, A->in[0])) norm = A->in[0];
  if (!match_rmsnorm(norm, &o->rm)) return false;
  o->norm = norm;
  int accounted = 0, view_readers = 0;
  for (cg_tensor *c : be->gemv_candidates) {
    if (c->op != N_MATMUL || !c->in[0]) continue;
    cg_tensor *in = c->in[0];
    if (rows_base(in) == A) {
      ++accounted;
      if (c->glu_user) {
        if (o->glu) return false;
        o->glu = c->glu_user;
      } else {
        o->plain.push_back(c);
      }
    } else if (in->op != N_REAL && keeps_rows(in, A)) {
      ExpertOperand eo;
      if ((o->view && o->view != in) || c->rank != 3 || !match_expert_operand(c->in[1], c->shape[0], &eo)) return false;
      if (!o->view) ++accounted;
      o->view = in;
      ++view_readers;
    }
  }
  if (o->view && refs(o->view) != view_readers) return false;
  if (o->glu) {
    if (!match_glu(o->glu, &o->gate, &o->up, &o->gelu)) return false;
    cg_tensor *um = rows_base(o->up);
    bool found = false;
    for (size_t i = 0; i < o->plain.size(); ++i)
      if (o->plain[i] == um) {
        o->plain.erase(o->plain.begin() + i);
        found = true;
        break;
      }
    if (!found) return false;
  }
  return accounted == refs(A);
}


// `view` (of `base`) is read by expert-indexed products only, and every other reader of `base` computes the
// RMSNorm that `base` is on its own way in: so may these products.
bool norm_row_readers_ok(cg_backend *be, cg_tensor *base, cg_tensor *view, RmsNormMatch *rm) {
  NormReaders nr;
  if (!norm_readers(be, base, &nr) || nr.view != view) return false;
  *rm = nr.rm;
  return true;
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
  if (rows < 1 || rows > GEMV_PRO_MAX_ROWS || X->size() != rows * K || g->size() != rows * N || K % 8 || K < 256 ||
      glu->size() != rows * N)
    return CG_OK;
  cg_tensor *ws[2] = {g->in[1], u->in[1]};
  for (cg_tensor *w : ws) {
    TRY(realize(be, w));
    if (!gemv_pro_rows_ok(w->stype, (uint32_t)rows, (uint32_t)K, PRO_NONE)) return CG_OK;
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
  // narrow plain products on the same rows ride along (the matrix-core form only), and with them the norm may
  // have further readers that compute it themselves
  std::vector<cg_tensor *> extras;
  bool shared_norm = false;
  if (X->op != N_REAL && refs(X) > 2 && rows > 1 && ws[0]->stype == ST_BF16 &&
      gemv_rows_mfma_ok(ST_BF16, (uint32_t)rows, (uint32_t)K, PRO_RMSNORM)) {
    NormReaders nr;
    if (norm_readers(be, X, &nr) && nr.glu == glu && nr.plain.size() <= 2) {
      shared_norm = true;
      for (cg_tensor *c : nr.plain) {
        cg_tensor *w = c->in[1];
        const int64_t nc = w->rank >= 2 ? w->shape[w->rank - 1] : 0;
        TRY(realize(be, w));
        bool ok = w->rank >= 2 && w->shape[w->rank - 2] == K && nc >= 1 && nc < 64 && c->size() == rows * nc && c->dtype == CG_F32 &&
                  w->stype == ST_BF16 && w->strides[w->rank - 2] == 1 && (uintptr_t)data_ptr(w) % 16 == 0 &&
                  (nc == 1 || w->strides[w->rank - 1] % 8 == 0) && !c->bias_user;
        for (int i = 0; ok && i + 2 < w->rank; ++i) ok = w->shape[i] == 1 || w->strides[i] == 0;
        shared_norm = shared_norm && ok;
      }
      if (shared_norm) {
        extras = nr.plain;
        rm = nr.rm;
      }
    }
  }
  if (X->op != N_REAL && (shared_norm || refs(X) == 2) && gemv_pro_rows_ok(ws[0]->stype, (uint32_t)rows, (uint32_t)K, PRO_RMSNORM) &&
      (shared_norm || match_rmsnorm(X, &rm))) {
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
  if (!a0) extras.clear();  // (the row is realised below, for every reader)
  if (!a0) {
    TRY(contiguous(be, X, &a0));
    if (a0->stype != ST_F32 || (uintptr_t)data_ptr(a0) % 16) {
      node_release(a0);
      return CG_OK;
    }
    d.pro = PRO_NONE;
  }
  int st = alloc_result(be, glu, ST_F32);
  for (size_t i = 0; i < extras.size() && !st; ++i) st = alloc_result(be, extras[i], ST_F32);
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
    double extra_bytes = 0, extra_flops = 0;
    for (cg_tensor *c : extras) {
      cg_tensor *w = c->in[1];
      auto &pr = d.m.p[d.m.n_prob++];
      pr.b = data_ptr(w);
      pr.c = (float *)c->st->ptr;
      pr.N = (uint32_t)w->shape[w->rank - 1];
      pr.sbn = pr.N > 1 ? w->strides[w->rank - 1] : K;  // (the stride between columns of a single column is never used)
      extra_bytes += (double)pr.N * K * 2 + (double)rows * pr.N * 4;
      extra_flops += 2.0 * rows * pr.N * K;
    }
    const char *base = rows > 1 && gemv_rows_mfma_ok(ws[0]->stype, (uint32_t)rows, (uint32_t)K, d.pro) ? "gemv_rows_bf16"
                       : ws[0]->stype == ST_BF16                                                          ? "gemv_rowdot_bf16"
                                                                                                          : "gemv_rowdot_f32";
    KernelScope ks(be, base, 2.0 * N * K * esize(ws[0]->stype) + (double)rows * (K * 8 + N * 4) + extra_bytes,
                   4.0 * rows * N * K + extra_flops);
    if (be->trace_shapes) {
      char buf[96];
      snprintf(buf, sizeof buf, "%s[%sgate*up%s,M%lld,K%lld,N%lld]", base, d.pro == PRO_RMSNORM ? "rmsnorm+" : "",
               extras.empty() ? "" : "+narrow", (long long)rows, (long long)K, (long long)(2 * N));
      ks.rename(buf);
    }
    hipError_t e = launch_gemv_pro(be->lc(), d);
    if (e != hipSuccess) st = fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
  }
  node_release(a0);
  node_release(a1);
  if (st) return st;
  for (cg_tensor *c : extras) {
    forget_gemv_candidate(c);
    c->op = N_REAL;
    drop_inputs(c);
  }
  finish_fused(glu);  // releases the activation chain and with it g and u
  *done = true;
  return CG_OK;
}


// A narrow product on the rows of a norm that a gated pair reads too (a MoE block's router, reached before its
// shared expert): the pair's launch takes it along.
int try_norm_reader_group(cg_backend *be, cg_tensor *n, bool *done) {
  if (!n->gemv_candidate || !n->in[0] || !(be->flags & CG_FLAG_BF16)) return CG_OK;
  cg_tensor *A = rows_base(n->in[0]);
  if (A->op == N_REAL || refs(A) < 3) return CG_OK;
  NormReaders nr;
  if (!norm_readers(be, A, &nr) || !nr.glu) return CG_OK;
  if (std::find(nr.plain.begin(), nr.plain.end(), n) == nr.plain.end()) return CG_OK;
  bool fused = false;
  TRY(try_gate_up_glu(be, nr.glu, nr.gate, nr.up, nr.gelu, &fused));
  *done = fused && n->op == N_REAL;
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
  if (rows < 1 || rows > GEMV_PRO_MAX_ROWS || A->size() != rows * K || K % 8 || K < 256) return CG_OK;
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
    if (!gemv_pro_rows_ok(w->stype, (uint32_t)rows, (uint32_t)K, pro)) return CG_OK;
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
    const char *base = rows > 1 && gemv_rows_mfma_ok(b_stype, (uint32_t)rows, (uint32_t)K, pro) ? "gemv_rows_bf16"
                       : b_stype == ST_BF16                                                      ? "gemv_rowdot_bf16"
                                                                                                 : "gemv_rowdot_f32";
    KernelScope ks(be, base, bytes, flops);
    if (be->trace_shapes) {
      char buf[96];
      snprintf(buf, sizeof buf, "%s[%s%d,M%lld,K%lld,N%.0f]", base, pro == PRO_RMSNORM ? "rmsnorm+multi" : "glu+multi",
               d.m.n_prob, (long long)rows, (long long)K, flops / (2.0 * rows * K));
      ks.rename(buf);
    }
    // the argmax over this row is wanted next: the launch leaves it in pieces
    Storage *records = nullptr;
    uint32_t n_records = be->amax_want == n && !bias_add[0] ? gemv_pro_amax_records(be->lc(), d) : 0;
    if (n_records && dev_alloc(be, (size_t)n_records * 12, &records) == CG_OK) d.amax_part = (uint32_t *)records->ptr;
    hipError_t e = launch_gemv_pro(be->lc(), d);
    if (e != hipSuccess) st = fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
    if (!st && records) {
      be->amax_records = records;
      be->amax_n_records = n_records;
    } else {
      storage_release(records);
    }
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


// o_proj of a decode step: a one-row product whose input row is the attention of this step, seen through
// the head merge (`transpose(1, 2)` + `reshape [b, 1, heads * d]`, models/llama.rs:107-110; one batch row, so
// both are views of the same memory order) and read by nobody else.  The attention is launched here and
// stops at the partial results of its key ranges; this product's kernel merges them on its way in, so
// the attention needs no hand-over between its workgroups and its value is never stored.
int try_gemv_attn_merge(cg_backend *be, cg_tensor *n, cg_tensor *addend, bool *added, bool *done) {
  if (!n->gemv_candidate) return CG_OK;
  cg_tensor *att = n->in[0];
  // The merge prologue reads the partials in the attention's own (head, d) order, so every view on the
  // way must keep the row-major element order: a reshape always does; a transpose does when at most one
  // axis in the swapped range has an extent other than 1 (it then only moves unit axes).
  auto keeps_order = [](const cg_tensor *t) {
    if (t->op == N_RESHAPE) return true;
    const int64_t lo = std::min(t->p0, t->p1), hi = std::max(t->p0, t->p1);
    int wide = 0;
    for (int64_t i = lo; i <= hi; ++i) wide += t->shape[i] != 1;
    return wide <= 1;
  };
  while ((att->op == N_RESHAPE || att->op == N_TRANSPOSE) && refs(att) == 1 && keeps_order(att)) att = att->in[0];
  if (att == n->in[0] || att->op != N_MATMUL || att->dtype != CG_F32 || att->rank != 4 || refs(att) != 1) return CG_OK;
  if (att->shape[0] != 1 || att->shape[2] != 1) return CG_OK;
  const int64_t K = att->shape[1] * att->shape[3];
  cg_tensor *w = n->in[1];
  if (n->in[0]->size() != K || K % 8 || K < 256 || K > 2048 || n->size() != n->shape[n->rank - 1]) return CG_OK;
  TRY(realize(be, w));
  if (w->rank < 2 || w->shape[w->rank - 2] != K || w->strides[w->rank - 2] != 1) return CG_OK;
  for (int i = 0; i + 2 < w->rank; ++i)
    if (w->shape[i] != 1 && w->strides[i] != 0) return CG_OK;
  if (w->stype != ST_F32 && w->stype != ST_BF16) return CG_OK;
  if ((uintptr_t)data_ptr(w) % 16 || w->strides[w->rank - 1] % (16 / esize(w->stype))) return CG_OK;
  if (addend && (addend->stype != ST_F32 || be->addend_is_row)) return CG_OK;
  if (att->shape[3] % 4) return CG_OK;  // (the merging prologue reads four values of a head at a time)
  // Once the attention has stopped at its partials its own value is never written, so everything that can
  // fail here comes first: the result's memory now; the launch's own checks are the conditions above plus the
  // split count and geometry try_attn_decode only defers for.
  int st = alloc_result(be, n, ST_F32);
  if (st) return st;
  AttnMergeLater later;
  bool att_done = false;
  st = try_attn_decode(be, att, &att_done, &later);
  if (st || !att_done || !later.deferred) {  // not an attention, or one that wrote its result: the usual path
    storage_release(n->st);
    n->st = nullptr;
    return st;
  }
  GemvProDesc d;
  std::memset(&d, 0, sizeof(d));
  d.pro = PRO_ATTN_MERGE;
  d.merge_part = later.part;
  d.merge_splits = later.splits;
  d.merge_heads = later.heads;
  d.merge_d = later.d;
  d.m.K = (uint32_t)K;
  d.m.n_prob = 1;
  d.m.b_stype = w->stype;
  d.m.p[0].b = data_ptr(w);
  d.m.p[0].c = (float *)n->st->ptr;
  d.m.p[0].c_add = addend ? (const float *)data_ptr(addend) : nullptr;
  d.m.p[0].sbn = w->strides[w->rank - 1];
  d.m.p[0].N = (uint32_t)w->shape[w->rank - 1];
  d.err = be->d_words;
  d.b_index_limit = 1;
  {
    const double N = (double)d.m.p[0].N;
    const char *base = w->stype == ST_BF16 ? "gemv_rowdot_bf16" : "gemv_rowdot_f32";
    KernelScope ks(be, base, N * K * esize(w->stype) + K * 4 + N * 4, 2.0 * N * K);
    if (be->trace_shapes) {
      char buf[96];
      snprintf(buf, sizeof buf, "%s[attn-merge,M1,K%lld,N%.0f]", base, (long long)K, N);
      ks.rename(buf);
    }
    hipError_t e = launch_gemv_pro(be->lc(), d);
    if (e != hipSuccess) return fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
  }
  if (addend) *added = true;
  forget_gemv_candidate(n);
  n->op = N_REAL;
  drop_inputs(n);  // lets go of the head-merge views and, with them, of the attention node
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
    if (!addend) TRY(try_norm_reader_group(be, n, &done));
    if (done) return CG_OK;
    TRY(try_gemv_prologue(be, n, addend, added, &done));
    if (done) return CG_OK;
    TRY(try_gemv_attn_merge(be, n, addend, added, &done));
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
  // an addend that is still the k-slices of an earlier product: the norm among this product's operands has
  // summed it by now; if there was none, it is summed here
  if (addend && addend->op == N_KSUM) TRY(realize(be, addend));
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
    // (a bf16 B that the k-major form of that kernel reads where it lies needs no copy at all)
    GemmDesc probe = g;
    probe.nb0 = nbo[0]; probe.nb1 = nbo[1];
    probe.sa_b0 = sao[0]; probe.sa_b1 = sao[1]; probe.sb_b0 = sbo[0]; probe.sb_b1 = sbo[1];
    probe.bf16_math = (be->flags & CG_FLAG_BF16) ? 1 : 0;
    if (g.bf16_math && M >= 64 && N >= 64 && K % 64 == 0 && g.a_stype == ST_BF16 && g.sak == 1 && g.sbn == 1 &&
        g.sbk != 1 && !ex.w && (g.b_stype == ST_F32 || g.b_stype == ST_BF16) && !gemm_dma_bkm_ok(probe)) {
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
    // The same for the few rows of a small batch against bf16 weights (the router and the shared expert's gate
    // of a MoE block, both narrow: 60 and 1 columns): the matrix-core kernel takes up to four products, and a
    // lone product of fewer than 64 columns too (the vector kernel needs 8 us for 4 x 60 x 2048).
    if (M >= 2 && N < 64 && batch == 1 && n->gemv_candidate && gemv_rows_group_ok(g)) {
      std::vector<cg_tensor *> members;
      for (cg_tensor *c : std::vector<cg_tensor *>(be->gemv_candidates)) {
        if (c == n || members.size() >= 3 || c->op != N_MATMUL || c->in[0] != n->in[0] || c->dtype != CG_F32) continue;
        cg_tensor *w = c->in[1];
        const int64_t nc = w->shape[w->rank - 1];
        if (w->rank != n->rank || w->shape[w->rank - 2] != (int64_t)K || nc < 1 || nc >= 64 ||  // (wide ones have fusions of their own)
            c->size() != (int64_t)M * nc)
          continue;
        TRY(realize(be, w));  // a view of the parameter
        if (w->stype != ST_BF16 || w->strides[w->rank - 2] != 1) continue;
        bool shared = true;  // one matrix for every row: batch axes of extent 1 or stride 0
        for (int i = 0; i + 2 < w->rank; ++i) shared = shared && (w->shape[i] == 1 || w->strides[i] == 0);
        // (the stride between columns of a single column is never used)
        if (!shared || (uintptr_t)data_ptr(w) % 16 || (nc > 1 && w->strides[w->rank - 1] % 8)) continue;
        members.push_back(c);
      }
      {
        GemvProDesc d;
        std::memset(&d, 0, sizeof(d));
        d.pro = PRO_NONE;
        d.a = (const float *)g.a;
        d.rows = M;
        d.a_rstride = g.sam;
        d.m.K = K;
        d.m.b_stype = ST_BF16;
        d.m.n_prob = 1;
        d.m.p[0].b = g.b;
        d.m.p[0].c = g.c;
        d.m.p[0].c_add = g.c_add;
        d.m.p[0].sbn = N > 1 ? g.sbn : (int64_t)K;  // (the stride between columns of a single column is never used)
        d.m.p[0].N = N;
        double bytes = uniq(A, sao) + uniq(B, sbo) + (double)n->size() * 4, flops = 2.0 * M * N * K;
        for (cg_tensor *c : members) {
          cg_tensor *w = c->in[1];
          TRY(alloc_result(be, c, ST_F32));
          auto &pr = d.m.p[d.m.n_prob++];
          pr.b = data_ptr(w);
          pr.c = (float *)c->st->ptr;
          pr.N = (uint32_t)w->shape[w->rank - 1];
          pr.sbn = pr.N > 1 ? w->strides[w->rank - 1] : (int64_t)K;
          bytes += (double)pr.N * K * 2 + (double)M * pr.N * 4;
          flops += 2.0 * M * pr.N * K;
        }
        {
          KernelScope ks(be, "gemv_rows_bf16", bytes, flops);
          if (be->trace_shapes) {
            char buf[96];
            snprintf(buf, sizeof buf, "gemv_rows_bf16[multi%d,M%u,K%u,N%.0f]", d.m.n_prob, M, K, flops / (2.0 * M * K));
            ks.rename(buf);
          }
          HIPCHK(be, launch_gemv_pro(be->lc(), d));
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
    std::vector<cg_tensor *> group, group_add, group_bias;  // a member, the add that takes its value, its bias vector
    const bool bias_row = addend && be->addend_is_row;  // `addend` is a vector added to every row
    if (n->gemm_candidate && (!addend || bias_row) && !ep && !ex.w && batch == 1 && g.bf16_math && g.a_stype == ST_BF16 &&
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
        // a sibling whose only reader adds a bias vector to it: the launch stores the sum, as that add's value
        cg_tensor *add = c->bias_user, *bv = nullptr;
        if (add) {
          if (refs(c) != 1 || add->op != N_BIN || add->bias_of != c || add->size() != c->size()) continue;
          bv = bias_vector_of(add->in[add->in[0] == c ? 1 : 0], add);
          if (!bv) continue;
          TRY(realize(be, bv));
          if (!bias_vector_ready(bv)) continue;
        }
        group.push_back(c);
        group_add.push_back(add);
        group_bias.push_back(bv);
      }
      if (group.size() < 2) group.clear();  // pairs (gate / up) keep their own launches and epilogues
    }
    if (!group.empty()) {
      g.n_group = 1;
      g.grp_b[0] = g.b;
      g.grp_c[0] = g.c;
      g.grp_n[0] = N;
      if (bias_row) {
        g.grp_bias[0] = (const float *)data_ptr(addend);
        *added = true;
      }
      for (size_t i = 0; i < group.size(); ++i) {
        cg_tensor *c = group[i], *dest = group_add[i] ? group_add[i] : c;
        TRY(alloc_result(be, dest, ST_F32));
        g.grp_b[g.n_group] = data_ptr(c->in[1]);
        g.grp_c[g.n_group] = (float *)dest->st->ptr;
        g.grp_bias[g.n_group] = group_bias[i] ? (const float *)data_ptr(group_bias[i]) : nullptr;
        g.grp_n[g.n_group] = (uint32_t)c->in[1]->shape[2];
        g.N += g.grp_n[g.n_group];
        ++g.n_group;
      }
    }
    // q / k / v of an attention that asked for its rotation and transposition in this launch's epilogue
    if (RopeGemmRequest *rq = be->rope_request; rq && group.size() == 2) {
      cg_tensor *members[3] = {n, group[0], group[1]};
      GemmDesc t = g;
      bool all = true;
      for (int i = 0; i < 3 && all; ++i) {
        int j = 0;
        while (j < 3 && rq->mm[j] != members[i]) ++j;
        if (j == 3) all = false;
        else if (j < 2) {
          t.rope_role[i] = 1;
          t.rope_out[i] = rq->out[j];
          t.rope_out16[i] = rq->out16[j];
          t.rope_cos[i] = rq->cos[j];
          t.rope_sin[i] = rq->sin[j];
          t.rope_cs_ss[i] = rq->cs_ss[j];
        } else {
          t.rope_role[i] = 2;
          t.rope_out16[i] = rq->out16[2];
        }
      }
      t.rope_s = rq->positions;
      t.rope_hd = rq->head_dim;
      if (all && gemm_rope_epilogue_ok(be->lc(), t)) {
        g = t;
        rq->applied = true;
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
        // ... and the caller may leave that pass to the norm that reads the sum
        if (be->ksum_request && n->size() % 4 == 0 && n->offset == 0) g.defer_reduce = 1;
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
                 g.dual_b ? ",gate*up" : group.empty() ? "" : g.rope_s ? ",grouped,rope" : ",grouped");
        ks.rename(buf);
      }
    }
    for (size_t i = 0; i < group.size(); ++i) {
      if (group_add[i]) {  // the add holds the value; letting go of its inputs deletes the product node
        if (e == hipSuccess) {
          finish_fused(group_add[i]);
        } else {
          storage_release(group_add[i]->st);
          group_add[i]->st = nullptr;
        }
        continue;
      }
      cg_tensor *c = group[i];
      forget_gemm_candidate(c);
      c->op = N_REAL;
      drop_inputs(c);
    }
    if (g.defer_reduce && e == hipSuccess) {  // the caller owns the slices now
      be->ksum_ws = ws;
      be->ksum_splits = splits;
    } else {
      storage_release(ws);
    }
    storage_release(bt);
    HIPCHK(be, e);
  }
  if (n->gemv_candidate) forget_gemv_candidate(n);
  if (n->gemm_candidate) forget_gemm_candidate(n);
  n->op = N_REAL;
  drop_inputs(n);
  return CG_OK;
}

}  // namespace cgrt
