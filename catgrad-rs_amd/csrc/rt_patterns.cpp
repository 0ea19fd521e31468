// rt_patterns.cpp — part of the host runtime behind include/catgrad_hip.h (layout: rt_internal.hpp).
#include "rt_internal.hpp"

namespace cgrt {


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
    // the bf16 copy is for a product that waits for these rows as its left operand: attention's p . V (a
    // batched product over heads, rank 4) or a recorded many-row product; for anybody else it would be a
    // third of the launch's traffic written for nobody
    bool only_gemms = false;
    if (root->rank >= 4 || gemm_readers(be, root, &only_gemms) > 0) st = twin_for_result(be, root, &d.y16);
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
  // The value may still be the k-slices of a split product (plus a residual): the kernel sums them on its way
  // in, in the order of the pass it replaces, and stores the sum where the value belongs.
  cg_tensor *ksum = view->op == N_KSUM && n % 4 == 0 && view->size() / n <= UINT32_MAX && view->stype == ST_F32 &&
                            (uintptr_t)data_ptr(view) % 16 == 0 && (uintptr_t)data_ptr(view->in[0]) % 16 == 0 &&
                            (!view->in[1] || (uintptr_t)data_ptr(view->in[1]) % 16 == 0)
                        ? view
                        : nullptr;
  if (!ksum) TRY(realize(be, view));
  if (ksum) {
    xs = retain(view);
    row_stride = n;
  } else if (rows_map(view, &rmap) && (rmap.d1 > 1 || rmap.d2 > 1) && (uintptr_t)data_ptr(view) % 16 == 0 &&
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
    double in_bytes = rs ? 8 : 4;
    if (ksum) {
      d.x_slices = (const float *)data_ptr(ksum->in[0]);
      d.x_n_slices = (uint32_t)ksum->p0;
      d.x_slice_stride = (uint64_t)ksum->size();
      d.x_add = ksum->in[1] ? (const float *)data_ptr(ksum->in[1]) : nullptr;
      d.x_out = (float *)data_ptr(ksum);
      in_bytes += 4.0 * ((double)d.x_n_slices + (d.x_add ? 1 : 0));  // (the 4 above: x_out, written)
    }
    if (only_gemms) {
      d.y16 = (uint16_t *)root->st->ptr;
    } else {
      d.y = (float *)root->st->ptr;
      if (to_gemms) st = twin_for_result(be, root, &d.y16);
    }
    KernelScope ks(be, "rmsnorm_fused", (double)root->size() * (in_bytes + (d.y ? 4 : 0) + (d.y16 ? 2 : 0)) + n * 4, 0);
    if (be->trace_shapes) {  // per-shape records: rmsnorm_fused[16384x1152,+res,f32+bf16]
      char buf[96];
      snprintf(buf, sizeof buf, "rmsnorm_fused[%ux%u%s%s%s,%s]", d.rows, d.n, ksum ? ",k-slices" : "", rs ? ",+res" : "",
               rmap.d1 > 1 || rmap.d2 > 1 ? ",strided" : "", !d.y ? "bf16" : d.y16 ? "f32+bf16" : "f32");
      ks.rename(buf);
    }
    hipError_t e = launch_rmsnorm(be->lc(), d);
    if (e != hipSuccess) st = fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
    else if (ksum) finish_fused(ksum);  // the sum is in memory now
  }
  node_release(xs);
  if (st) return st;
  finish_fused(root);
  *done = true;
  return CG_OK;
}


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


// realises the cos / sin tables of a matched rope; *ok = the kernels' layout requirements hold
int rope_tables(cg_backend *be, const RopeMatch &m, bool *ok) {
  TRY(realize(be, m.cb));
  TRY(realize(be, m.sb));
  auto table_ok = [&](const cg_tensor *t) {
    return t->stype == ST_F32 && t->strides[0] * (t->shape[0] != 1) == 0 &&
           t->strides[1] * (t->shape[1] != 1) == 0 && t->strides[3] == 1 && t->strides[2] % 4 == 0 &&
           (uintptr_t)data_ptr(t) % 16 == 0;
  };
  *ok = table_ok(m.cb) && table_ok(m.sb) && m.cb->strides[2] == m.sb->strides[2];
  return CG_OK;
}

// ... and the rotated tensor too
int rope_operands(cg_backend *be, const RopeMatch &m, bool *ok) {
  TRY(realize(be, m.x));
  return rope_tables(be, m, ok);
}


// gemma3.rs:99-117: q and k are RMS-normed per head - folded to [b * heads * s, head_dim] - between the head
// transpose and the rotation.  When the rotated tensor of `m` is such a norm, still deferred and read by nothing
// but the rotation, the rotation's kernel can norm each row on its way in: *out says so and holds what it reads
// (the norm's input as a [b, h, s, d] view, realised here, and gamma).  out->on = false: not that shape.
static int rope_normed_input(cg_backend *be, cg_tensor *root, const RopeMatch &m, RopeNormed *out) {
  *out = RopeNormed();
  if (be->flags & CG_FLAG_NO_PATTERNS) return CG_OK;
  const int64_t n = root->shape[3];
  if ((n != 64 && n != 128 && n != 256) || m.x->op == N_REAL || refs(m.x) != 3) return CG_OK;
  cg_tensor *t = m.x;
  while (t->op == N_RESHAPE && t->in[0] && (t == m.x || refs(t) == 1) && t->in[0]->rank >= 1 &&
         t->in[0]->shape[t->in[0]->rank - 1] == n)
    t = t->in[0];
  if (t->op == N_REAL || (t != m.x && refs(t) != 1)) return CG_OK;
  RmsNormMatch rm;
  if (!match_rmsnorm(t, &rm)) return CG_OK;
  cg_tensor *v = rm.x;
  while (v->op == N_RESHAPE && v->in[0] && v->in[0]->rank >= 1 && v->in[0]->shape[v->in[0]->rank - 1] == n) v = v->in[0];
  if (v->rank != 4 || !std::equal(v->shape, v->shape + 4, root->shape) || v->dtype != CG_F32) return CG_OK;
  if (rm.gamma) {
    bool vec = false;
    TRY(gamma_row_vector(be, rm.gamma, &vec));
    if (!vec) return CG_OK;
  }
  TRY(realize(be, v));
  bool fits = v->stype == ST_F32 && v->strides[3] == 1 && (uintptr_t)data_ptr(v) % 16 == 0;
  for (int i = 0; i < 3; ++i)
    if (v->strides[i] % 4) fits = false;
  if (!fits) return CG_OK;
  out->on = true;
  out->rm = rm;
  out->view = v;
  out->gamma = rm.gamma ? (const float *)data_ptr(rm.gamma) : nullptr;
  return CG_OK;
}


// Fills the rope kernel's descriptor for `root` (matched as m) writing to `out` with the given element
// strides.  *xs receives a retained tensor the descriptor reads from (release it after the launch);
// *ok = false: layout requirements not met, nothing to launch.
int rope_describe(cg_backend *be, cg_tensor *root, const RopeMatch &m, float *out, const int64_t *o_strides,
                  uint16_t *out16, RopeDesc *dsc, cg_tensor **xs_out, bool *ok, const RopeNormed *normed) {
  *ok = false;
  *xs_out = nullptr;
  bool tables = false;
  const bool nrm = normed && normed->on;
  if (nrm) TRY(rope_tables(be, m, &tables));  // (the rotated tensor itself stays deferred: the kernel norms its input)
  else TRY(rope_operands(be, m, &tables));
  if (!tables) return CG_OK;
  cg_tensor *x = nrm ? normed->view : m.x, *cb = m.cb, *sb = m.sb;
  cg_tensor *xs = retain(x);
  bool fits = x->stype == ST_F32 && x->strides[3] == 1 && (uintptr_t)data_ptr(x) % 16 == 0;
  for (int i = 0; i < 3; ++i)
    if (x->strides[i] % 4) fits = false;
  if (!fits) {
    node_release(xs);
    xs = nullptr;
    TRY(materialize(be, x, &xs));
  }
  const int64_t dim = root->shape[3];
  RopeDesc &d = *dsc;
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
  if (nrm) {
    d.norm = 1;
    d.gamma = normed->gamma;
    d.n_as_float = normed->rm.n_as_float;
    d.eps = normed->rm.eps;
    d.gamma_offset = normed->rm.gamma_offset;
  }
  *xs_out = xs;
  *ok = true;
  return CG_OK;
}

// Launches the rope kernel for `root` (matched as m) into `out` with the given element strides.
// *done = false: layout requirements not met, nothing was launched.
int rope_into(cg_backend *be, cg_tensor *root, const RopeMatch &m, float *out, const int64_t *o_strides,
              const char *name, bool *done, uint16_t *out16) {
  RopeDesc d;
  cg_tensor *xs = nullptr;
  bool ok = false;
  TRY(rope_describe(be, root, m, out, o_strides, out16, &d, &xs, &ok));
  if (!ok) return CG_OK;
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

// The queries and the keys of an attention, both straight from apply_rope_embedding and both still
// deferred: one launch rotates both.  *done = false: nothing was changed (each is then realised alone).
int try_rope_pair(cg_backend *be, cg_tensor *rq, cg_tensor *rk, bool *done) {
  *done = false;
  if (be->flags & CG_FLAG_NO_PATTERNS) return CG_OK;
  if (rq == rk || rq->op == N_REAL || rk->op == N_REAL) return CG_OK;
  RopeMatch mq, mk;
  if (!match_rope(rq, &mq) || !match_rope(rk, &mk)) return CG_OK;
  bool tq = false, tk = false;
  RopeNormed norms[2];
  TRY(rope_normed_input(be, rq, mq, &norms[0]));
  TRY(rope_normed_input(be, rk, mk, &norms[1]));
  if (norms[0].on) TRY(rope_tables(be, mq, &tq));
  else TRY(rope_operands(be, mq, &tq));
  if (norms[1].on) TRY(rope_tables(be, mk, &tk));
  else TRY(rope_operands(be, mk, &tk));
  if (!tq || !tk) return CG_OK;
  cg_tensor *roots[2] = {rq, rk};
  const RopeMatch *ms[2] = {&mq, &mk};
  RopeDesc d[2];
  cg_tensor *xs[2] = {nullptr, nullptr};
  int st = CG_OK;
  bool ok = true;
  for (int i = 0; i < 2 && !st && ok; ++i) {
    st = alloc_result(be, roots[i], ST_F32);
    uint16_t *y16 = nullptr;
    if (!st) st = twin_for_result(be, roots[i], &y16);
    if (!st) st = rope_describe(be, roots[i], *ms[i], (float *)roots[i]->st->ptr, roots[i]->strides, y16, &d[i], &xs[i], &ok, &norms[i]);
  }
  if (!st && ok) {
    KernelScope ks(be, "rope_fused", (double)(rq->size() + rk->size()) * 8, 0);
    if (be->trace_shapes && (norms[0].on || norms[1].on)) ks.rename("rope_fused[normed]");
    hipError_t e = launch_rope_pair(be->lc(), d[0], d[1]);
    if (e != hipSuccess) st = fail(be, CG_ERR_DEVICE, hipGetErrorString(e));
  }
  for (int i = 0; i < 2; ++i) node_release(xs[i]);
  if (st || !ok) {  // nothing was launched: both stay deferred
    for (int i = 0; i < 2; ++i) {
      storage_release(roots[i]->st);
      roots[i]->st = nullptr;
    }
    return st;
  }
  finish_fused(rq);
  finish_fused(rk);
  *done = true;
  return CG_OK;
}

// The queries, keys and values of a prefill attention whose projections are all still deferred (models/llama.rs:77-94:
// three linears on one input - with or without a bias -, `reshape [b, s, heads, d]`, `transpose(1, 2)`, then
// apply_rope_embedding on q and k): the grouped launch of the three products rotates q and k where they are still
// accumulators and stores a transposed bf16 copy of v beside v itself, so neither the rotation nor the
// transposition is a launch of its own.  Heads of 64 or 128 columns; the linears see the batch folded into the rows.
// *done = false: nothing was changed beyond realising the products.  On success *vt owns the transposed values
// ([sequences][kv heads][d][positions], bf16) of the storage *v_st.
int try_qkv_rope_gemm(cg_backend *be, cg_tensor *rq, cg_tensor *rk, cg_tensor *v, Storage **vt, const Storage **v_st,
                      bool *done) {
  *done = false;
  *vt = nullptr;
  *v_st = nullptr;
  if (!(be->flags & CG_FLAG_BF16) || (be->flags & CG_FLAG_NO_PATTERNS)) return CG_OK;
  if (rq == rk || rq->op == N_REAL || rk->op == N_REAL || !v || v->op == N_REAL) return CG_OK;
  RopeMatch mq, mk;
  if (!match_rope(rq, &mq) || !match_rope(rk, &mk)) return CG_OK;
  const int64_t hd = rq->shape[3];
  if (hd != 64 && hd != 128) return CG_OK;
  // x = transpose(1, 2) of reshapes of a deferred product [1, b * s, heads * hd], or of that product plus its bias
  // vector; `readers`: the references x must have (the rotation reads it three times and nobody else may: its
  // product is never stored as such), 0 = any.  *top: the node whose realisation launches the product.
  auto product_under = [hd](cg_tensor *x, int readers, cg_tensor **top) -> cg_tensor * {
    if (x->op != N_TRANSPOSE || x->rank != 4 || (readers && refs(x) != readers)) return nullptr;
    if (!((x->p0 == 1 && x->p1 == 2) || (x->p0 == 2 && x->p1 == 1)) || x->shape[3] != hd) return nullptr;
    cg_tensor *t = x->in[0];
    while (t->op == N_RESHAPE && (!readers || refs(t) == 1)) t = t->in[0];
    *top = t;
    if (t->op == N_BIN && t->bias_of && (!readers || refs(t) == 1) && (t->in[0] == t->bias_of || t->in[1] == t->bias_of)) t = t->bias_of;
    if (t->op != N_MATMUL || (readers && refs(t) != 1) || !t->gemm_candidate || t->dtype != CG_F32 || t->rank != 3) return nullptr;
    if (t->shape[0] != 1 || t->shape[1] != x->shape[0] * x->shape[2] || t->shape[2] != x->shape[1] * hd) return nullptr;
    return t;
  };
  cg_tensor *top_q = nullptr, *top_k = nullptr, *top_v = nullptr;
  cg_tensor *pq = product_under(mq.x, 3, &top_q), *pk = product_under(mk.x, 3, &top_k), *pv = product_under(v, 0, &top_v);
  if (!pq || !pk || !pv || pq == pk || pq == pv || pk == pv) return CG_OK;
  const int64_t positions = rq->shape[2], seqs = rq->shape[0];
  if (rk->shape[2] != positions || rk->shape[0] != seqs || v->shape[2] != positions || v->shape[0] != seqs ||
      pk->shape[2] != pv->shape[2] || positions % 4)
    return CG_OK;
  bool tq = false, tk = false;
  TRY(rope_tables(be, mq, &tq));
  TRY(rope_tables(be, mk, &tk));
  if (!tq || !tk) return CG_OK;
  RopeGemmRequest req;
  cg_tensor *roots[2] = {rq, rk};
  const RopeMatch *ms[2] = {&mq, &mk};
  int st = CG_OK;
  for (int i = 0; i < 2 && !st; ++i) {
    st = alloc_result(be, roots[i], ST_F32);
    if (!st) st = twin_for_result(be, roots[i], &req.out16[i]);
    if (!st) {
      req.out[i] = (float *)roots[i]->st->ptr;
      req.cos[i] = (const float *)data_ptr(ms[i]->cb);
      req.sin[i] = (const float *)data_ptr(ms[i]->sb);
      req.cs_ss[i] = positions == 1 ? 0 : ms[i]->cb->strides[2];
    }
  }
  Storage *t = nullptr;
  if (!st) st = dev_alloc(be, (size_t)pv->shape[1] * pv->shape[2] * 2, &t);
  if (!st) {
    req.out16[2] = (uint16_t *)t->ptr;
    req.mm[0] = pq;
    req.mm[1] = pk;
    req.mm[2] = pv;
    req.positions = (uint32_t)positions;
    req.head_dim = (uint32_t)hd;
    cg_tensor *keep = retain(top_v);  // (the products leave the graph as they are realised)
    be->rope_request = &req;
    st = realize(be, top_q);
    be->rope_request = nullptr;
    if (!st && req.applied && keep->op == N_REAL) *v_st = keep->st;
    node_release(keep);
  }
  if (st || !req.applied) {  // the rotation and the transposition stay with their own kernels
    for (int i = 0; i < 2; ++i) {
      storage_release(roots[i]->st);
      roots[i]->st = nullptr;
    }
    storage_release(t);
    return st;
  }
  finish_fused(rq);
  finish_fused(rk);
  *vt = t;
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


// The gate of `act(gate) * up` by structure alone (no reference counts: while a term is being recorded the
// caller still holds values that it lets go of before anything is realised), or null.
cg_tensor *glu_gate_of(const cg_tensor *root) {
  if (root->dtype != CG_F32 || !is_bin(root, E_MUL_F)) return nullptr;
  const cg_tensor *act = root->in[0], *g = nullptr;
  if (is_bin(act, E_MUL_F) && is_sigmoid_of(act->in[1], &g) && g == act->in[0]) return const_cast<cg_tensor *>(g);
  if (is_gelu_of(act, &g)) return const_cast<cg_tensor *>(g);
  return nullptr;
}


// the same tensor, or two reshapes of one tensor to one shape (each linear folds the batch into its rows itself)
bool same_rows(const cg_tensor *a, const cg_tensor *b) {
  if (a == b) return true;
  return a->op == N_RESHAPE && b->op == N_RESHAPE && a->in[0] == b->in[0] && a->rank == b->rank &&
         std::equal(a->shape, a->shape + a->rank, b->shape);
}


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
    if (cg_tensor *bv = (!folded && !plain_row && (mm->gemv_candidate || (mm->gemm_candidate && mm->bias_user == root)))
                            ? bias_vector_of(other, root)
                            : nullptr) {
      // linear(x) + bias: the grouped product launch adds the vector to every row (few rows: always; many rows:
      // where q / k / v go out as one launch - otherwise *added stays false and the add runs as an op of its own)
      TRY(realize(be, bv));
      if (!bias_vector_ready(bv)) return CG_OK;
      be->addend_is_row = true;
      int st = realize_matmul(be, mm, bv, &added, nullptr);
      be->addend_is_row = false;
      if (st) return st;
    } else {
      // A residual that is itself the unsummed k-slices of the previous block's product stays that way for
      // now: the norm under this many-row product sums it (realize_matmul sees to it that it is summed by
      // the time it is added).
      if (other->op != N_KSUM || mm->gemv_candidate) TRY(realize(be, other));
      if (other->stype != ST_F32 || !is_contiguous(other)) return CG_OK;
      be->ksum_request = be->ksum_flush_node == root;
      be->ksum_ws = nullptr;
      const int st = realize_matmul(be, mm, other, &added, nullptr);
      be->ksum_request = false;
      if (st) {
        storage_release(be->ksum_ws);
        be->ksum_ws = nullptr;
        return st;
      }
    }
    if (!added) return CG_OK;  // the product is realised; the generic add takes it from here
    // mm now holds the sum and nobody else can see it: root takes over its storage
    root->st = mm->st;
    root->st->rc.fetch_add(1);
    root->stype = mm->stype;
    root->offset = mm->offset;
    if (folded) contiguous_strides(root->rank, root->shape, root->strides);  // products are dense
    else std::copy(mm->strides, mm->strides + mm->rank, root->strides);
    if (Storage *ws = be->ksum_ws) {
      // the product was left as its k-slices: root becomes their pending sum (plus the residual)
      be->ksum_ws = nullptr;
      const int64_t len = (int64_t)be->ksum_splits * root->size();
      cg_tensor *slices = new_node(be, CG_F32, 1, &len);
      slices->st = ws;
      slices->stype = ST_F32;
      slices->strides[0] = 1;
      cg_tensor *keep = retain(other);
      drop_inputs(root);
      root->op = N_KSUM;
      root->ew = 0;
      root->in[0] = slices;
      root->in[1] = keep;
      root->p0 = be->ksum_splits;
      *done = true;
      return CG_OK;
    }
    finish_fused(root);
    *done = true;
    return CG_OK;
  }
  return CG_OK;
}


// ---- a sum of rows, each scaled by a value of its own -------------------------------------------------
// How a MoE block ends (llm/qwen_moe.py after deepseek.rs:163-165 and qwen3.rs:104-123):
//   sum_k h_k * broadcast(value_k)  +  shared * broadcast(sigmoid(gate))  +  residual
// with transposes and reshapes in between that only move axes of extent 1.  One op at a time that is four
// launches of the generic evaluator (its operand limit, the views and the broadcast of a computed value each
// end a program); launch_row_scaled_sum adds the terms in the same order, each product and sum rounded alone.
namespace {
struct SumTerm {
  cg_tensor *x, *s;  // rows; one value per row (or null)
  bool sigmoid;
};

// rows of `d` values with at most one leading axis longer than 1: views between such shapes keep the row order
bool rows_shape(const cg_tensor *t, int64_t d) {
  if (t->rank < 1 || t->shape[t->rank - 1] != d) return false;
  int big = 0;
  for (int i = 0; i + 1 < t->rank; ++i) big += t->shape[i] != 1;
  return big <= 1;
}

// through deferred reshapes / transposes that nobody else reads and that only move axes of extent 1
cg_tensor *under_unit_views(cg_tensor *n, const cg_tensor *root, int64_t d) {
  while ((n->op == N_RESHAPE || n->op == N_TRANSPOSE) && (n == root || refs(n) == 1) && n->in[0] &&
         n->in[0]->size() == n->size() && rows_shape(n, d) && rows_shape(n->in[0], d))
    n = n->in[0];
  return n;
}

// one value per row: a realised f32 view whose axes are broadcast (stride 0), of extent 1, or step through
// `rows` values at one stride
bool row_scalar_view(const cg_tensor *t, int64_t rows, int64_t *stride) {
  if (t->op != N_REAL || t->stype != ST_F32) return false;
  int64_t count = 1, st = 0, expect = -1;
  for (int i = t->rank - 1; i >= 0; --i) {
    if (t->shape[i] == 1 || t->strides[i] == 0) continue;
    if (expect < 0) st = t->strides[i];
    else if (t->strides[i] != expect) return false;
    expect = t->strides[i] * t->shape[i];
    count *= t->shape[i];
  }
  if (count != rows) return false;
  *stride = st;
  return true;
}

// x, or x * (one value per row), the value possibly through a sigmoid
bool sum_term(cg_tensor *n, const cg_tensor *root, int64_t rows, int64_t d, SumTerm *out) {
  n = under_unit_views(n, root, d);
  out->x = n;
  out->s = nullptr;
  out->sigmoid = false;
  if (n->op == N_REAL || !is_bin(n, E_MUL_F) || refs(n) != 1) return rows_shape(n, d) && n->size() == rows * d;
  for (int side = 0; side < 2; ++side) {
    cg_tensor *sc = under_unit_views(n->in[side], root, d), *x = under_unit_views(n->in[1 - side], root, d);
    if (!rows_shape(x, d) || x->size() != rows * d || sc->size() != rows * d) continue;
    int64_t st;
    if (sc->op == N_REAL && sc->strides[sc->rank - 1] == 0 && row_scalar_view(sc, rows, &st)) {
      out->x = x;
      out->s = sc;  // a broadcast of values in memory is a view
      return true;
    }
    // the same still deferred: views, ending in a broadcast, of a value that takes a launch of its own whoever
    // reads it (the values a top-k chose); the caller checks the strides once the views are realised
    if (sc->op == N_BROADCAST && refs(sc) == 1) {
      const cg_tensor *src = sc->in[0];
      while ((src->op == N_RESHAPE || src->op == N_SLICE || src->op == N_TRANSPOSE || src->op == N_BROADCAST) && src->in[0])
        src = src->in[0];
      if ((src->op == N_TOPK || src->op == N_REAL) && src->dtype == CG_F32 && sc->in[0]->size() == rows) {
        out->x = x;
        out->s = sc;
        return true;
      }
    }
    const cg_tensor *arg = nullptr;
    if (sc->op == N_BROADCAST && refs(sc) == 1 && sc->in[0]->size() == rows && is_sigmoid_of(sc->in[0], &arg) &&
        arg->size() == rows) {
      out->x = x;
      out->s = const_cast<cg_tensor *>(arg);
      out->sigmoid = true;
      return true;
    }
  }
  return rows_shape(n, d) && n->size() == rows * d;  // some other product: a term like any value
}

// the terms of a chain of additions, left to right (a + b == b + a exactly, so either side may be the chain)
bool sum_chain(cg_tensor *n, const cg_tensor *root, int64_t rows, int64_t d, std::vector<SumTerm> &terms, int depth) {
  n = under_unit_views(n, root, d);
  if (depth < 16 && n->op != N_REAL && is_bin(n, E_ADD_F) && (n == root || refs(n) == 1) && n->size() == rows * d) {
    for (int side = 0; side < 2; ++side) {
      cg_tensor *chain = under_unit_views(n->in[side], root, d), *leaf = n->in[1 - side];
      const bool zero = chain->op == N_CONST && is_constf(chain, 0u);  // the accumulator's first value: 0 + t = t
      if (!zero && !(chain->op != N_REAL && is_bin(chain, E_ADD_F) && refs(chain) == 1)) continue;
      if (!zero && !sum_chain(chain, root, rows, d, terms, depth + 1)) return false;
      SumTerm t;
      if (!sum_term(leaf, root, rows, d, &t)) return false;
      terms.push_back(t);
      return true;
    }
    // two values
    SumTerm a, b;
    if (!sum_term(n->in[0], root, rows, d, &a) || !sum_term(n->in[1], root, rows, d, &b)) return false;
    terms.push_back(a);
    terms.push_back(b);
    return true;
  }
  SumTerm t;
  if (!sum_term(n, root, rows, d, &t)) return false;
  terms.push_back(t);
  return true;
}
}  // namespace

int try_row_scaled_sum(cg_backend *be, cg_tensor *root, bool *done) {
  if (root->dtype != CG_F32 || !is_bin(root, E_ADD_F) || root->rank < 2) return CG_OK;
  const int64_t d = root->shape[root->rank - 1];
  if (d < 4 || d % 4 || !rows_shape(root, d)) return CG_OK;
  const int64_t rows = root->size() / d;
  if (rows < 1 || rows > 4096) return CG_OK;
  std::vector<SumTerm> terms;
  if (!sum_chain(root, root, rows, d, terms, 0)) return CG_OK;
  int scaled = 0;
  for (const SumTerm &t : terms) scaled += t.s != nullptr;
  // (two terms, or none with a scale: the product epilogues and the plain kernels do those)
  if (terms.size() < 3 || terms.size() > ROW_SUM_MAX_TERMS || !scaled) return CG_OK;
  RowSumDesc g;
  std::memset(&g, 0, sizeof(g));
  g.rows = (uint32_t)rows;
  g.d = (uint32_t)d;
  g.n_terms = (uint32_t)terms.size();
  for (size_t j = 0; j < terms.size(); ++j) {
    cg_tensor *x = terms[j].x, *sc = terms[j].s;
    TRY(realize(be, x));
    if (sc) TRY(realize(be, sc));
    int64_t rs = 0, ss = 0;
    if (!rows_view(x, &rs) || x->strides[x->rank - 1] != 1 || rs % 4 || (uintptr_t)data_ptr(x) % 16) return CG_OK;
    if (sc && !row_scalar_view(sc, rows, &ss)) return CG_OK;
    g.t[j].x = (const float *)data_ptr(x);
    g.t[j].x_rs = rs;
    g.t[j].s = sc ? (const float *)data_ptr(sc) : nullptr;
    g.t[j].s_rs = ss;
    g.t[j].sigmoid = terms[j].sigmoid ? 1 : 0;
  }
  TRY(alloc_result(be, root, ST_F32));
  g.out = (float *)root->st->ptr;
  g.out_rs = d;
  {
    KernelScope ks(be, "row_scaled_sum", (double)rows * d * 4 * (terms.size() + 1), 2.0 * rows * d * terms.size());
    HIPCHK(be, launch_row_scaled_sum(be->lc(), g));
  }
  finish_fused(root);
  *done = true;
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
  TRY(try_row_scaled_sum(be, root, done));
  if (*done) return CG_OK;
  TRY(try_gemv_add(be, root, done));
  if (*done) return CG_OK;
  return try_binary(be, root, done);
}

}  // namespace cgrt
