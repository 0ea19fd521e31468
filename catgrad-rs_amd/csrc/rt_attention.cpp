// rt_attention.cpp — part of the host runtime behind include/catgrad_hip.h (layout: rt_internal.hpp).
#include "rt_internal.hpp"

namespace cgrt {


// Attention of a decode step (models/llama.rs:77-112 with one query row):
//   matmul(softmax(matmul(q, K^T) / sqrt(d) + mask), V)
// in one launch that reads K and V rows in place from the cache; the [b, h, 1, T] scores and
// probabilities never exist in HBM.
// Attention over many query rows (prefill; models/llama.rs:95-107, gemma3.rs:153-186):
//   matmul(softmax(matmul(q, K^T) / sqrt(d) + mask), V)
// as one pass with online softmax (k_attn.hip); the [b, h, S, T] scores and probabilities are
// never written.  With the bf16 flag the products run on bf16 MFMA (keys from their bf16 twin, values
// from a bf16 V^T made once per call); without it every product is f32 and K / V are read as they lie.
int try_attn_prefill(cg_backend *be, cg_tensor *n, bool *done) {
  const bool f32 = !(be->flags & CG_FLAG_BF16);
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
  // (bf16 mode from 256 keys on: 4 x 16 heads x 256 x 256, d = 128 - two batched GEMMs, a softmax, the copy
  // of the transposed result and two casts, 44 us - take 21 us in one pass)
  if (T < (f32 ? 512 : 256) && !(be->flags & CG_FLAG_ATTN_ONE_PASS)) return CG_OK;
  if (nb > 65535 || heads > 65535) return CG_OK;
  cg_tensor *q = S->in[0];
  // queries and keys both still to be rotated: one launch for the two (each alone otherwise, below)
  // (the transposed bf16 values, when the projections' own launch has made them: released on every way out)
  struct Held {
    Storage *s = nullptr;
    ~Held() { storage_release(s); }
  } vt_made;
  const Storage *vt_of = nullptr;
  if (cg_tensor *kr = node_under_repeat_kv(S->in[1])) {
    bool paired = false;
    // ... or none at all: the projections still deferred rotate q and k in their epilogue
    if (!f32 && (d == 64 || d == 128)) TRY(try_qkv_rope_gemm(be, q, kr, node_under_repeat_kv(n->in[1]), &vt_made.s, &vt_of, &paired));
    if (!paired) TRY(try_rope_pair(be, q, kr, &paired));
  }
  MatOperand Kop, Vop;
  bool pk = false, pv = false;
  TRY(peel_repeat_kv(be, S->in[1], &Kop, &pk));
  TRY(peel_repeat_kv(be, n->in[1], &Vop, &pv));
  if (!pk || !pv) return CG_OK;  // operands get realised by the generic path below
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
  if (!f32 && (Kop.t->offset % 8 || Kop.strides[0] % 8 || Kop.strides[1] % 8 || Kop.strides[2] % 8 || Kop.strides[4] % 8)) return CG_OK;
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
  // the kernel reads mask rows and value columns 16 bytes at a time, and (bf16) the keys from their bf16 twin
  Storage *ksh = nullptr;
  const bool twin_ok = f32 || (Kop.t->st->grow_dim < 0 && Kop.t->st->bytes % 32 == 0);
  if ((mask && !a.m_vec) || T % 8 || !twin_ok) {
    storage_release(n->st);
    n->st = nullptr;
    return CG_OK;
  }
  Storage *vt = nullptr;
  bool vt_ready = false;
  const int64_t kvh = Kop.shape[1];
  if (f32) {
    a.f32 = 1;
    a.k = (const float *)data_ptr(Kop.t);
  } else {
    TRY(bf16_shadow(be, Kop.t->st, &ksh));
    a.k16 = (const uint16_t *)ksh->ptr + Kop.t->offset;
    // the values as the projections left them, [T, kv heads * d] read as [kv heads][T][d]: their transposed copy is there
    if (vt_made.s && vt_of == Vop.t->st && Vop.t->offset == 0 && Vop.strides[1] == d && Vop.strides[3] == kvh * d &&
        Vop.strides[4] == 1 && (nb == 1 || Vop.strides[0] == T * kvh * d) && (size_t)nb * kvh * d * T * 2 <= vt_made.s->bytes) {
      vt = vt_made.s;
      vt_made.s = nullptr;
      vt_ready = true;
    } else {
      TRY(dev_alloc(be, (size_t)nb * kvh * d * T * 2, &vt));
    }
  }
  if (!f32 && !vt_ready) {
    KernelScope ks(be, "transpose_cast_bf16", (double)nb * kvh * d * T * 6, 0);
    hipError_t te = launch_transpose_cast_bf16(be->lc(), data_ptr(Vop.t), ST_F32, vt->ptr, (uint32_t)T, (uint32_t)d,
                                               Vop.strides[3], (uint32_t)nb, (uint32_t)kvh, Vop.strides[0], Vop.strides[1]);
    if (te != hipSuccess) {
      storage_release(vt);
      return fail(be, CG_ERR_DEVICE, hipGetErrorString(te));
    }
  }
  if (vt) a.vt16 = (const uint16_t *)vt->ptr;
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


// The tensor that repeat_kv (helpers.rs:147-161: reshape, broadcast, reshape) and an optional transpose of the
// last two axes were applied to, when nobody else reads the views in between; null otherwise.
cg_tensor *node_under_repeat_kv(cg_tensor *t) {
  if (t->op == N_TRANSPOSE && refs(t) == 1 && t->rank == 4 &&
      ((t->p0 == 2 && t->p1 == 3) || (t->p0 == 3 && t->p1 == 2)))
    t = t->in[0];
  if (t->op != N_RESHAPE || refs(t) != 1 || t->rank != 4) return nullptr;
  cg_tensor *u = t->in[0];
  if (u->op != N_BROADCAST || refs(u) != 1 || u->rank != 5) return nullptr;
  cg_tensor *r5 = u->in[0];
  if (r5->op != N_RESHAPE || refs(r5) != 1 || r5->rank != 5 || r5->shape[2] != 1) return nullptr;
  return r5->in[0];
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


int try_attn_decode(cg_backend *be, cg_tensor *n, bool *done, AttnMergeLater *later) {
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
    // When the reader merges the partials (every one of its workgroups reads all of them), fewer and
    // longer key ranges pay: about one pass of a workgroup each, three ranges at least.  Swept on the
    // whole decode loop: T ~ 540: 4 ranges 1367, 5 1392, 6 1382, 8 1372 tokens/s; T ~ 200: 2 1415, 3 1421,
    // 4 1421, 8 1397.
    if (later && nb == 1 && ns <= ATTN_MERGE_MAX_SPLITS) ns = std::max<int64_t>((T + 109) / 110, std::min<int64_t>(3, (T + 31) / 32));
    if (ns >= 2 || T > ATTN_DECODE_MAX_T) {
      const int64_t chunk = (T + ns - 1) / ns;
      a.chunk = (uint32_t)chunk;
      a.splits = (uint32_t)((T + chunk - 1) / chunk);
      // the reader of the result merges the partials when it can (one row, few splits)
      if (later && nb == 1 && a.splits >= 2 && a.splits <= ATTN_MERGE_MAX_SPLITS && heads * a.splits <= 256 &&
          heads * d <= 2048 && d % 4 == 0)
        a.merge_later = 1;
      TRY(attn_decode_scratch(be, (size_t)bh * a.splits * (d + 4), (size_t)bh));
      a.part = be->attn_part;
      a.count = be->attn_count;
      if (a.merge_later) {
        later->part = a.part;
        later->splits = a.splits;
        later->heads = (uint32_t)heads;
        later->d = (uint32_t)d;
        later->deferred = true;
      }
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

}  // namespace cgrt
