// rt_moe.cpp — part of the host runtime behind include/catgrad_hip.h (layout: rt_internal.hpp).
#include "rt_internal.hpp"

namespace cgrt {


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
          const size_t words = 2 * (size_t)d.n_expert + (size_t)S * d.n_slot + 1 + moe_route_max_tiles(d);
          st = dev_alloc(be, words * 4, &route);
          if (st) {
            drop_h();
            return st;
          }
          uint32_t *rc = (uint32_t *)route->ptr, *ro = rc + d.n_expert, *rl = ro + d.n_expert, *rt = rl + (size_t)S * d.n_slot;
          {
            KernelScope ks(be, "experts_route", (double)S * d.n_slot * 8, 0);
            e = launch_moe_route(be->lc(), d, rc, ro, rl, rt);
          }
          f.route_tiles = d.route_tiles = rt;
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
  // The indices may be the router's choice that nothing has computed yet - column i of topk(softmax(logits))
  // for slot i (models/qwen3.rs:64-80) - and then this launch makes the choice itself, token by token, and
  // leaves values and indices in memory for their other readers: the router needs no launch of its own.
  cg_tensor *topk_ix = nullptr;
  SoftmaxMatch rsm;
  if (!glu) {
    bool fold = K < 4096;  // (deeper rows split k over the waves: another form of the kernel)
    for (const Member &m : members) {
      cg_tensor *t = m.idx;
      int64_t col = -1;
      while (fold && t->op != N_TOPK_INDEX) {
        if (t->op == N_RESHAPE && t->in[0] && t->in[0]->size() == t->size()) {
          t = t->in[0];
        } else if (t->op == N_SLICE && col < 0 && t->in[0] && t->p0 == t->rank - 1 && t->shape[t->rank - 1] == 1 && t->size() == S) {
          col = t->p1;  // one column of rows of choices
          t = t->in[0];
        } else {
          fold = false;
        }
      }
      if (!fold) break;
      if (topk_ix && t != topk_ix) fold = false;
      topk_ix = t;
      const int64_t k = t->shape[t->rank - 1];
      if (col < 0 || col >= k || k > 8 || t->size() != S * k || m.slot >= 8) fold = false;
      else d.router_col[m.slot] = (uint8_t)col;
    }
    if (fold && topk_ix) {
      cg_tensor *v = topk_ix->in[0], *x = v && v->op == N_TOPK ? v->in[0] : nullptr;
      const int64_t ne = x ? x->shape[x->rank - 1] : 0;
      fold = x && x->op != N_REAL && refs(x) == 1 && ne >= 1 && ne <= 64 && x->size() == S * ne && match_softmax(x, &rsm) &&
             !rsm.has_scale && !rsm.has_mask_const && !rsm.mask && rsm.src == rsm.x;
    }
    if (!fold) topk_ix = nullptr;
  }
  // indices: u32, one stride between consecutive tokens, the same stride in every slot
  int64_t istride0 = -1;
  for (const Member &m : members) {
    if (topk_ix) break;
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
  cg_tensor *norm_x = nullptr;
  if (!glu) {
    // the rows are an RMSNorm that every reader computes on its way in (norm_row_readers_ok): so does this launch
    RmsNormMatch rm;
    if (A->op != N_REAL && A->in[0] && norm_row_readers_ok(be, A->in[0], A, &rm) && gemv_pro_rows_ok(b_stype, 1, (uint32_t)K, PRO_RMSNORM)) {
      bool vec = true;
      if (rm.gamma) TRY(gamma_row_vector(be, rm.gamma, &vec));
      TRY(realize(be, rm.x));
      if (vec && rm.x->stype == ST_F32 && is_contiguous(rm.x) && (uintptr_t)data_ptr(rm.x) % 16 == 0 && rm.x->size() == S * K) {
        norm_x = rm.x;
        d.pro = PRO_RMSNORM;
        d.a = (const float *)data_ptr(rm.x);
        d.aux = rm.gamma ? (const float *)data_ptr(rm.gamma) : nullptr;
        d.a_bstride = K;
        d.aux_bstride = 0;
        d.a_by_token = 1;
        d.n_as_float = rm.n_as_float;
        d.eps = rm.eps;
        d.gamma_offset = rm.gamma_offset;
      }
    }
  }
  if (!glu && !norm_x) {
    TRY(realize(be, A));
    if (A->stype != ST_F32 || A->strides[2] != 1 || A->strides[0] % 4 || (uintptr_t)data_ptr(A) % 16) return CG_OK;
    d.pro = PRO_NONE;
    d.a = (const float *)data_ptr(A);
    d.a_bstride = A->strides[0];
    d.a_by_token = 1;
  } else if (glu) {
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
  cg_tensor *logits = nullptr;
  if (topk_ix) {
    // the logits (their launch comes first), then both results of the top-k as values in memory that the launch
    // below fills
    cg_tensor *v = retain(topk_ix->in[0]);
    int st = contiguous(be, rsm.src, &logits);
    if (!st && logits->stype != ST_F32) st = fail(be, CG_ERR_INTERNAL, "router logits are not f32");
    if (!st) st = alloc_result(be, v, ST_F32);
    if (!st) st = alloc_result(be, topk_ix, ST_U32);
    if (st) {
      node_release(logits);
      node_release(v);
      drop_outs();
      return st;
    }
    d.router_logits = (const float *)data_ptr(logits);
    d.router_n = (uint32_t)logits->shape[logits->rank - 1];
    d.router_stride = d.router_n;
    d.router_k = (uint32_t)v->p0;
    d.router_values = (float *)v->st->ptr;
    d.router_indices = (uint32_t *)topk_ix->st->ptr;
    v->op = N_REAL;
    v->pair = nullptr;
    drop_inputs(v);
    topk_ix->op = N_REAL;
    drop_inputs(topk_ix);
    node_release(v);
  }
  hipError_t e;
  {
    KernelScope ks(be, b_stype == ST_BF16 ? "gemv_experts_bf16" : "gemv_experts_f32", bytes, flops);
    e = launch_gemv_pro(be->lc(), d);
  }
  node_release(logits);
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

}  // namespace cgrt
