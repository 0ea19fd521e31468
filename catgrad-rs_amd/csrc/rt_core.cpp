// rt_core.cpp — part of the host runtime behind include/catgrad_hip.h (layout: rt_internal.hpp).
#include "rt_internal.hpp"

namespace cgrt {


int fail(cg_backend *be, int code, const std::string &msg) {
  if (be) be->err = msg;
  return code;
}


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
  noalloc_release_slot(be->device, be->noalloc_slot);
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
    if (n->glu_of && n->glu_of->glu_user == n) n->glu_of->glu_user = nullptr;
    if (n->op == N_TOPK_INDEX && n->in[0] && n->in[0]->pair == n) n->in[0]->pair = nullptr;
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
  if (n->glu_of) {
    if (n->glu_of->glu_user == n) n->glu_of->glu_user = nullptr;
    n->glu_of = nullptr;
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

}  // namespace cgrt
