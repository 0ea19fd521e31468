// rt.hpp — host runtime of the HIP backend: device allocator, ref-counted tensor handles with
// shape/stride views, deferred op nodes, and the scheduler that turns them into kernel launches.
//
// The `Backend` trait is called one op at a time (catgrad/src/interpreter/tensor_op.rs:15-41)
// and cannot see the graph, so fusion has to happen behind the interface: every call only
// checks shapes and records a node; kernels run when a value is needed on the host
// (to_vec / compare / cg_sync).  Views (transpose, slice, broadcast, mergeable reshape) never
// move data.
#pragma once
#include <hip/hip_runtime_api.h>

#include <atomic>
#include <cstdint>
#include <deque>
#include <map>
#include <unordered_map>
#include <string>
#include <vector>

#include "../../include/catgrad_hip.h"
#include "launch.hpp"

namespace cgrt {

struct RopeGemmRequest;

struct Storage {
  std::atomic<int> rc{1};
  void *ptr = nullptr;
  size_t bytes = 0;  // size class actually allocated
  cg_backend *be = nullptr;
  // set by concat when the buffer was laid out with spare room along one axis (KV cache)
  int grow_dim = -1;
  int64_t grow_cap = 0;
  // the layout the spare room belongs to: rank and element strides of the tensor it was allocated for.
  // Only a view with exactly these strides may be appended to in place (a transposed or regrouped
  // view of the same storage would write its new rows over live elements).
  int grow_rank = 0;
  int64_t grow_strides[CG_MAX_RANK] = {};
  // bf16 copy of this (f32) storage, element for element, made on demand for the MFMA GEMM and
  // shared by every matmul that reads a view of it (q/k/v, gate/up read the same activations)
  Storage *shadow = nullptr;
  // an attention mask's table of tile classes (launch_mask_tiles), made on demand and shared by every
  // layer that reads the mask; tiles_key = {element offset of the mask, rows, keys, query rows per tile, keys per tile}
  Storage *tiles = nullptr;
  int64_t tiles_key[5] = {-1, 0, 0, 0, 0};
};

enum NodeOp : uint8_t {
  N_REAL = 0,   // has storage
  N_CONST,      // every element equals cbits; no storage until someone needs a buffer
  N_ARANGE,
  N_BIN,        // ew = EwOp, in[0], in[1]
  N_UN,         // ew = EwOp, in[0]
  N_TRANSPOSE,  // p0, p1
  N_BROADCAST,
  N_RESHAPE,
  N_SLICE,      // p0 = dim, p1 = start
  N_MATMUL,
  N_REDUCE,     // p0 = ReduceKind
  N_CONCAT,     // p0 = dim
  N_INDEX,      // p0 = dim; in[0] = x, in[1] = indices
  N_KSUM,       // the k-slices of a split product, still to be summed: in[0] = the slices ([p0, size] floats),
                // in[1] = a value added to the sum (or null); the node already owns the storage of the result
  N_TOPK,       // p0 = k; in[0] = x: the k largest values of every row; `pair` is the node of their indices
  N_TOPK_INDEX  // in[0] = the N_TOPK node: realised together with it
};

struct TraceRec {
  uint64_t launches = 0;
  double ms = 0, bytes = 0, flops = 0;
};

struct PendingEvent {
  std::string name;
  hipEvent_t start, stop;
  double bytes, flops;
};

// ---- shared with noalloc.cpp -------------------------------------------------------------------
// Resolves, once per device and with that device current, the address of the library's fixed scratch
// array; cg_backend_create calls it.
int noalloc_init_device(int device);
void noalloc_release_slot(int device, int slot);  // a destroyed backend's slice of the scratch array
int reduce_into(cg_backend *be, int kind, cg_tensor *x, cg_tensor *out, uint32_t *scratch, size_t scratch_bytes);
int fail_with(cg_backend *be, int code, const std::string &msg);
bool tensor_is_contiguous(const cg_tensor *t);

}  // namespace cgrt

struct cg_tensor {
  std::atomic<int> rc{1};
  cg_backend *be = nullptr;
  cg_dtype dtype = CG_F32;
  int rank = 0;
  int64_t shape[CG_MAX_RANK] = {};
  // realised state
  cgrt::Storage *st = nullptr;
  int stype = cgk::ST_F32;
  int64_t strides[CG_MAX_RANK] = {};  // in elements
  int64_t offset = 0;                 // in elements
  // deferred state
  uint8_t op = cgrt::N_REAL;
  uint8_t ew = 0;
  cg_tensor *in[2] = {nullptr, nullptr};
  int64_t p0 = 0, p1 = 0;
  uint32_t cbits = 0;
  bool gemv_candidate = false;  // listed in cg_backend::gemv_candidates (a weak reference)
  bool gemm_candidate = false;  // listed in cg_backend::gemm_candidates (a weak reference)
  // `linear(x) + bias`: on a deferred few-row product, the add that reads it next to a broadcast bias
  // vector (a weak reference, cleared when that add lets go of its inputs); on the add, the product
  cg_tensor *bias_user = nullptr, *bias_of = nullptr;
  // `act(gate_proj(x)) * up_proj(x)`: on a deferred few-row product, the multiplication that gates with it (a
  // weak reference, cleared like bias_user); on that multiplication, the product
  cg_tensor *glu_user = nullptr, *glu_of = nullptr;
  // on a deferred N_TOPK node: its N_TOPK_INDEX node while that is alive (a weak reference)
  cg_tensor *pair = nullptr;
  // a value that depends on nothing but constants and aranges (a causal mask, say); such nodes are
  // shared: cse_key is this node's entry in cg_backend::shared_nodes while it is still deferred
  bool const_like = false;
  std::string *cse_key = nullptr;
  // cg_tensor_prefetch: a pinned host copy in flight (data, then the backend's error words) and the
  // event recorded behind the copy
  void *host_copy = nullptr;
  hipEvent_t host_ev = nullptr;

  int64_t size() const {
    int64_t n = 1;
    for (int i = 0; i < rank; ++i) n *= shape[i];
    return n;
  }
};

struct cg_backend {
  std::atomic<int> rc{1};
  int device = 0;
  uint32_t flags = 0;
  hipStream_t stream = nullptr;
  int n_cus = 256;
  std::string err;
  uint32_t *d_words = nullptr;  // [0] kernel error flags, [1] compare flag
  uint32_t *h_words = nullptr;  // pinned mirror
  // caching allocator
  std::map<size_t, std::vector<void *>> pool;
  uint64_t pool_bytes = 0, device_bytes = 0, launches = 0;
  // launches by kernel family (the names of the trace records), counted always: which hand-written
  // pattern kernels ran and how many launches fell to the generic programs ("ew_fused", "row_fused", ...)
  std::map<std::string, uint64_t> launch_counts;
  uint64_t uid = 0;  // distinct for every backend ever created in the process
  int noalloc_slot = -1;  // cg_argmax_into: this backend's slice of its device's scratch array, taken at the first call
  // tracing
  bool trace = false;
  bool trace_shapes = false;  // cg_trace_enable(be, 2): matmul records carry their shape
  std::map<std::string, cgrt::TraceRec> trace_recs;
  std::vector<cgrt::PendingEvent> trace_pending;

  // deferred small-M matmuls, so that those sharing their left operand (q/k/v, gate/up) can be
  // issued as one launch; weak references, removed when a node is realised or deleted
  std::vector<cg_tensor *> gemv_candidates;
  // the same for many-row products in bf16 mode (q/k/v of a prefill as one grouped GEMM)
  std::vector<cg_tensor *> gemm_candidates;
  hipEvent_t cur_start = nullptr, cur_stop = nullptr;  // set while a traced launch is issued
  // arange(n) is immutable and models ask for the same few n over and over (masks, RoPE tables of
  // every layer): one node per n, realised once
  std::map<int64_t, cg_tensor *> arange_cache;
  std::deque<int64_t> arange_order;  // the cached extents, oldest first (the oldest leaves when the cache is full)
  // deferred nodes built from constants and aranges only, by structure: every layer of a model asks
  // for the same causal mask, and gets the same node (weak references; an entry goes when its node is
  // realised or deleted)
  std::unordered_map<std::string, cg_tensor *> shared_nodes;
  // the most recent of them are kept alive (a realised mask survives from one block to the next, and
  // from one run to the next), oldest first
  std::deque<cg_tensor *> shared_keep;
  // a block-closing value (residual + linear over many rows) to realise at the next call, when its
  // creator has let go of the operands
  cg_tensor *flush_node = nullptr;
  // A block-closing `residual + linear(x)` realised ahead of its readers (run_pending_flush) may stop at the
  // k-slices of its product (N_KSUM): the RMSNorm that reads it next sums them on its way in.
  cg_tensor *ksum_flush_node = nullptr;  // that add, while it is being realised (a weak reference)
  bool ksum_request = false;   // set by try_gemv_add around its product
  // set by try_qkv_rope_gemm around the realisation of a q projection: the grouped q / k / v launch may rotate
  // the queries and keys and transpose the values in its epilogue
  cgrt::RopeGemmRequest *rope_request = nullptr;
  cgrt::Storage *ksum_ws = nullptr;  // handed back by realize_matmul: the slices (the caller owns them now)
  uint32_t ksum_splits = 0;
  // argmax over the row a one-row product is about to store (the logits of a greedy decode step): realize_reduce
  // names the product, try_gemv_prologue's launch leaves the argmax in pieces (GemvProDesc::amax_part) and hands
  // the records back
  cg_tensor *amax_want = nullptr;
  cgrt::Storage *amax_records = nullptr;
  uint32_t amax_n_records = 0;
  // set by try_gemv_add around realize_matmul when the addend it passes is a bias vector (one row added
  // to every row of the product) instead of a tensor shaped like the product
  bool addend_is_row = false;
  // recycled pinned buffers (PREFETCH_BYTES each) and events of cg_tensor_prefetch
  std::vector<void *> pinned_pool;
  std::vector<hipEvent_t> event_pool;
  // scratch of the decode attention that divides the keys over several workgroups: partial results
  // and one counter per (batch, head); the counters are zero whenever no launch is running
  float *attn_part = nullptr;
  uint32_t *attn_count = nullptr;
  size_t attn_part_floats = 0, attn_count_words = 0;

  // kernel launches go through this thread's queue; null when the backend launches inline (CG_FLAG_EAGER)
  cgk::LaunchQueue *queue = nullptr;
  cgk::LaunchCtx lc() const { return cgk::LaunchCtx{stream, n_cus, d_words, cur_start, cur_stop, queue}; }
  // the stream, once every launch handed to the queue has reached it: what anything but a kernel launch
  // (copies, events, synchronisation, frees) must use to keep program order
  hipStream_t ordered_stream() const {
    if (queue) queue->drain();
    return stream;
  }
};
