// noalloc.cpp — the one entry point of the library that allocates nothing.
//
// cg_argmax_into is cg_argmax (catgrad/src/interpreter/backend/mod.rs:57, ndarray.rs:240-246,
// 469-493) for callers that cannot allocate device memory: code under HIP graph capture, serving
// loops with a fixed footprint, harnesses that forbid hipMalloc.  The caller brings the input and the
// output; the one piece of memory cg_argmax would otherwise take from the allocator - the per-chunk
// accumulators of a few long rows split over many workgroups (the argmax over a vocabulary) - lives
// in a fixed array in device memory that the library's code object carries.
//
// Every GPU the library runs on holds its own copy of that array, at its own address, until the
// process ends.  The array is cut into SLOTS slices; a backend takes a free slice of its device at its
// first call and keeps it until it is destroyed, so calls of different backends (different streams) never
// share scratch memory, and the calls of one backend are ordered by its stream.  A slice keeps the last
// call's contents: the split pass writes every word the merge pass reads, so nothing needs clearing.  When
// every slice of a device is taken the call is refused.
#include "rt.hpp"

#include <mutex>

using namespace cgk;

namespace {

// 12 bytes per (row, chunk); rows are split into at most 2 x CUs / rows chunks, so 16 KiB covers every
// shape on a device of up to 682 CUs.  Beyond it the call is refused.
enum : size_t { SCRATCH_BYTES = 16 * 1024 };
enum : int { MAX_DEVICES = 64, SLOTS = 8 };

// Device memory (128 KiB per GPU).  In host code this name is only a handle for hipGetSymbolAddress, never an
// address: the pointers below are what host code passes to kernels.
static __device__ __align__(256) unsigned char scratch[SLOTS * SCRATCH_BYTES];

std::mutex g_lock;
void *g_scratch_ptr[MAX_DEVICES];
uint32_t g_slots_taken[MAX_DEVICES];  // bit s: slice s of this device's array belongs to a live backend

}  // namespace

namespace cgrt {

int noalloc_init_device(int device) {
  if (device < 0 || device >= MAX_DEVICES) return CG_ERR_DEVICE;
  std::lock_guard<std::mutex> lk(g_lock);
  if (g_scratch_ptr[device]) return CG_OK;
  void *ptr = nullptr;
  if (hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) {
    (void)hipGetLastError();
    return CG_ERR_DEVICE;
  }
  g_scratch_ptr[device] = ptr;
  return CG_OK;
}

void noalloc_release_slot(int device, int slot) {
  if (device < 0 || device >= MAX_DEVICES || slot < 0 || slot >= SLOTS) return;
  std::lock_guard<std::mutex> lk(g_lock);
  g_slots_taken[device] &= ~(1u << slot);
}

}  // namespace cgrt

extern "C" int cg_argmax_into(cg_backend *be, cg_tensor *x, cg_tensor *out) {
  using cgrt::fail_with;
  if (!be || !x || !out || x->be != be || out->be != be) return fail_with(be, CG_ERR_ARG, "null or foreign argument");
  if (x->op != cgrt::N_REAL)
    return fail_with(be, CG_ERR_ARG, "cg_argmax_into: x is a deferred value; computing it would allocate "
                                     "(cg_tensor_realize it beforehand)");
  if (out->op != cgrt::N_REAL || out->host_copy)
    return fail_with(be, CG_ERR_ARG, "cg_argmax_into: out must be a tensor in memory with no host read in flight");
  if (x->rank == 0) return fail_with(be, CG_ERR_SHAPE, "reduction of a rank-0 tensor");
  const int64_t cols = x->shape[x->rank - 1];
  if (cols == 0) return fail_with(be, CG_ERR_SHAPE, "argmax of an empty lane");
  if (out->dtype != CG_U32 || out->stype != ST_U32) return fail_with(be, CG_ERR_DTYPE, "cg_argmax_into: out must be U32");
  bool shape_ok = out->rank == x->rank && out->shape[out->rank - 1] == 1;
  for (int i = 0; shape_ok && i + 1 < x->rank; ++i) shape_ok = out->shape[i] == x->shape[i];
  if (!shape_ok || !cgrt::tensor_is_contiguous(out))
    return fail_with(be, CG_ERR_SHAPE, "cg_argmax_into: out must be contiguous and shaped like x with a last axis of 1");
  if (x->size() == 0) return CG_OK;
  if (x->size() >= ((int64_t)1 << 32)) return fail_with(be, CG_ERR_ARG, "cg_argmax_into: tensor above 2^32 elements");
  uint32_t *ptr = nullptr;
  {
    std::lock_guard<std::mutex> lk(g_lock);
    if (be->device >= 0 && be->device < MAX_DEVICES) {
      if (be->noalloc_slot < 0)
        for (int s = 0; s < SLOTS; ++s)
          if (!(g_slots_taken[be->device] & (1u << s))) {
            g_slots_taken[be->device] |= 1u << s;
            be->noalloc_slot = s;
            break;
          }
      if (be->noalloc_slot >= 0 && g_scratch_ptr[be->device])
        ptr = (uint32_t *)((unsigned char *)g_scratch_ptr[be->device] + (size_t)be->noalloc_slot * SCRATCH_BYTES);
    }
  }
  if (!ptr)
    return fail_with(be, CG_ERR_DEVICE, "cg_argmax_into: every scratch slice of this device belongs to another live "
                                        "backend (8 per device)");
  if (hipSetDevice(be->device) != hipSuccess) return fail_with(be, CG_ERR_DEVICE, "hipSetDevice failed");
  return cgrt::reduce_into(be, x->dtype == CG_F32 ? R_ARGMAX_F : R_ARGMAX_U, x, out, ptr, SCRATCH_BYTES);
}
