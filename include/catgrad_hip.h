/*
 * catgrad_hip.h — C ABI of the MI355X (gfx950) tensor backend for catgrad's Interpreter.
 *
 * One function per method of `trait Backend`
 * (catgrad/src/interpreter/backend/mod.rs:22-82).  A Rust shim implements
 * `Backend for HipBackend` by forwarding every trait method to the function of the
 * same name below; the evaluator half of this header (cg_term_*, cg_interp_*) is the
 * stand-in caller used where no Rust toolchain exists: it restates
 * catgrad/src/abstract_interpreter/eval.rs and catgrad/src/interpreter/tensor_op.rs.
 *
 * Conventions
 *  - every function returns an int status (CG_OK == 0); no C++ exception crosses the ABI;
 *  - tensor arguments are BORROWED (the callee never consumes a reference);
 *    every `cg_tensor **out` receives a NEW reference the caller must cg_tensor_release;
 *  - the dtype tag (F32 / U32) is carried by the handle, like `TaggedTensor`
 *    (catgrad/src/interpreter/types.rs:16-26);
 *  - binary ops demand identical shape and dtype, reductions act on the last axis and
 *    keep the rank (backend/mod.rs:16-21);
 *  - where the reference panics (shape mismatch, sin/cos/topk on U32, matmul asserts,
 *    u32 division by zero) the call returns a non-zero status and cg_last_error()
 *    holds the message;
 *  - a backend instance owns one HIP stream; calls on one backend must not overlap.
 */
#ifndef CATGRAD_HIP_H
#define CATGRAD_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
/* the functions declared here are the library's exported symbols (it is built with hidden visibility) */
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

typedef struct cg_backend cg_backend;
typedef struct cg_tensor cg_tensor;

/* core::Dtype (catgrad/src/category/core.rs:20-24) */
typedef enum { CG_F32 = 0, CG_U32 = 1 } cg_dtype;

enum {
  CG_OK = 0,
  CG_ERR_SHAPE = 1,    /* BackendError::ShapeError and every "Shape mismatch" panic */
  CG_ERR_DTYPE = 2,    /* op not defined for this dtype, or mixed dtypes */
  CG_ERR_ARG = 3,      /* null pointer, axis out of range, ... */
  CG_ERR_DEVICE = 4,   /* a HIP call failed */
  CG_ERR_OOM = 5,
  CG_ERR_ARITH = 6,    /* u32 division by zero (Rust panics) */
  CG_ERR_INTERNAL = 7,
  /* evaluator errors: abstract_interpreter/types.rs:95-112 */
  CG_ERR_MULTIPLE_READ = 20,
  CG_ERR_MULTIPLE_WRITE = 21,
  CG_ERR_CYCLE = 22,
  CG_ERR_TYPE = 23,
  CG_ERR_ARITY = 24,
  CG_ERR_LOAD = 25,
  CG_ERR_APPLY = 26,
  /* weight files */
  CG_ERR_IO = 40,      /* open / stat / mmap failed */
  CG_ERR_FORMAT = 41   /* not a well-formed safetensors file */
};

/* cg_backend_create flags */
enum {
  /* F32 tensors of rank >= 2 handed over with cg_from_f32 are stored as bf16 and every
   * matmul rounds its operands to bf16 (f32 accumulation).  Everything else stays f32, except a
   * value computed only to be such an operand (the gated activation of an MLP over many rows),
   * which may be kept in the rounded form the matmul would read anyway. */
  CG_FLAG_BF16 = 1u,
  /* run every op when it is issued instead of deferring and fusing */
  CG_FLAG_EAGER = 2u,
  /* keep deferring, but never dispatch to the hand-written pattern kernels (softmax, RMSNorm,
   * RoPE, gated activations): everything goes through the generic fused-program kernels */
  CG_FLAG_NO_PATTERNS = 4u,
  /* use the one-pass attention kernels over many query rows for every sequence length (by default
   * only from 512 keys on - 256 with CG_FLAG_BF16 -, where the score tensor they avoid is large); bf16 or f32 products, as
   * CG_FLAG_BF16 says */
  CG_FLAG_ATTN_ONE_PASS = 8u
};

#define CG_MAX_RANK 8

/* ---- backend lifetime ---------------------------------------------------------- */
int cg_backend_create(int device, uint32_t flags, cg_backend **out);
void cg_backend_destroy(cg_backend *be);
/* message of the last failed call on this backend (never NULL) */
const char *cg_last_error(const cg_backend *be);
/* wait for the stream; reports errors only the data can reveal (u32 division by zero, gather index
 * out of bounds) raised by kernels since the last wait */
int cg_sync(cg_backend *be);
/* issue the kernels a deferred tensor still needs, without waiting.  No counterpart in the reference,
 * whose backends compute inside every call: the HIP backend records calls and computes when a value
 * is read (cg_to_f32 / cg_to_u32 / cg_compare) or here; a no-op for the oracle */
int cg_tensor_realize(cg_backend *be, cg_tensor *t);
/* cg_tensor_realize, then start copying a small tensor (<= 4088 bytes, e.g. the sampled token) to
 * pinned host memory behind the work queued so far.  A later cg_to_f32 / cg_to_u32 of the same
 * handle waits for that copy only, so the caller can keep the device busy with the next step while
 * it reads this one.  Larger or strided tensors are left alone (their read synchronises as usual).
 * No counterpart in the reference, whose to_vec is the only way out of a tensor. */
int cg_tensor_prefetch(cg_backend *be, cg_tensor *t);
/* "hip-gfx950" or "ndarray-oracle" */
const char *cg_backend_name(const cg_backend *be);

/* ---- handles: BackendTensor: Clone + BackendTensorOps (backend/mod.rs:84-86) ----- */
cg_tensor *cg_tensor_retain(cg_tensor *t);     /* Clone: O(1) */
void cg_tensor_release(cg_tensor *t);          /* Drop */
int cg_tensor_rank(const cg_tensor *t);
int cg_tensor_shape(const cg_tensor *t, size_t *dims); /* BackendTensorOps::shape; host only */
cg_dtype cg_tensor_dtype(const cg_tensor *t);
size_t cg_tensor_size(const cg_tensor *t);     /* Shape::size (core.rs:35-37) */

/* ---- Backend methods -------------------------------------------------------------- */
/* zeros (mod.rs:26, ndarray.rs:53-65) */
int cg_zeros(cg_backend *be, const size_t *dims, int rank, cg_dtype dtype, cg_tensor **out);
/* ndarray_from_vec_f32 / _u32 (mod.rs:28-38, ndarray.rs:67-89): CG_ERR_SHAPE when
 * n != product(dims) */
int cg_from_f32(cg_backend *be, const float *data, size_t n, const size_t *dims, int rank,
                cg_tensor **out);
int cg_from_u32(cg_backend *be, const uint32_t *data, size_t n, const size_t *dims, int rank,
                cg_tensor **out);
/* An F32 tensor from bf16 bit patterns: what the weight loader of
 * catgrad-llm/examples/llama/main.rs:309-312 does on the host (widen every bf16 to f32, then
 * ndarray_from_vec_f32), with the widening left to the device.  With CG_FLAG_BF16 a tensor of
 * rank >= 2 keeps the file's bits as its storage: nothing is widened or rounded. */
int cg_from_bf16(cg_backend *be, const uint16_t *bits, size_t n, const size_t *dims, int rank,
                 cg_tensor **out);
/* `n` tensors of one shape and dtype as one tensor of shape [n, ...]: the value of the chain
 * reshape([1, ...]) + concat(.., 0) in concat_moe_experts (catgrad-llm/examples/llama/main.rs:217-236),
 * built with one allocation and n copies instead of n - 1 growing concatenations. */
int cg_stack(cg_backend *be, cg_tensor *const *parts, size_t n, cg_tensor **out);
/* cast (mod.rs:40, ndarray.rs:97-114): f32->u32 is Rust `as` (truncate, saturate, NaN->0) */
int cg_cast(cg_backend *be, cg_tensor *x, cg_dtype target, cg_tensor **out);
/* matmul (mod.rs:41, ndarray.rs:116-122, 549-615) */
int cg_matmul(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **out);
/* add sub mul div pow lt eq (mod.rs:42-48, ndarray.rs:124-198, 401-453) */
int cg_add(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **out);
int cg_sub(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **out);
int cg_mul(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **out);
int cg_div(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **out);
int cg_pow(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **out);
int cg_lt(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **out);
int cg_eq(cg_backend *be, cg_tensor *a, cg_tensor *b, cg_tensor **out);
/* sin cos neg (mod.rs:49-51, ndarray.rs:200-222, 433-441) */
int cg_sin(cg_backend *be, cg_tensor *x, cg_tensor **out);
int cg_cos(cg_backend *be, cg_tensor *x, cg_tensor **out);
int cg_neg(cg_backend *be, cg_tensor *x, cg_tensor **out);
/* broadcast reshape transpose (mod.rs:52-54, ndarray.rs:259-273, 311-317, 347-371) */
int cg_broadcast(cg_backend *be, cg_tensor *x, const size_t *dims, int rank, cg_tensor **out);
int cg_reshape(cg_backend *be, cg_tensor *x, const size_t *dims, int rank, cg_tensor **out);
int cg_transpose(cg_backend *be, cg_tensor *x, size_t dim0, size_t dim1, cg_tensor **out);
/* max sum argmax (mod.rs:55-57, ndarray.rs:224-246, 455-493, 522-529) */
int cg_max(cg_backend *be, cg_tensor *x, cg_tensor **out);
int cg_sum(cg_backend *be, cg_tensor *x, cg_tensor **out);
int cg_argmax(cg_backend *be, cg_tensor *x, cg_tensor **out);
/* cg_argmax into memory the caller brings.  No counterpart in the reference: it is for callers that
 * cannot allocate device memory (code under HIP graph capture, serving loops with a fixed footprint,
 * harnesses that forbid hipMalloc).  `x` must already be in memory (an uploaded tensor, or one passed
 * through cg_tensor_realize) and `out` a contiguous U32 tensor in memory shaped like x with a last
 * axis of 1; both stay the caller's.  The call makes no hipMalloc / hipFree and creates no handle: the
 * per-chunk accumulators of long rows that are split over workgroups go to a fixed 16 KiB slice of an
 * array in the library's device image (12 bytes per row and chunk; a shape needing more is refused with
 * CG_ERR_ARG).  Each GPU holds one such array of 8 slices (128 KiB); a backend takes a free slice of its
 * device at its first call and keeps it until it is destroyed, so calls of different backends never share
 * scratch memory and the calls of one backend are ordered by its stream; with all 8 slices of a device
 * taken by live backends the call is refused (CG_ERR_DEVICE).  A slice keeps the last call's contents. */
int cg_argmax_into(cg_backend *be, cg_tensor *x, cg_tensor *out);
/* topk (mod.rs:58, ndarray.rs:248-257, 495-520): f32 only; values f32, indices u32 */
int cg_topk(cg_backend *be, cg_tensor *x, size_t k, cg_tensor **values, cg_tensor **indices);
/* compare (mod.rs:59, ndarray.rs:337-343): *equal = 1 iff same shape and all elements == */
int cg_compare(cg_backend *be, cg_tensor *a, cg_tensor *b, int *equal);
/* concat index slice arange (mod.rs:60-79, ndarray.rs:275-335, 373-399, 91-95) */
int cg_concat(cg_backend *be, cg_tensor *x, cg_tensor *y, size_t dim, cg_tensor **out);
int cg_index(cg_backend *be, cg_tensor *x, size_t dim, cg_tensor *indices, cg_tensor **out);
int cg_slice(cg_backend *be, cg_tensor *x, size_t dim, size_t start, size_t len,
             cg_tensor **out);
int cg_arange(cg_backend *be, size_t end, cg_tensor **out);
/* to_vec (mod.rs:81, ndarray.rs:46-51): row-major copy-out; n must equal the size */
int cg_to_f32(cg_backend *be, cg_tensor *x, float *dst, size_t n);
int cg_to_u32(cg_backend *be, cg_tensor *x, uint32_t *dst, size_t n);

/* ---- tracing (no counterpart in the reference) -------------------------------------
 * When enabled every kernel launch is bracketed by two events on the backend's stream.
 * cg_trace_report writes one line per kernel name: "name launches total_ms bytes flops".
 * on = 2 additionally keys the records of matmuls, RMSNorms and elementwise programs by problem shape
 * ("gemm_mfma_bf16[b1,512x2048x2048,s4]", "rmsnorm_fused[16384x1152,+res,+norm,bf16]", "ew_fused[n8192,i5,in3]").
 */
int cg_trace_enable(cg_backend *be, int on);
/* Peak probes (no counterpart in the reference): what this device gives a plain 16-byte grid-stride
 * copy of `bytes` (GB/s, read + write counted) and a register-resident MFMA issue loop
 * (operand CG_F32: v_mfma_f32_32x32x2_f32, otherwise bf16 v_mfma_f32_32x32x16_bf16; TFLOP/s).
 * Benchmarks report them beside the data-sheet peaks. */
int cg_peak_copy_gbs(cg_backend *be, size_t bytes, int iters, double *gbs);
int cg_peak_mfma_tflops(cg_backend *be, cg_dtype operand, int iters, double *tflops);
/* Clock probe (no counterpart in the reference): `iters` launches of the bf16 product C[m, n] = A[m, k] . B[n, k]^T
 * on pseudo-random operands (m, n multiples of 128, k of 64) through the library's own GEMM dispatch; *tflops is
 * their rate and *clock_mhz the shader clock their main loops ran at (shader-clock ticks over 100 MHz ticks,
 * read inside the kernel).  m == 0: the register-resident bf16 MFMA loop of cg_peak_mfma_tflops instead.  A
 * GEMM draws more power than the bare loop and is clocked lower; its MFMA fraction is a fraction of that clock. */
int cg_peak_gemm_clock(cg_backend *be, size_t m, size_t n, size_t k, int iters, double *tflops, double *clock_mhz);
int cg_trace_reset(cg_backend *be);
/* returns the number of bytes needed (including the NUL); writes at most cap bytes */
size_t cg_trace_report(cg_backend *be, char *buf, size_t cap);
/* Launches by kernel family since the backend was created (or since the last call with reset != 0),
 * one line per name, "name count"; counted whether or not tracing is on.  The hand-written pattern
 * kernels have names of their own ("softmax_fused", "rmsnorm_fused", "rope_fused", "swiglu_fused",
 * "attn_decode", "gemv_rowdot_bf16", ...); what no pattern took runs as a generic program ("ew_fused",
 * "row_fused", "reduce_sum" / "reduce_max" / "reduce_argmax").  A caller that expects a model's hot ops
 * to be pattern kernels can assert that here.  Returns the bytes needed (including the NUL); writes at
 * most cap bytes.  Zero-count names are listed after a reset. */
size_t cg_launch_counts(cg_backend *be, int reset, char *buf, size_t cap);
/* counters: launches issued, bytes allocated from the device, bytes held in the pool */
int cg_stats(cg_backend *be, uint64_t *launches, uint64_t *device_bytes, uint64_t *pool_bytes);

/* ==================================================================================
 * Evaluator: core::Term, Environment, Parameters, Interpreter::{new,eval}
 * (catgrad/src/category/core.rs, catgrad/src/interpreter/interpreter.rs:14-37,
 *  catgrad/src/abstract_interpreter/eval.rs:18-184)
 * ================================================================================== */
typedef struct cg_term cg_term;
typedef struct cg_env cg_env;
typedef struct cg_params cg_params;

/* core::Object (core.rs:69-76) */
typedef enum { CG_OBJ_NAT = 0, CG_OBJ_DTYPE = 1, CG_OBJ_TYPE = 2, CG_OBJ_SHAPE = 3,
               CG_OBJ_TENSOR = 4 } cg_object;

/* core::Operation flattened (core.rs:92-241); order of TensorOp follows tensor_op.rs:15-41 */
typedef enum {
  CG_OP_COPY = 0,
  CG_OP_LOAD,            /* payload: path */
  CG_OP_DEF,             /* payload: path of a definition in the environment */
  CG_OP_PACK, CG_OP_UNPACK, CG_OP_SHAPE, CG_OP_DTYPE,      /* TypeOp */
  CG_OP_NAT_CONST,       /* payload: nat */
  CG_OP_NAT_MUL, CG_OP_NAT_ADD,
  CG_OP_DTYPE_CONST,     /* payload: dtype */
  CG_OP_ADD, CG_OP_SUB, CG_OP_MUL, CG_OP_DIV, CG_OP_NEG, CG_OP_POW, CG_OP_LT, CG_OP_EQ,
  CG_OP_COS, CG_OP_SIN,                                    /* Map(ScalarOp) */
  CG_OP_NAT_TO_U32, CG_OP_CAST, CG_OP_MATMUL,
  CG_OP_SCALAR_F32,      /* payload: f32 */
  CG_OP_SCALAR_U32,      /* payload: u32 */
  CG_OP_SUM, CG_OP_MAX, CG_OP_ARGMAX, CG_OP_TOPK, CG_OP_BROADCAST, CG_OP_RESHAPE,
  CG_OP_TRANSPOSE, CG_OP_SLICE, CG_OP_CONCAT, CG_OP_ARANGE, CG_OP_INDEX,
  CG_OP__COUNT
} cg_opcode;

/* abstract_interpreter::Value (types.rs:69-75) */
typedef enum { CG_VAL_NAT = 0, CG_VAL_DTYPE = 1, CG_VAL_SHAPE = 2, CG_VAL_TENSOR = 4 } cg_value_kind;
typedef struct cg_value {
  int kind;                 /* cg_value_kind */
  size_t nat;               /* CG_VAL_NAT */
  int dtype;                /* CG_VAL_DTYPE */
  int rank;                 /* CG_VAL_SHAPE */
  size_t dims[CG_MAX_RANK]; /* CG_VAL_SHAPE */
  cg_tensor *tensor;        /* CG_VAL_TENSOR */
} cg_value;

/* Term construction: nodes are numbered from 0 in creation order. */
int cg_term_create(cg_term **out);
void cg_term_destroy(cg_term *t);
int cg_term_add_node(cg_term *t, cg_object label, uint32_t *node_id);
/* payload: path for LOAD/DEF (NUL-terminated, '.'-separated), else NULL;
 * scalar: nat for NAT_CONST, dtype for DTYPE_CONST, the bit pattern for SCALAR_F32/U32 */
int cg_term_add_op(cg_term *t, cg_opcode op, const char *path, uint64_t scalar,
                   const uint32_t *sources, size_t n_sources,
                   const uint32_t *targets, size_t n_targets, uint32_t *edge_id);
int cg_term_set_boundary(cg_term *t, const uint32_t *sources, size_t n_sources,
                         const uint32_t *targets, size_t n_targets);
/* number of hyperedges, and of layers of the layered topological order
 * (ssa/mod.rs:24-76); CG_ERR_CYCLE if the term is cyclic */
int cg_term_stats(cg_term *t, size_t *n_ops, size_t *n_layers);

/* Environment.definitions (pass/to_core.rs:19-22): path -> term.  The env borrows the term. */
int cg_env_create(cg_env **out);
void cg_env_destroy(cg_env *e);
int cg_env_define(cg_env *e, const char *path, cg_term *term);

/* Parameters (abstract_interpreter/parameters.rs:9): path -> tensor (retained) */
int cg_params_create(cg_params **out);
void cg_params_destroy(cg_params *p);
int cg_params_set(cg_params *p, const char *path, cg_tensor *t);

/* the table itself: number of entries, the i-th path (valid until the table changes), lookup
 * (*out is a new reference; CG_ERR_LOAD when the path is absent), removal (0 or 1 entries go) */
size_t cg_params_len(const cg_params *p);
const char *cg_params_key(const cg_params *p, size_t i);
int cg_params_get(const cg_params *p, const char *path, cg_tensor **out);
int cg_params_remove(cg_params *p, const char *path);

/* Interpreter::eval (interpreter.rs:29-31).  args are borrowed; results[i].tensor are new
 * references.  n_results must equal the number of term targets.  On failure *err_id holds the
 * offending node or edge id (may be NULL). */
int cg_interp_eval(cg_backend *be, const cg_env *env, const cg_params *params, cg_term *term,
                   const cg_value *args, size_t n_args, cg_value *results, size_t n_results,
                   uint32_t *err_id);
/* The same, taking its values by value as Interpreter::run does (interpreter.rs:33-37): the caller's
 * reference to every tensor argument passes to the evaluator, on success and on failure.  A cache
 * tensor handed over this way is owned by nobody else while the term runs, which is what lets
 * `concat(2, cache, new)` append in place even when an op inside the term forces evaluation. */
int cg_interp_eval_owned(cg_backend *be, const cg_env *env, const cg_params *params, cg_term *term,
                         const cg_value *args, size_t n_args, cg_value *results, size_t n_results,
                         uint32_t *err_id);
/* message of the last failed cg_interp_eval / cg_term_* call in this thread */
const char *cg_interp_last_error(void);
/* counts Backend calls issued by cg_interp_eval since the last reset (per thread) */
uint64_t cg_interp_backend_calls(int reset);

/* ==================================================================================
 * Weight files: safetensors -> Parameters
 * (the loading loop of catgrad-llm/examples/llama/main.rs:288-333 and its post-processing,
 *  concat_moe_experts, main.rs:171-262)
 * ================================================================================== */
typedef struct cg_weights cg_weights;
typedef enum { CG_WDT_F32 = 0, CG_WDT_BF16 = 1, CG_WDT_OTHER = 2 } cg_weight_dtype;

/* Map a safetensors file and parse its header (main.rs:290-292: File::open, Mmap::map,
 * SafeTensors::deserialize).  Host only: no backend, no device.  CG_ERR_IO / CG_ERR_FORMAT with
 * the reason in cg_weights_last_error(). */
int cg_weights_open(const char *path, cg_weights **out);
void cg_weights_close(cg_weights *w);
size_t cg_weights_count(const cg_weights *w);
/* name, dtype, shape (up to 8 dims) and byte count of the i-th tensor, in file order of the header;
 * dtype_name receives the header's dtype string ("F32", "BF16", "F16", ...) */
const char *cg_weights_name(const cg_weights *w, size_t i);
int cg_weights_info(const cg_weights *w, size_t i, cg_weight_dtype *dtype, const char **dtype_name,
                    int *rank, size_t *dims, uint64_t *nbytes);
/* The i-th tensor on the device as an F32-tagged tensor (main.rs:297-321): F32 bytes as they are,
 * BF16 through cg_from_bf16; any other dtype is CG_ERR_DTYPE ("Unsupported dtype", main.rs:314-316). */
int cg_weights_tensor(cg_backend *be, const cg_weights *w, size_t i, cg_tensor **out);
/* Every tensor of `file` into `params` under the path prefix + name (main.rs:294-333);
 * *n_loaded (may be NULL) receives their number. */
int cg_params_load(cg_backend *be, cg_params *params, const char *file, const char *prefix,
                   size_t *n_loaded);
/* concat_moe_experts (main.rs:171-262): for every layer l < num_layers and every projection in
 * {down_proj, gate_proj, up_proj}, the entries prefix + "model.layers.{l}.mlp.experts.{e}.{proj}.weight",
 * e < num_experts, become one entry prefix + "model.layers.{l}.mlp.experts.{proj}.weight" of shape
 * [num_experts, ...] and are removed.  A (layer, projection) with no expert entry is skipped; one
 * with some but not all is CG_ERR_LOAD ("Expected {} experts for layer {} {}, found {}"). */
int cg_params_stack_experts(cg_backend *be, cg_params *params, const char *prefix,
                            size_t num_layers, size_t num_experts);
/* message of the last failed cg_weights_* / cg_params_load / cg_params_stack_experts call in
 * this thread */
const char *cg_weights_last_error(void);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif
#ifdef __cplusplus
}
#endif
#endif /* CATGRAD_HIP_H */
