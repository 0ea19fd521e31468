// launch.hpp — host-callable launchers of the gfx950 kernels (one per kernel family).
// Every launcher enqueues on lc.stream and returns the launch status; nothing synchronises.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>
#include "program.hpp"
#include "launch_queue.hpp"

namespace cgk {

// bits of the device-side error word (checked by the host at synchronisation points)
enum : uint32_t { ERRF_DIV_ZERO = 1u, ERRF_INDEX_OOB = 2u };

struct LaunchCtx {
  hipStream_t stream;
  int n_cus;
  uint32_t *err_flag;  // device word
  // when tracing: events that receive the kernel's own begin / end timestamps
  hipEvent_t ev_start, ev_stop;
  // when set, launches are handed to this queue's thread instead of being made by the caller
  LaunchQueue *queue;
};

// Every kernel is launched through this: with null events it is an ordinary launch (made by the
// queue's thread when there is one); with events the runtime stamps them at the kernel's start and
// end (what a profiler reports as duration), and the launch is made here, after the queue drained.
template <typename... KArgs, typename... Args>
inline void cg_launch(const LaunchCtx &lc, void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t smem, Args &&...args) {
  if (lc.queue && !lc.ev_start && !lc.ev_stop) {
    lc.queue->launch(kernel, grid, block, smem, lc.stream, std::forward<Args>(args)...);
    return;
  }
  if (lc.queue) lc.queue->drain();
  hipExtLaunchKernelGGL(kernel, grid, block, smem, lc.stream, lc.ev_start, lc.ev_stop, 0, static_cast<KArgs>(args)...);
}
#define CG_LAUNCH(lc, kernel, grid, block, ...) cgk::cg_launch((lc), kernel, dim3(grid), dim3(block), 0, __VA_ARGS__)

// ---- k_ew.hip
hipError_t launch_ew(const LaunchCtx &lc, const Program &p, const OutDesc &o, uint64_t n_elems,
                     bool vec4);
// chunks > 1 (from reduce_split_chunks) splits every row over several workgroups; scratch then
// needs rows * chunks * 3 words
uint32_t reduce_split_chunks(const LaunchCtx &lc, uint32_t rows, uint32_t n);
hipError_t launch_reduce(const LaunchCtx &lc, int kind, const Program &p, void *out, uint32_t rows,
                         uint32_t n, bool vec4, uint32_t *scratch, uint32_t chunks);
// last-axis reduction of rows already in memory (unit stride along the row, n % 4 == 0, rows 16-byte
// aligned; bf16 rows are widened); kind = ReduceKind
hipError_t launch_reduce_plain(const LaunchCtx &lc, int kind, const void *x, int bf16, int64_t row_stride, void *out,
                               uint32_t rows, uint32_t n);
// reduction stages + final segment of a row program in one launch
hipError_t launch_row(const LaunchCtx &lc, const Program &p, const OutDesc &o, uint32_t rows,
                      uint32_t n, bool vec4);

// ---- k_misc.hip
// out[o, i, inner] = x[o, idx[i], inner]; x is read through its strides, out is contiguous
struct GatherDesc {
  const void *x;
  const uint32_t *idx;
  void *out;
  int32_t x_stype;         // ST_F32 / ST_U32 / ST_BF16 (bf16 is widened to f32)
  int32_t n_dims;          // rank of x (== rank of out)
  int32_t dim;             // gathered axis
  uint32_t out_dims[MAX_DIMS + 2];
  int64_t x_stride[MAX_DIMS + 2];
  uint32_t x_dim_size;     // extent of x along `dim`
  int32_t vec;             // 16-byte moves along the innermost axis are legal
};
hipError_t launch_gather(const LaunchCtx &lc, const GatherDesc &g, uint64_t n_out);
// stable descending top-k per row of a contiguous [rows, n] f32 tensor
// topk(softmax(x)) of rows of at most 256 values (row r at x + r * x_row_stride), probabilities as the softmax
// kernel for such rows computes them
hipError_t launch_softmax_topk(const LaunchCtx &lc, const float *x, int64_t x_row_stride, float *values, uint32_t *indices,
                               uint32_t rows, uint32_t n, uint32_t k);
hipError_t launch_topk(const LaunchCtx &lc, const float *x, float *values, uint32_t *indices,
                       uint32_t rows, uint32_t n, uint32_t k);
// *flag |= 1 if any element differs (u32: bit compare, f32: IEEE ==, so NaN differs)
hipError_t launch_compare(const LaunchCtx &lc, const void *a, const void *b, uint64_t n,
                          int is_f32, uint32_t *flag);
hipError_t launch_fill_u32(const LaunchCtx &lc, uint32_t *dst, uint32_t value, uint64_t n);
// Contiguous copy of a strided view whose unit-stride axis is not the last one (a materialised
// transpose): 64 x 64 tiles through LDS, reads along the input's unit-stride axis `j`, writes
// along the output's last axis.  4-byte output elements (bf16 input widened), or bf16 to bf16.
struct TransposeDesc {
  const void *x;
  void *out;
  int32_t x_stype, out_bf16;  // out_bf16: bf16 in, bf16 out (otherwise 4-byte output)
  uint32_t R, C;            // extents of axis j and of the last axis
  int64_t x_sc;             // input stride of the last axis (axis j has input stride 1)
  int64_t o_sj;             // output stride of axis j (the last axis has output stride 1)
  int32_t n_other;          // remaining axes, outermost first
  uint32_t odims[MAX_DIMS + 2];
  int64_t x_so[MAX_DIMS + 2], o_so[MAX_DIMS + 2];
};
hipError_t launch_transpose_copy(const LaunchCtx &lc, const TransposeDesc &d);
// peak probes: plain 16-byte copy; MFMA issue loop (out: grid * 256 floats)
hipError_t launch_peak_copy(const LaunchCtx &lc, const void *in, void *out, uint64_t bytes);
hipError_t launch_peak_mfma(const LaunchCtx &lc, int bf16, float *out, unsigned grid, int iters,
                            unsigned long long *clock_ticks = nullptr);

// ---- k_fused.hip
struct RmsNormDesc {
  const float *x;        // rows of n contiguous floats, row r at x + r * x_row_stride; with x_d1 or x_d2 above 1
                         // the row index splits as ((i0 * x_d1) + i1) * x_d2 + i2 and the row sits at
                         // x + i0 * x_row_stride + i1 * x_s1 + i2 * x_s2 (a transposed view, read in place)
  const float *gamma;    // n floats or null
  const float *residual; // contiguous [rows, n] added to the result, or null
  uint16_t *y16;         // bf16 copy of y (the operand of the GEMMs that follow), or null
  float *y;              // contiguous [rows, n]; null when only the bf16 form is wanted
  int64_t x_row_stride, x_s1, x_s2;
  uint32_t x_d1, x_d2;   // 0 counts as 1
  uint32_t rows, n;
  float n_as_float, eps, gamma_offset;  // gamma_offset: 0 (llama) or 1 (gemma's 1 + gamma)
  // x as the sum of the k-slices of a split product (non-null x_slices: x_n_slices slices, x_slice_stride
  // floats apart, each contiguous [rows, n]) plus x_add (contiguous [rows, n], or null), summed in the order
  // of launch_splitk_sum and also stored to x_out (contiguous [rows, n]); x itself is not read
  const float *x_slices, *x_add;
  float *x_out;
  uint32_t x_n_slices;
  uint64_t x_slice_stride;
  // Two norms in a row (non-null y_mid): the first result (with its residual) goes to y_mid, contiguous
  // [rows, n], and is normed again with gamma2 (n floats, not null) into y / y16.
  float *y_mid;
  const float *gamma2;
  float eps2, gamma2_offset;
};
hipError_t launch_rmsnorm(const LaunchCtx &lc, const RmsNormDesc &d);
// c[i] = ws[0][i] + ws[1][i] + ... + ws[splits - 1][i] (+ cadd[i]): the k-slices of a split product, n floats each
hipError_t launch_splitk_sum(const LaunchCtx &lc, const float *ws, float *c, uint64_t n, uint32_t splits, const float *cadd);

struct SoftmaxDesc {
  const float *x;        // row r at x + r * x_row_stride, unit stride along the row
  const float *mask;     // or null; row r reads mask + (r / mask_rows) * group + (r % mask_rows) * row
  float *y;              // contiguous [rows, n]
  uint16_t *y16;         // optional bf16 copy of y (vector kernels only), or null
  int64_t x_row_stride, mask_group_stride, mask_row_stride, mask_col_stride;
  uint32_t rows, n, mask_rows;
  int32_t has_scale, has_mask_const;
  float scale, mask_const;
  int32_t x_bf16;        // x points at bf16 rows (vector kernels only: n % 4 == 0, n >= 256, 8-byte aligned rows)
};
hipError_t launch_softmax(const LaunchCtx &lc, const SoftmaxDesc &d);

struct RopeDesc {
  const float *x, *cos, *sin;
  float *out;            // [b, h, s, dim] through o_sb / o_sh / o_ss (e.g. a slot of the KV cache)
  int64_t x_sb, x_sh, x_ss, cs_ss;  // element strides (unit stride along dim everywhere)
  int64_t o_sb, o_sh, o_ss;
  uint16_t *out16;       // optional bf16 copy, same layout as out, or null
  uint32_t b, h, s, dim, half;
  // optional (norm != 0, dim 64, 128 or 256): every row of x is RMS-normed first, the arithmetic of rmsnorm_kernel -
  // x / sqrt(sum(x * x) / n_as_float + eps) * (gamma_offset + gamma), gamma: dim floats or null
  int32_t norm;
  const float *gamma;
  float n_as_float, eps, gamma_offset;
};
hipError_t launch_rope(const LaunchCtx &lc, const RopeDesc &d);
// two rotations (the queries and the keys of an attention) as one launch
hipError_t launch_rope_pair(const LaunchCtx &lc, const RopeDesc &d0, const RopeDesc &d1);
// out = silu(gate) * up (gelu = 0) or gelu(gate) * up (gelu = 1); contiguous, n % 4 == 0
// out[r, :] = sum_j w_j[r] * x_j[r, :] in the order of the terms, w_j = 1 (s null), s_j[r] or sigmoid(s_j[r]):
// how a MoE block ends (models/qwen3.rs:104-123, deepseek.rs:163-165: the routed experts' rows weighted by
// their router values, the shared expert's row through its gate, the residual) as one launch.  Every product
// and every sum is rounded on its own (no fused multiply-add), like the one-op-at-a-time evaluation.
// rows of d floats, d % 4 == 0; x_j and out 16-byte aligned with row strides that are multiples of 4
enum { ROW_SUM_MAX_TERMS = 8 };
struct RowSumDesc {
  float *out;
  int64_t out_rs;
  uint32_t rows, d, n_terms;
  struct {
    const float *x, *s;
    int64_t x_rs, s_rs;
    int32_t sigmoid;
  } t[ROW_SUM_MAX_TERMS];
};
hipError_t launch_row_scaled_sum(const LaunchCtx &lc, const RowSumDesc &g);
hipError_t launch_glu(const LaunchCtx &lc, int gelu, const float *gate, const float *up, float *out,
                      uint64_t n, uint16_t *out16 = nullptr);  // out16: optional bf16 copy of out
// op: 0 add, 1 sub, 2 mul, 3 div; b is contiguous (b_period = 0) or a vector of b_period floats
// repeated; n % 4 == 0, b_period % 4 == 0
hipError_t launch_binary_f32(const LaunchCtx &lc, int op, const float *a, const float *b, float *out,
                             uint64_t n, uint32_t b_period, bool a_bf16 = false);  // a_bf16: a points at bf16 values

// One-query attention (a decode step): out[b, h, :] = softmax(q[b, h, :] . K[b, h, t, :] / scale + mask_const) . V
// K and V rows are read in place from the (growable) cache through strides; head h of a
// grouped-query model reads kv head h / rep (stride 0 along the repeat axis).
struct AttnDecodeDesc {
  const float *q, *k, *v;
  float *out;                       // contiguous [b, heads, d]
  int64_t q_sb, q_sh;               // q strides (unit stride along d)
  int64_t k_sb, k_skv, k_srep, k_st;  // K[b, kv, rep, t, :] strides (unit stride along d)
  int64_t v_sb, v_skv, v_srep, v_st;
  uint32_t b, heads, rep, t, d;
  int32_t has_scale, has_mask_const;
  float scale, mask_const;
  // optional: q is the projection before apply_rope_embedding; the kernel rotates it with this
  // position's cos / sin rows (d floats each, half-split) as it loads it
  const float *q_cos, *q_sin;
  // optional: the key / value rows of this step are not in the cache yet.  Row t_new (= t - 1) of
  // K and V is taken from k_new / v_new ([b, kv, d] through the strides; k_new is rotated with
  // kn_cos / kn_sin when those are set) and the first head of every kv group also stores both rows
  // into the cache (k and v are written through in that case).
  const float *k_new, *v_new, *kn_cos, *kn_sin;
  int64_t kn_sb, kn_skv, vn_sb, vn_skv;
  uint32_t t_new;
  // optional: the keys of one (batch, head) divided over `splits` workgroups of `chunk` keys each
  // (splits * chunk >= t).  part: b * heads * splits * (d + 2) floats of scratch; count: b * heads
  // words that are zero before the launch and zero again after it.  splits = 0: one workgroup per
  // (batch, head), t <= ATTN_DECODE_MAX_T.
  uint32_t splits, chunk;
  float *part;
  uint32_t *count;
  // splits >= 2 only: stop after the partials and leave their merge to the kernel that reads the result
  // (GemvProDesc::pro == PRO_ATTN_MERGE).  part then holds, per (batch, head, split), d values, the
  // maximum, the sum and two unused floats (stride d + 4: every record 16-byte aligned); out and count
  // are not touched.
  int32_t merge_later;
};
enum { ATTN_DECODE_MAX_T = 8192, ATTN_DECODE_MAX_D = 256 };
// keys one workgroup of the split form visits per pass over its chunk
uint32_t attn_decode_rows_per_pass(uint32_t d);
hipError_t launch_attn_decode(const LaunchCtx &lc, const AttnDecodeDesc &d);

// ---- k_attn.hip
// Attention over s query rows per head (bf16 MFMA, online softmax):
//   out[b, h, i, :] = softmax_j(q[b,h,i,:] . k[b,h,j,:] / scale + mask[b,h,i,j]) . v[b,h,j,:]
// q, v: f32 with unit stride along d (v through the kv-head strides as in AttnDecodeDesc; only read for
// rows whose every key is masked); k16: the keys as bf16 through the same kind of strides; vt16: the
// values as bf16, transposed, contiguous [b, kv heads, d, t]; t % 8 == 0;
// mask: additive f32 through its strides (0 = broadcast) or a constant; out [b, heads, s, d] through its strides.
struct AttnPrefillDesc {
  const float *q, *v, *mask;
  const uint16_t *k16, *vt16;          // bf16 products: keys as bf16 rows, values as bf16 V^T [b, kv, d, T]
  const float *k;                      // f32 products (f32 != 0): keys as f32 rows; k16 / vt16 unused
  int32_t f32;
  float *out;
  uint16_t *out16;                     // optional bf16 copy of out, same indexing
  int64_t o_sb, o_sh, o_ss;            // out[b, h, s, :] strides (unit stride along d)
  int64_t q_sb, q_sh, q_ss;
  int64_t k_sb, k_skv, k_srep, k_st;
  int64_t v_sb, v_skv, v_srep, v_st;
  int64_t m_sb, m_sh, m_ss, m_st;
  uint32_t b, heads, rep, s, t, d;
  int32_t has_scale, has_mask_const, m_vec;  // m_vec: mask rows allow 16-byte loads
  float scale, mask_const;
  // optional, for a mask shared by every batch and head (m_sb == m_sh == 0): the class of every
  // (query tile, key tile) pair from launch_mask_tiles with the tiling of attn_prefill_tiling - 0 = every
  // pair masked (the tile is skipped without being fetched), 2 = every value zero (the tile is computed
  // without reading the mask), 1 = anything else; row q of the table has tile_cols entries
  const uint8_t *tile_class;
  uint32_t tile_cols;
};
hipError_t launch_attn_prefill(const LaunchCtx &lc, const AttnPrefillDesc &d);
// query rows and keys per tile that launch_attn_prefill uses for this problem
void attn_prefill_tiling(const LaunchCtx &lc, const AttnPrefillDesc &d, uint32_t *q_rows, uint32_t *keys);
// out[qt * ceil(t / keys) + kt] = class of mask[qt * q_rows .., kt * keys ..] (values <= -3e38 count as masked);
// mask is [s, t] with unit stride along t and row stride m_ss
hipError_t launch_mask_tiles(const LaunchCtx &lc, const float *mask, int64_t m_ss, uint32_t s, uint32_t t, uint32_t q_rows,
                             uint32_t keys, uint8_t *out);

// ---- k_gemm.hip
struct GemmDesc {
  const void *a, *b;
  float *c;                  // contiguous [batch, M, N]
  int32_t a_stype, b_stype;  // ST_F32 or ST_BF16
  uint32_t M, N, K;
  int64_t sam, sak;          // element strides of A[m, k]
  int64_t sbk, sbn;          // element strides of B[k, n]
  uint32_t nb0, nb1;         // batch = nb0 * nb1 (row-major)
  int64_t sa_b0, sa_b1, sb_b0, sb_b1;  // batch strides (0 = broadcast)
  int32_t bf16_math;         // 1: operands rounded to bf16, bf16 MFMA; 0: f32 MFMA
  // split-K (bf16 fast path only): partial products go to workspace[split][batch][M][N]
  float *workspace;
  uint32_t splits, k_per_split;
  // optional epilogue of the one-row kernels: C = A . B + c_add (c_add laid out like C)
  const float *c_add;
  // split along k (splits > 1): leave the slices in the workspace; the caller sums them (launch_splitk_sum, or
  // the RMSNorm kernel on its way in)
  int32_t defer_reduce;
  // expert-indirect batches (one-row kernels only): when b_index is set, batch z reads its B
  // matrix at b + b_index[z * b_index_stride] * sb_index instead of the batch strides; an
  // index >= b_index_limit raises ERRF_INDEX_OOB in *err and is clamped
  const uint32_t *b_index;
  int64_t b_index_stride, sb_index;
  uint32_t b_index_limit;
  uint32_t *err;
  // optional epilogue of the direct-to-LDS bf16 GEMM without split-K (gemm_epilogue_ok):
  // C = act(glu_gate) * (A . B), glu_gate laid out like C (glu_kind 0 = silu, 1 = gelu), i.e. the
  // gated activation of an MLP applied where up_proj's product is still in registers;
  // c16: a bf16 copy of C, same indexing
  const float *glu_gate;
  int32_t glu_kind;
  uint16_t *c16;
  // optional (same conditions): a second B matrix laid out like b (same strides, same N).  The kernel computes
  // both products and stores C = act(A . b) * (A . dual_b) - gate_proj, up_proj and the gated activation of an
  // MLP in one launch; c may be null when only the bf16 copy c16 is wanted
  const void *dual_b;
  // optional (same kernel, one batch, no split-K): n_group products that share A, K and the strides of
  // B (q/k/v of a prefill) as one launch.  N is the sum of grp_n; columns [0, grp_n[0]) belong to the
  // first product, and so on; every grp_n is a multiple of 128; b and c are ignored.
  uint32_t n_group;
  const void *grp_b[3];
  float *grp_c[3];
  uint32_t grp_n[3];
  // optional, with n_group: a vector of grp_n[p] floats added to every row of product p (the bias of a linear)
  const float *grp_bias[3];
  // optional, with n_group (gemm_rope_epilogue_ok): the products are the q / k / v projections of M / rope_s
  // sequences of rope_s positions each (row m = sequence m / rope_s, position m % rope_s) with heads of rope_hd
  // (64 or 128) columns.  A group with rope_role 1 leaves the kernel rotated (apply_rope_embedding, cos / sin
  // rows of rope_hd floats at rope_cs_ss apart, indexed by position) as [sequence][head][position][rope_hd] at
  // rope_out (f32) and rope_out16 (bf16, optional) instead of grp_c; a group with rope_role 2 is stored as usual
  // and also transposed, as bf16 [sequence][head][rope_hd][position], at rope_out16.
  uint32_t rope_s, rope_hd;
  uint32_t rope_role[3];
  float *rope_out[3];
  uint16_t *rope_out16[3];
  const float *rope_cos[3], *rope_sin[3];
  int64_t rope_cs_ss[3];
  // optional (the direct-to-LDS bf16 GEMM, for the clock probe): every workgroup adds the shader-clock ticks and
  // the 100 MHz ticks its main loop took to clock_ticks[0] and [1]
  unsigned long long *clock_ticks;
};
// split factor launch_matmul should be given for this problem (1 = none)
uint32_t gemm_split_k(const LaunchCtx &lc, const GemmDesc &g);
// whether launch_matmul would run this problem (splits as given) on the kernel that honours
// glu_gate / c16
bool gemm_epilogue_ok(const GemmDesc &g);
// whether launch_matmul would run this grouped problem on the tile whose epilogue honours rope_role
bool gemm_rope_epilogue_ok(const LaunchCtx &lc, const GemmDesc &g);
hipError_t launch_matmul(const LaunchCtx &lc, const GemmDesc &g, const char **kernel_name);
// contiguous f32 -> bf16 (RNE); n % 8 == 0, 16-byte aligned
hipError_t launch_cast_bf16(const LaunchCtx &lc, const float *in, void *out, uint64_t n);
// B[k, n] (unit stride along n, row stride sbk, f32 or bf16, nb0 x nb1 batches through sb_b0 / sb_b1)
// -> contiguous bf16 [nb0 * nb1][N][K]
hipError_t launch_transpose_cast_bf16(const LaunchCtx &lc, const void *b, int b_stype, void *out, uint32_t K,
                                      uint32_t N, int64_t sbk, uint32_t nb0, uint32_t nb1, int64_t sb_b0,
                                      int64_t sb_b1);
// Several GEMVs y_p = x . B_p^T that share x (M == 1, B_p k-contiguous, 16-byte aligned rows):
// one launch, problem p on grid.y
struct GemvMultiDesc {
  const float *x;
  uint32_t K;
  int32_t n_prob, b_stype;
  struct {
    const void *b;
    float *c;
    const float *c_add;  // optional: c = x . b^T + c_add
    int64_t sbn;
    uint32_t N;
    // several input rows (GemvProDesc::rows): c_add is a vector added to every row (a bias) instead of
    // a [rows, N] matrix (a residual)
    int32_t c_add_is_row;
  } p[4];
};
hipError_t launch_gemv_multi(const LaunchCtx &lc, const GemvMultiDesc &g);
// The same, with x produced inside the kernel (once per workgroup, kept in LDS) from the op that
// feeds these projections in a decoder layer, so that op needs no launch of its own:
//   PRO_RMSNORM: x = a / sqrt(sum(a*a) / n + eps) * (gamma_offset + gamma)   (gamma may be null)
//   PRO_SWIGLU / PRO_GEGLU: x = silu(a) * aux  /  gelu(a) * aux
// K <= GEMV_PRO_MAX_K, K % 8 == 0; a, aux, gamma contiguous, 16-byte aligned
//   PRO_NONE: x = a (staged once per workgroup)
// Batched form (the routed experts of a MoE layer, models/qwen3.rs:104-123): batch z has its own
// input row (a + z * a_bstride, aux + z * aux_bstride), its own output rows (c + z * N) and reads
// the weight matrices of expert b_index[z * b_index_stride] (b + index * sb_index); an index >=
// b_index_limit raises ERRF_INDEX_OOB in *err and is clamped.
//   PRO_ATTN_MERGE: x = the output row of a split decode attention launched with merge_later, merged here
//     from its partials (one row, K = heads * d <= 2048, at most 8 splits, heads * splits <= 256); a is unused
enum { PRO_NONE = 0, PRO_RMSNORM = 1, PRO_SWIGLU = 2, PRO_GEGLU = 3, PRO_ATTN_MERGE = 4, GEMV_PRO_MAX_K = 8192 };
enum { ATTN_MERGE_MAX_SPLITS = 8 };
struct GemvProDesc {
  GemvMultiDesc m;  // m.x is ignored
  int32_t pro;
  const float *a, *aux;
  float n_as_float, eps, gamma_offset;
  // 0, or PRO_SWIGLU / PRO_GEGLU: two problems of equal N (gate, up); a single output
  // p[0].c[n] = act(x . gate_n) * (x . up_n) replaces the two product vectors
  // (several rows against bf16 weights on the matrix cores: problems 2 and 3, if any, are plain products of
  // the same input rows, computed by glu_extra_blocks further workgroups - set by the launcher)
  int32_t glu_epilogue;
  uint32_t glu_extra_blocks;
  uint32_t batch;   // 0 or 1: a single row
  int64_t a_bstride, aux_bstride;
  // 0 / 1, or several input rows that share the weights (gemv_pro_rows_ok; no batch, no b_index):
  // row r of the input is a + r * a_rstride (aux + r * aux_rstride; gamma is one vector for all rows) and
  // the outputs (and c_add) are the rows of contiguous [rows, N] matrices
  uint32_t rows;
  int64_t a_rstride, aux_rstride;
  const uint32_t *b_index;
  int64_t b_index_stride, sb_index;
  uint32_t b_index_limit;
  uint32_t *err;
  // Several slots of a MoE layer in one batched launch (slot_tokens > 0): batch z is token z % slot_tokens
  // of slot z / slot_tokens and reads expert b_index_slot[slot][token * b_index_stride] (b_index is unused);
  // outputs and - unless a_by_token - inputs are laid out [slot][token]; with a_by_token every slot reads
  // the same input rows a + token * a_bstride
  uint32_t slot_tokens;
  int32_t a_by_token;
  const uint32_t *b_index_slot[8];
  // ... and the router's choice made here (router_logits != null: rows of router_n <= 64 logits, router_stride
  // apart, one per token): every workgroup computes topk(softmax(row)) of its token - router_k <= 8 choices,
  // as launch_softmax_topk would - and slot s reads choice router_col[s]; b_index_slot is unused.  One workgroup
  // per token also stores the k values and indices (rows of router_k) for whoever reads them next.
  const float *router_logits;
  int64_t router_stride;
  uint32_t router_n, router_k;
  float *router_values;
  uint32_t *router_indices;
  uint8_t router_col[8];
  // PRO_ATTN_MERGE: the attention's partials (AttnDecodeDesc::part with merge_later) and their geometry
  const float *merge_part;
  uint32_t merge_splits, merge_heads, merge_d;
  // optional: gemv_pro_amax_records(lc, g) records of 3 words, the argmax of the stored row in pieces
  // (launch_argmax_merge finishes it)
  uint32_t *amax_part;
};
hipError_t launch_gemv_pro(const LaunchCtx &lc, const GemvProDesc &g);
// the number of argmax records launch_gemv_pro would write for this product (0: it cannot)
uint32_t gemv_pro_amax_records(const LaunchCtx &lc, const GemvProDesc &g);
// out[0] = the argmax (Backend::argmax's order) over `records` records of (key, column, any)
hipError_t launch_argmax_merge(const LaunchCtx &lc, const uint32_t *records, uint32_t *out, uint32_t n_records);
// largest K the several-row form on the vector ALUs takes for weights of this storage type
uint32_t gemv_pro_multi_row_max_k(int b_stype);
// most input rows any several-row form takes
enum { GEMV_PRO_MAX_ROWS = 16 };
// whether launch_gemv_pro takes `rows` input rows of K values with prologue `pro` against weights of this
// storage type: one row; up to 4 on the vector ALUs; up to 16 against bf16 weights on the matrix cores
// (K % 128 == 0, rows * (K + 8) <= 20480, inputs rounded to bf16)
bool gemv_pro_rows_ok(int b_stype, uint32_t rows, uint32_t K, int pro);
bool gemv_rows_mfma_ok(int b_stype, uint32_t rows, uint32_t K, int pro);
// a plain product of 2 to 16 rows that launch_gemv_pro's matrix-core form takes as one of up to four problems
bool gemv_rows_group_ok(const GemmDesc &g);
// a bf16 product whose right operand is [K, N] with unit stride along n and that the direct-to-LDS kernel takes
// as it lies (no transposed copy of B)
bool gemm_dma_bkm_ok(const GemmDesc &g);
// The routed experts of a MoE layer over many tokens (a prefill; models/qwen3.rs:104-123), expert by
// expert.  A slot is one of the k choices of every token: its index vector, its input rows and its
// outputs.  A problem is one stacked weight tensor [E, N, K] (bf16): gate_proj and up_proj share
// input rows and indices, so they go out together (n_prob = 2); down_proj (n_prob = 1) computes its
// rows from gate and up (pro = PRO_SWIGLU / PRO_GEGLU, aux = up).  All slots of a layer go out in one
// launch, so an expert's matrix is read once per 128 columns for every token that chose it in any
// slot.  Inputs are rounded to bf16 like every many-row product in bf16 mode.
struct MoeGemmDesc {
  uint32_t S, K, n_slot, n_prob, n_expert;  // S <= 65535 tokens, n_slot <= 8, n_prob <= 2
  int32_t pro;                              // PRO_NONE, PRO_SWIGLU or PRO_GEGLU (f32 input rows only)
  // 0, or PRO_SWIGLU / PRO_GEGLU with n_prob == 2 problems of equal N (gate, up): a workgroup computes
  // both products of its tokens and stores act(first) * second as bf16 into slot[].h16; c is unused
  int32_t fuse_glu;
  int64_t sb_index;                         // elements between two experts' matrices
  struct {
    const uint32_t *idx;                    // idx[t * idx_stride] = expert of token t in this slot
    int64_t idx_stride;
    const float *a, *aux;                   // f32 input rows: a + t * a_bs (aux + t * aux_bs), unit stride along k
    const uint16_t *a16;                    // or bf16 input rows (a16 + t * a_bs), taken as they are
    int64_t a_bs, aux_bs;
    float *c[2];                            // outputs per problem, contiguous [S, N]
    uint16_t *h16;                          // fuse_glu: gated activations, contiguous bf16 [S, N]
  } slot[8];
  struct {
    const void *w;                          // [E, N, K], unit stride along k, row stride sbn
    int64_t sbn;
    uint32_t N;
  } prob[2];
  uint32_t *err;                            // ERRF_INDEX_OOB for an index >= n_expert (served by the last expert)
  // optional: the (slot, token) pairs already sorted by expert (launch_moe_route): pairs
  // route_list[route_offset[e] .. + route_count[e]) = slot << 16 | token chose expert e
  const uint32_t *route_count, *route_offset, *route_list;
  // optional, with the above: the row tiles of all experts as a work list (launch_moe_route's `tiles`)
  const uint32_t *route_tiles;
};
hipError_t launch_moe_gemm(const LaunchCtx &lc, const MoeGemmDesc &g);
// Sorts the S * n_slot (slot, token) pairs of g by expert into count / offset (n_expert words each) and
// list (S * n_slot words); n_expert <= MOE_ROUTE_MAX_EXPERTS.  With these in g.route_*, bf16 input rows
// (slot[].a16 for every slot) and K % 64 == 0, launch_moe_gemm streams the weights through a
// multi-stage direct-to-LDS pipeline.
enum { MOE_ROUTE_MAX_EXPERTS = 4096 };
// tiles (optional, 1 + moe_route_max_tiles(g) words): the number of 128-pair row tiles over all experts, then
// expert << 16 | row tile for each; with it in g.route_tiles a workgroup of launch_moe_gemm owns one row tile
// of one expert, so the launch stays balanced when most tokens choose the same few experts.
hipError_t launch_moe_route(const LaunchCtx &lc, const MoeGemmDesc &g, uint32_t *count, uint32_t *offset, uint32_t *list,
                            uint32_t *tiles);
uint32_t moe_route_max_tiles(const MoeGemmDesc &g);
bool moe_gemm_pipelined_ok(const MoeGemmDesc &g);
// wrapping u32 matmul (ndarray's generic dot); all operands contiguous
hipError_t launch_matmul_u32(const LaunchCtx &lc, const uint32_t *a, const uint32_t *b, uint32_t *c,
                             uint32_t batch, uint32_t M, uint32_t N, uint32_t K);

}  // namespace cgk
