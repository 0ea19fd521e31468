// program.hpp — the fused-elementwise "program" shared by host and device code.
//
// A chain of broadcast/elementwise/cast ops (the Map(ScalarOp) family of
// catgrad/src/category/core.rs:212-223 plus Cast and constants) is not run op by op: the host
// flattens the expression tree into a short postfix program, and one kernel evaluates it per
// output element, reading every operand through its own strides (so broadcast, transpose and
// slice views cost nothing).  The same program is the prologue of the row reductions.
#pragma once
#include <stdint.h>

namespace cgk {

enum : int { MAX_IN = 8, MAX_INSTR = 96, MAX_DIMS = 6, MAX_STACK = 8, MAX_STAGES = 2 };

// storage element types
enum SType : int { ST_F32 = 0, ST_U32 = 1, ST_BF16 = 2 };

enum EwOp : uint8_t {
  E_LOAD = 0,   // push input[arg]
  E_CONST,      // push imm[arg]
  E_IOTA,       // push linear element index (u32); only in rank-1 programs
  E_ROW0,       // push the row value produced by reduction stage 0 / 1 (row programs only)
  E_ROW1,
  // binary: pop b, pop a, push f(a, b)
  E_ADD_F, E_SUB_F, E_MUL_F, E_DIV_F, E_POW_F, E_LT_F, E_EQ_F,
  E_ADD_U, E_SUB_U, E_MUL_U, E_DIV_U, E_POW_U, E_LT_U, E_EQ_U,
  // unary
  E_NEG_F, E_NEG_U, E_SIN_F, E_COS_F, E_F2U, E_U2F,
  // specialisations the host derives from constant operands (same results as the general op
  // within the f32 tolerance): pow(e, x), pow(x, 0.5), pow(x, 3), 1 / x
  E_EXP_F, E_SQRT_F, E_CUBE_F, E_RCP_F,
  E__COUNT
};

struct Instr {
  uint8_t op;
  uint8_t depth;  // stack depth before the instruction runs
  uint16_t arg;   // input slot / immediate slot
};

struct Operand {
  const void *ptr;            // already offset to the view's first element
  int64_t stride[MAX_DIMS];   // element strides per collapsed dim (0 = broadcast)
  int32_t stype;              // SType
  int32_t vec;                // 1 if the innermost stride is 1 and 16-byte vector loads are legal
};

// A program is up to three code segments over one operand table.  Segment s < n_stages is the
// per-element value fed to row reduction s (red_kind[s]); its result is visible to all later
// segments as E_ROW<s>.  The last segment is the value that is stored.  Plain elementwise
// programs have n_stages = 0 and one segment.  This is how softmax (max, then sum, then the
// quotient), RMSNorm and LayerNorm run as ONE kernel without being special-cased.
struct Program {
  int32_t n_instr, n_in, n_dims, n_stages;
  int32_t seg_end[MAX_STAGES + 1];  // code[seg_end[s-1] .. seg_end[s]) is segment s
  int32_t red_kind[MAX_STAGES];     // ReduceKind of each stage (sum / max only)
  uint32_t dims[MAX_DIMS];    // collapsed extents, outermost first; dims[n_dims-1] innermost
  Instr code[MAX_INSTR];
  uint32_t imm[MAX_INSTR];
  Operand in[MAX_IN];
};

// output of an elementwise launch
struct OutDesc {
  void *ptr;
  int64_t stride[MAX_DIMS];
  int32_t stype;  // ST_F32 / ST_U32 / ST_BF16
  int32_t vec;
};

enum ReduceKind : int { R_SUM_F = 0, R_SUM_U, R_MAX_F, R_MAX_U, R_ARGMAX_F, R_ARGMAX_U };

}  // namespace cgk
