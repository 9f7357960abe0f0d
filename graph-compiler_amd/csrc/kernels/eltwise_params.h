// Argument blocks of the generic element-wise / reduce / softmax kernels.
#pragma once
#include <stdint.h>

namespace gcmi {

static constexpr int ELT_MAX_RANK = 6;

enum EltOp : int {
  ELT_COPY = 0, ELT_ADD, ELT_SUB, ELT_MUL, ELT_DIV, ELT_RELU, ELT_SIGMOID, ELT_GELU_ERF, ELT_GELU_TANH, ELT_POW,
  ELT_DEQUANT, ELT_QUANT, ELT_MAX, ELT_EXP, ELT_NEG,
  ELT_ROWSUM, // only inside a FusedParams program: the row sum of a register
  ELT_MIN, ELT_ABS, ELT_CEIL, ELT_FLOOR, ELT_ERF, ELT_LOG, ELT_ROUND, ELT_RSQRT, ELT_SQRT, ELT_SQUARE, ELT_TANH, ELT_RECIP
};

struct EltParams {
  const void *a;
  const void *b; // null for unary ops
  void *out;     // dense row-major over dims
  int64_t n;
  int64_t dims[ELT_MAX_RANK]; // left-padded with 1
  int64_t sa[ELT_MAX_RANK];   // element strides of a (0 on broadcast dims)
  int64_t sb[ELT_MAX_RANK];
  int32_t op, a_dt, b_dt, out_dt;
  float alpha;          // Pow exponent
  const float *scales;  // (de)quantise: device arrays
  const int32_t *zps;
  int32_t n_scales, ch_axis; // ch_axis indexes dims[] (after left padding)
};

struct ReduceParams {
  const void *in;
  void *out;
  int64_t n_out, n_red;
  int64_t kdims[ELT_MAX_RANK], kstr[ELT_MAX_RANK]; // kept dims and their input strides
  int64_t rdims[ELT_MAX_RANK], rstr[ELT_MAX_RANK]; // reduced dims and their input strides
  int32_t dt, mean;
};

// A group of point-wise ops fused into one launch: a straight-line program over f32 registers, evaluated once per
// element of the iteration space.  Registers 0 .. n_in-1 hold the inputs (read through broadcast strides),
// instruction j writes register n_in + j.  Every instruction rounds its result to the storage type its op has in
// the graph (dt), so the fused group computes bit for bit what the ops compute one launch at a time.
//
// With a sum inside (sum_ins >= 0) the iteration space is [n / n_red rows, n_red]: instructions before sum_ins run
// per element and read inputs 0 .. n_in_pre-1; instruction sum_ins (ELT_ROWSUM) is the sum (or mean) over the row
// of its register a; the instructions after it run once per row, may read the remaining inputs (whose strides
// over the row's own dims are 0) and the output has one value per row.
static constexpr int FUSED_MAX_IN = 8, FUSED_MAX_INS = 24;

struct FusedIns {
  int32_t op;   // EltOp (not the (de)quantise ops)
  int32_t a, b; // source registers (b unused by unary ops)
  int32_t dt;   // storage type of the result: DT_F32 / DT_BF16 / DT_F16
  float imm;    // Pow exponent
};

struct FusedParams {
  const void *in[FUSED_MAX_IN];
  void *out;
  int64_t in_str[FUSED_MAX_IN][ELT_MAX_RANK]; // element strides per iteration dim (0 on broadcast dims)
  int64_t dims[ELT_MAX_RANK];                 // iteration space, left-padded with 1
  int64_t n;                                  // its element count
  int64_t n_red;                              // row length (1 without a sum)
  int32_t in_dt[FUSED_MAX_IN];
  int32_t out_dt, out_reg;
  int32_t n_in, n_in_pre, n_ins, sum_ins; // sum_ins: -1 without a sum
  int32_t rank, rank_red;                 // dims after merging, and how many of them lie inside a row (set by the launcher)
  int32_t mean;
  FusedIns ins[FUSED_MAX_INS];
};

struct SoftmaxParams {
  const void *in;
  void *out;
  int64_t outer, len, inner;
  int32_t in_dt, out_dt;
};

} // namespace gcmi
