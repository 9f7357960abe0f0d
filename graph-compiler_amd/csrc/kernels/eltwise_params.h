// Argument blocks of the generic element-wise / reduce / softmax kernels.
#pragma once
#include <stdint.h>

namespace gcmi {

static constexpr int ELT_MAX_RANK = 6;

enum EltOp : int {
  ELT_COPY = 0, ELT_ADD, ELT_SUB, ELT_MUL, ELT_DIV, ELT_RELU, ELT_SIGMOID, ELT_GELU_ERF, ELT_GELU_TANH, ELT_POW,
  ELT_DEQUANT, ELT_QUANT, ELT_MAX, ELT_EXP, ELT_NEG
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

struct SoftmaxParams {
  const void *in;
  void *out;
  int64_t outer, len, inner;
  int32_t in_dt, out_dt;
};

} // namespace gcmi
