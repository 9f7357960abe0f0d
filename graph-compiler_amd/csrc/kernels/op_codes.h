// Op, activation and data-type codes shared by the host-side planner, the kernels built with the library and the
// kernels generated at run time.  Plain enums, no includes: this text is also handed to the run-time compiler.
#ifndef GCMI_OP_CODES_H
#define GCMI_OP_CODES_H

namespace gcmi {

// post-op kinds fused into a GEMM epilogue
enum Act : int { ACT_NONE = 0, ACT_RELU = 1, ACT_GELU_ERF = 2, ACT_GELU_TANH = 3, ACT_SIGMOID = 4 };

// dnnl_data_type_t values used across the C ABI
enum DType : int { DT_F16 = 1, DT_BF16 = 2, DT_F32 = 3, DT_S32 = 4, DT_S8 = 5, DT_U8 = 6 };

enum EltOp : int {
  ELT_COPY = 0, ELT_ADD, ELT_SUB, ELT_MUL, ELT_DIV, ELT_RELU, ELT_SIGMOID, ELT_GELU_ERF, ELT_GELU_TANH, ELT_POW,
  ELT_DEQUANT, ELT_QUANT, ELT_MAX, ELT_EXP, ELT_NEG,
  ELT_ROWSUM, // only inside a FusedParams program: the row sum of a register
  ELT_MIN, ELT_ABS, ELT_CEIL, ELT_FLOOR, ELT_ERF, ELT_LOG, ELT_ROUND, ELT_RSQRT, ELT_SQRT, ELT_SQUARE, ELT_TANH, ELT_RECIP
};

} // namespace gcmi

#endif
