// Device-side arithmetic shared by every kernel: bf16 rounding, the activations of the GEMM epilogues and the table
// of point-wise ops.  No includes (the including file supplies the HIP runtime, the fixed-width integer types and
// op_codes.h): this text is also handed to the run-time compiler, so that generated kernels and the kernels built
// with the library compute the same bits.
#ifndef GCMI_DEVICE_MATH_HPP
#define GCMI_DEVICE_MATH_HPP

namespace gcmi {

// f32 -> bf16, round to nearest even, NaN -> 0x7FC0: the reference's bf16_t
// constructor (include/gc/ExecutionEngine/CPURuntime/Microkernel/
// BrgemmInterface.h:83-92).
// The rounding itself is the hardware's v_cvt_pk_bf16_f32: it gives (bits + 0x7FFF + ((bits >> 16) & 1)) >> 16 for
// every one of the 2^32 inputs that is not a NaN (checked exhaustively on the GPU) and keeps a NaN's sign and
// payload, which is where the select comes in.
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float v) {
  typedef __bf16 gcmi_bf16x2_ __attribute__((ext_vector_type(2)));
  typedef float gcmi_f32x2_ __attribute__((ext_vector_type(2)));
  const gcmi_f32x2_ pair = {v, v};
  const uint32_t r = __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, gcmi_bf16x2_));
  return (v != v) ? (uint16_t)0x7FC0u : (uint16_t)r;
}
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }
__device__ __forceinline__ float round_bf16(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }

// erf for the GELU below, where it is added to 1: for x >= 0, erf(x) = 1 - 2^(-x q(x)) with q a polynomial of degree 6
// fitted to -log2(erfc(x)) / x on [0, 4.2] (weighted for the error of erf itself), odd in x; absolute error below
// 2e-7 (relative accuracy near 0 is not kept).  The reference evaluates erf with approximations of the same class (a
// table of degree-5 polynomials, or Abramowitz-Stegun 7.1.26 with absolute error 1.5e-7:
// legacy/core/src/compiler/ir/transform/cpu/target_specific_lower.cpp:1012-1130), so nothing finer than that is
// pinned by it.  |x| is clamped to 4.2, where 2^(-x q) < 2^-28 and the difference is exactly 1, so large arguments,
// infinities included, give +-1 with no comparison; 14 issue slots per element (the exponential counts four), no
// branch, and the four elements of a row interleave.  (An odd rational P(x^2) x / Q(x^2) of the same accuracy took 19;
// a conditional `|x| >= bound ? +-1 : ...` makes the compiler branch around the polynomial per element: six scalar
// instructions each, and the chains serialise.)
__device__ __forceinline__ float erf_rational(float x) {
  const float a = fminf(fabsf(x), 4.2f);
  float q = -1.0021075286203995e-04f;
  q = fmaf(q, a, 4.615070065483451e-04f);
  q = fmaf(q, a, 2.3023963440209627e-03f);
  q = fmaf(q, a, -2.9452694579958916e-02f);
  q = fmaf(q, a, 1.4896376430988312e-01f);
  q = fmaf(q, a, 9.183286428451538e-01f);
  q = fmaf(q, a, 1.6279137134552002f);
  return copysignf(1.0f - __builtin_amdgcn_exp2f(-(q * a)), x);
}

// GELU (erf form) of a FINITE x whose result is stored as bf16: x Phi(x) with Phi(-|x|) = erfc(t) / 2 = 2^(-t q(t) - 1),
// t = |x| / sqrt 2, q of degree 4 fitted to -log2(erfc(t)) / t on [0, 4.2]:
//   x < 0:  x Phi(x) = x e          x >= 0:  x (1 - e) = x - x e          (e = 2^(-t q(t) - 1))
// both as max(x, -0) - |x e|.  Relative error of the result below 2^-11.9 wherever |gelu| > 1e-5 (absolute error below
// 1.1e-9 elsewhere): a quarter of the last place of a bf16 -- about 4 % of the results in |x| < 6 round to the
// neighbouring bf16 value of the exactly rounded one, none differs by more.  q has positive derivative for all t >= 0, so no clamp is
// needed: for |x| > 13 the power underflows to 0 and the result is x or -0 exactly, as with the reference's
// saturated erf (legacy/core/src/ops/gelu.cpp:110-131 gives (erf + 1) * x * 0.5 = -0 there).  12 issue slots (the
// exponential counts four) against 19 for erf_rational + 1, * x, * 0.5.  Not for infinite or NaN x (inf * 0).
__device__ __forceinline__ float gelu_erf_bf16_result(float x) {
  // q(t) t with t = |x| / sqrt 2 written as a polynomial in |x| (the factors of 1 / sqrt 2 are in the coefficients;
  // |x| is an operand modifier, not an instruction)
  const float a = fabsf(x);
  float q = 2.5154993636533618e-04f;
  q = fmaf(q, a, -5.1113637164235115e-03f);
  q = fmaf(q, a, 4.5734334737062454e-02f);
  q = fmaf(q, a, 4.6741172671318054e-01f);
  q = fmaf(q, a, 1.1480368375778198f);
  const float g = x * __builtin_amdgcn_exp2f(fmaf(-a, q, -1.0f));
  return fmaxf(x, -0.0f) - fabsf(g);
}

// tanh for the GELU below, where it is added to 1: 1 - 2 / (e^(2|t|) + 1) with the sign of t, absolute error about
// 2e-7 (relative accuracy near 0 is not kept: the math library's tanhf keeps it with a polynomial branch per element,
// which costs the epilogues what the conditional in erf did).  Infinite and NaN arguments come out as +-1 and NaN.
__device__ __forceinline__ float tanh_by_exp(float t) {
  const float e = __builtin_amdgcn_exp2f(fabsf(t) * 2.885390081777927f); // 2 log2 e
  const float r = fmaf(__builtin_amdgcn_rcpf(e + 1.0f), -2.0f, 1.0f);
  return copysignf(r, t);
}

// Activation in f32.  Operation order follows the reference graphs:
// ReLU   = max(x, 0), NaN propagates (lib/gc/Transforms/OneDNNGraphToLinalg.cpp:355-358)
// GELU   = ((erf(x*c)+1)*x)*0.5, c = 0x3f3504f3 (legacy/core/src/ops/gelu.cpp:110-131)
// tanh   = (x*(tanh((((x*x)*0.044715+1)*x)*0.79788458)+1))*0.5 (gelu.cpp:78-108)
// sigmoid= 1/(1+exp(-x)) (lib/gc/Dialect/Linalgx/LinalgxOps.cpp:42-61)
__device__ __forceinline__ float apply_act(float x, int act) {
  switch (act) {
  case ACT_RELU:
    return (x != x) ? x : fmaxf(x, 0.0f);
  case ACT_GELU_ERF: {
    const float c = __uint_as_float(0x3f3504f3u);
    return ((erf_rational(x * c) + 1.0f) * x) * 0.5f;
  }
  case ACT_GELU_TANH: {
    float t = (((x * x) * 0.044715f + 1.0f) * x) * 0.79788458f;
    return (x * (tanh_by_exp(t) + 1.0f)) * 0.5f;
  }
  case ACT_SIGMOID:
    return 1.0f / (1.0f + expf(-x));
  default:
    return x;
  }
}

// one point-wise op in f32 (shared by the single-op kernel and the fused programs)
__device__ __forceinline__ float round_to_storage(float v, int dt) {
  switch (dt) {
  case DT_BF16: return bf16_bits_to_f32(f32_to_bf16_bits(v));
  case DT_F16: return (float)(_Float16)v;
  default: return v;
  }
}

__device__ __forceinline__ float fused_op(int op, float x, float y, float imm) {
  switch (op) {
  case ELT_ADD: return x + y;
  case ELT_SUB: return x - y;
  case ELT_MUL: return x * y;
  case ELT_DIV: return x / y;
  case ELT_MAX: return (x != x || y != y) ? x + y : fmaxf(x, y);
  case ELT_EXP: return expf(x);
  case ELT_NEG: return -x;
  case ELT_RELU: return apply_act(x, ACT_RELU);
  case ELT_SIGMOID: return apply_act(x, ACT_SIGMOID);
  case ELT_GELU_ERF: return apply_act(x, ACT_GELU_ERF);
  case ELT_GELU_TANH: return apply_act(x, ACT_GELU_TANH);
  case ELT_POW: return imm == 2.0f ? x * x : (imm == 1.0f ? x : (imm == 0.5f ? sqrtf(x) : powf(x, imm)));
  case ELT_MIN: return (x != x || y != y) ? x + y : fminf(x, y); // arith.minimumf: NaN propagates
  case ELT_ABS: return fabsf(x);
  case ELT_CEIL: return ceilf(x);
  case ELT_FLOOR: return floorf(x);
  case ELT_ERF: return erff(x);
  case ELT_LOG: return __builtin_logf(x); // spelled as the builtin: the offline headers and the run-time compiler's resolve logf differently
  case ELT_ROUND: return roundf(x); // math.round: halves away from zero
  case ELT_RSQRT: return 1.0f / sqrtf(x);
  case ELT_SQRT: return sqrtf(x);
  case ELT_SQUARE: return x * x;
  case ELT_TANH: return tanhf(x);
  case ELT_RECIP: return 1.0f / x;
  default: return x; // ELT_COPY
  }
}

} // namespace gcmi

#endif
