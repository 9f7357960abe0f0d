// Shared device-side vocabulary for the gfx950 kernels: vector types, bf16
// rounding, post-op (epilogue) math.  Wave size is 64 throughout.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace gcmi {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef int i32x16_t __attribute__((ext_vector_type(16)));
typedef int i32x4_t __attribute__((ext_vector_type(4)));
typedef int i32x2_t __attribute__((ext_vector_type(2)));
typedef unsigned short u16x4_t __attribute__((ext_vector_type(4)));

#define GCMI_LDS __attribute__((address_space(3)))

// post-op kinds fused into a GEMM epilogue
enum Act : int { ACT_NONE = 0, ACT_RELU = 1, ACT_GELU_ERF = 2, ACT_GELU_TANH = 3, ACT_SIGMOID = 4 };

// dnnl_data_type_t values used across the C ABI
enum DType : int { DT_F16 = 1, DT_BF16 = 2, DT_F32 = 3, DT_S32 = 4, DT_S8 = 5, DT_U8 = 6 };

// f32 -> bf16, round to nearest even, NaN -> 0x7FC0: the reference's bf16_t
// constructor (include/gc/ExecutionEngine/CPURuntime/Microkernel/
// BrgemmInterface.h:83-92).
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float v) {
  uint32_t bits = __float_as_uint(v);
  uint32_t r = (bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16;
  return (v != v) ? (uint16_t)0x7FC0u : (uint16_t)r;
}
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }
__device__ __forceinline__ float round_bf16(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }

// erf(x) as an odd rational P(x^2)*x / Q(x^2) on |x| <= 3.95 (beyond that erf
// rounds to +-1 in f32); absolute error below 5e-7.  The reference evaluates erf
// with approximations of the same class (a table of degree-5 polynomials, or
// Abramowitz-Stegun 7.1.26 with absolute error 1.5e-7:
// legacy/core/src/compiler/ir/transform/cpu/target_specific_lower.cpp:1012-1130),
// so nothing finer than that is pinned by it.  About 20 VALU operations, no branches.
__device__ __forceinline__ float erf_rational(float x) {
  const float xc = __builtin_amdgcn_fmed3f(x, -3.95f, 3.95f);
  const float x2 = xc * xc;
  float p = -2.72614225801306e-10f;
  p = fmaf(p, x2, 2.77068142495902e-08f);
  p = fmaf(p, x2, -2.10102402082508e-06f);
  p = fmaf(p, x2, -5.69250639462346e-05f);
  p = fmaf(p, x2, -7.34990630326855e-04f);
  p = fmaf(p, x2, -2.95459980854025e-03f);
  p = fmaf(p, x2, -1.60960333262415e-02f);
  float q = -1.45660718464996e-05f;
  q = fmaf(q, x2, -2.13374055278905e-04f);
  q = fmaf(q, x2, -1.68282697438203e-03f);
  q = fmaf(q, x2, -7.37332916720468e-03f);
  q = fmaf(q, x2, -1.42647390514189e-02f);
  const float r = __builtin_amdgcn_fmed3f((p * xc) * __builtin_amdgcn_rcpf(q), -1.0f, 1.0f);
  return fabsf(x) >= 3.95f ? copysignf(1.0f, x) : r;
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
    return (x * (tanhf(t) + 1.0f)) * 0.5f;
  }
  case ACT_SIGMOID:
    return 1.0f / (1.0f + expf(-x));
  default:
    return x;
  }
}

} // namespace gcmi

// compute units of the current device (host side, cached per device)
static inline int gcmi_num_cus() {
  static int cache[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
    return 256;
  if (cache[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    cache[dev] = n;
  }
  return cache[dev];
}
