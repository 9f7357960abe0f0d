// Generic element-wise, reduction, softmax and (de)quantise kernels for the ops
// of a partition that are not fused into a GEMM or attention kernel.  Every op
// reads its operands in their storage type (f32 / bf16 / f16 / s8 / u8 / s32),
// computes in f32 and rounds once to the result type, which is what the
// reference's bf16->f32 emulation does to each op
// (lib/gc/Transforms/Pipeline.cpp:79-95).  Semantics per op:
//   Add/Subtract/Multiply/Divide  numpy broadcasting
//                                 (lib/gc/Transforms/OneDNNGraphToLinalg.cpp:64-118)
//   Maximum / Exp / Neg           linalg.max, linalg.exp, linalg.negf of the MLIR front end
//   ReLU max(x,0), Sigmoid 1/(1+exp(-x)), Pow x^beta, Typecast = copy with rounding
//                                 (OneDNNGraphToLinalg.cpp:331-358)
//   ReduceSum / ReduceMean        sum over axes, mean divides by the count (:505-559)
//   SoftMax                       max, sub, exp, sum, div along one axis
//                                 (lib/gc/Transforms/DecomposeAggregatedOps.cpp:24-38)
//   Dequantize (q - zp) * scale, Quantize sat(rne(x / scale) + zp)
//                                 (legacy/core/src/compiler/ir/graph/quantization/quantize_op.cpp:107-277)
#include "common.hpp"
#include "eltwise_params.h"

namespace gcmi {

__device__ __forceinline__ float load_as_f32(const void *p, int64_t i, int dt) {
  switch (dt) {
  case DT_F32: return reinterpret_cast<const float *>(p)[i];
  case DT_BF16: return bf16_bits_to_f32(reinterpret_cast<const uint16_t *>(p)[i]);
  case DT_F16: return (float)reinterpret_cast<const _Float16 *>(p)[i];
  case DT_S32: return (float)reinterpret_cast<const int32_t *>(p)[i];
  case DT_S8: return (float)reinterpret_cast<const int8_t *>(p)[i];
  case DT_U8: return (float)reinterpret_cast<const uint8_t *>(p)[i];
  default: return 0.0f;
  }
}
__device__ __forceinline__ void store_from_f32(void *p, int64_t i, int dt, float v) {
  switch (dt) {
  case DT_F32: reinterpret_cast<float *>(p)[i] = v; break;
  case DT_BF16: reinterpret_cast<uint16_t *>(p)[i] = f32_to_bf16_bits(v); break;
  case DT_F16: reinterpret_cast<_Float16 *>(p)[i] = (_Float16)v; break; // RNE
  case DT_S32: reinterpret_cast<int32_t *>(p)[i] = (int32_t)v; break;
  case DT_S8: reinterpret_cast<int8_t *>(p)[i] = (int8_t)fminf(fmaxf(v, -128.f), 127.f); break;
  case DT_U8: reinterpret_cast<uint8_t *>(p)[i] = (uint8_t)fminf(fmaxf(v, 0.f), 255.f); break;
  default: break;
  }
}

// out[idx] = op(a[idx . sa], b[idx . sb]); out is dense row-major over dims
__global__ void eltwise_kernel(EltParams p) {
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < p.n; idx += (int64_t)gridDim.x * blockDim.x) {
    int64_t rem = idx, ia = 0, ib = 0, ch = 0;
#pragma unroll
    for (int d = ELT_MAX_RANK - 1; d >= 0; d--) {
      int64_t c = rem % p.dims[d];
      rem /= p.dims[d];
      ia += c * p.sa[d];
      ib += c * p.sb[d];
      if (d == p.ch_axis)
        ch = c;
    }
    float x = load_as_f32(p.a, ia, p.a_dt), y = 0.0f, r;
    if (p.b)
      y = load_as_f32(p.b, ib, p.b_dt);
    switch (p.op) {
    case ELT_ADD: r = x + y; break;
    case ELT_SUB: r = x - y; break;
    case ELT_MUL: r = x * y; break;
    case ELT_DIV: r = x / y; break;
    case ELT_MAX: r = (x != x || y != y) ? x + y : fmaxf(x, y); break; // arith.maximumf: NaN propagates
    case ELT_EXP: r = expf(x); break;
    case ELT_NEG: r = -x; break;
    case ELT_RELU: r = apply_act(x, ACT_RELU); break;
    case ELT_SIGMOID: r = apply_act(x, ACT_SIGMOID); break;
    case ELT_GELU_ERF: r = apply_act(x, ACT_GELU_ERF); break;
    case ELT_GELU_TANH: r = apply_act(x, ACT_GELU_TANH); break;
    case ELT_POW: r = p.alpha == 2.0f ? x * x : (p.alpha == 1.0f ? x : (p.alpha == 0.5f ? sqrtf(x) : powf(x, p.alpha))); break;
    case ELT_DEQUANT: {
      float sc = p.scales ? p.scales[p.n_scales > 1 ? ch : 0] : 1.0f;
      float zp = p.zps ? (float)p.zps[p.n_scales > 1 ? ch : 0] : 0.0f;
      r = (x - zp) * sc;
      break;
    }
    case ELT_QUANT: {
      float sc = p.scales ? p.scales[p.n_scales > 1 ? ch : 0] : 1.0f;
      float zp = p.zps ? (float)p.zps[p.n_scales > 1 ? ch : 0] : 0.0f;
      r = rintf(x / sc) + zp;
      break;
    }
    default: r = x; break; // ELT_COPY: typecast / strided gather
    }
    store_from_f32(p.out, idx, p.out_dt, r);
  }
}

// one thread per output element; the reduced sub-space is walked serially in
// row-major order (k ascending, like the linalg.reduce loop nest)
__global__ void reduce_kernel(ReduceParams p) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= p.n_out)
    return;
  int64_t rem = idx, base = 0;
#pragma unroll
  for (int d = ELT_MAX_RANK - 1; d >= 0; d--) {
    int64_t c = rem % p.kdims[d];
    rem /= p.kdims[d];
    base += c * p.kstr[d];
  }
  float s = 0.0f;
  for (int64_t r = 0; r < p.n_red; r++) {
    int64_t rr = r, off = 0;
#pragma unroll
    for (int d = ELT_MAX_RANK - 1; d >= 0; d--) {
      int64_t c = rr % p.rdims[d];
      rr /= p.rdims[d];
      off += c * p.rstr[d];
    }
    s += load_as_f32(p.in, base + off, p.dt);
  }
  if (p.mean)
    s = s / (float)p.n_red;
  store_from_f32(p.out, idx, p.dt, s);
}

// softmax along an axis of length `len` and element stride `stride`; one wave
// per row, rows enumerated as outer*inner
__global__ __launch_bounds__(256) void softmax_kernel(SoftmaxParams p) {
  const int lane = threadIdx.x & 63;
  int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= p.outer * p.inner)
    return;
  int64_t o = row / p.inner, in = row % p.inner;
  int64_t base = o * p.len * p.inner + in;
  float mx = -INFINITY;
  for (int64_t i = lane; i < p.len; i += 64)
    mx = fmaxf(mx, load_as_f32(p.in, base + i * p.inner, p.in_dt));
#pragma unroll
  for (int s = 32; s > 0; s >>= 1)
    mx = fmaxf(mx, __shfl_xor(mx, s));
  float sum = 0.0f;
  for (int64_t i = lane; i < p.len; i += 64)
    sum += expf(load_as_f32(p.in, base + i * p.inner, p.in_dt) - mx);
#pragma unroll
  for (int s = 32; s > 0; s >>= 1)
    sum += __shfl_xor(sum, s);
  for (int64_t i = lane; i < p.len; i += 64)
    store_from_f32(p.out, base + i * p.inner, p.out_dt, expf(load_as_f32(p.in, base + i * p.inner, p.in_dt) - mx) / sum);
}

} // namespace gcmi

using namespace gcmi;

extern "C" int gcmi_launch_eltwise(const EltParams *pp, hipStream_t stream) {
  EltParams p = *pp;
  if (p.n <= 0)
    return 0;
  int64_t blocks = (p.n + 255) / 256;
  if (blocks > 65536)
    blocks = 65536;
  hipLaunchKernelGGL(eltwise_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, p);
  return hipGetLastError() == hipSuccess ? 0 : 5;
}
extern "C" int gcmi_launch_reduce(const ReduceParams *pp, hipStream_t stream) {
  ReduceParams p = *pp;
  if (p.n_out <= 0)
    return 0;
  hipLaunchKernelGGL(reduce_kernel, dim3((unsigned)((p.n_out + 255) / 256)), dim3(256), 0, stream, p);
  return hipGetLastError() == hipSuccess ? 0 : 5;
}
extern "C" int gcmi_launch_softmax(const SoftmaxParams *pp, hipStream_t stream) {
  SoftmaxParams p = *pp;
  int64_t rows = p.outer * p.inner;
  if (rows <= 0 || p.len <= 0)
    return 0;
  hipLaunchKernelGGL(softmax_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, p);
  return hipGetLastError() == hipSuccess ? 0 : 5;
}
