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

// ---------------------------------------------------------------------------
// Fused point-wise groups (FusedParams).  The register file lives in LDS, one column per thread
// (regs[r][tid]: conflict free, and a register number that is only known at run time costs nothing extra).
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
  default: return x; // ELT_COPY
  }
}

static constexpr int FUSED_THREADS = 256;
static constexpr int FUSED_REGS = FUSED_MAX_IN + FUSED_MAX_INS;

// inputs k0 .. k1-1 of element idx into their registers
template <typename IDX>
__device__ __forceinline__ void fused_load(const FusedParams &p, float (*regs)[FUSED_THREADS], int tid, IDX idx, int k0,
                                           int k1) {
  IDX off[FUSED_MAX_IN];
#pragma unroll
  for (int k = 0; k < FUSED_MAX_IN; k++)
    off[k] = 0;
  IDX rem = idx;
  for (int d = ELT_MAX_RANK - 1; d >= ELT_MAX_RANK - p.rank; d--) {
    const IDX dim = (IDX)p.dims[d];
    const IDX c = rem % dim;
    rem /= dim;
#pragma unroll
    for (int k = 0; k < FUSED_MAX_IN; k++)
      if (k >= k0 && k < k1)
        off[k] += c * (IDX)p.in_str[k][d];
  }
#pragma unroll
  for (int k = 0; k < FUSED_MAX_IN; k++)
    if (k >= k0 && k < k1)
      regs[k][tid] = load_as_f32(p.in[k], (int64_t)off[k], p.in_dt[k]);
}

// instructions j0 .. j1-1
__device__ __forceinline__ void fused_run(const FusedParams &p, float (*regs)[FUSED_THREADS], int tid, int j0, int j1) {
  for (int j = j0; j < j1; j++) {
    const FusedIns in = p.ins[j];
    const float x = regs[in.a][tid], y = regs[in.b][tid];
    regs[p.n_in + j][tid] = round_to_storage(fused_op(in.op, x, y, in.imm), in.dt);
  }
}

__global__ __launch_bounds__(FUSED_THREADS) void fused_pointwise_kernel(FusedParams p) {
  __shared__ float regs[FUSED_REGS][FUSED_THREADS];
  const int tid = threadIdx.x;
  const bool small = p.n < ((int64_t)1 << 31); // 32-bit index arithmetic when the whole space fits
  for (int64_t idx = (int64_t)blockIdx.x * FUSED_THREADS + tid; idx < p.n; idx += (int64_t)gridDim.x * FUSED_THREADS) {
    if (small)
      fused_load<uint32_t>(p, regs, tid, (uint32_t)idx, 0, p.n_in);
    else
      fused_load<int64_t>(p, regs, tid, idx, 0, p.n_in);
    fused_run(p, regs, tid, 0, p.n_ins);
    store_from_f32(p.out, idx, p.out_dt, regs[p.out_reg][tid]);
  }
}

// ROWS rows per workgroup, FUSED_THREADS / ROWS threads per row (a multiple of 64: whole waves per row).
// Partial sums are combined in a fixed tree, so results do not vary from run to run.
template <int ROWS> __global__ __launch_bounds__(FUSED_THREADS) void fused_rowsum_kernel(FusedParams p) {
  __shared__ float regs[FUSED_REGS][FUSED_THREADS];
  __shared__ float wave_sum[FUSED_THREADS / 64];
  constexpr int TPR = FUSED_THREADS / ROWS;
  const int tid = threadIdx.x, sub = tid % TPR;
  const int64_t rows = p.n / p.n_red;
  const int64_t row = (int64_t)blockIdx.x * ROWS + tid / TPR;
  const bool small = p.n < ((int64_t)1 << 31);
  const FusedIns sum = p.ins[p.sum_ins];
  float acc = 0.0f;
  if (row < rows) {
    for (int64_t r = sub; r < p.n_red; r += TPR) {
      const int64_t idx = row * p.n_red + r;
      if (small)
        fused_load<uint32_t>(p, regs, tid, (uint32_t)idx, 0, p.n_in_pre);
      else
        fused_load<int64_t>(p, regs, tid, idx, 0, p.n_in_pre);
      fused_run(p, regs, tid, 0, p.sum_ins);
      acc += regs[sum.a][tid];
    }
  }
#pragma unroll
  for (int s = 32; s > 0; s >>= 1)
    acc += __shfl_xor(acc, s);
  if constexpr (TPR > 64) {
    if ((tid & 63) == 0)
      wave_sum[tid >> 6] = acc;
    __syncthreads();
    if (sub == 0) {
      acc = 0.0f;
      for (int w = 0; w < TPR / 64; w++)
        acc += wave_sum[(tid >> 6) + w];
    }
  }
  if (sub == 0 && row < rows) {
    if (p.mean)
      acc = acc / (float)p.n_red;
    regs[p.n_in + p.sum_ins][tid] = round_to_storage(acc, sum.dt);
    const int64_t idx = row * p.n_red; // the per-row inputs have stride 0 along the row
    if (small)
      fused_load<uint32_t>(p, regs, tid, (uint32_t)idx, p.n_in_pre, p.n_in);
    else
      fused_load<int64_t>(p, regs, tid, idx, p.n_in_pre, p.n_in);
    fused_run(p, regs, tid, p.sum_ins + 1, p.n_ins);
    store_from_f32(p.out, row, p.out_dt, regs[p.out_reg][tid]);
  }
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
extern "C" int gcmi_launch_fused(const FusedParams *pp, hipStream_t stream) {
  FusedParams p = *pp;
  if (p.n <= 0)
    return 0;
  const bool has_sum = p.sum_ins >= 0;
  if (p.n_in < 1 || p.n_in > FUSED_MAX_IN || p.n_ins < 0 || p.n_ins > FUSED_MAX_INS || p.sum_ins >= p.n_ins)
    return 2;
  if (!has_sum)
    p.n_in_pre = p.n_in, p.n_red = 1;
  if (p.n_in_pre < 0 || p.n_in_pre > p.n_in || p.n_red < 1 || p.n % p.n_red != 0)
    return 2;
  for (int j = 0; j < p.n_ins; j++) {
    // an instruction reads registers that are already written; before the sum, only per-element inputs
    const FusedIns &f = p.ins[j];
    const bool unary_sum = f.op == ELT_ROWSUM;
    if ((f.op == ELT_ROWSUM) != (j == p.sum_ins))
      return 2;
    for (int r : {f.a, unary_sum ? f.a : f.b}) {
      if (r < 0 || r >= p.n_in + j)
        return 2;
      if (has_sum && j <= p.sum_ins && r >= p.n_in_pre && r < p.n_in)
        return 2;
      if (has_sum && j > p.sum_ins && (r < p.n_in_pre || (r >= p.n_in && r < p.n_in + p.sum_ins)))
        return 2; // per-element values do not exist after the sum
    }
  }
  if (p.out_reg < 0 || p.out_reg >= p.n_in + p.n_ins || (has_sum && p.out_reg < p.n_in + p.sum_ins))
    return 2;
  // merge neighbouring iteration dims that every input walks contiguously (or not at all): fewer divisions per
  // element.  The boundary between rows and the inside of a row is never merged across.
  int64_t dims[ELT_MAX_RANK], str[FUSED_MAX_IN][ELT_MAX_RANK];
  int nd = 0;
  int64_t inner = 1; // elements of the dims to the right of d
  for (int d = ELT_MAX_RANK - 1; d >= 0; d--) {
    if (p.dims[d] == 1)
      continue;
    bool merge = nd > 0 && !(has_sum && inner == p.n_red);
    for (int k = 0; k < p.n_in && merge; k++)
      merge = p.in_str[k][d] == str[k][nd - 1] * dims[nd - 1];
    if (merge) {
      dims[nd - 1] *= p.dims[d];
    } else {
      dims[nd] = p.dims[d];
      for (int k = 0; k < p.n_in; k++)
        str[k][nd] = p.in_str[k][d];
      nd++;
    }
    inner *= p.dims[d];
  }
  for (int d = 0; d < ELT_MAX_RANK; d++) {
    const int src = ELT_MAX_RANK - 1 - d; // dims[] was filled innermost first
    p.dims[d] = src < nd ? dims[src] : 1;
    for (int k = 0; k < p.n_in; k++)
      p.in_str[k][d] = src < nd ? str[k][src] : 0;
  }
  p.rank = nd;
  if (has_sum) {
    const int64_t rows = p.n / p.n_red;
    if (p.n_red >= 1024 || rows < 64) {
      if (rows > 0x7fffffff)
        return 2;
      hipLaunchKernelGGL(fused_rowsum_kernel<1>, dim3((unsigned)rows), dim3(FUSED_THREADS), 0, stream, p);
    } else {
      const int64_t blocks = (rows + 3) / 4;
      if (blocks > 0x7fffffff)
        return 2;
      hipLaunchKernelGGL(fused_rowsum_kernel<4>, dim3((unsigned)blocks), dim3(FUSED_THREADS), 0, stream, p);
    }
  } else {
    int64_t blocks = (p.n + FUSED_THREADS - 1) / FUSED_THREADS;
    if (blocks > 16384)
      blocks = 16384;
    hipLaunchKernelGGL(fused_pointwise_kernel, dim3((unsigned)blocks), dim3(FUSED_THREADS), 0, stream, p);
  }
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
