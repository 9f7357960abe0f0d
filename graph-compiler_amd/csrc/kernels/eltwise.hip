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
  case ELT_LOG: return logf(x);
  case ELT_ROUND: return roundf(x); // math.round: halves away from zero
  case ELT_RSQRT: return 1.0f / sqrtf(x);
  case ELT_SQRT: return sqrtf(x);
  case ELT_SQUARE: return x * x;
  case ELT_TANH: return tanhf(x);
  case ELT_RECIP: return 1.0f / x;
  default: return x; // ELT_COPY
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
    default: r = fused_op(p.op, x, y, p.alpha); break; // ELT_COPY (typecast / strided gather) and the arithmetic ops
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
static constexpr int FUSED_THREADS = 256;

// The register file: register r of thread tid is regs[r * blockDim.x + tid] in dynamic LDS, sized by the launcher
// to the registers the program uses.
struct FusedRegs {
  float *base;
  int threads, tid;
  __device__ __forceinline__ float &operator[](int r) const { return base[r * threads + tid]; }
};

// adds to off[k] (inputs k0 .. k1-1) the contribution of the coordinates of `idx` over iteration dims d_lo .. d_hi-1
// (innermost first); a single dim needs no division
template <typename IDX>
__device__ __forceinline__ void fused_offsets(const FusedParams &p, IDX idx, int d_lo, int d_hi, int k0, int k1,
                                              IDX (&off)[FUSED_MAX_IN]) {
  if (d_hi - d_lo == 1) {
#pragma unroll
    for (int k = 0; k < FUSED_MAX_IN; k++)
      if (k >= k0 && k < k1)
        off[k] += idx * (IDX)p.in_str[k][d_lo];
    return;
  }
  IDX rem = idx;
  for (int d = d_hi - 1; d >= d_lo; d--) {
    const IDX dim = (IDX)p.dims[d];
    const IDX c = rem % dim;
    rem /= dim;
#pragma unroll
    for (int k = 0; k < FUSED_MAX_IN; k++)
      if (k >= k0 && k < k1)
        off[k] += c * (IDX)p.in_str[k][d];
  }
}

// instructions j0 .. j1-1
__device__ __forceinline__ void fused_run(const FusedParams &p, const FusedRegs &regs, int j0, int j1) {
  for (int j = j0; j < j1; j++) {
    const FusedIns in = p.ins[j];
    const float x = regs[in.a], y = regs[in.b];
    regs[p.n_in + j] = round_to_storage(fused_op(in.op, x, y, in.imm), in.dt);
  }
}

// The parameter block is read many times (once per instruction per element) and the kernel-argument segment is
// slow to reach on a first touch: all threads copy it into LDS together, one word each, so its cache lines are
// fetched side by side instead of one after the other.
__device__ __forceinline__ void fused_params_to_lds(FusedParams *dst) {
  const uint32_t *src = (const uint32_t *)__builtin_amdgcn_kernarg_segment_ptr();
  uint32_t *d = reinterpret_cast<uint32_t *>(dst);
  for (unsigned w = threadIdx.x; w < sizeof(FusedParams) / 4; w += blockDim.x)
    d[w] = src[w];
  __syncthreads();
}

template <typename IDX> __device__ __forceinline__ void fused_pointwise_body(const FusedParams &p, const FusedRegs &regs) {
  const int d0 = ELT_MAX_RANK - p.rank;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < p.n; idx += (int64_t)gridDim.x * blockDim.x) {
    IDX off[FUSED_MAX_IN];
#pragma unroll
    for (int k = 0; k < FUSED_MAX_IN; k++)
      off[k] = 0;
    fused_offsets<IDX>(p, (IDX)idx, d0, ELT_MAX_RANK, 0, p.n_in, off);
#pragma unroll
    for (int k = 0; k < FUSED_MAX_IN; k++)
      if (k < p.n_in)
        regs[k] = load_as_f32(p.in[k], (int64_t)off[k], p.in_dt[k]);
    fused_run(p, regs, 0, p.n_ins);
    store_from_f32(p.out, idx, p.out_dt, regs[p.out_reg]);
  }
}

__global__ __launch_bounds__(FUSED_THREADS) void fused_pointwise_kernel(FusedParams) {
  extern __shared__ float fused_lds[];
  __shared__ FusedParams p;
  fused_params_to_lds(&p);
  const FusedRegs regs{fused_lds, (int)blockDim.x, (int)threadIdx.x};
  if (p.n < ((int64_t)1 << 31)) // 32-bit index arithmetic when the whole space fits
    fused_pointwise_body<uint32_t>(p, regs);
  else
    fused_pointwise_body<int64_t>(p, regs);
}

// TPR threads work on one row (a multiple of 64: whole waves), THREADS / TPR rows per workgroup.  The loads of
// several elements per thread are in flight together; partial sums are combined in a fixed tree, so results do not
// vary from run to run.
template <typename IDX, int THREADS, int TPR>
__device__ __forceinline__ void fused_rowsum_body(const FusedParams &p, const FusedRegs &regs, float *wave_sum) {
  constexpr int U = TPR >= 1024 ? 2 : 4; // 1024 threads leave 128 registers per lane
  const int tid = threadIdx.x, sub = tid % TPR;
  const int64_t rows = p.n / p.n_red;
  const int64_t row = (int64_t)blockIdx.x * (THREADS / TPR) + tid / TPR;
  const int d0 = ELT_MAX_RANK - p.rank, d_row = ELT_MAX_RANK - p.rank_red;
  const FusedIns sum = p.ins[p.sum_ins];
  float acc = 0.0f;
  IDX base[FUSED_MAX_IN];
#pragma unroll
  for (int k = 0; k < FUSED_MAX_IN; k++)
    base[k] = 0;
  if (row < rows) {
    fused_offsets<IDX>(p, (IDX)row, d0, d_row, 0, p.n_in, base);
    for (int64_t r0 = sub; r0 < p.n_red; r0 += (int64_t)TPR * U) {
      float v[U][FUSED_MAX_IN];
#pragma unroll
      for (int u = 0; u < U; u++) {
        const int64_t r = r0 + (int64_t)u * TPR;
        if (r < p.n_red) {
          IDX off[FUSED_MAX_IN];
#pragma unroll
          for (int k = 0; k < FUSED_MAX_IN; k++)
            off[k] = base[k];
          fused_offsets<IDX>(p, (IDX)r, d_row, ELT_MAX_RANK, 0, p.n_in_pre, off);
#pragma unroll
          for (int k = 0; k < FUSED_MAX_IN; k++)
            if (k < p.n_in_pre)
              v[u][k] = load_as_f32(p.in[k], (int64_t)off[k], p.in_dt[k]);
        }
      }
#pragma unroll
      for (int u = 0; u < U; u++) {
        if (r0 + (int64_t)u * TPR < p.n_red) {
#pragma unroll
          for (int k = 0; k < FUSED_MAX_IN; k++)
            if (k < p.n_in_pre)
              regs[k] = v[u][k];
          fused_run(p, regs, 0, p.sum_ins);
          acc += regs[sum.a];
        }
      }
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
    regs[p.n_in + p.sum_ins] = round_to_storage(acc, sum.dt);
#pragma unroll
    for (int k = 0; k < FUSED_MAX_IN; k++) // the per-row inputs have stride 0 along the row
      if (k >= p.n_in_pre && k < p.n_in)
        regs[k] = load_as_f32(p.in[k], (int64_t)base[k], p.in_dt[k]);
    fused_run(p, regs, p.sum_ins + 1, p.n_ins);
    store_from_f32(p.out, row, p.out_dt, regs[p.out_reg]);
  }
}

template <int THREADS, int TPR> __global__ __launch_bounds__(THREADS) void fused_rowsum_kernel(FusedParams) {
  extern __shared__ float fused_lds[];
  __shared__ float wave_sum[THREADS / 64];
  __shared__ FusedParams p;
  fused_params_to_lds(&p);
  const FusedRegs regs{fused_lds, THREADS, (int)threadIdx.x};
  if (p.n < ((int64_t)1 << 31))
    fused_rowsum_body<uint32_t, THREADS, TPR>(p, regs, wave_sum);
  else
    fused_rowsum_body<int64_t, THREADS, TPR>(p, regs, wave_sum);
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
  // collapsed dims that lie inside a row
  p.rank_red = 0;
  for (int64_t in_row = 1; has_sum && in_row < p.n_red && p.rank_red < nd; p.rank_red++)
    in_row *= dims[p.rank_red];
  const size_t n_regs = (size_t)(p.n_in + p.n_ins);
  if (has_sum) {
    const int64_t rows = p.n / p.n_red;
    if (rows > 0x7fffffff)
      return 2;
    // few long rows: 1024 threads per row when their registers fit the 64 KiB a launch may ask for
    if (p.n_red >= 2048 && rows < 1024 && n_regs * 1024 * 4 + sizeof(FusedParams) + 256 <= 65536) {
      hipLaunchKernelGGL((fused_rowsum_kernel<1024, 1024>), dim3((unsigned)rows), dim3(1024), n_regs * 1024 * 4, stream, p);
    } else if (p.n_red >= 512 || rows < 64) {
      hipLaunchKernelGGL((fused_rowsum_kernel<256, 256>), dim3((unsigned)rows), dim3(256), n_regs * 256 * 4, stream, p);
    } else {
      hipLaunchKernelGGL((fused_rowsum_kernel<256, 64>), dim3((unsigned)((rows + 3) / 4)), dim3(256), n_regs * 256 * 4, stream,
                         p);
    }
  } else {
    int64_t blocks = (p.n + FUSED_THREADS - 1) / FUSED_THREADS;
    if (blocks > 16384)
      blocks = 16384;
    hipLaunchKernelGGL(fused_pointwise_kernel, dim3((unsigned)blocks), dim3(FUSED_THREADS), n_regs * FUSED_THREADS * 4, stream,
                       p);
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
