// Element-wise, reduction, softmax and (de)quantise kernels for the ops of a
// partition that are not fused into a GEMM or attention kernel: single-op
// kernels, and the kernels that run a whole group of point-wise ops (with an
// optional row sum inside) as one launch.  Every op
// reads its operands in their storage type (f32 / bf16 / f16 / s8 / u8 / s32),
// computes in f32 and rounds once to the result type, which is what the
// reference's bf16->f32 emulation does to each op
// (lib/gc/Transforms/Pipeline.cpp:79-95).  Semantics per op:
//   Add/Subtract/Multiply/Divide  numpy broadcasting
//                                 (lib/gc/Transforms/OneDNNGraphToLinalg.cpp:64-118)
//   Maximum / Minimum / Exp / Neg / Abs / Ceil / Floor / Erf / Log / Round / Rsqrt / Sqrt / Square / Tanh /
//   Reciprocal                    the named linalg ops of the MLIR front end (arith / math semantics; Round is
//                                 math.round, halves away from zero)
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
static constexpr int FU = 4; // elements a thread carries through the program together

// fused groups hold float storage types only: one 4-byte or one 2-byte load
__device__ __forceinline__ float fused_load_f32(const void *p, int64_t i, int dt) {
  if (dt == DT_F32)
    return reinterpret_cast<const float *>(p)[i];
  const uint16_t h = reinterpret_cast<const uint16_t *>(p)[i];
  return dt == DT_BF16 ? bf16_bits_to_f32(h) : (float)__builtin_bit_cast(_Float16, h);
}
__device__ __forceinline__ void fused_store_f32(void *p, int64_t i, int dt, float v) {
  if (dt == DT_F32)
    reinterpret_cast<float *>(p)[i] = v;
  else
    reinterpret_cast<uint16_t *>(p)[i] = dt == DT_BF16 ? f32_to_bf16_bits(v) : __builtin_bit_cast(uint16_t, (_Float16)v);
}

// The register file: register r of thread t is the 16-byte slot (r * threads + t) of dynamic LDS, holding the FU
// elements the thread carries (one ds_read_b128 / ds_write_b128 per access, conflict free).  Register numbers are
// only known at run time, which costs nothing extra this way.
typedef float fused_vec __attribute__((ext_vector_type(FU)));
struct FusedRegs {
  fused_vec *base;
  int threads, tid;
  __device__ __forceinline__ fused_vec get(int r) const { return base[r * threads + tid]; }
  __device__ __forceinline__ void set(int r, fused_vec v) const { base[r * threads + tid] = v; }
};

// The parameter block is read many times (once per instruction per step) and the kernel-argument segment is slow to
// reach on a first touch: all threads copy it into LDS together, one word each, so its cache lines are fetched side
// by side instead of one after the other.
__device__ __forceinline__ void fused_params_to_lds(FusedParams *dst) {
  const uint32_t *src = (const uint32_t *)__builtin_amdgcn_kernarg_segment_ptr();
  uint32_t *d = reinterpret_cast<uint32_t *>(dst);
  for (unsigned w = threadIdx.x; w < sizeof(FusedParams) / 4; w += blockDim.x)
    d[w] = src[w];
  __syncthreads();
}

// instructions j0 .. j1-1 on the FU elements a thread holds
__device__ __forceinline__ void fused_run(const FusedParams &p, const FusedRegs &f, int j0, int j1) {
  for (int j = j0; j < j1; j++) {
    const FusedIns in = p.ins[j];
    const int op = __builtin_amdgcn_readfirstlane(in.op), dt = __builtin_amdgcn_readfirstlane(in.dt);
    const float imm = in.imm;
    const fused_vec x = f.get(in.a), y = f.get(in.b);
    fused_vec v;
    switch (op) {
#define EACH(expr)                                                                                                        \
  _Pragma("unroll") for (int u = 0; u < FU; u++) v[u] = (expr);                                                           \
  break;
    case ELT_ADD: v = x + y; break;
    case ELT_SUB: v = x - y; break;
    case ELT_MUL: v = x * y; break;
    case ELT_DIV: EACH(x[u] / y[u])
    case ELT_NEG: v = -x; break;
    case ELT_SQUARE: v = x * x; break;
    case ELT_COPY: v = x; break;
    default: EACH(fused_op(op, x[u], y[u], imm))
#undef EACH
    }
    if (dt == DT_BF16) {
#pragma unroll
      for (int u = 0; u < FU; u++)
        v[u] = bf16_bits_to_f32(f32_to_bf16_bits(v[u]));
    } else if (dt == DT_F16) {
#pragma unroll
      for (int u = 0; u < FU; u++)
        v[u] = (float)(_Float16)v[u];
    }
    f.set(in.d, v);
  }
}

// offsets of inputs k0 .. k1-1 for element idx, coordinates taken over iteration dims d_lo .. d_hi-1 (innermost
// first), added to off[]; a single dim needs no division
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

// Four consecutive elements of one input: one 16- or 8-byte load when the input is contiguous there (vec), else
// four loads `step` elements apart (step 0: a broadcast along the innermost dim)
__device__ __forceinline__ fused_vec fused_load_quad(const void *p, int64_t i, int dt, bool vec, int64_t step) {
  fused_vec v;
  if (vec) {
    if (dt == DT_F32) {
      const f32x4_t q = *reinterpret_cast<const f32x4_t *>(reinterpret_cast<const float *>(p) + i);
      v[0] = q[0], v[1] = q[1], v[2] = q[2], v[3] = q[3];
    } else {
      const uint2 q = *reinterpret_cast<const uint2 *>(reinterpret_cast<const uint16_t *>(p) + i);
      const uint16_t h[4] = {(uint16_t)q.x, (uint16_t)(q.x >> 16), (uint16_t)q.y, (uint16_t)(q.y >> 16)};
#pragma unroll
      for (int u = 0; u < 4; u++)
        v[u] = dt == DT_BF16 ? bf16_bits_to_f32(h[u]) : (float)__builtin_bit_cast(_Float16, h[u]);
    }
  } else {
#pragma unroll
    for (int u = 0; u < 4; u++)
      v[u] = fused_load_f32(p, i + u * step, dt);
  }
  return v;
}
__device__ __forceinline__ void fused_store_quad(void *p, int64_t i, int dt, bool vec, int64_t step, fused_vec v) {
  if (vec) {
    if (dt == DT_F32) {
      *reinterpret_cast<f32x4_t *>(reinterpret_cast<float *>(p) + i) = f32x4_t{v[0], v[1], v[2], v[3]};
    } else {
      uint16_t h[4];
#pragma unroll
      for (int u = 0; u < 4; u++)
        h[u] = dt == DT_BF16 ? f32_to_bf16_bits(v[u]) : __builtin_bit_cast(uint16_t, (_Float16)v[u]);
      *reinterpret_cast<uint2 *>(reinterpret_cast<uint16_t *>(p) + i) =
          make_uint2(h[0] | ((uint32_t)h[1] << 16), h[2] | ((uint32_t)h[3] << 16));
    }
  } else {
#pragma unroll
    for (int u = 0; u < 4; u++)
      fused_store_f32(p, i + u * step, dt, v[u]);
  }
}
static_assert(FU == 4, "the quad loads and stores move four elements");

// Inputs k0 .. k1-1 of the four elements a thread holds into their registers.  quad: the elements are e0 .. e0+3
// of one innermost row (the launcher sets it when the innermost dim is a multiple of 4), so one set of offsets
// serves all four; otherwise they are the separate elements e[u] (ok[u] false: skipped).
template <typename IDX>
__device__ __forceinline__ void fused_load(const FusedParams &p, const FusedRegs &f, const IDX (&e)[FU], const bool (&ok)[FU],
                                           const IDX (&base)[FUSED_MAX_IN], int d_lo, int d_hi, int k0, int k1) {
  if (p.quad) {
    if (!ok[0])
      return;
    IDX off[FUSED_MAX_IN];
#pragma unroll
    for (int k = 0; k < FUSED_MAX_IN; k++)
      off[k] = base[k];
    fused_offsets<IDX>(p, e[0], d_lo, d_hi, k0, k1, off);
    fused_vec v[FUSED_MAX_IN];
#pragma unroll
    for (int k = 0; k < FUSED_MAX_IN; k++) // all loads are issued before the first LDS write waits for one
      if (k >= k0 && k < k1)
        v[k] = fused_load_quad(p.in[k], (int64_t)off[k], p.in_dt[k], (p.vec_mask >> k) & 1,
                               p.in_str[k][ELT_MAX_RANK - 1]);
#pragma unroll
    for (int k = 0; k < FUSED_MAX_IN; k++)
      if (k >= k0 && k < k1)
        f.set(p.in_reg[k], v[k]);
    return;
  }
  fused_vec v[FUSED_MAX_IN];
#pragma unroll
  for (int u = 0; u < FU; u++) {
    IDX off[FUSED_MAX_IN];
#pragma unroll
    for (int k = 0; k < FUSED_MAX_IN; k++)
      off[k] = base[k];
    if (ok[u])
      fused_offsets<IDX>(p, e[u], d_lo, d_hi, k0, k1, off);
#pragma unroll
    for (int k = 0; k < FUSED_MAX_IN; k++)
      if (k >= k0 && k < k1)
        v[k][u] = ok[u] ? fused_load_f32(p.in[k], (int64_t)off[k], p.in_dt[k]) : 0.0f;
  }
#pragma unroll
  for (int k = 0; k < FUSED_MAX_IN; k++)
    if (k >= k0 && k < k1)
      f.set(p.in_reg[k], v[k]);
}

// the four elements of thread `t` in the step that starts at element c0, `threads` threads taking part
template <typename IDX>
__device__ __forceinline__ void fused_elements(const FusedParams &p, int64_t c0, int64_t limit, int t, int threads,
                                               IDX (&e)[FU], bool (&ok)[FU]) {
#pragma unroll
  for (int u = 0; u < FU; u++) {
    // quad: four consecutive elements per thread; otherwise consecutive threads take consecutive elements
    const int64_t idx = p.quad ? c0 + (int64_t)FU * t + u : c0 + (int64_t)u * threads + t;
    ok[u] = idx < limit;
    e[u] = (IDX)idx;
  }
}

// IDX: 32-bit index arithmetic when the whole iteration space fits (the launcher picks), 64-bit otherwise.
// A workgroup takes FU * FUSED_THREADS consecutive elements per step.
template <typename IDX> __global__ __launch_bounds__(FUSED_THREADS) void fused_pointwise_kernel(FusedParams) {
  extern __shared__ fused_vec fused_lds[];
  __shared__ FusedParams p;
  fused_params_to_lds(&p);
  const FusedRegs f{fused_lds, FUSED_THREADS, (int)threadIdx.x};
  const int d0 = ELT_MAX_RANK - p.rank;
  IDX zero[FUSED_MAX_IN];
#pragma unroll
  for (int k = 0; k < FUSED_MAX_IN; k++)
    zero[k] = 0;
  const int64_t chunk = (int64_t)FU * FUSED_THREADS;
  for (int64_t c0 = (int64_t)blockIdx.x * chunk; c0 < p.n; c0 += (int64_t)gridDim.x * chunk) {
    IDX e[FU];
    bool ok[FU];
    fused_elements<IDX>(p, c0, p.n, threadIdx.x, FUSED_THREADS, e, ok);
    fused_load<IDX>(p, f, e, ok, zero, d0, ELT_MAX_RANK, 0, p.n_in);
    fused_run(p, f, 0, p.n_ins);
    const fused_vec v = f.get(p.out_reg);
    if (p.quad) { // the output is dense: four consecutive elements are contiguous
      if (ok[0])
        fused_store_quad(p.out, (int64_t)e[0], p.out_dt, p.out_vec, 1, v);
    } else {
#pragma unroll
      for (int u = 0; u < FU; u++)
        if (ok[u])
          fused_store_f32(p.out, (int64_t)e[u], p.out_dt, v[u]);
    }
  }
}

// TPR threads work on one row (a multiple of 64: whole waves), THREADS / TPR rows per workgroup.  Every thread of a
// row ends up with the row's sum (partial sums are combined in a fixed tree: results do not vary from run to run)
// and runs the per-row instructions itself, so the second pass needs no exchange.
// (Four waves per SIMD are asked for: the kernel is latency bound, and 128 registers with a few spilled words
// measured 10-25 % faster on row counts from 1024 up than the 144 registers the compiler takes by itself.)
template <typename IDX, int THREADS, int TPR>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(4, 8))) void fused_rowsum_kernel(FusedParams) {
  extern __shared__ fused_vec fused_lds[];
  __shared__ float wave_sum[THREADS / 64];
  __shared__ FusedParams p;
  fused_params_to_lds(&p);
  const FusedRegs f{fused_lds, THREADS, (int)threadIdx.x};
  const int tid = threadIdx.x, sub = tid % TPR;
  const int64_t rows = p.n / p.n_red;
  const int64_t row_raw = (int64_t)blockIdx.x * (THREADS / TPR) + tid / TPR;
  const bool live = row_raw < rows;
  const int64_t row = live ? row_raw : rows - 1; // threads past the last row shadow it and store nothing
  const int d0 = ELT_MAX_RANK - p.rank, d_row = ELT_MAX_RANK - p.rank_red;
  const int sum_a = p.ins[p.sum_ins].a, sum_d = p.ins[p.sum_ins].d, sum_dt = p.ins[p.sum_ins].dt;
  IDX base[FUSED_MAX_IN];
#pragma unroll
  for (int k = 0; k < FUSED_MAX_IN; k++)
    base[k] = 0;
  fused_offsets<IDX>(p, (IDX)row, d0, d_row, 0, p.n_in, base);

  float acc = 0.0f;
  for (int64_t r0 = 0; r0 < p.n_red; r0 += (int64_t)TPR * FU) {
    IDX e[FU];
    bool ok[FU];
    fused_elements<IDX>(p, r0, p.n_red, sub, TPR, e, ok);
    fused_load<IDX>(p, f, e, ok, base, d_row, ELT_MAX_RANK, 0, p.n_in_pre);
    fused_run(p, f, 0, p.sum_ins);
    const fused_vec v = f.get(sum_a);
#pragma unroll
    for (int u = 0; u < FU; u++)
      if (p.quad ? ok[0] : ok[u])
        acc += v[u];
  }
#pragma unroll
  for (int s = 32; s > 0; s >>= 1)
    acc += __shfl_xor(acc, s);
  if constexpr (TPR > 64) {
    if ((tid & 63) == 0)
      wave_sum[tid >> 6] = acc;
    __syncthreads();
    acc = 0.0f;
    const int w0 = (tid / TPR) * (TPR / 64);
    for (int w = 0; w < TPR / 64; w++)
      acc += wave_sum[w0 + w];
  }
  if (p.mean)
    acc = acc / (float)p.n_red;
  acc = sum_dt == DT_BF16 ? bf16_bits_to_f32(f32_to_bf16_bits(acc)) : sum_dt == DT_F16 ? (float)(_Float16)acc : acc;
  f.set(sum_d, fused_vec(acc));
  // per-row inputs (stride 0 along the row): the same value in every element slot
#pragma unroll
  for (int k = 0; k < FUSED_MAX_IN; k++)
    if (k >= p.n_in_pre && k < p.n_in_row)
      f.set(p.in_reg[k], fused_vec(fused_load_f32(p.in[k], (int64_t)base[k], p.in_dt[k])));
  fused_run(p, f, p.sum_ins + 1, p.row_end);
  if (p.row_end >= p.n_ins) { // no second pass: one value per row
    const fused_vec v = f.get(p.out_reg);
    if (sub == 0 && live)
      fused_store_f32(p.out, row, p.out_dt, v[0]);
    return;
  }
  // second pass: the output is walked through its own strides
  auto out_offset = [&](IDX idx, int d_lo, int d_hi) {
    IDX o = 0, rem = idx;
    for (int d = d_hi - 1; d >= d_lo; d--) {
      const IDX dim = (IDX)p.dims[d];
      o += (rem % dim) * (IDX)p.out_str[d];
      rem /= dim;
    }
    return o;
  };
  const IDX obase = out_offset((IDX)row, d0, d_row);
  for (int64_t r0 = 0; r0 < p.n_red; r0 += (int64_t)TPR * FU) {
    IDX e[FU];
    bool ok[FU];
    fused_elements<IDX>(p, r0, p.n_red, sub, TPR, e, ok);
    fused_load<IDX>(p, f, e, ok, base, d_row, ELT_MAX_RANK, p.n_in_row, p.n_in);
    fused_run(p, f, p.row_end, p.n_ins);
    const fused_vec v = f.get(p.out_reg);
    if (!live)
      continue;
    if (p.quad) {
      if (ok[0])
        fused_store_quad(p.out, (int64_t)(obase + out_offset(e[0], d_row, ELT_MAX_RANK)), p.out_dt, p.out_vec,
                         p.out_str[ELT_MAX_RANK - 1], v);
    } else {
#pragma unroll
      for (int u = 0; u < FU; u++)
        if (ok[u])
          fused_store_f32(p.out, (int64_t)(obase + out_offset(e[u], d_row, ELT_MAX_RANK)), p.out_dt, v[u]);
    }
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
  const int bad = fused_prepare(p, false);
  if (bad)
    return bad;
  const bool has_sum = p.sum_ins >= 0;
  if (fused_allocate(p) > FUSED_MAX_PHYS)
    return 3;
  const size_t lds = (size_t)p.n_phys * 256 * sizeof(float) * FU; // the kernels with 256 threads
  const bool small = p.n < ((int64_t)1 << 31);
  if (has_sum) {
    const int64_t rows = p.n / p.n_red;
    if (rows > 0x7fffffff)
      return 2;
    // few long rows: as many threads per row as the registers leave room for in 64 KiB of LDS
    const size_t per_thread = (size_t)p.n_phys * sizeof(float) * FU, room = 65536 - sizeof(FusedParams) - 512;
    if (rows < 512 && p.n_red >= 2048 && per_thread * 512 <= room) { // (1024 threads leave 128 registers: spills)
      const dim3 grid((unsigned)rows), block(512);
      if (small)
        hipLaunchKernelGGL((fused_rowsum_kernel<uint32_t, 512, 512>), grid, block, per_thread * 512, stream, p);
      else
        hipLaunchKernelGGL((fused_rowsum_kernel<int64_t, 512, 512>), grid, block, per_thread * 512, stream, p);
    } else if (p.n_red >= 512 || rows < 64) { // a workgroup of 256 per row
      const dim3 grid((unsigned)rows), block(256);
      if (small)
        hipLaunchKernelGGL((fused_rowsum_kernel<uint32_t, 256, 256>), grid, block, lds, stream, p);
      else
        hipLaunchKernelGGL((fused_rowsum_kernel<int64_t, 256, 256>), grid, block, lds, stream, p);
    } else { // a wave per row
      const dim3 grid((unsigned)((rows + 3) / 4)), block(256);
      if (small)
        hipLaunchKernelGGL((fused_rowsum_kernel<uint32_t, 256, 64>), grid, block, lds, stream, p);
      else
        hipLaunchKernelGGL((fused_rowsum_kernel<int64_t, 256, 64>), grid, block, lds, stream, p);
    }
  } else {
    int64_t blocks = (p.n + FU * FUSED_THREADS - 1) / (FU * FUSED_THREADS);
    if (blocks > 16384)
      blocks = 16384;
    if (small)
      hipLaunchKernelGGL(fused_pointwise_kernel<uint32_t>, dim3((unsigned)blocks), dim3(FUSED_THREADS), lds, stream, p);
    else
      hipLaunchKernelGGL(fused_pointwise_kernel<int64_t>, dim3((unsigned)blocks), dim3(FUSED_THREADS), lds, stream, p);
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
