// f32 GEMM (exact f32 FMA, no reduced-precision matrix path) and the
// batch-reduce microkernel with the reference's operand layouts.
//
// gemm_f32_kernel: C[M,N] = act(beta*C + A.B + bias), arbitrary element strides
// on A and B so that transpose_a / transpose_b of onednn_graph.matmul
// (lib/gc/Transforms/OneDNNGraphToLinalg.cpp:421-499) need no copy.
// 64/32/16-square workgroup tiles, 32-deep K slices through LDS with register
// prefetch, k ascending per output element.
//
// brgemm_kernel: C[m*LDC+n] (+)= sum_i sum_k a(i,m,k) * b(i,k,n) with
//   f32 : b at i*stride_b + k*LDB + n
//   bf16: b at i*stride_b + (k - k%2)*LDB + 2n + k%2      (VNNI-2)
//   8bit: b at i*stride_b + (k - k%4)*LDB + 4n + k%4      (VNNI-4)
// (lib/gc/ExecutionEngine/CPURuntime/Microkernel/BrgemmNaive.cpp:46-140).
// Microkernel calls are small (typically 32x32x32 with a batch of 8-16); one
// thread per C element, batch-major then k ascending as the reference sums.
#include "common.hpp"
#include "gemm_params.h"

namespace gcmi {

// BT x BT workgroup tile (BT = 64, 32 or 16: small problems take small tiles so
// that more compute units take part), 256 threads, (BT/16)^2 outputs per thread,
// 32-deep K slices through LDS.  The next slice is fetched into registers while
// the current one is multiplied, so global latency is paid once, not per slice.
template <int BT> __global__ __launch_bounds__(256) void gemm_f32_kernel(F32GemmParams p) {
  constexpr int BK = 32, MT = BT / 16, PER = BT * BK / 256; // elements per thread per operand slice
  __shared__ float As[BK][BT + 4];
  __shared__ float Bs[BK][BT + 4];
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const int64_t m0 = (int64_t)blockIdx.y * BT, n0 = (int64_t)blockIdx.x * BT;
  p.A += (int64_t)blockIdx.z * p.a_bs, p.B += (int64_t)blockIdx.z * p.b_bs, p.C += (int64_t)blockIdx.z * p.c_bs;
  // slice element e of this thread: (row/col within the tile, k within the slice);
  // the contiguous direction of each operand runs along consecutive threads
  int am[PER], ak[PER], bn[PER], bk[PER];
#pragma unroll
  for (int e = 0; e < PER; e++) {
    const int idx = threadIdx.x + 256 * e;
    if (p.a_cs == 1) {
      ak[e] = idx % BK;
      am[e] = idx / BK;
    } else {
      am[e] = idx % BT;
      ak[e] = idx / BT;
    }
    if (p.b_rs == 1 && p.b_cs != 1) {
      bk[e] = idx % BK;
      bn[e] = idx / BK;
    } else {
      bn[e] = idx % BT;
      bk[e] = idx / BT;
    }
  }
  float ra[PER], rb[PER];
  auto fetch = [&](int64_t k0) {
#pragma unroll
    for (int e = 0; e < PER; e++) {
      const int64_t gm = m0 + am[e], gk = k0 + ak[e];
      ra[e] = (gm < p.M && gk < p.K) ? p.A[gm * p.a_rs + gk * p.a_cs] : 0.0f;
      const int64_t gn = n0 + bn[e], gk2 = k0 + bk[e];
      rb[e] = (gn < p.N && gk2 < p.K) ? p.B[gk2 * p.b_rs + gn * p.b_cs] : 0.0f;
    }
  };
  float acc[MT][MT] = {};
  fetch(0);
  for (int64_t k0 = 0; k0 < p.K; k0 += BK) {
#pragma unroll
    for (int e = 0; e < PER; e++) {
      As[ak[e]][am[e]] = ra[e];
      Bs[bk[e]][bn[e]] = rb[e];
    }
    __syncthreads();
    if (k0 + BK < p.K)
      fetch(k0 + BK);
#pragma unroll
    for (int k = 0; k < BK; k++) { // k ascending per output element
      float a[MT], b[MT];
#pragma unroll
      for (int i = 0; i < MT; i++)
        a[i] = As[k][ty * MT + i];
#pragma unroll
      for (int j = 0; j < MT; j++)
        b[j] = Bs[k][tx * MT + j];
#pragma unroll
      for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < MT; j++)
          acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < MT; i++) {
    int64_t m = m0 + ty * MT + i;
    if (m >= p.M)
      continue;
#pragma unroll
    for (int j = 0; j < MT; j++) {
      int64_t n = n0 + tx * MT + j;
      if (n >= p.N)
        continue;
      float x = acc[i][j];
      if (p.beta != 0.0f)
        x = x + p.C[m * p.ldc + n];
      if (p.bias)
        x = x + p.bias[n];
      p.C[m * p.ldc + n] = apply_act(x, p.act);
    }
  }
}

struct BrgemmParams {
  const void *A, *B;
  void *C;
  int64_t M, N, K, LDA, LDB, LDC, stride_a, stride_b;
  int32_t num, beta_zero, dtA, dtB;
};

__global__ __launch_bounds__(256) void brgemm_kernel(BrgemmParams p) {
  const int64_t n = (int64_t)blockIdx.x * 16 + (threadIdx.x & 15);
  const int64_t m = (int64_t)blockIdx.y * 16 + (threadIdx.x >> 4);
  if (m >= p.M || n >= p.N)
    return;
  if (p.dtA == DT_F32) {
    const float *a = (const float *)p.A, *b = (const float *)p.B;
    float *c = (float *)p.C + m * p.LDC + n;
    float s = p.beta_zero ? 0.0f : *c;
    for (int i = 0; i < p.num; i++)
      for (int64_t k = 0; k < p.K; k++)
        s += a[i * p.stride_a + m * p.LDA + k] * b[i * p.stride_b + k * p.LDB + n];
    *c = s;
  } else if (p.dtA == DT_BF16) {
    const uint16_t *a = (const uint16_t *)p.A, *b = (const uint16_t *)p.B;
    float *c = (float *)p.C + m * p.LDC + n;
    float s = p.beta_zero ? 0.0f : *c;
    for (int i = 0; i < p.num; i++)
      for (int64_t k = 0; k < p.K; k++)
        s += bf16_bits_to_f32(a[i * p.stride_a + m * p.LDA + k]) *
             bf16_bits_to_f32(b[i * p.stride_b + (k & ~(int64_t)1) * p.LDB + 2 * n + (k & 1)]);
    *c = s;
  } else {
    const uint8_t *a = (const uint8_t *)p.A, *b = (const uint8_t *)p.B;
    int32_t *c = (int32_t *)p.C + m * p.LDC + n;
    int32_t s = p.beta_zero ? 0 : *c;
    for (int i = 0; i < p.num; i++)
      for (int64_t k = 0; k < p.K; k++) {
        uint8_t ar = a[i * p.stride_a + m * p.LDA + k];
        uint8_t br = b[i * p.stride_b + (k & ~(int64_t)3) * p.LDB + 4 * n + (k & 3)];
        int av = p.dtA == DT_S8 ? (int)(int8_t)ar : (int)ar;
        int bv = p.dtB == DT_S8 ? (int)(int8_t)br : (int)br;
        s += av * bv;
      }
    *c = s;
  }
}

} // namespace gcmi

using namespace gcmi;

extern "C" int gcmi_launch_gemm_f32(const F32GemmParams *pp, hipStream_t stream) {
  F32GemmParams p = *pp;
  if (p.M <= 0 || p.N <= 0)
    return 0;
  // the largest tile that still gives every compute unit a workgroup
  const int64_t nbatch = p.batch > 1 ? p.batch : 1;
  if (nbatch > 65535)
    return 2;
  auto tiles = [&](int bt) { return ((p.N + bt - 1) / bt) * ((p.M + bt - 1) / bt) * nbatch; };
  const int bt = tiles(64) >= 256 ? 64 : tiles(32) >= 256 ? 32 : 16;
  dim3 grid((unsigned)((p.N + bt - 1) / bt), (unsigned)((p.M + bt - 1) / bt), (unsigned)nbatch), block(256);
  if (grid.y > 65535)
    return 2;
  if (bt == 64)
    hipLaunchKernelGGL(gemm_f32_kernel<64>, grid, block, 0, stream, p);
  else if (bt == 32)
    hipLaunchKernelGGL(gemm_f32_kernel<32>, grid, block, 0, stream, p);
  else
    hipLaunchKernelGGL(gemm_f32_kernel<16>, grid, block, 0, stream, p);
  return hipGetLastError() == hipSuccess ? 0 : 5;
}

extern "C" int gcmi_launch_brgemm(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K, int64_t LDA,
                                  int64_t LDB, int64_t LDC, int64_t stride_a, int64_t stride_b, int num, int beta_zero,
                                  int dtA, int dtB, hipStream_t stream) {
  if (M <= 0 || N <= 0)
    return 0;
  BrgemmParams p{A, B, C, M, N, K, LDA, LDB, LDC, stride_a, stride_b, num, beta_zero, dtA, dtB};
  dim3 grid((unsigned)((N + 15) / 16), (unsigned)((M + 15) / 16)), block(256);
  hipLaunchKernelGGL(brgemm_kernel, grid, block, 0, stream, p);
  return hipGetLastError() == hipSuccess ? 0 : 5;
}
