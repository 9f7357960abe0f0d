// f32 GEMM (exact f32 FMA, no reduced-precision matrix path) and the
// batch-reduce microkernel with the reference's operand layouts.
//
// gemm_f32_kernel: C[M,N] = act(beta*C + A.B + bias), arbitrary element strides
// on A and B so that transpose_a / transpose_b of onednn_graph.matmul
// (lib/gc/Transforms/OneDNNGraphToLinalg.cpp:421-499) need no copy.
// 64x64 workgroup tile, 16-deep K slices through LDS, 4x4 outputs per thread,
// k ascending per output element.
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

__global__ __launch_bounds__(256) void gemm_f32_kernel(F32GemmParams p) {
  __shared__ float As[16][64 + 4];
  __shared__ float Bs[16][64 + 4];
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const int64_t m0 = (int64_t)blockIdx.y * 64, n0 = (int64_t)blockIdx.x * 64;
  float acc[4][4] = {};
  for (int64_t k0 = 0; k0 < p.K; k0 += 16) {
    // 64x16 of A and 16x64 of B: 1024 elements each, 4 per thread
#pragma unroll
    for (int e = 0; e < 4; e++) {
      int idx = threadIdx.x + 256 * e;
      int am = idx & 63, ak = idx >> 6; // consecutive threads along m
      if (p.a_cs == 1) {                // k contiguous: walk k fastest instead
        ak = idx & 15;
        am = idx >> 4;
      }
      int64_t gm = m0 + am, gk = k0 + ak;
      As[ak][am] = (gm < p.M && gk < p.K) ? p.A[gm * p.a_rs + gk * p.a_cs] : 0.0f;
      int bn = idx & 63, bk = idx >> 6;
      if (p.b_rs == 1 && p.b_cs != 1) {
        bk = idx & 15;
        bn = idx >> 4;
      }
      int64_t gn = n0 + bn, gk2 = k0 + bk;
      Bs[bk][bn] = (gn < p.N && gk2 < p.K) ? p.B[gk2 * p.b_rs + gn * p.b_cs] : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 16; k++) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; i++)
        a[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; j++)
        b[j] = Bs[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
          acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; i++) {
    int64_t m = m0 + ty * 4 + i;
    if (m >= p.M)
      continue;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      int64_t n = n0 + tx * 4 + j;
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
  dim3 grid((unsigned)((p.N + 63) / 64), (unsigned)((p.M + 63) / 64)), block(256);
  hipLaunchKernelGGL(gemm_f32_kernel, grid, block, 0, stream, p);
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
