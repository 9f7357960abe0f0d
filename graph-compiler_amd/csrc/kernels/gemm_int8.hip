// (u8|s8) x s8 -> s32 instantiation of the 256x256 MFMA GEMM (see
// gemm_tile256.hpp) and the weight column-sum kernel.
#include "gemm_tile256.hpp"

namespace gcmi {

// column sums of an s8 [K,N] weight in s32 (weight-only constant of the
// asymmetric-activation compensation, legacy/core/src/ops/matmul_core.cpp:
// 546-557).  One thread per column, coalesced along n; K split over blockDim.y
// with an LDS reduction.
__global__ void colsum_s8_kernel(const int8_t *W, int64_t K, int64_t N, int64_t ldw, int32_t *out) {
  __shared__ int part[8][64];
  const int64_t n = (int64_t)blockIdx.x * 64 + threadIdx.x;
  int s = 0;
  if (n < N)
    for (int64_t k = threadIdx.y; k < K; k += 8)
      s += (int)W[k * ldw + n];
  part[threadIdx.y][threadIdx.x] = s;
  __syncthreads();
  if (threadIdx.y == 0 && n < N) {
    int t = 0;
#pragma unroll
    for (int y = 0; y < 8; y++)
      t += part[y][threadIdx.x];
    out[n] = t;
  }
}

} // namespace gcmi

using namespace gcmi;

extern "C" int gcmi_launch_gemm_int8(const GemmParams *p, hipStream_t stream) { return launch_tile256<1>(p, stream); }

extern "C" int gcmi_launch_gemm_int8_config(const GemmParams *p, GemmTileConfig *cfg) {
  return launch_tile256<1>(p, (hipStream_t)-1, nullptr, cfg);
}

extern "C" int gcmi_launch_colsum_s8(const void *W, int64_t K, int64_t N, int64_t ldw, void *out, hipStream_t stream) {
  if (N <= 0)
    return 0;
  dim3 grid((unsigned)((N + 63) / 64)), block(64, 8);
  hipLaunchKernelGGL(colsum_s8_kernel, grid, block, 0, stream, (const int8_t *)W, K, N, ldw, (int32_t *)out);
  return hipGetLastError() == hipSuccess ? 0 : 5;
}
