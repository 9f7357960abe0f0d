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

// The same for 16-byte aligned rows (HBM bound: the weight is read once, 16 bytes per lane).  A workgroup takes a
// strip of 256 columns and one of CS_SLICES slices of K: thread t reads columns 16*(t%16)..+15 of rows t/16, t/16+16,
// ...; a byte is picked out of a dword and added with one v_dot4_i32_i8 against a one-hot selector.  The 16 row lanes
// of a column add up through LDS, slices through integer atomics (exact in any order) into a zeroed result.
static constexpr int CS_SLICES = 16;
__global__ __launch_bounds__(256) void colsum_s8_zero_kernel(int32_t *out, int64_t N) {
  const int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (n < N)
    out[n] = 0;
}
__global__ __launch_bounds__(256) void colsum_s8_wide_kernel(const int8_t *W, int64_t K, int64_t N, int64_t ldw, int32_t *out) {
  __shared__ int part[16][257];
  const int cchunk = threadIdx.x & 15, rlane = threadIdx.x >> 4;
  const int64_t n0 = (int64_t)blockIdx.x * 256 + cchunk * 16;
  const int64_t per = (K + CS_SLICES - 1) / CS_SLICES, k0 = blockIdx.y * per, k1 = min(K, k0 + per);
  int acc[16];
#pragma unroll
  for (int c = 0; c < 16; c++)
    acc[c] = 0;
  if (n0 < N) { // N is a multiple of 16: a chunk is inside or outside as a whole
    const int8_t *p = W + n0;
    for (int64_t k = k0 + rlane; k < k1; k += 64) { // four loads in flight per lane
      i32x4_t v[4];
#pragma unroll
      for (int u = 0; u < 4; u++)
        v[u] = k + 16 * u < k1 ? *reinterpret_cast<const i32x4_t *>(p + (k + 16 * u) * ldw) : i32x4_t{0, 0, 0, 0};
#pragma unroll
      for (int u = 0; u < 4; u++)
#pragma unroll
        for (int d = 0; d < 4; d++)
#pragma unroll
          for (int b = 0; b < 4; b++)
            acc[4 * d + b] = __builtin_amdgcn_sdot4(v[u][d], 1 << (8 * b), acc[4 * d + b], false);
    }
  }
#pragma unroll
  for (int c = 0; c < 16; c++)
    part[rlane][cchunk * 16 + c] = acc[c];
  __syncthreads();
  const int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (n < N) {
    int t = 0;
#pragma unroll
    for (int r = 0; r < 16; r++)
      t += part[r][threadIdx.x];
    atomicAdd(out + n, t);
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
  if (N % 16 == 0 && ldw % 16 == 0 && (reinterpret_cast<uintptr_t>(W) & 15) == 0 && K >= 256) {
    const unsigned strips = (unsigned)((N + 255) / 256);
    hipLaunchKernelGGL(colsum_s8_zero_kernel, dim3(strips), dim3(256), 0, stream, (int32_t *)out, N);
    hipLaunchKernelGGL(colsum_s8_wide_kernel, dim3(strips, CS_SLICES), dim3(256), 0, stream, (const int8_t *)W, K, N, ldw,
                       (int32_t *)out);
    return hipGetLastError() == hipSuccess ? 0 : 5;
  }
  dim3 grid((unsigned)((N + 63) / 64)), block(64, 8);
  hipLaunchKernelGGL(colsum_s8_kernel, grid, block, 0, stream, (const int8_t *)W, K, N, ldw, (int32_t *)out);
  return hipGetLastError() == hipSuccess ? 0 : 5;
}
