// f32 GEMM (f32 multiply-add throughout: vector FMAs, or the f32 matrix
// instruction on whole tiles; no reduced precision) and the
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
// thread per C element, operands staged through LDS, batch-major then k ascending as the reference sums, and
// every product and every sum rounded on its own (no fused multiply-add: the
// reference's loop is plain C++ built for baseline x86-64, which has none), so
// f32 results equal the reference's bit for bit; bf16 products are exact in f32
// and integer sums are exact anyway.
#include "common.hpp"
#include <type_traits>
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

// The same GEMM on the matrix cores for whole 128 x 128 tiles of row-major operands: v_mfma_f32_32x32x2_f32 multiplies
// and adds in f32 (no reduced precision), 256 flop per clock and compute unit against 128 for the vector ALU's FMA.
// 256 threads = 4 waves as 2 x 2, a wave owns 64 x 64 = four 32 x 32 tiles (64 accumulator registers); 16-deep K
// slices through LDS, the next slice prefetched into registers.  A is stored k-major in LDS ([k][m]) so that a
// fragment read (lane = row, k = lane / 32) is one conflict-free ds_read_b32 per tile, B as it lies in memory.
__global__ __launch_bounds__(256) void gemm_f32_mfma_kernel(F32GemmParams p) {
  constexpr int BT = 128, BK = 16;
  __shared__ float As[BK][BT + 4];
  __shared__ float Bs[BK][BT + 4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, lh = lane >> 5;
  const int64_t m0 = (int64_t)blockIdx.y * BT, n0 = (int64_t)blockIdx.x * BT;
  p.A += (int64_t)blockIdx.z * p.a_bs, p.B += (int64_t)blockIdx.z * p.b_bs, p.C += (int64_t)blockIdx.z * p.c_bs;
  // slice loads, 16 bytes per thread and operand piece: A 128 rows x 16 k = 512 float4 (two per thread: row = idx / 4,
  // k = 4 * (idx % 4)), B 16 k x 128 n = 512 float4 (k = idx / 32, n = 4 * (idx % 32))
  f32x4_t ra[2], rb[2];
  auto fetch = [&](int64_t k0) {
#pragma unroll
    for (int e = 0; e < 2; e++) {
      const int idx = tid + 256 * e;
      ra[e] = *reinterpret_cast<const f32x4_t *>(p.A + (m0 + idx / 4) * p.a_rs + k0 + 4 * (idx % 4));
      rb[e] = *reinterpret_cast<const f32x4_t *>(p.B + (k0 + idx / 32) * p.b_rs + n0 + 4 * (idx % 32));
    }
  };
  f32x16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int r = 0; r < 16; r++)
        acc[i][j][r] = 0.0f;
  fetch(0);
  for (int64_t k0 = 0; k0 < p.K; k0 += BK) {
#pragma unroll
    for (int e = 0; e < 2; e++) {
      const int idx = tid + 256 * e;
#pragma unroll
      for (int c = 0; c < 4; c++)
        As[4 * (idx % 4) + c][idx / 4] = ra[e][c];
      *reinterpret_cast<f32x4_t *>(&Bs[idx / 32][4 * (idx % 32)]) = rb[e];
    }
    __syncthreads();
    if (k0 + BK < p.K)
      fetch(k0 + BK);
#pragma unroll
    for (int ks = 0; ks < BK; ks += 2) { // k ascending per output element
      float a[2], b[2];
#pragma unroll
      for (int i = 0; i < 2; i++)
        a[i] = As[ks + lh][wm * 64 + i * 32 + l32];
#pragma unroll
      for (int j = 0; j < 2; j++)
        b[j] = Bs[ks + lh][wn * 64 + j * 32 + l32];
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
  }
  // lane (l32, lh) holds column l32 and rows 8 * (r / 4) + 4 * lh + r % 4 of every tile: 32 lanes write 128 bytes
#pragma unroll
  for (int j = 0; j < 2; j++) {
    const int64_t n = n0 + wn * 64 + j * 32 + l32;
    const float bias = p.bias ? p.bias[n] : 0.0f;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int64_t m = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
        float x = acc[i][j][r];
        if (p.beta != 0.0f)
          x = x + p.C[m * p.ldc + n];
        if (p.bias)
          x = x + bias;
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

// One workgroup = one 16 x 16 tile of C, one thread per element.  The terms of an element's sum keep the reference's
// order (batch-major, k ascending, each product and each sum rounded on its own), so the only freedom is where the
// operands come from: the workgroup stages BRG_CH terms' worth of its 16 rows of A and 16 columns of B in LDS as
// widened values (f32, or s32 for the 8-bit types), both with the terms contiguous so that four terms come out of
// one 16-byte read per operand -- and the loads of the next chunk are in flight in registers while this chunk is
// summed.  A chunk is a run of whole batches when K is small (the usual 32 x 32 x 32 call) or a slice of one batch's
// K.  K tails of the packed layouts are never read and never added (adding a zero would turn a -0 sum into +0).
// A wave issues a vector instruction that needs its predecessor's result only every 8-9 cycles, so the chain of num*K dependent sums
// is the floor; everything else is kept short: element offsets are worked out once, a chunk adds two scalars.
static constexpr int BRG_CH = 128, BRG_PITCH = BRG_CH + 4, BRG_PER = 16 * BRG_CH / 256;

template <typename ACC, int V> // V: the k elements packed beside each other in B (1 f32, 2 bf16, 4 8-bit)
__global__ __launch_bounds__(256) void brgemm_kernel(BrgemmParams p) {
#pragma clang fp contract(off) // a product and the sum it goes into are rounded separately, as the reference's are
  __shared__ __attribute__((aligned(16))) ACC As[16][BRG_PITCH]; // [row of the tile][term of the chunk]
  __shared__ __attribute__((aligned(16))) ACC Bs[16][BRG_PITCH]; // [column of the tile][term of the chunk]
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const int64_t n0 = (int64_t)blockIdx.x * 16, m0 = (int64_t)blockIdx.y * 16;
  // chunk geometry: kc terms of K per batch and chunk, nb batches per chunk; chunks run batch group by batch group
  // and, inside one, K slice by K slice
  const int kc = p.K < BRG_CH ? (int)p.K : BRG_CH;
  const int nb = p.K < BRG_CH ? BRG_CH / (kc > 0 ? kc : 1) : 1;
  const int64_t kchunks = p.K > 0 ? (p.K + kc - 1) / kc : 0;
  const int64_t nchunks = ((p.num + nb - 1) / nb) * kchunks;
  const bool a_signed = p.dtA == DT_S8, b_signed = p.dtB == DT_S8;

  // Loads keep the raw element (a register each); widening waits until the value goes to LDS, one chunk later, so
  // that nothing between a load and the sums of the current chunk needs the loaded value.
  typedef typename std::conditional<V == 1, float, uint32_t>::type RAW;
  auto load = [&](const void *base, int64_t idx) -> RAW {
    if constexpr (V == 1)
      return ((const float *)base)[idx];
    else if constexpr (V == 2)
      return ((const uint16_t *)base)[idx];
    else
      return ((const uint8_t *)base)[idx];
  };
  auto widen = [&](RAW v, bool is_signed) -> ACC {
    if constexpr (V == 1)
      return v;
    else if constexpr (V == 2)
      return __uint_as_float(v << 16);
    else
      return is_signed ? (int)(v ^ 0x80u) - 0x80 : (int)v;
  };
  // Slot e of a chunk.  A: (row, term), terms along consecutive threads.  B: (term group, column, k within the
  // group), the order B lies in memory.  Term t of a chunk = (batch t / kc, k t % kc) relative to the chunk's first
  // batch and first k (a multiple of V, so the packed position of k does not depend on the chunk).
  int64_t a_off[BRG_PER], b_off[BRG_PER];
  int a_bat[BRG_PER], a_k[BRG_PER], b_bat[BRG_PER], b_k[BRG_PER];
#pragma unroll
  for (int e = 0; e < BRG_PER; e++) {
    const int idx = threadIdx.x + 256 * e;
    const int ta = idx % BRG_CH, tb = (idx / (16 * V)) * V + idx % V;
    const int kd = kc > 0 ? kc : 1;
    const int64_t m = m0 + idx / BRG_CH, n = n0 + (idx % (16 * V)) / V;
    a_bat[e] = (ta < nb * kc && m < p.M) ? ta / kd : 1 << 30, a_k[e] = ta % kd; // 1 << 30: never a valid batch
    b_bat[e] = (tb < nb * kc && n < p.N) ? tb / kd : 1 << 30, b_k[e] = tb % kd;
    a_off[e] = (int64_t)(ta / kd) * p.stride_a + m * p.LDA + a_k[e];
    b_off[e] = (int64_t)(tb / kd) * p.stride_b + (int64_t)(b_k[e] - b_k[e] % V) * p.LDB + V * n + b_k[e] % V;
  }
  RAW ra[BRG_PER], rb[BRG_PER];
  auto fetch = [&](int64_t b0, int64_t k0) {
    const int64_t a_chunk = b0 * p.stride_a + k0, b_chunk = b0 * p.stride_b + k0 * p.LDB;
    const int64_t bats = p.num - b0, ks = p.K - k0; // batches and k left from here
#pragma unroll
    for (int e = 0; e < BRG_PER; e++) {
      ra[e] = (a_bat[e] < bats && a_k[e] < ks) ? load(p.A, a_off[e] + a_chunk) : RAW(0);
      rb[e] = (b_bat[e] < bats && b_k[e] < ks) ? load(p.B, b_off[e] + b_chunk) : RAW(0);
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int e = 0; e < BRG_PER; e++) {
      const int idx = threadIdx.x + 256 * e;
      As[idx / BRG_CH][idx % BRG_CH] = widen(ra[e], a_signed);
      Bs[(idx % (16 * V)) / V][(idx / (16 * V)) * V + idx % V] = widen(rb[e], b_signed);
    }
  };
  auto term = [](ACC s, ACC a, ACC b) -> ACC {
    if constexpr (V == 4)
      return __mul24(a, b) + s; // 8-bit values: one 24-bit multiply-add, exact
    else
      return s + a * b;
  };
  const int64_t m = m0 + ty, n = n0 + tx;
  const bool mine = m < p.M && n < p.N;
  ACC *c = (ACC *)p.C + m * p.LDC + n;
  ACC s = (p.beta_zero || !mine) ? ACC(0) : *c;
  int64_t b0 = 0, k0 = 0, b0n = 0, k0n = 0; // this chunk's first batch and k, and the next chunk's
  auto advance = [&]() {
    k0n += kc;
    if (k0n >= p.K)
      k0n = 0, b0n += nb;
  };
  if (nchunks > 0) {
    fetch(0, 0);
    advance();
  }
  typedef ACC acc4 __attribute__((ext_vector_type(4)));
  for (int64_t ch = 0; ch < nchunks; ch++) {
    stash();
    __syncthreads();
    if (ch + 1 < nchunks)
      fetch(b0n, k0n);
    const int nbat = (int)((p.num - b0) < nb ? (p.num - b0) : nb);
    const int klen = (int)((p.K - k0) < kc ? (p.K - k0) : kc);
    for (int bi = 0; bi < nbat; bi++) {
      const int t0 = bi * kc;
      int k = 0;
      if ((kc & 3) == 0) { // every batch of the chunk starts on a 16-byte boundary
#pragma unroll 2
        for (; k + 4 <= klen; k += 4) {
          const acc4 a = *reinterpret_cast<const acc4 *>(&As[ty][t0 + k]);
          const acc4 b = *reinterpret_cast<const acc4 *>(&Bs[tx][t0 + k]);
          s = term(s, a.x, b.x);
          s = term(s, a.y, b.y);
          s = term(s, a.z, b.z);
          s = term(s, a.w, b.w);
        }
      }
      for (; k < klen; k++)
        s = term(s, As[ty][t0 + k], Bs[tx][t0 + k]);
    }
    __syncthreads();
    b0 = b0n, k0 = k0n;
    advance();
  }
  if (mine)
    *c = s;
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
  // whole 128 x 128 tiles of row-major operands with 16-byte aligned rows, and enough of them: the matrix cores
  auto al16 = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  if (p.a_cs == 1 && p.b_cs == 1 && p.M % 128 == 0 && p.N % 128 == 0 && p.K % 16 == 0 && p.K > 0 && p.a_rs % 4 == 0 &&
      p.b_rs % 4 == 0 && al16(p.A) && al16(p.B) && (nbatch == 1 || (p.a_bs % 4 == 0 && p.b_bs % 4 == 0)) &&
      (p.M / 128) * (p.N / 128) * nbatch >= 64 && p.M / 128 <= 65535) {
    dim3 grid((unsigned)(p.N / 128), (unsigned)(p.M / 128), (unsigned)nbatch);
    hipLaunchKernelGGL(gemm_f32_mfma_kernel, grid, dim3(256), 0, stream, p);
    return hipGetLastError() == hipSuccess ? 0 : 5;
  }
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
  if (grid.y > 65535)
    return 2;
  if (dtA == DT_F32)
    hipLaunchKernelGGL((brgemm_kernel<float, 1>), grid, block, 0, stream, p);
  else if (dtA == DT_BF16)
    hipLaunchKernelGGL((brgemm_kernel<float, 2>), grid, block, 0, stream, p);
  else
    hipLaunchKernelGGL((brgemm_kernel<int32_t, 4>), grid, block, 0, stream, p);
  return hipGetLastError() == hipSuccess ? 0 : 5;
}
