// bf16 GEMM for a short A (M <= 128) against wide weights, stored [N,K] (k contiguous) or [K,N]:
// C[M,N] = epilogue(A . W).
// This is the decode-time shape of the reference's llama2 case (test/benchgc/cases/llama2.mlir: 32 tokens against
// 4096 x 4096 .. 4096 x 11008 weights), where the reference splits K over threads (KThreads,
// lib/gc/Analysis/MatmulConfigAnalysis.cpp:149-166).  The arithmetic is negligible; the job is to pull the weights
// from HBM once at the rate the memory system gives.  Measured on MI355X with read-only probes of the same 32-90 MB:
// requests whose 64 lanes cover whole 128-byte lines reach 5.1-5.5 TB/s from 8-wave workgroups that follow their
// rows along K (5.7-6.1 TB/s for one linear sweep of the buffer), 64-byte pieces of 16 rows 4.5-5.2, 32-byte pieces
// of 32 rows 3.2-4.4 -- the vector memory pipe pays per cache line it looks up -- and every fragment of A that a
// wave fetches for itself costs look-ups of its own.  Hence:
//   * a workgroup is 8 waves on a panel of 64 columns and one slice of K; a stage is 256 bytes of K per row: the A
//     tile (32 rows, 8 KiB, shared by all waves; 64 or 128 rows past that) and the panel's weights (16 KiB) go to
//     an LDS ring by global_load_lds_dwordx4, 4 rows x 256 bytes per request, one request (two, four) for A and
//     two for the weights per wave;
//   * A is re-read once per panel (half the weights' traffic, from L2) instead of once per 16 columns;
//   * wave w owns column tile w % 4 and k-steps 2 * (w / 4), 2 * (w / 4) + 1 of the stage's four; the two halves are
//     added through LDS at the end (upper onto lower: a fixed order); one barrier per stage.
// A row's 16 chunks of 16 bytes sit at chunk ^ (row % 16), so the 16 rows of a fragment read fall on 16 different
// bank groups.  With 172 panels or more (N >= 11008) K is not sliced and the epilogue runs here in the one launch;
// narrower weights are cut into K slices (blockIdx.y) whose f32 partial sums go to the workspace, and
// gemm_splitk_reduce_kernel adds them in slice order and runs the epilogue: no result depends on timing.  (Adding the
// slices in the same launch -- the workgroup that takes a panel's last ticket reads the others' sums -- was built
// twice and is slower than the second kernel: with device-scope fences every workgroup writes back and invalidates
// an L2 that the others stream through, 59 against 14 us; with device-scope stores and loads instead of fences the
// word-sized write-through stores cost more than the launch saves, 12.9 against 11.2 us.)
// Measured, [N,K] / [K,N]: 32 x 4096 x 4096 11.0 / 11.1 us (13.2 us with 32-byte pieces straight into registers; 16 us
// on K slices of 128 x 128 tiles), 32 x 11008 x 4096 22.7 / 23.1 us in one launch (28.9; 24), 32 x 4096 x 11008
// 23.5 / 24.0 us (28.4; 24).
#pragma once
#include "gemm_tile256.hpp"

namespace gcmi {

static constexpr int R32_BM = 32, R32_BN = 64, R32_KB = 256, R32_NST = 3;

// Four results of row m, columns n .. n+3, from their f32 sums: the rounding points of a bf16 graph (after the
// matmul and after every op, lib/gc/Transforms/Pipeline.cpp:79-95), or one f32 epilogue.
__device__ __forceinline__ void rows32_store4(const GemmParams &p, const f32x4_t &v, int64_t m, int64_t n) {
  float o32[4];
  uint16_t o16[4];
#pragma unroll
  for (int c = 0; c < 4; c++) {
    float b = 0.0f;
    if (p.bias)
      b = p.bias_dt == DT_BF16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t *>(p.bias)[n + c])
                               : reinterpret_cast<const float *>(p.bias)[n + c];
    float x = v[c], r = 0.0f;
    if (p.residual)
      r = p.residual_dt == DT_BF16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t *>(p.residual)[m * p.ldr + n + c])
                                   : reinterpret_cast<const float *>(p.residual)[m * p.ldr + n + c];
    if (p.out_dt == DT_BF16) {
      x = round_bf16(x);
      if (p.bias)
        x = round_bf16(x + b);
      if (p.act != ACT_NONE)
        x = round_bf16(apply_act(x, p.act));
      if (p.residual)
        x = round_bf16(x + r);
    } else {
      if (p.bias)
        x = x + b;
      x = apply_act(x, p.act);
      if (p.residual) { // kept apart from the activation's last multiply: the sum equals a separate add
#pragma clang fp contract(off)
        x = x + r;
      }
    }
    o32[c] = x;
    o16[c] = f32_to_bf16_bits(x);
  }
  if (p.out_dt == DT_BF16)
    *reinterpret_cast<uint2 *>(reinterpret_cast<uint16_t *>(p.C) + m * p.ldc + n) =
        make_uint2(o16[0] | ((uint32_t)o16[1] << 16), o16[2] | ((uint32_t)o16[3] << 16));
  else
    *reinterpret_cast<f32x4_t *>(reinterpret_cast<float *>(p.C) + m * p.ldc + n) = f32x4_t{o32[0], o32[1], o32[2], o32[3]};
}

// MT: 16-row tiles of A (2: up to 32 rows; 4: up to 64; 8: up to 128, with an A tile of 16 / 32 KiB per stage)
// TB: the weights are stored [N,K]; else [K,N]: a stage's weights are then 128 k-rows of 128 bytes (the panel's 64
// columns), requested 8 k-rows at a time (whole lines again) and read through the transposing LDS load; a k-row's 8
// chunks sit at chunk ^ 2 * (k / 2 % 2 + 2 * (k / 8 % 2)), which spreads the 8 k-rows that 32 lanes of a transposing
// read touch over all banks.
template <int MT, bool TB> __global__ __launch_bounds__(512, 1) void gemm_rows32_kernel(GemmParams p) {
  static_assert(MT == 2 || MT == 4 || MT == 8, "32, 64 or 128 rows");
  constexpr int KB = R32_KB, BK = KB / 2, NST = R32_NST, BN = R32_BN;
  constexpr int A_BYTES = 16 * MT * KB, B_BYTES = BN * KB, STAGE = A_BYTES + B_BYTES; // 8 (16) + 16 KiB
  constexpr int NA_DMA = MT / 2;    // A requests per wave and stage
  constexpr int PER = NA_DMA + 2;   // requests per wave and stage
  __shared__ __align__(1024) char smem[NST * STAGE];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ct = wave & 3, half = wave >> 2;
  const int r16 = lane & 15, g16 = lane >> 4;
  const int64_t n0 = (int64_t)blockIdx.x * BN;
  const int cols_in = (int)min((int64_t)BN, p.N - n0);
  const int64_t lda_b = p.lda * 2, ldb_b = p.ldb * 2;

  int KT = (int)(p.K / BK), k_first = 0;
  const int slice = blockIdx.y;
  if (p.splits > 1) {
    const int g0 = (int)((int64_t)slice * KT / p.splits), g1 = (int)((int64_t)(slice + 1) * KT / p.splits);
    k_first = g0, KT = g1 - g0;
  }
  uint32_t a_src[NA_DMA], b_src[2];
  {
    const int pos = lane & 15;
#pragma unroll
    for (int i = 0; i < NA_DMA; i++) {
      const int row = 4 * (NA_DMA * wave + i) + (lane >> 4);
      a_src[i] = (uint32_t)(min(row, (int)p.M - 1) * lda_b + ((pos ^ (row & 15)) << 4));
    }
#pragma unroll
    for (int i = 0; i < 2; i++) {
      if constexpr (TB) {
        const int rb = 4 * (2 * wave + i) + (lane >> 4);
        b_src[i] = (uint32_t)(min(rb, cols_in - 1) * ldb_b + ((pos ^ (rb & 15)) << 4));
      } else {
        const int krow = 8 * (2 * wave + i) + (lane >> 3), c8 = lane & 7;
        const int swz = (((krow >> 1) & 1) | (((krow >> 3) & 1) << 1)) << 1;
        b_src[i] = (uint32_t)(krow * ldb_b + (min(c8 ^ swz, cols_in / 8 - 1) << 4));
      }
    }
  }
  const char *a_ptr = reinterpret_cast<const char *>(p.A) + (int64_t)k_first * KB;
  const int64_t b_step = TB ? (int64_t)KB : (int64_t)BK * ldb_b; // bytes from one stage of the weights to the next
  const char *b_ptr = reinterpret_cast<const char *>(p.B) + (TB ? n0 * ldb_b : n0 * 2) + (int64_t)k_first * b_step;
  // (the __restrict__ pointers give the requests and the fragment reads separate alias scopes: without them the
  // compiler makes every fragment read wait for all requests in flight)
  auto issue = [&](char *__restrict__ stage, int kt) {
#pragma unroll
    for (int i = 0; i < NA_DMA; i++)
      __builtin_amdgcn_global_load_lds((GCMI_GLB const void *)(a_ptr + (int64_t)kt * KB + a_src[i]),
                                       (GCMI_LDS void *)(stage + (NA_DMA * wave + i) * 1024), 16, 0, 0);
#pragma unroll
    for (int i = 0; i < 2; i++)
      __builtin_amdgcn_global_load_lds((GCMI_GLB const void *)(b_ptr + kt * b_step + b_src[i]),
                                       (GCMI_LDS void *)(stage + A_BYTES + (2 * wave + i) * 1024), 16, 0, 0);
  };
  const uint32_t a_ld = (uint32_t)(r16 * KB);
  uint32_t b_ld = (uint32_t)(A_BYTES + (16 * ct + r16) * KB);
  if constexpr (!TB) { // the 16 lanes of a group hand the transposing read 4 k-rows x 16 columns in 8-byte pieces
    const int kk = r16 >> 2, cc = r16 & 3;
    const int swz = (((kk >> 1) & 1) | ((g16 & 1) << 1)) << 1; // of k-row 8 * g16 + kk (+ 4, + 32 per k-step: the same)
    b_ld = (uint32_t)(A_BYTES + (8 * g16 + kk) * 128 + (((2 * ct + (cc >> 1)) ^ swz) << 4) + (cc & 1) * 8);
  }
  f32x4_t acc[MT];
#pragma unroll
  for (int it = 0; it < MT; it++)
    acc[it] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  auto compute = [&](const char *__restrict__ st) {
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const int sw = ((4 * (2 * half + u) + g16) ^ r16) << 4; // rows 16 * x + r16: row % 16 = r16
      uint4 fa[MT];
#pragma unroll
      for (int it = 0; it < MT; it++)
        fa[it] = *reinterpret_cast<const uint4 *>(st + a_ld + it * 16 * KB + sw);
      uint4 fb;
      if constexpr (TB) {
        fb = *reinterpret_cast<const uint4 *>(st + b_ld + sw);
      } else {
        const uint2 lo = MfmaOp<2>::tr_read(st + b_ld + (2 * half + u) * 4096);
        const uint2 hi = MfmaOp<2>::tr_read(st + b_ld + (2 * half + u) * 4096 + 512);
        fb = make_uint4(lo.x, lo.y, hi.x, hi.y);
      }
#pragma unroll
      for (int it = 0; it < MT; it++)
        acc[it] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, fb), __builtin_bit_cast(bf16x8_t, fa[it]), acc[it],
                                                          0, 0, 0);
    }
  };
#pragma unroll
  for (int d = 0; d < NST - 1; d++)
    if (d < KT)
      issue(smem + d * STAGE, d);
  for (int kt = 0; kt < KT; kt++) {
    // this wave's requests of stage kt have landed (those of the NST - 2 stages behind it may be in flight; near the
    // end fewer were issued, so everything is awaited); barrier: stage kt is visible, the slot of stage kt - 1 is free
    if (kt + NST - 2 < KT)
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NST - 2) * PER) : "memory");
    else
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    if (kt + NST - 1 < KT)
      issue(smem + ((kt + NST - 1) % NST) * STAGE, kt + NST - 1);
    compute(smem + (kt % NST) * STAGE);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // this wave's reads of the stage are over before the next barrier
  }
  // upper k half onto the lower one
  __syncthreads();
  float *red = reinterpret_cast<float *>(smem);
  if (half == 1) {
#pragma unroll
    for (int it = 0; it < MT; it++)
      *reinterpret_cast<f32x4_t *>(red + ((ct * MT + it) * 64 + lane) * 4) = acc[it];
  }
  __syncthreads();
  float *part = p.partial + (int64_t)slice * p.M * p.N;
  if (half == 0) {
#pragma unroll
    for (int it = 0; it < MT; it++) {
      const f32x4_t o = *reinterpret_cast<const f32x4_t *>(red + ((ct * MT + it) * 64 + lane) * 4);
      const f32x4_t v = {acc[it][0] + o[0], acc[it][1] + o[1], acc[it][2] + o[2], acc[it][3] + o[3]};
      const int64_t m = 16 * it + r16;
      const int col = 16 * ct + 4 * g16;
      if (m >= p.M || col >= cols_in)
        continue;
      if (p.splits > 1)
        *reinterpret_cast<f32x4_t *>(part + m * p.N + n0 + col) = v;
      else
        rows32_store4(p, v, m, n0 + col);
    }
  }
}

// Takes the call when the shape is this kernel's (returns -1 otherwise: the other kernels handle it).
// want != null: nothing is launched; *want receives the floats of workspace this call would use if it had them.
static int launch_rows32(const GemmParams *pp, hipStream_t stream, int64_t *want = nullptr, GemmTileConfig *cfg = nullptr) {
  GemmParams p = *pp;
  if (want)
    *want = 0;
  const bool dry = want != nullptr || (cfg != nullptr && stream == (hipStream_t)-1);
  const int64_t ws_cap = want ? INT64_MAX : (p.partial ? p.partial_cap : 0);
  auto al16 = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  const int res_es = p.residual_dt == DT_BF16 ? 2 : 4;
  if (p.batch > 1 || p.M < 1 || p.M > 4 * R32_BM || p.N % (p.trans_b ? 4 : 8) != 0 || p.K % 128 != 0 || p.K < 512 || !al16(p.A) || !al16(p.B) ||
      !al16(p.C) || (p.lda * 2) % 16 != 0 || (p.ldb * 2) % 16 != 0 || p.ldc % 4 != 0 || p.out_dt == DT_S32 ||
      (p.residual && (!al16(p.residual) || (p.ldr * res_es) % 8 != 0)) || p.cfg_tile == 128)
    return -1;
  // [K,N] weights: a caller's MatmulConfig names a workgroup tile, and that tile it gets (with [N,K] weights only the
  // slice count of such a config is used)
  if (!p.trans_b && p.cfg_tile != 0)
    return -1;
  // rows reachable with 32-bit byte offsets from the tile's first row
  if (p.lda * 2 * 4 * R32_BM >= (int64_t)1 << 31 || p.ldb * 2 * 128 >= (int64_t)1 << 31)
    return -1;
  // the weights must be worth streaming: with few of them the tile kernels' launch is as good
  if (p.N * p.K < (int64_t)1 << 22 || p.N < 512)
    return -1;
  const int n_cu = gcmi_num_cus(), stages = (int)(p.K / 128);
  const int panels = (int)((p.N + R32_BN - 1) / R32_BN);
  if (panels > 0x3fffff)
    return -1;
  // K slices: one workgroup per compute unit where the panels alone leave a third of them idle, four stages or more
  // each, and a workspace that holds the partial sums.  A caller's slice count (its KThreads) replaces the choice.
  int s = 3 * panels >= 2 * n_cu ? 1 : (n_cu + panels / 2) / panels;
  if (p.M > R32_BM && panels * s > n_cu) // (the larger rings leave room for one workgroup per compute unit)
    s = n_cu / panels > 1 ? n_cu / panels : 1;
  if (p.cfg_split_k > 0)
    s = p.cfg_split_k;
  if (s > stages / 4)
    s = stages / 4;
  while (s > 1 && (int64_t)s * p.M * p.N > ws_cap)
    s--;
  if (s < 1)
    s = 1;
  if (want)
    *want = s > 1 ? (int64_t)s * p.M * p.N : 0;
  if (cfg) {
    GemmTileConfig c{};
    const int bm = p.M <= R32_BM ? R32_BM : (p.M <= 2 * R32_BM ? 2 * R32_BM : 4 * R32_BM);
    c.kernel = GK_STREAM, c.bm = bm, c.bn = R32_BN, c.kbytes = R32_KB, c.stages = R32_NST;
    c.waves_m = 1, c.waves_n = 4, c.wave_m = bm, c.wave_n = 16, c.mfma_m = c.mfma_n = 16, c.mfma_k = 32;
    c.split_k = s, c.group_m = 1, c.workgroups = panels * s;
    c.from_attrs = p.cfg_split_k > 0 ? 1 : 0;
    *cfg = c;
  }
  if (dry)
    return 0;
  p.splits = s;
  const dim3 grid((unsigned)panels, (unsigned)s), block(512);
  const int mt = p.M <= R32_BM ? 2 : (p.M <= 2 * R32_BM ? 4 : 8);
  if (p.trans_b) {
    if (mt == 2)
      hipLaunchKernelGGL((gemm_rows32_kernel<2, true>), grid, block, 0, stream, p);
    else if (mt == 4)
      hipLaunchKernelGGL((gemm_rows32_kernel<4, true>), grid, block, 0, stream, p);
    else
      hipLaunchKernelGGL((gemm_rows32_kernel<8, true>), grid, block, 0, stream, p);
  } else {
    if (mt == 2)
      hipLaunchKernelGGL((gemm_rows32_kernel<2, false>), grid, block, 0, stream, p);
    else if (mt == 4)
      hipLaunchKernelGGL((gemm_rows32_kernel<4, false>), grid, block, 0, stream, p);
    else
      hipLaunchKernelGGL((gemm_rows32_kernel<8, false>), grid, block, 0, stream, p);
  }
  if (s > 1)
    launch_splitk_reduce(p, stream);
  return hipGetLastError() == hipSuccess ? 0 : 5;
}

} // namespace gcmi
