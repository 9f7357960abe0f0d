// bf16 GEMM for a short A against weights stored [N,K] (k contiguous): C[M,N] = epilogue(A[M,K] . Bt[N,K]^T),
// M <= 64.  This is the decode-time shape of the reference's llama2 case (test/benchgc/cases/llama2.mlir:
// 32 tokens against 4096x4096 .. 4096x11008 weights), where the reference splits K over threads
// (KThreads, lib/gc/Analysis/MatmulConfigAnalysis.cpp:149-166).  The job is to stream the weights from HBM once
// at full rate; the arithmetic is negligible.
//
// No LDS tile, no barrier in the main loop: every wave streams its own 32 weight rows x K slice straight into
// registers in MFMA operand layout and keeps SK_DEPTH stages of 4 KiB in flight.
//   * v_mfma_f32_32x32x16_bf16 with the weight fragment as first operand (rows = n) and the A fragment as
//     second (columns = m): lane (l32, lh) owns weight row n0 + l32 and A row l32 (+32 for the second row tile).
//   * One loop step covers 64 k (128 bytes of each row, one cache line): load t of 4 reads bytes
//     [32t + 16 lh, +16) of that line for both operands, so an instruction reads 32 contiguous bytes of each of
//     32 rows, and the four loads of a step use up the line.  Which k a lane holds does not matter as long as
//     both operands agree.
//   * A is tiny and stays in cache, but its loads share the in-order memory counter with the weight loads, so
//     they are requested SK_DEPTH steps ahead as well.
// A workgroup is four waves on the same 32 weight rows and four consecutive K slices; their accumulators are added
// through LDS in wave order, and the workgroup's f32 partial sums go to the split-K workspace.  The second kernel
// (gemm_splitk_reduce_kernel) adds the workgroup slices in order and runs the epilogue: results do not vary from
// run to run.
#pragma once
#include "gemm_tile256.hpp"

namespace gcmi {

static constexpr int SK_DEPTH = 6;   // stages in flight per wave (MT = 1); 4 with two row tiles
static constexpr int SK_WAVES = 4;

template <int MT> struct SkinnyStage {
  uint4 w[4];
  uint4 x[MT][4];
};

template <int MT> __global__ __launch_bounds__(SK_WAVES * 64, 2) void gemm_skinny_nt_kernel(GemmParams p) {
  constexpr int D = MT == 1 ? SK_DEPTH : 4;
  __shared__ float red[SK_WAVES][MT * 16][64];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int l32 = lane & 31, lh = lane >> 5;
  const int nblocks = (int)(p.N / 32);
  const int nb = (int)blockIdx.x % nblocks, wg_slice = (int)blockIdx.x / nblocks;
  const int64_t n0 = (int64_t)nb * 32;
  // this wave's K slice, in steps of 64 k: slices differ by at most one step
  const int steps = (int)(p.K / 64), slices = p.splits * SK_WAVES, sl = wg_slice * SK_WAVES + wave;
  const int it0 = (int)((int64_t)sl * steps / slices), it1 = (int)((int64_t)(sl + 1) * steps / slices);
  const int n_it = it1 - it0;

  const char *wrow = reinterpret_cast<const char *>(p.B) + (n0 + l32) * p.ldb * 2 + lh * 16 + (int64_t)it0 * 128;
  const char *xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; mt++) {
    const int64_t m = min((int64_t)(mt * 32 + l32), p.M - 1); // rows past M: read the last row, results are dropped
    xrow[mt] = reinterpret_cast<const char *>(p.A) + m * p.lda * 2 + lh * 16 + (int64_t)it0 * 128;
  }

  f32x16_t acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; mt++)
#pragma unroll
    for (int r = 0; r < 16; r++)
      acc[mt][r] = 0.0f;

  SkinnyStage<MT> st[D];
  auto load = [&](SkinnyStage<MT> &s, int it) {
#pragma unroll
    for (int t = 0; t < 4; t++)
      s.w[t] = *reinterpret_cast<const uint4 *>(wrow + (int64_t)it * 128 + t * 32);
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
      for (int t = 0; t < 4; t++)
        s.x[mt][t] = *reinterpret_cast<const uint4 *>(xrow[mt] + (int64_t)it * 128 + t * 32);
  };
  auto compute = [&](const SkinnyStage<MT> &s) {
#pragma unroll
    for (int t = 0; t < 4; t++)
#pragma unroll
      for (int mt = 0; mt < MT; mt++)
        acc[mt] = MfmaOp<2>::run(s.w[t], s.x[mt][t], acc[mt]);
  };

#pragma unroll
  for (int s = 0; s < D; s++)
    if (s < n_it)
      load(st[s], s);
  for (int base = 0; base < n_it; base += D) {
#pragma unroll
    for (int s = 0; s < D; s++) {
      const int i = base + s;
      if (i < n_it) { // wave-uniform
        compute(st[s]);
        if (i + D < n_it)
          load(st[s], i + D);
      }
    }
  }

  // add the four waves' accumulators in wave order: wave w sums the quads {w*MT .. w*MT+MT-1} of all four
#pragma unroll
  for (int mt = 0; mt < MT; mt++)
#pragma unroll
    for (int r = 0; r < 16; r++)
      red[wave][mt * 16 + r][lane] = acc[mt][r];
  __syncthreads();
  float *part = p.partial + (int64_t)wg_slice * p.M * p.N;
#pragma unroll
  for (int u = 0; u < MT; u++) {
    const int quad = wave * MT + u, mt = quad >> 2, q = quad & 3;
    f32x4_t v;
#pragma unroll
    for (int c = 0; c < 4; c++) {
      float sum = red[0][quad * 4 + c][lane];
#pragma unroll
      for (int w = 1; w < SK_WAVES; w++)
        sum += red[w][quad * 4 + c][lane];
      v[c] = sum;
    }
    const int64_t m = mt * 32 + l32, n = n0 + 8 * q + 4 * lh;
    if (m >= p.M)
      continue;
    if (p.splits > 1) {
      *reinterpret_cast<f32x4_t *>(part + m * p.N + n) = v;
      continue;
    }
    // one slice: this workgroup holds the whole sum, the epilogue runs here (same rounding points as the second pass)
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
}

// Takes the call when the shape is this kernel's (returns -1 otherwise: the tile kernels handle it).
// want != null: nothing is launched; *want receives the floats of workspace this call would use if it had them.
static int launch_skinny_nt(const GemmParams *pp, hipStream_t stream, int64_t *want = nullptr, GemmTileConfig *cfg = nullptr) {
  GemmParams p = *pp;
  if (want)
    *want = 0;
  const bool dry = want != nullptr || (cfg != nullptr && stream == (hipStream_t)-1);
  const int64_t ws_cap = want ? INT64_MAX : (p.partial ? p.partial_cap : 0);
  auto al16 = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  const int out_es = p.out_dt == DT_BF16 ? 2 : 4;
  if (!p.trans_b || p.batch > 1 || p.M < 1 || p.M > 64 || p.N % 32 != 0 || p.K % 64 != 0 || p.K < 256 || !al16(p.A) || !al16(p.B) ||
      !al16(p.C) || (p.lda * 2) % 16 != 0 || (p.ldb * 2) % 16 != 0 || (p.ldc * out_es) % 16 != 0 || p.out_dt == DT_S32 ||
      p.N / 32 > 0x3fffff)
    return -1;
  // the weights must be worth streaming this way: with few of them the tile kernel's launch is as good
  if (p.N * p.K < (int64_t)1 << 20)
    return -1;
  // Left to its own choice the launcher keeps this kernel for what it wins: up to 32 rows against up to 24 Mi
  // weights (32 x 4096 x 4096: 13.2 us against 14 us for K slices of 128 x 128 tiles).  With more rows or wider
  // weights the tile kernels are ahead (64 x 11008 x 4096: 41 us here, 26 us there).  A caller's slice count
  // (its KThreads) still selects it for any shape it can run.
  if (p.cfg_split_k <= 0 && (p.M > 32 || p.N * p.K > (int64_t)3 << 23))
    return -1;
  const int mt = p.M <= 32 ? 1 : 2;
  const int n_cu = gcmi_num_cus(), nblocks = (int)(p.N / 32), steps = (int)(p.K / 64);
  // workgroup slices: whole rounds of one workgroup per compute unit (measured: 32 x 4096 x 4096 takes 20 us with
  // 128 workgroups, 15 us with 256, 17 us with 512; a compute unit pulls about 17 GB/s whatever it has in flight, so
  // all of them must pull, evenly), every wave at two or more steps, and little partial-sum traffic (S x M x N f32,
  // written and read) against the weights.  One slice needs no second kernel: the epilogue runs in place.
  int best = 1;
  double best_score = -1.0;
  for (int s = 1; s <= 16; s++) {
    if (steps / (s * SK_WAVES) < 2 || (s > 1 && (int64_t)s * p.M * p.N > ws_cap))
      break;
    const double rounds = (double)nblocks * s / (double)n_cu;
    const double fill = rounds / (double)(int64_t)(rounds + 0.999999);
    const double extra = (double)s * (32.0 * mt) * 8.0 / ((double)p.K * 2.0);
    const double score = fill / (1.0 + extra);
    if (score > best_score + 1e-9)
      best_score = score, best = s;
  }
  if (p.cfg_split_k > 0) { // the caller's slice count (its KThreads), as far as the shape and the workspace allow
    int s = (p.cfg_split_k + SK_WAVES - 1) / SK_WAVES;
    while (s > 1 && (steps / (s * SK_WAVES) < 2 || (int64_t)s * p.M * p.N > ws_cap))
      s--;
    best = s;
  }
  if (steps / (best * SK_WAVES) < 2)
    return -1;
  if (want)
    *want = best > 1 ? (int64_t)best * p.M * p.N : 0;
  if (cfg) {
    GemmTileConfig c{};
    c.kernel = GK_STREAM, c.bm = 32 * mt, c.bn = 32, c.kbytes = 128, c.stages = mt == 1 ? SK_DEPTH : 4;
    c.waves_m = 1, c.waves_n = 1, c.wave_m = 32 * mt, c.wave_n = 32, c.mfma_m = c.mfma_n = 32, c.mfma_k = 16;
    c.split_k = best * SK_WAVES, c.group_m = 1, c.workgroups = nblocks * best;
    *cfg = c;
  }
  if (dry)
    return 0;
  p.splits = best;
  const dim3 grid((unsigned)(nblocks * best)), block(SK_WAVES * 64);
  if (mt == 1)
    hipLaunchKernelGGL(gemm_skinny_nt_kernel<1>, grid, block, 0, stream, p);
  else
    hipLaunchKernelGGL(gemm_skinny_nt_kernel<2>, grid, block, 0, stream, p);
  if (best == 1) // the epilogue ran in the kernel
    return hipGetLastError() == hipSuccess ? 0 : 5;
  launch_splitk_reduce(p, stream);
  return hipGetLastError() == hipSuccess ? 0 : 5;
}

} // namespace gcmi
