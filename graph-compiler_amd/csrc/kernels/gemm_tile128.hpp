// The 128 x 128 tile kernel.  Included by gemm_tile256.hpp (inside namespace gcmi, behind the pieces it shares with
// the 256 x 256 kernels: tile_of_block, MfmaOp, the 4-wave kernel's epilogue); the launcher there chooses between the
// tiles.
#pragma once

// ---------------------------------------------------------------------------
// 128 x 128 tiles for problems whose 256 x 256 tiles would leave most of the GPU idle (a 256 x 256 tile keeps
// one compute unit busy for 1.9 us per 128 elements of K whatever else the GPU does).  4 waves as 2 x 2, each owning
// 64 x 64 as 4 x 4 tiles of 16 x 16 (v_mfma_f32_16x16x32_bf16 or v_mfma_i32_16x16x64_i8, 64 accumulator registers),
// two workgroups per compute unit so that one computes while the other waits at its barrier.  Ring of 4 stages of
// 64 bytes of K (A 8 KiB + B 8 KiB each), filled by global_load_lds_dwordx4 with the swizzles of the 256 x 256 kernels (A rows of 64 bytes:
// chunk ^ (row / 4 % 4); B rows of 256 bytes read through the transposing LDS load: chunk ^ 4 * (k % 4)).  A stage
// computes k-block s from registers while the fragments of block s+1 are read and block s+3 is requested; one
// barrier per stage.  Rows past M and columns past N (N a multiple of 8) are fetched from the last row / chunk
// inside and never stored.  The epilogue is the 4-wave kernel's: accumulators through a wave-private LDS region,
// then rows of four columns per lane.  blockIdx.y: the batch, or with GemmParams::splits the K slice.
static constexpr int T128_B = 128, T128_KB = 64, T128_NST = 4;
static constexpr int T128_A_BYTES = T128_B * T128_KB, T128_STAGE_BYTES = 2 * T128_A_BYTES;
static constexpr int T128_DUMP_WAVE_BYTES = 64 * W4_DUMP_PITCH; // 17408 per wave
static constexpr int T128_SMEM_BYTES = 4 * T128_DUMP_WAVE_BYTES + 3 * 256 * 4; // accumulator regions / ring, column parameters
static_assert(T128_NST * T128_STAGE_BYTES <= 4 * T128_DUMP_WAVE_BYTES, "the ring overlaps the column parameters");

template <bool TB = false, int ES = 2> __global__ __launch_bounds__(256, 2) void gemm_tile128_kernel(GemmParams p) {
  static_assert(!TB || ES == 2, "B stored [N,K]: bf16 only");
  constexpr int KB = T128_KB, BK = KB / ES, NST = T128_NST, A_BYTES = T128_A_BYTES, STAGE = T128_STAGE_BYTES;
  // a k-row of the B tile: 256 bytes of bf16 (4 k-rows per transposing read, chunk ^ 4 * (k % 4)) or 128 bytes of
  // int8 (8 k-rows per read, chunk ^ 2 * (k % 8 / 2): the read of 8 k-rows x 16 columns touches every bank once)
  constexpr int RG = ES == 2 ? 4 : 8, B_ROW_BYTES = T128_B * ES, B_CPR = B_ROW_BYTES / 16;
  typedef typename std::conditional<ES == 2, f32x4_t, i32x4_t>::type acc4_t;
  __shared__ __align__(1024) char smem[T128_SMEM_BYTES];
  float *colp = reinterpret_cast<float *>(smem + 4 * T128_DUMP_WAVE_BYTES); // [0..127] bias, [256..] scale, [512..] comp * colsum
  auto b_swz = [](int krow) { return ES == 2 ? (krow % 4) * 4 : ((krow % 8) >> 1) * 2; };

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int r16 = lane & 15, g16 = lane >> 4;

  const int tiles_m = (int)((p.M + T128_B - 1) / T128_B), tiles_n = (int)((p.N + T128_B - 1) / T128_B);
  int tm, tn;
  tile_of_block(blockIdx.x, gridDim.x, tiles_m, tiles_n, p.group_m, tm, tn);
  tm = __builtin_amdgcn_readfirstlane(tm), tn = __builtin_amdgcn_readfirstlane(tn);
  const int64_t m0 = (int64_t)tm * T128_B, n0 = (int64_t)tn * T128_B;
  const int64_t lda_b = p.lda * ES, ldb_b = p.ldb * ES;
  const int64_t b_step = TB ? (int64_t)KB : (int64_t)BK * ldb_b;
  int KT = (int)(p.K / BK); // k-blocks: a positive multiple of NST (checked by the launcher)
  int64_t k_first = 0;      // first k-block of this workgroup
  if (p.splits > 1) {
    // K slices: blockIdx.y is the slice, whole ring groups each (they differ by at most one group); its f32 sums go
    // to the workspace as they are, the second kernel adds the slices and runs the epilogue
    const int slice = blockIdx.y, groups = KT / NST;
    const int g0 = (int)((int64_t)slice * groups / p.splits), g1 = (int)((int64_t)(slice + 1) * groups / p.splits);
    k_first = (int64_t)g0 * NST, KT = (g1 - g0) * NST;
    p.C = p.partial + (int64_t)slice * p.M * p.N, p.ldc = p.N, p.out_dt = DT_F32;
    p.bias = nullptr, p.act = ACT_NONE, p.residual = nullptr;
  } else {
    const int64_t bz = blockIdx.y; // strided batch
    p.A = reinterpret_cast<const char *>(p.A) + bz * p.a_bs * ES;
    p.B = reinterpret_cast<const char *>(p.B) + bz * p.b_bs * ES;
    p.C = reinterpret_cast<char *>(p.C) + bz * p.c_bs * (p.out_dt == DT_BF16 ? 2 : 4);
    if (p.residual)
      p.residual = reinterpret_cast<const char *>(p.residual) + bz * p.c_bs * (p.residual_dt == DT_BF16 ? 2 : 4);
  }
  const int rows_in = (int)min((int64_t)T128_B, p.M - m0), cols_in = (int)min((int64_t)T128_B, p.N - n0);

  // this wave's two DMA instructions per operand and stage: 1 KiB each = 16 rows of A (or of B stored [N,K]), 4 k-rows of B
  uint32_t a_src[2], b_src[2];
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const int d = wave * 2 + i;
    const int row = d * 16 + lane / 4;
    const int c = (lane % 4) ^ ((row >> 2) & 3);
    a_src[i] = (uint32_t)(min(row, rows_in - 1) * lda_b + c * 16);
    const int krow = d * (1024 / B_ROW_BYTES) + lane / B_CPR;
    const int cb = min((lane % B_CPR) ^ b_swz(krow), cols_in * ES / 16 - 1);
    b_src[i] = TB ? (uint32_t)(min(row, cols_in - 1) * ldb_b + c * 16) : (uint32_t)(krow * ldb_b + cb * 16);
  }
  auto issue = [&](char *__restrict__ stage, const char *a_base, const char *b_base) {
#pragma unroll
    for (int i = 0; i < 2; i++)
      __builtin_amdgcn_global_load_lds((GCMI_GLB const void *)(a_base + a_src[i]),
                                       (GCMI_LDS void *)(stage + (wave * 2 + i) * 1024), 16, 0, 0);
#pragma unroll
    for (int i = 0; i < 2; i++)
      __builtin_amdgcn_global_load_lds((GCMI_GLB const void *)(b_base + b_src[i]),
                                       (GCMI_LDS void *)(stage + A_BYTES + (wave * 2 + i) * 1024), 16, 0, 0);
  };
  // fragment reads as in gemm_tile256_mi16_kernel: A tile `it` = rows wm*64 + 16*it .., B tile `jt` = columns wn*64 + 16*jt ..
  const int row_a = wm * 64 + r16;
  const uint32_t a_ld = (uint32_t)(row_a * KB + ((g16 ^ ((row_a >> 2) & 3)) << 4));
  uint32_t b_ld[4];
  {
    // the 16 lanes of a group hand the transposing read RG k-rows x 16 columns in 8-byte pieces (bf16: k row
    // lane%16/4, 4 columns at lane%4; int8: k row lane%16/2, 8 columns at lane%2) and get back column lane%16
    const int kk = ES == 2 ? (r16 >> 2) : (r16 >> 1), cc = ES == 2 ? (r16 & 3) : (r16 & 1);
#pragma unroll
    for (int jt = 0; jt < 4; jt++) {
      const int chunk = ES == 2 ? (wn * 4 + jt) * 2 + (cc >> 1) : (wn * 4 + jt);
      const int sub = ES == 2 ? (cc & 1) * 8 : cc * 8;
      b_ld[jt] = (uint32_t)(A_BYTES + (2 * RG * g16 + kk) * B_ROW_BYTES + ((chunk ^ b_swz(kk)) << 4) + sub);
      if (TB) {
        const int row_b = wn * 64 + jt * 16 + r16;
        b_ld[jt] = (uint32_t)(A_BYTES + row_b * KB + ((g16 ^ ((row_b >> 2) & 3)) << 4));
      }
    }
  }
  auto load_frags = [&](const char *__restrict__ st, uint4(&a)[4], uint4(&b)[4]) {
#pragma unroll
    for (int it = 0; it < 4; it++)
      a[it] = *reinterpret_cast<const uint4 *>(st + a_ld + it * (16 * KB));
#pragma unroll
    for (int jt = 0; jt < 4; jt++) {
      if constexpr (TB) {
        b[jt] = *reinterpret_cast<const uint4 *>(st + b_ld[jt]);
      } else {
        const uint2 lo = MfmaOp<ES>::tr_read(st + b_ld[jt]);
        const uint2 hi = MfmaOp<ES>::tr_read(st + b_ld[jt] + RG * B_ROW_BYTES);
        b[jt] = make_uint4(lo.x, lo.y, hi.x, hi.y);
      }
    }
  };
  acc4_t acc[4][4]; // [jt][it]: rows 16*it + lane%16, columns 16*jt + 4*(lane/16) .. +3 (B fragment as first operand)
#pragma unroll
  for (int jt = 0; jt < 4; jt++)
#pragma unroll
    for (int it = 0; it < 4; it++)
      acc[jt][it] = acc4_t{0, 0, 0, 0};
  const uint32_t a_xor = p.a_xor;
  auto mfma_all = [&](const uint4(&a)[4], const uint4(&b)[4]) {
    if constexpr (ES == 2) {
#pragma unroll
      for (int jt = 0; jt < 4; jt++)
#pragma unroll
        for (int it = 0; it < 4; it++)
          acc[jt][it] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, b[jt]),
                                                                __builtin_bit_cast(bf16x8_t, a[it]), acc[jt][it], 0, 0, 0);
    } else {
      // row tile by row tile; its bytes are flipped (u8 activations: a - 128 as s8 == a ^ 0x80) just before its four
      // MFMAs, a whole stage after they were read, so no flip waits for LDS
#pragma unroll
      for (int it = 0; it < 4; it++) {
        const uint4 f = make_uint4(a[it].x ^ a_xor, a[it].y ^ a_xor, a[it].z ^ a_xor, a[it].w ^ a_xor);
#pragma unroll
        for (int jt = 0; jt < 4; jt++)
          acc[jt][it] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(i32x4_t, b[jt]), __builtin_bit_cast(i32x4_t, f),
                                                              acc[jt][it], 0, 0, 0);
      }
    }
  };

  const char *a_ptr = reinterpret_cast<const char *>(p.A) + m0 * lda_b + k_first * KB;
  const char *b_ptr = reinterpret_cast<const char *>(p.B) + (TB ? n0 * ldb_b : n0 * ES) + k_first * b_step;

  float cp_bias = -0.0f, cp_scale = 1.0f; // an absent bias adds nothing, not even to -0.0
  int cp_cs = 0;
  if (tid < cols_in) {
    if (p.bias)
      cp_bias = p.bias_dt == DT_BF16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t *>(p.bias)[n0 + tid])
                                     : reinterpret_cast<const float *>(p.bias)[n0 + tid];
    if (ES == 1) {
      if (p.scale)
        cp_scale = p.scale[n0 + tid];
      if (p.colsum)
        cp_cs = p.comp * p.colsum[n0 + tid];
    }
  }
#pragma unroll
  for (int d = 0; d < NST - 1; d++)
    issue(smem + d * STAGE, a_ptr + d * KB, b_ptr + d * b_step);
  if (tid < T128_B) {
    colp[tid] = cp_bias;
    if (ES == 1) {
      colp[256 + tid] = cp_scale;
      reinterpret_cast<int *>(colp)[512 + tid] = cp_cs;
    }
  }
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"((NST - 2) * 4) : "memory");
  __builtin_amdgcn_s_barrier();
  uint4 fa0[4], fb0[4], fa1[4], fb1[4];
  load_frags(smem, fa0, fb0);

  // One stage: k-block kt is in the `cur` registers.  Request block kt+NST-1 into the slot block kt-1 was read from
  // (every wave's reads of it had returned before it passed the previous barrier); wait for this wave's share of
  // block kt+1 and for its own LDS reads; barrier: block kt+1 is visible; read its fragments under the MFMAs of kt.
  auto stage = [&](auto has_fill, auto has_next, auto behindc, const char *__restrict__ nxt, char *__restrict__ fill,
                   const char *a_fill, const char *b_fill, uint4(&ca)[4], uint4(&cb)[4], uint4(&na)[4], uint4(&nb)[4]) {
    constexpr bool HAS_FILL = decltype(has_fill)::value, HAS_NEXT = decltype(has_next)::value;
    constexpr int BEHIND = decltype(behindc)::value;
    if constexpr (HAS_FILL)
      issue(fill, a_fill, b_fill);
    if constexpr (HAS_NEXT) {
      asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(BEHIND * 4) : "memory");
      __builtin_amdgcn_s_barrier();
      load_frags(nxt, na, nb);
    }
    mfma_all(ca, cb);
    // MFMA, two LDS reads, MFMA, two LDS reads ... then the remaining MFMAs
    if constexpr (HAS_NEXT) {
      constexpr int N_DS = TB ? 8 : 12;
      static_for<0, 16>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        constexpr int left = N_DS - 2 * i;
        if constexpr (left > 0)
          __builtin_amdgcn_sched_group_barrier(0x100, left < 2 ? left : 2, 0);
      });
    }
  };
  typedef std::integral_constant<bool, true> T;
  typedef std::integral_constant<bool, false> F;
  int kt0 = 0;
  for (; kt0 + 2 * NST <= KT; kt0 += NST) {
    static_for<0, NST>([&](auto sc) {
      constexpr int st = decltype(sc)::value;
      constexpr int nxt = (st + 1) % NST, fill = (st + NST - 1) % NST;
      const int kf = kt0 + st + NST - 1;
      if constexpr (st % 2 == 0)
        stage(T{}, T{}, std::integral_constant<int, NST - 2>{}, smem + nxt * STAGE, smem + fill * STAGE, a_ptr + (int64_t)kf * KB,
              b_ptr + kf * b_step, fa0, fb0, fa1, fb1);
      else
        stage(T{}, T{}, std::integral_constant<int, NST - 2>{}, smem + nxt * STAGE, smem + fill * STAGE, a_ptr + (int64_t)kf * KB,
              b_ptr + kf * b_step, fa1, fb1, fa0, fb0);
    });
  }
  static_for<0, NST>([&](auto sc) { // last group: only its first stage requests a block; the ring drains
    constexpr int st = decltype(sc)::value;
    constexpr int nxt = (st + 1) % NST, fill = (st + NST - 1) % NST;
    constexpr int behind = NST - 2 - st > 0 ? NST - 2 - st : 0;
    const int kf = kt0 + st + NST - 1;
    if constexpr (st % 2 == 0)
      stage(std::integral_constant<bool, st == 0>{}, std::integral_constant<bool, (st < NST - 1)>{}, std::integral_constant<int, behind>{},
            smem + nxt * STAGE, smem + fill * STAGE, a_ptr + (int64_t)kf * KB, b_ptr + kf * b_step, fa0, fb0, fa1, fb1);
    else
      stage(std::integral_constant<bool, st == 0>{}, std::integral_constant<bool, (st < NST - 1)>{}, std::integral_constant<int, behind>{},
            smem + nxt * STAGE, smem + fill * STAGE, a_ptr + (int64_t)kf * KB, b_ptr + kf * b_step, fa1, fb1, fa0, fb0);
  });

  // the accumulator regions lie over the ring: every wave's reads of the last block must have returned
  __syncthreads();
  char *dump = smem + wave * T128_DUMP_WAVE_BYTES;
#pragma unroll
  for (int jt = 0; jt < 4; jt++)
#pragma unroll
    for (int it = 0; it < 4; it++)
      *reinterpret_cast<acc4_t *>(dump + (it * 16 + r16) * W4_DUMP_PITCH + (jt * 16 + 4 * g16) * 4) = acc[jt][it];
  const int out_kind = p.out_dt == DT_BF16 ? 0 : ((ES == 1 && p.out_dt == DT_S32) ? 2 : 1);
  const int kind = (out_kind == 2 ? (int)ACT_NONE : p.act) + 8 * out_kind;
  if (rows_in < T128_B || cols_in < T128_B)
    w4_epilogue_half_any<ES, true, 64, 64>(p, kind, 0, m0, n0, wm, wn, lane, dump, colp, rows_in, cols_in);
  else
    w4_epilogue_half_any<ES, false, 64, 64>(p, kind, 0, m0, n0, wm, wn, lane, dump, colp, T128_B, T128_B);
}
