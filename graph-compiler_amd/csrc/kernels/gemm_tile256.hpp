// Whole-problem MFMA GEMM for gfx950 with a register-fused epilogue.
//
// Replaces the reference's "outer loops + brgemm microkernel call" structure
// (lib/gc/Transforms/DeepTileContractionOp.cpp:506-540 calling
// dnnl_brgemm_execute, lib/gc/ExecutionEngine/CPURuntime/Microkernel/
// BrgemmOnednn.cpp:145-168) by one kernel per matmul:
//   C[M,N] = epilogue( A[M,K] . B[K,N] ),  A and B plain row-major.
// ES = 2: bf16 x bf16 -> f32 accumulate (v_mfma_f32_32x32x16_bf16)
// ES = 1: (u8|s8) x s8 -> s32 accumulate (v_mfma_i32_32x32x32_i8)
//
// Workgroup tile 256 x 256, 128 bytes of K per stage (64 bf16 / 128 int8),
// 8 waves as 2 (M) x 4 (N), wave tile 128 x 64 = 4 x 2 MFMA tiles of 32 x 32.
// LDS: two stages of {A 256 rows x 128 B, B (128/ES) rows x 256*ES B} = 128 KiB.
//
// Operand roles are swapped on purpose: the MFMA's first operand is the B
// fragment (rows = n), the second the A fragment (columns = m).  The 32x32
// accumulator then gives every lane 4 consecutive n for one m, so the epilogue
// stores 8 (bf16) or 16 (f32/s32) contiguous bytes per lane and reads bias /
// scale / colsum as 4-vectors.
//
// B is row-major [K,N] (n contiguous) while the MFMA wants k-contiguous
// fragments: the transposition happens in the LDS read with
// ds_read_b64_tr_b16 / ds_read_b64_tr_b8, so the tile is stored exactly as it
// lies in memory.  This is the GPU analogue of the VNNI re-layout the
// reference's brgemm requires of B (lib/gc/Dialect/Microkernel/
// MicrokernelOps.cpp:380-389) without a separate packing pass.
//
// LDS swizzles (16-byte chunk index XOR):
//   A: chunk ^= (row >> 1) & 7        -> ds_read_b128 of 32 rows x 16 B is
//                                        conflict free over 64 banks
//   B: chunk ^= (krow % RG) * CW      -> RG = rows per transpose group (4 for
//                                        16-bit, 8 for 8-bit), CW = 16-byte
//                                        chunks one read touches per row
#pragma once
#include <type_traits>

#include "common.hpp"
#include "gemm_params.h"

namespace gcmi {

static constexpr int G_BM = 256, G_BN = 256, G_KBYTES = 128;
static constexpr int G_THREADS = 512;
static constexpr int G_STAGE_BYTES = 65536; // A 32 KiB + B 32 KiB
#ifndef G_FAST_WJ
// wave layout of the fast path: 2 = 8 waves of 128 x 64 (two per SIMD), 4 = 4 waves of 128 x 128 (one per
// SIMD, a third less LDS read traffic).  Measured on MI355X: the 4-wave layout is 5-7 % slower on bf16
// 4096^3 / 8192^3 and 19 % slower on the int8 MLP layer (nothing overlaps its epilogue), so 2 it is.
#define G_FAST_WJ 2
#endif
#ifndef G_FAST_KS
#define G_FAST_KS 2 // MFMA k-steps per LDS stage of the fast path: 2 (4-stage ring) or 4 (2-stage ring)
#endif

template <int ES> struct MfmaOp;
template <> struct MfmaOp<2> {
  typedef f32x16_t acc_t;
  typedef float acc_elem_t;
  static __device__ __forceinline__ acc_t run(const uint4 &a, const uint4 &b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c,
                                                   0, 0, 0);
  }
  // 8 bytes: k..k+3 of one n
  static __device__ __forceinline__ uint2 tr_read(const char *p) {
    bf16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((GCMI_LDS bf16x4_t *)p);
    return __builtin_bit_cast(uint2, v);
  }
};
template <> struct MfmaOp<1> {
  typedef i32x16_t acc_t;
  typedef int acc_elem_t;
  static __device__ __forceinline__ acc_t run(const uint4 &a, const uint4 &b, acc_t c) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4_t, a), __builtin_bit_cast(i32x4_t, b), c, 0,
                                                 0, 0);
  }
  // 8 bytes: k..k+7 of one n
  static __device__ __forceinline__ uint2 tr_read(const char *p) {
    i32x2_t v = __builtin_amdgcn_ds_read_tr8_b64_v2i32((GCMI_LDS i32x2_t *)p);
    return __builtin_bit_cast(uint2, v);
  }
};

// 16-byte chunk from global memory, zero filled outside [0,rows) x [0,row_bytes)
template <bool EDGE>
__device__ __forceinline__ uint4 load_chunk(const char *base, int64_t row, int64_t rows, int64_t col_byte,
                                            int64_t row_bytes, int64_t ld_bytes) {
  if (!EDGE) {
    return *reinterpret_cast<const uint4 *>(base + row * ld_bytes + col_byte);
  } else {
    uint4 v = make_uint4(0, 0, 0, 0);
    if (row >= rows || col_byte >= row_bytes)
      return v;
    const char *p = base + row * ld_bytes + col_byte;
    int64_t nvalid = row_bytes - col_byte;
    if (nvalid >= 16 && ((reinterpret_cast<uintptr_t>(p) & 15) == 0))
      return *reinterpret_cast<const uint4 *>(p);
    unsigned char tmp[16];
#pragma unroll
    for (int i = 0; i < 16; i++)
      tmp[i] = i < nvalid ? (unsigned char)p[i] : (unsigned char)0;
    v.x = tmp[0] | (tmp[1] << 8) | (tmp[2] << 16) | ((uint32_t)tmp[3] << 24);
    v.y = tmp[4] | (tmp[5] << 8) | (tmp[6] << 16) | ((uint32_t)tmp[7] << 24);
    v.z = tmp[8] | (tmp[9] << 8) | (tmp[10] << 16) | ((uint32_t)tmp[11] << 24);
    v.w = tmp[12] | (tmp[13] << 8) | (tmp[14] << 16) | ((uint32_t)tmp[15] << 24);
    return v;
  }
}

// Map a linear workgroup id to a tile so that the workgroups one XCD receives
// (hardware deals consecutive ids round-robin over 8 XCDs) cover a compact
// rectangle of tiles and share A/B panels in that XCD's L2.
__device__ __forceinline__ void tile_of_block(int bid, int nblk, int tiles_m, int tiles_n, int group_m, int &tm,
                                              int &tn) {
  int id = bid;
  if ((nblk & 7) == 0)
    id = (bid & 7) * (nblk >> 3) + (bid >> 3);
  int per_group = group_m * tiles_n;
  int g = id / per_group;
  int first_m = g * group_m;
  int gm = min(group_m, tiles_m - first_m);
  int in_g = id - g * per_group;
  tm = first_m + in_g % gm;
  tn = in_g / gm;
}

// compile-time loop: the body receives std::integral_constant<int, I>, so every
// accumulator index is a constant and the accumulators stay in registers
template <int I, int N, typename F> __device__ __forceinline__ void static_for(F &&f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

template <int ACT> __device__ __forceinline__ float act_const(float x) { return apply_act(x, ACT); }

// two f32 -> two bf16 in one instruction (v_cvt_pk_bf16_f32: round to nearest even; not for NaNs, whose sign and
// payload it keeps); lo in bits 0-15
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// Epilogue shared by both kernels.  acc[j][i][r] holds
//   m = m0 + wm*128 + i*32 + (lane & 31),  n = n0 + wn*64 + j*32 + 8*(r/4) + 4*(lane >> 5) + r%4.
// Instantiated once per activation so that each copy unrolls completely.
// STAGED (whole tiles, bf16 output): the wave first lays its 128 x 64 result out
// in a private LDS region (rows of 128 B at a 144 B pitch), then reads it back
// row-wise so that every global store instruction writes eight complete
// 128-byte lines (16 B per lane) instead of 32 scattered 16-byte pieces.
static constexpr int G_STG_PITCH = 144;
static constexpr int G_STG_WAVE_BYTES = 128 * G_STG_PITCH; // 18 KiB per wave

// WJ = MFMA tiles along n per wave: 2 (8 waves as 2 x 4, wave tile 128 x 64) or 4
// (4 waves as 2 x 2, wave tile 128 x 128).
// LDSP (whole-tile kernels): the tile's 256 column parameters were laid out in LDS when the kernel started
// (colp[0..255] bias as f32, -0.0 when there is none; [256..511] scale; [512..767] comp * colsum as s32), so a
// lane fetches its four columns with one ds_read_b128 per array instead of scalar global loads behind a wait.
// MI16: the accumulators come from 16x16x32 MFMAs.  acc[j][i] still covers columns j*32.. and rows i*32.. of the wave
// tile, as four 16 x 16 tiles: elements 4q..4q+3 belong to the tile at columns 16*(q/2), rows 16*(q%2), where a
// lane holds columns 4*(lane/16)..+3 of row lane%16.
template <int ES, bool EDGE, int ACT, bool STAGED, int WJ = 2, bool LDSP = false, bool MI16 = false>
__device__ __forceinline__ void gemm_epilogue_act(const GemmParams &p, typename MfmaOp<ES>::acc_t (&acc)[WJ][4],
                                                  int64_t m0, int64_t n0, int wm, int wn, int l32, int lh,
                                                  char *stg, const float *colp = nullptr) {
  constexpr int PITCH = 64 * WJ + 16; // staging row: 32*WJ bf16 + 16 bytes of padding
  const int out_dt = STAGED ? (int)DT_BF16 : p.out_dt; // only bf16 results are staged
  const int out_es = out_dt == DT_BF16 ? 2 : 4;
  char *Cb = reinterpret_cast<char *>(p.C);
  static_for<0, WJ>([&](auto jc) {
    constexpr int j = decltype(jc)::value;
    static_for<0, 4>([&](auto qc) {
      constexpr int q = decltype(qc)::value;
      // this lane's four columns and its row inside the 32 x 32 block (j, i)
      const int n_off = MI16 ? 16 * (q >> 1) + 4 * (2 * lh + (l32 >> 4)) : 8 * q + 4 * lh;
      const int m_off = MI16 ? 16 * (q & 1) + (l32 & 15) : l32;
      const int64_t n = n0 + wn * (32 * WJ) + j * 32 + n_off;
      float bias4[4] = {0.f, 0.f, 0.f, 0.f}, scale4[4] = {1.f, 1.f, 1.f, 1.f};
      int cs4[4] = {0, 0, 0, 0}; // comp * colsum
      if constexpr (LDSP) {
        const int col = wn * (32 * WJ) + j * 32 + n_off;
        const f32x4_t b = *reinterpret_cast<const f32x4_t *>(colp + col);
        bias4[0] = b[0], bias4[1] = b[1], bias4[2] = b[2], bias4[3] = b[3];
        if (ES == 1) {
          const f32x4_t sc = *reinterpret_cast<const f32x4_t *>(colp + 256 + col);
          const i32x4_t cs = *reinterpret_cast<const i32x4_t *>(colp + 512 + col);
          scale4[0] = sc[0], scale4[1] = sc[1], scale4[2] = sc[2], scale4[3] = sc[3];
          cs4[0] = cs[0], cs4[1] = cs[1], cs4[2] = cs[2], cs4[3] = cs[3];
        }
      } else {
#pragma unroll
        for (int e = 0; e < 4; e++) {
          if (!EDGE || n + e < p.N) {
            if (p.bias)
              bias4[e] = p.bias_dt == DT_BF16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t *>(p.bias)[n + e])
                                              : reinterpret_cast<const float *>(p.bias)[n + e];
            if (ES == 1) {
              if (p.scale)
                scale4[e] = p.scale[n + e];
              if (p.colsum)
                cs4[e] = p.comp * p.colsum[n + e];
            }
          }
        }
      }
      static_for<0, 4>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        const int64_t m = m0 + wm * 128 + i * 32 + m_off;
        if (EDGE && m >= p.M)
          return;
        uint32_t o32[4];
        uint16_t o16[4];
        float xf[4] = {0.f, 0.f, 0.f, 0.f};
        float res4[4] = {0.f, 0.f, 0.f, 0.f};
        if (ES == 2 && p.residual) {
          const int64_t at = m * p.ldr + n;
          if (!EDGE) { // the launcher sends unaligned residuals to the EDGE kernels
            if (p.residual_dt == DT_BF16) {
              const uint2 v = *reinterpret_cast<const uint2 *>(reinterpret_cast<const uint16_t *>(p.residual) + at);
              res4[0] = __uint_as_float(v.x << 16), res4[1] = __uint_as_float(v.x & 0xffff0000u);
              res4[2] = __uint_as_float(v.y << 16), res4[3] = __uint_as_float(v.y & 0xffff0000u);
            } else {
              const f32x4_t v = *reinterpret_cast<const f32x4_t *>(reinterpret_cast<const float *>(p.residual) + at);
              res4[0] = v[0], res4[1] = v[1], res4[2] = v[2], res4[3] = v[3];
            }
          } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
              if (n + e < p.N)
                res4[e] = p.residual_dt == DT_BF16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t *>(p.residual)[at + e])
                                                   : reinterpret_cast<const float *>(p.residual)[at + e];
          }
        }
        if constexpr (ES == 2 && LDSP && STAGED) {
          // bf16 graph, whole tiles: the same rounding points as below (after the matmul and after every bf16 op,
          // lib/gc/Transforms/Pipeline.cpp:79-95), rounded in pairs by v_cvt_pk_bf16_f32.  A NaN stays a NaN
          // through the ops that follow, so only the last conversion has to give it the reference's 0x7FC0.
          float x[4] = {(float)acc[j][i][4 * q], (float)acc[j][i][4 * q + 1], (float)acc[j][i][4 * q + 2],
                        (float)acc[j][i][4 * q + 3]};
          uint32_t p0, p1;
          auto rnd = [&]() {
            p0 = pack_bf16x2(x[0], x[1]), p1 = pack_bf16x2(x[2], x[3]);
            x[0] = __uint_as_float(p0 << 16), x[1] = __uint_as_float(p0 & 0xffff0000u);
            x[2] = __uint_as_float(p1 << 16), x[3] = __uint_as_float(p1 & 0xffff0000u);
          };
          rnd();
          if (p.bias) {
#pragma unroll
            for (int e = 0; e < 4; e++)
              x[e] = x[e] + bias4[e];
            rnd();
          }
          if (ACT != ACT_NONE) {
#pragma unroll
            for (int e = 0; e < 4; e++)
              x[e] = act_const<ACT>(x[e]);
            if (ACT == ACT_RELU) { // max(x, 0) of a bf16 value is a bf16 value: nothing to round
              p0 = (__float_as_uint(x[0]) >> 16) | (__float_as_uint(x[1]) & 0xffff0000u);
              p1 = (__float_as_uint(x[2]) >> 16) | (__float_as_uint(x[3]) & 0xffff0000u);
            } else {
              rnd();
            }
          }
          if (p.residual) {
#pragma unroll
            for (int e = 0; e < 4; e++)
              x[e] = x[e] + res4[e];
            rnd();
          }
          const float any_nan = (x[0] + x[1]) + (x[2] + x[3]); // a NaN if one of them is (or opposite infinities)
          if (__builtin_expect(any_nan != any_nan, 0)) {
            if (x[0] != x[0]) p0 = (p0 & 0xffff0000u) | 0x7FC0u;
            if (x[1] != x[1]) p0 = (p0 & 0x0000ffffu) | 0x7FC00000u;
            if (x[2] != x[2]) p1 = (p1 & 0xffff0000u) | 0x7FC0u;
            if (x[3] != x[3]) p1 = (p1 & 0x0000ffffu) | 0x7FC00000u;
          }
          *reinterpret_cast<uint2 *>(stg + (i * 32 + m_off) * PITCH + (j * 32 + n_off) * 2) = make_uint2(p0, p1);
          return;
        }
#pragma unroll
        for (int e = 0; e < 4; e++) {
          if (ES == 1) {
            // s32 accumulator of (a ^ 0x80) * w; comp restores / applies the
            // zero-point term in exact integer arithmetic.
            int c = (int)acc[j][i][4 * q + e] + cs4[e];
            if (out_dt == DT_S32) {
              o32[e] = (uint32_t)c;
              o16[e] = 0;
            } else {
              float x;
              if constexpr (LDSP) { // an absent bias is -0.0: the fused multiply-add then equals the product
                x = fmaf((float)c, scale4[e], bias4[e]);
              } else {
                x = (float)c * scale4[e];
                if (p.bias)
                  x = x + bias4[e];
              }
              x = act_const<ACT>(x);
              o32[e] = __float_as_uint(x);
              if constexpr (LDSP && STAGED)
                xf[e] = x; // converted in pairs below
              else
                o16[e] = f32_to_bf16_bits(x);
            }
          } else {
            float x = (float)acc[j][i][4 * q + e];
            const float r = res4[e];
            if (out_dt == DT_BF16) {
              // bf16 graph: round after the matmul and after every bf16 op
              // (lib/gc/Transforms/Pipeline.cpp:79-95)
              x = round_bf16(x);
              if (p.bias)
                x = round_bf16(x + bias4[e]);
              if (ACT != ACT_NONE)
                x = round_bf16(act_const<ACT>(x));
              if (p.residual)
                x = round_bf16(x + r);
              o16[e] = f32_to_bf16_bits(x);
              o32[e] = 0;
            } else {
              if (p.bias)
                x = x + bias4[e];
              x = act_const<ACT>(x);
              if (p.residual) { // kept apart from the activation's last multiply: the sum equals a separate add
#pragma clang fp contract(off)
                x = x + r;
              }
              o32[e] = __float_as_uint(x);
              o16[e] = 0;
            }
          }
        }
        if (STAGED) {
          uint2 packed;
          if constexpr (LDSP && ES == 1) {
            // v_cvt_pk_bf16_f32 rounds to nearest even like the scalar routine but keeps a NaN's sign (the
            // hardware's own invalid-operation NaN is negative), so four values with a NaN among them (their sum
            // is one; so is the sum of opposite infinities) take the scalar routine: NaN -> 0x7FC0
            const float any_nan = (xf[0] + xf[1]) + (xf[2] + xf[3]);
            if (__builtin_expect(any_nan != any_nan, 0))
              packed = make_uint2(f32_to_bf16_bits(xf[0]) | ((uint32_t)f32_to_bf16_bits(xf[1]) << 16),
                                  f32_to_bf16_bits(xf[2]) | ((uint32_t)f32_to_bf16_bits(xf[3]) << 16));
            else
              packed = make_uint2(pack_bf16x2(xf[0], xf[1]), pack_bf16x2(xf[2], xf[3]));
          } else {
            packed = make_uint2(o16[0] | ((uint32_t)o16[1] << 16), o16[2] | ((uint32_t)o16[3] << 16));
          }
          *reinterpret_cast<uint2 *>(stg + (i * 32 + m_off) * PITCH + (j * 32 + n_off) * 2) = packed;
          return;
        }
        char *dst = Cb + (m * p.ldc + n) * out_es;
        if (!EDGE) {
          if (out_es == 2)
            *reinterpret_cast<uint2 *>(dst) =
                make_uint2(o16[0] | ((uint32_t)o16[1] << 16), o16[2] | ((uint32_t)o16[3] << 16));
          else
            *reinterpret_cast<uint4 *>(dst) = make_uint4(o32[0], o32[1], o32[2], o32[3]);
        } else {
#pragma unroll
          for (int e = 0; e < 4; e++) {
            if (n + e < p.N) {
              if (out_es == 2)
                reinterpret_cast<uint16_t *>(dst)[e] = o16[e];
              else
                reinterpret_cast<uint32_t *>(dst)[e] = o32[e];
            }
          }
        }
      });
    });
  });
  if (STAGED) {
    // wave-private region: only this wave's own LDS writes have to land
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    const int lane = lh * 32 + l32;
    constexpr int LPR = 4 * WJ, RPP = 64 / LPR; // lanes per row (16 B each), rows per pass
    const int rr = lane / LPR, cc = lane % LPR;
#pragma unroll
    for (int it = 0; it < 128 / RPP; it++) {
      const int row = it * RPP + rr;
      uint4 v = *reinterpret_cast<const uint4 *>(stg + row * PITCH + cc * 16);
      typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
      u32x4_t vv = {v.x, v.y, v.z, v.w};
      __builtin_nontemporal_store(vv, reinterpret_cast<u32x4_t *>(Cb + ((m0 + wm * 128 + row) * p.ldc + n0 + wn * (32 * WJ) + cc * 8) * 2));
    }
  }
}

template <int ES, bool EDGE, bool STAGED, int WJ = 2, bool LDSP = false, bool MI16 = false>
__device__ __forceinline__ void gemm_epilogue(const GemmParams &p, typename MfmaOp<ES>::acc_t (&acc)[WJ][4], int64_t m0,
                                              int64_t n0, int wm, int wn, int l32, int lh, char *stg,
                                              const float *colp = nullptr) {
  switch (p.act) {
  case ACT_RELU:
    gemm_epilogue_act<ES, EDGE, ACT_RELU, STAGED, WJ, LDSP, MI16>(p, acc, m0, n0, wm, wn, l32, lh, stg, colp);
    break;
  case ACT_GELU_ERF:
    gemm_epilogue_act<ES, EDGE, ACT_GELU_ERF, STAGED, WJ, LDSP, MI16>(p, acc, m0, n0, wm, wn, l32, lh, stg, colp);
    break;
  case ACT_GELU_TANH:
    gemm_epilogue_act<ES, EDGE, ACT_GELU_TANH, STAGED, WJ, LDSP, MI16>(p, acc, m0, n0, wm, wn, l32, lh, stg, colp);
    break;
  case ACT_SIGMOID:
    gemm_epilogue_act<ES, EDGE, ACT_SIGMOID, STAGED, WJ, LDSP, MI16>(p, acc, m0, n0, wm, wn, l32, lh, stg, colp);
    break;
  default:
    gemm_epilogue_act<ES, EDGE, ACT_NONE, STAGED, WJ, LDSP, MI16>(p, acc, m0, n0, wm, wn, l32, lh, stg, colp);
    break;
  }
}

// TB: B is stored [N,K] (k contiguous).  Its tile then has the geometry of the A tile (256 rows x 128 bytes of K),
// takes the same swizzle, and its fragments are plain 16-byte reads like A's: no transposing LDS read is needed.
template <int ES, bool EDGE, bool TB = false> __global__ __launch_bounds__(G_THREADS) void gemm_tile256_kernel(GemmParams p) {
  typedef MfmaOp<ES> Op;
  typedef typename Op::acc_t acc_t;
  constexpr int BK = G_KBYTES / ES;        // K elements per stage
  constexpr int B_ROW_BYTES = G_BN * ES;   // bytes per k-row of the B tile
  constexpr int B_CPR = B_ROW_BYTES / 16;  // 16-byte chunks per B row
  constexpr int RG = ES == 2 ? 4 : 8;      // k-rows per transpose-read group
  constexpr int CW = ES == 2 ? 4 : 2;      // chunks per row one transpose read spans
  constexpr int KSTEP = 32 / ES;           // K elements one MFMA consumes

  __shared__ __align__(16) char smem[2 * G_STAGE_BYTES];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 2, wn = wave & 3;
  const int l32 = lane & 31, lh = lane >> 5;

  const int tiles_m = (int)((p.M + G_BM - 1) / G_BM), tiles_n = (int)((p.N + G_BN - 1) / G_BN);
  int tm, tn;
  tile_of_block(blockIdx.x, gridDim.x, tiles_m, tiles_n, p.group_m, tm, tn);
  const int64_t m0 = (int64_t)tm * G_BM, n0 = (int64_t)tn * G_BN;

  const int64_t lda_b = p.lda * ES, ldb_b = p.ldb * ES;
  const int64_t bz = blockIdx.y; // batch
  const char *Ab = reinterpret_cast<const char *>(p.A) + bz * p.a_bs * ES;
  const char *Bb = reinterpret_cast<const char *>(p.B) + bz * p.b_bs * ES;
  p.C = reinterpret_cast<char *>(p.C) + bz * p.c_bs * (p.out_dt == DT_BF16 ? 2 : 4);
  if (p.residual)
    p.residual = reinterpret_cast<const char *>(p.residual) + bz * p.c_bs * (p.residual_dt == DT_BF16 ? 2 : 4);

  // ---- global -> register staging assignment: 4 A chunks + 4 B chunks per thread
  const int a_row0 = tid >> 3, a_c = tid & 7;             // rows a_row0 + 64*i
  const int b_row0 = tid / B_CPR, b_c = tid % B_CPR;      // rows b_row0 + (512/B_CPR)*i
  constexpr int B_ROW_STEP = G_THREADS / B_CPR;
  uint32_t a_st[4], b_st[4]; // LDS store offsets inside a stage
#pragma unroll
  for (int i = 0; i < 4; i++) {
    int row = a_row0 + 64 * i;
    a_st[i] = row * 128 + ((a_c ^ ((row >> 1) & 7)) << 4);
    int krow = b_row0 + B_ROW_STEP * i;
    b_st[i] = TB ? 32768 + a_st[i] : 32768 + krow * B_ROW_BYTES + ((b_c ^ ((krow % RG) * CW)) << 4);
  }

  // ---- LDS read offsets of this lane's MFMA fragments
  const int sw = (l32 >> 1) & 7;
  uint32_t a_ld[4]; // per k-step chunk offset; + lane row base + i*4096
#pragma unroll
  for (int ks = 0; ks < 4; ks++)
    a_ld[ks] = (wm * 128 + l32) * 128 + (((2 * ks + lh) ^ sw) << 4);
  const int g = lane >> 4, i16 = lane & 15;
  uint32_t b_ld[2]; // + ks*8192 + jj*2048
  {
    const int kk = ES == 2 ? (i16 >> 2) : (i16 >> 1);
    const int cc = ES == 2 ? (i16 & 3) : (i16 & 1);
#pragma unroll
    for (int j = 0; j < 2; j++) {
      int chunk = ES == 2 ? (wn * 8 + j * 4 + 2 * (g & 1) + (cc >> 1)) : (wn * 4 + j * 2 + (g & 1));
      int sub = ES == 2 ? (cc & 1) * 8 : cc * 8;
      int krow_lane = (ES == 2 ? 8 : 16) * (g >> 1) + kk;
      b_ld[j] = 32768 + krow_lane * B_ROW_BYTES + ((chunk ^ (kk * CW)) << 4) + sub;
      if (TB) // row of the tile; + the k-step's chunk (swizzled like A's)
        b_ld[j] = 32768 + (wn * 64 + j * 32 + l32) * 128;
    }
  }

  acc_t acc[2][4];
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
      for (int r = 0; r < 16; r++)
        acc[j][i][r] = 0;

  const int64_t k_bytes = p.K * ES;
  const int KT = (int)((p.K + BK - 1) / BK);
  uint4 ra[4], rb[4];

  auto gload = [&](int kt) {
    const int64_t kb = (int64_t)kt * G_KBYTES; // byte offset along K of A
#pragma unroll
    for (int i = 0; i < 4; i++)
      ra[i] = load_chunk<EDGE>(Ab, m0 + a_row0 + 64 * i, p.M, kb + a_c * 16, k_bytes, lda_b);
#pragma unroll
    for (int i = 0; i < 4; i++)
      rb[i] = TB ? load_chunk<EDGE>(Bb, n0 + a_row0 + 64 * i, p.N, kb + a_c * 16, k_bytes, ldb_b)
                 : load_chunk<EDGE>(Bb, (int64_t)kt * BK + b_row0 + B_ROW_STEP * i, p.K, n0 * ES + b_c * 16,
                                    p.N * ES, ldb_b);
  };
  auto lstore = [&](int stage) {
    char *s = smem + stage * G_STAGE_BYTES;
    const uint32_t x = p.a_xor;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      uint4 v = ra[i];
      if (ES == 1) { // u8 activations: a - 128 as s8 == a ^ 0x80
        v.x ^= x;
        v.y ^= x;
        v.z ^= x;
        v.w ^= x;
      }
      *reinterpret_cast<uint4 *>(s + a_st[i]) = v;
    }
#pragma unroll
    for (int i = 0; i < 4; i++)
      *reinterpret_cast<uint4 *>(s + b_st[i]) = rb[i];
  };

  gload(0);
  lstore(0);
  __syncthreads();

  for (int kt = 0; kt < KT; kt++) {
    const int cur = kt & 1;
    if (kt + 1 < KT)
      gload(kt + 1);
    const char *s = smem + cur * G_STAGE_BYTES;
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
      uint4 af[4], bf[2];
#pragma unroll
      for (int i = 0; i < 4; i++)
        af[i] = *reinterpret_cast<const uint4 *>(s + a_ld[ks] + i * 4096);
#pragma unroll
      for (int j = 0; j < 2; j++) {
        if (TB) {
          bf[j] = *reinterpret_cast<const uint4 *>(s + b_ld[j] + (((2 * ks + lh) ^ sw) << 4));
        } else {
          uint2 lo = Op::tr_read(s + b_ld[j] + ks * 8192);
          uint2 hi = Op::tr_read(s + b_ld[j] + ks * 8192 + 2048);
          bf[j] = make_uint4(lo.x, lo.y, hi.x, hi.y);
        }
      }
#pragma unroll
      for (int j = 0; j < 2; j++)
#pragma unroll
        for (int i = 0; i < 4; i++)
          acc[j][i] = Op::run(bf[j], af[i], acc[j][i]);
    }
    if (kt + 1 < KT)
      lstore(cur ^ 1);
    __syncthreads();
  }
  (void)KSTEP;

  gemm_epilogue<ES, EDGE, false>(p, acc, m0, n0, wm, wn, l32, lh, nullptr);
}

// ---------------------------------------------------------------------------
// Fast path: every dimension a multiple of the tile, 16-byte aligned operands.
//  * K is consumed in stages of KS MFMA k-steps (KS*32 bytes of K per row); the
//    LDS holds a ring of NST = 8/KS such stages (KS=2: 4 x 32 KiB, KS=4:
//    2 x 64 KiB).  Stage kt+NST-1 is requested while stage kt is computed, so
//    two to three stages of global->LDS traffic are always in flight: a CU's
//    L2->LDS path only delivers ~100 GB/s and has to stream without gaps.
//  * global -> LDS goes through global_load_lds_dwordx4: each wave instruction
//    drops 1 KiB straight into LDS (lane l at base + 16*l), no staging
//    registers and no ds_write.  The swizzle is applied on the GLOBAL side: the
//    lane that fills physical chunk P fetches logical chunk P ^ f(row).
//  * MFMA fragments are double buffered in registers: the LDS reads of k-step
//    s+1 are issued in the shadow of the MFMAs of k-step s, interleaved 1:1 by
//    the scheduler hints; the reads of the next stage's first k-step are issued
//    right after the stage barrier, under the last 8 MFMAs of the stage.
//  * The stage loop is unrolled over the ring, so every LDS address is static.
#define GCMI_GLB __attribute__((address_space(1)))

// SPLIT (split-K on a short A): only the first `mi` 32-row tiles of a wave hold rows of A; the others are
// neither read from LDS nor multiplied.
// TB (B stored [N,K]): the B tile is staged and read exactly like the A tile.
template <int ES, int KS, int WJ = 2, bool SPLIT = false, bool TB = false> struct FastGemm {
  static constexpr int NWAVES = 16 / WJ; // 8 or 4
  int mi = 4;
  typedef MfmaOp<ES> Op;
  typedef typename Op::acc_t acc_t;
  static constexpr int NST = 8 / KS;                  // stages in the LDS ring
  static constexpr int KB = KS * 32;                  // bytes of K per A row per stage
  static constexpr int BK = KB / ES;                  // K elements per stage
  static constexpr int A_BYTES = G_BM * KB;           // 16 or 32 KiB
  static constexpr int STAGE_BYTES = 2 * A_BYTES;     // B tile has the same size
  static constexpr int A_CPR = KB / 16;               // 16-byte chunks per A row: 4 or 8
  static constexpr int A_ROWS_PER_DMA = 1024 / KB;    // 16 or 8
  static constexpr int B_ROW_BYTES = G_BN * ES;
  static constexpr int RG = ES == 2 ? 4 : 8;
  static constexpr int CW = ES == 2 ? 4 : 2;
  static constexpr int B_ROWS_PER_DMA = 1024 / B_ROW_BYTES; // 2 (bf16) or 4 (int8)
  static constexpr int B_CPR = B_ROW_BYTES / 16;
  static constexpr int NDMA = KS * 8 / NWAVES;        // DMA instructions per operand per wave per stage

  static __device__ __forceinline__ int a_swz(int row) { return KS == 4 ? ((row >> 1) & 7) : ((row >> 2) & 3); }

  uint32_t a_src[NDMA], b_src[NDMA]; // per-lane byte offsets of this wave's DMA instructions
  uint32_t a_ld[KS], b_ld[TB ? KS : WJ]; // fragment read offsets
  uint32_t a_xor;
  int wave_u; // wave id, wave-uniform

  __device__ __forceinline__ void issue_loads(char *__restrict__ stage, const char *a_base, const char *b_base) const {
#pragma unroll
    for (int i = 0; i < NDMA; i++)
      __builtin_amdgcn_global_load_lds((GCMI_GLB const void *)(a_base + a_src[i]),
                                       (GCMI_LDS void *)(stage + (wave_u * NDMA + i) * 1024), 16, 0, 0);
#pragma unroll
    for (int i = 0; i < NDMA; i++)
      __builtin_amdgcn_global_load_lds((GCMI_GLB const void *)(b_base + b_src[i]),
                                       (GCMI_LDS void *)(stage + A_BYTES + (wave_u * NDMA + i) * 1024), 16, 0, 0);
  }

  __device__ __forceinline__ void load_frags(const char *__restrict__ s, int ks, uint4 (&af)[4], uint4 (&bf)[WJ]) const {
    if (SPLIT && mi == 0)
      return;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      if (SPLIT && i >= mi)
        break;
      uint4 v = *reinterpret_cast<const uint4 *>(s + a_ld[ks] + i * 32 * KB);
      if (ES == 1) // u8 activations: a - 128 as s8 == a ^ 0x80
        v = make_uint4(v.x ^ a_xor, v.y ^ a_xor, v.z ^ a_xor, v.w ^ a_xor);
      af[i] = v;
    }
#pragma unroll
    for (int j = 0; j < WJ; j++) {
      if (TB) {
        bf[j] = *reinterpret_cast<const uint4 *>(s + A_BYTES + b_ld[ks] + j * 32 * KB);
      } else {
        uint2 lo = Op::tr_read(s + b_ld[j] + ks * 8192);
        uint2 hi = Op::tr_read(s + b_ld[j] + ks * 8192 + 2048);
        bf[j] = make_uint4(lo.x, lo.y, hi.x, hi.y);
      }
    }
  }

  __device__ __forceinline__ void mfma_all(acc_t (&acc)[WJ][4], const uint4 (&af)[4], const uint4 (&bf)[WJ]) const {
#pragma unroll
    for (int j = 0; j < WJ; j++)
#pragma unroll
      for (int i = 0; i < 4; i++)
        if (!SPLIT || i < mi)
          acc[j][i] = Op::run(bf[j], af[i], acc[j][i]);
  }

  // ask the scheduler for MFMA, DS read, MFMA, DS read, ... over the region
  static __device__ __forceinline__ void interleave_hint() {
    if (SPLIT)
      return;
    // the fragment reads of the next k-step go out with the first MFMAs, two per MFMA, so that they have landed
    // when the group ends and the wait in front of the next group finds little outstanding (1-4 % over one read
    // per MFMA spread over the whole group)
    constexpr int N_DS = 4 + (TB ? WJ : 2 * WJ);
    static_for<0, 4 * WJ>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // 1 MFMA
      constexpr int left = N_DS - 2 * i;
      if constexpr (left > 0)
        __builtin_amdgcn_sched_group_barrier(0x100, left < 2 ? left : 2, 0); // DS reads
    });
  }

  // wait until at most BEHIND later stages of this wave's DMA are still in flight
  // (and all of its LDS reads have returned)
  template <int BEHIND> static __device__ __forceinline__ void wait_dma() {
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(BEHIND * 2 * NDMA) : "memory");
  }

  // One stage, branch free.  `cur` holds k-block kt (landed and barriered;
  // fragments of its k-step 0 are in a0/b0); the DMA of k-block kt+NST-1 goes
  // into `fill`, the buffer that was computed from one stage ago; `nxt` holds
  // k-block kt+1, behind which BEHIND more blocks are in flight.
  template <bool HAS_FILL, bool HAS_NEXT, int BEHIND>
  __device__ __forceinline__ void stage(char *__restrict__ cur, char *__restrict__ nxt, char *__restrict__ fill,
                                        const char *a_fill, const char *b_fill, acc_t (&acc)[WJ][4], uint4 (&a0)[4],
                                        uint4 (&b0)[WJ], uint4 (&a1)[4], uint4 (&b1)[WJ]) const {
    if (HAS_FILL)
      issue_loads(fill, a_fill, b_fill);
#pragma unroll
    for (int ks = 0; ks + 1 < KS; ks++) {
      if (ks & 1) {
        load_frags(cur, ks + 1, a0, b0);
        mfma_all(acc, a1, b1);
      } else {
        load_frags(cur, ks + 1, a1, b1);
        mfma_all(acc, a0, b0);
      }
      interleave_hint();
    }
    // every wave has its last fragments of `cur` in registers and its share of
    // k-block kt+1 landed in `nxt` before anyone moves on
    wait_dma<BEHIND>();
    __builtin_amdgcn_s_barrier();
    // with a 2-stage ring the next block lives in the buffer just filled: read it
    // through the same pointer the DMA was issued with
    if (HAS_NEXT)
      load_frags(NST == 2 ? fill : nxt, 0, a0, b0);
    mfma_all(acc, a1, b1);
    interleave_hint();
  }
};

template <int ES, int KS, int WJ, bool SPLIT = false, bool TB = false>
__global__ __launch_bounds__(1024 / WJ, 1) void gemm_tile256_fast_kernel(GemmParams p) {
  typedef FastGemm<ES, KS, WJ, SPLIT, TB> FG;
  typedef typename FG::acc_t acc_t;
  constexpr int NST = FG::NST;
  // ring of NST stages (128 KiB); the epilogue reuses the whole array as 8 x 18 KiB staging regions
  // behind them the tile's column parameters for the epilogue: bias, scale, comp * colsum (see gemm_epilogue_act).
  // One array on purpose: with a second LDS variable in the kernel the compiler puts a full vmcnt(0) wait in
  // front of the fragment reads of every stage (it then treats every LDS read as a reader of the DMA's target).
  __shared__ __align__(1024) char smem[8 * G_STG_WAVE_BYTES + (SPLIT ? 0 : 3 * G_BN * 4)];
  float *colp = reinterpret_cast<float *>(smem + 8 * G_STG_WAVE_BYTES);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = WJ == 2 ? wave >> 2 : wave >> 1, wn = WJ == 2 ? wave & 3 : wave & 1;
  const int l32 = lane & 31, lh = lane >> 5;

  const int tiles_m = (int)((p.M + G_BM - 1) / G_BM), tiles_n = (int)(p.N / G_BN);
  int tm, tn, slice = 0;
  if (SPLIT) { // the tiles of one K slice are neighbours in the grid; K slice = blockIdx / tiles
    const int tiles = tiles_m * tiles_n, tile = (int)blockIdx.x % tiles;
    tm = tile / tiles_n;
    tn = tile % tiles_n;
    slice = (int)blockIdx.x / tiles;
  } else {
    tile_of_block(blockIdx.x, gridDim.x, tiles_m, tiles_n, p.group_m, tm, tn);
  }
  const int64_t m0 = (int64_t)tm * G_BM, n0 = (int64_t)tn * G_BN;
  const int64_t lda_b = p.lda * ES, ldb_b = p.ldb * ES;
  if (!SPLIT) { // strided batch in blockIdx.y
    const int64_t bz = blockIdx.y;
    p.A = reinterpret_cast<const char *>(p.A) + bz * p.a_bs * ES;
    p.B = reinterpret_cast<const char *>(p.B) + bz * p.b_bs * ES;
    p.C = reinterpret_cast<char *>(p.C) + bz * p.c_bs * (p.out_dt == DT_BF16 ? 2 : 4);
  if (p.residual)
    p.residual = reinterpret_cast<const char *>(p.residual) + bz * p.c_bs * (p.residual_dt == DT_BF16 ? 2 : 4);
  }

  FG g;
  g.wave_u = wave;
  if (SPLIT) { // 32-row tiles of this wave that hold rows of A
    const int64_t left = p.M - m0 - wm * 128;
    g.mi = left <= 0 ? 0 : (int)min((int64_t)4, (left + 31) / 32);
  }
  g.a_xor = p.a_xor;
#pragma unroll
  for (int i = 0; i < FG::NDMA; i++) {
    // A: this instruction fills 1 KiB = A_ROWS_PER_DMA rows; lane -> (row, physical chunk)
    int row = (wave * FG::NDMA + i) * FG::A_ROWS_PER_DMA + lane / FG::A_CPR;
    int c = (lane % FG::A_CPR) ^ FG::a_swz(row);
    // rows past M (split-K on a short A): fetch the last row instead, its results are dropped
    const int row_src = (int)min((int64_t)row, p.M - 1 - m0);
    g.a_src[i] = (uint32_t)(row_src * lda_b + c * 16);
    // B: B_ROWS_PER_DMA k-rows; lane -> (krow, physical chunk)
    int krow = (wave * FG::NDMA + i) * FG::B_ROWS_PER_DMA + lane / FG::B_CPR;
    int cb = (lane % FG::B_CPR) ^ ((krow % FG::RG) * FG::CW);
    g.b_src[i] = TB ? (uint32_t)(row * ldb_b + c * 16) : (uint32_t)(krow * ldb_b + cb * 16);
  }
#pragma unroll
  for (int ks = 0; ks < KS; ks++) {
    int row = wm * 128 + l32; // + i*32: a multiple of 32 leaves the swizzle unchanged
    g.a_ld[ks] = row * FG::KB + (((2 * ks + lh) ^ FG::a_swz(row)) << 4);
  }
  {
    const int gq = lane >> 4, i16 = lane & 15;
    const int kk = ES == 2 ? (i16 >> 2) : (i16 >> 1);
    const int cc = ES == 2 ? (i16 & 3) : (i16 & 1);
    if constexpr (TB) {
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        int row = wn * 32 * WJ + l32; // + j*32
        g.b_ld[ks] = row * FG::KB + (((2 * ks + lh) ^ FG::a_swz(row)) << 4);
      }
    } else {
#pragma unroll
      for (int j = 0; j < WJ; j++) {
        const int nb = wn * WJ + j; // 32-column block of the tile
        int chunk = ES == 2 ? (nb * 4 + 2 * (gq & 1) + (cc >> 1)) : (nb * 2 + (gq & 1));
        int sub = ES == 2 ? (cc & 1) * 8 : cc * 8;
        int krow_lane = (ES == 2 ? 8 : 16) * (gq >> 1) + kk;
        g.b_ld[j] = FG::A_BYTES + krow_lane * FG::B_ROW_BYTES + ((chunk ^ (kk * FG::CW)) << 4) + sub;
      }
    }
  }

  acc_t acc[WJ][4];
#pragma unroll
  for (int j = 0; j < WJ; j++)
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
      for (int r = 0; r < 16; r++)
        acc[j][i][r] = 0;

  const int64_t b_step = TB ? (int64_t)FG::KB : (int64_t)FG::BK * ldb_b; // bytes from one k-block of B to the next
  // K slice of this workgroup in ring groups (NST stages each): slices differ by at most one group
  const int groups = (int)(p.K / FG::BK) / NST, nsl = SPLIT ? p.splits : 1;
  const int g0 = (int)((int64_t)slice * groups / nsl), g1 = (int)((int64_t)(slice + 1) * groups / nsl);
  const int KT = (g1 - g0) * NST;
  const char *a_ptr = reinterpret_cast<const char *>(p.A) + m0 * lda_b + (int64_t)g0 * NST * FG::KB; // first k-block; KB bytes each
  const char *b_ptr = reinterpret_cast<const char *>(p.B) + (TB ? n0 * ldb_b : n0 * ES) + (int64_t)g0 * NST * b_step;

  uint4 a0[4], b0[WJ], a1[4], b1[WJ];
  // column parameters of this tile: requested before the operand traffic, written to LDS in front of the
  // prologue's barrier (which also publishes them to every wave)
  float cp_bias = -0.0f, cp_scale = 1.0f;
  int cp_cs = 0;
  if constexpr (!SPLIT) {
    if (tid < G_BN) {
      const int64_t n = n0 + tid;
      if (p.bias)
        cp_bias = p.bias_dt == DT_BF16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t *>(p.bias)[n])
                                       : reinterpret_cast<const float *>(p.bias)[n];
      if (ES == 1) {
        if (p.scale)
          cp_scale = p.scale[n];
        if (p.colsum)
          cp_cs = p.comp * p.colsum[n];
      }
    }
  }
  // prologue: request k-blocks 0 .. NST-2 (KT is a positive multiple of NST), wait for block 0
#pragma unroll
  for (int d = 0; d < NST - 1; d++)
    g.issue_loads(smem + d * FG::STAGE_BYTES, a_ptr + d * FG::KB, b_ptr + d * b_step);
  if constexpr (!SPLIT) {
    if (tid < G_BN) {
      colp[tid] = cp_bias;
      colp[G_BN + tid] = cp_scale;
      reinterpret_cast<int *>(colp)[2 * G_BN + tid] = cp_cs;
    }
  }
  FG::template wait_dma<NST - 2>();
  __builtin_amdgcn_s_barrier();
  g.load_frags(smem, 0, a0, b0);

  // steady state: groups of NST stages in which every stage still has a block to request
  int kt0 = 0;
  for (; kt0 + 2 * NST <= KT; kt0 += NST) {
    static_for<0, NST>([&](auto sc) {
      constexpr int st = decltype(sc)::value;
      constexpr int cur = st, nxt = (st + 1) % NST, fill = (st + NST - 1) % NST;
      const int kf = kt0 + st + NST - 1;
      g.template stage<true, true, NST - 2>(smem + cur * FG::STAGE_BYTES, smem + nxt * FG::STAGE_BYTES,
                                            smem + fill * FG::STAGE_BYTES, a_ptr + (int64_t)kf * FG::KB,
                                            b_ptr + kf * b_step, acc, a0, b0, a1, b1);
    });
  }
  // last group: only its first stage requests a block (the last one); the ring drains
  static_for<0, NST>([&](auto sc) {
    constexpr int st = decltype(sc)::value;
    constexpr int cur = st, nxt = (st + 1) % NST, fill = (st + NST - 1) % NST;
    constexpr int behind = NST - 2 - st > 0 ? NST - 2 - st : 0;
    const int kf = kt0 + st + NST - 1;
    g.template stage<st == 0, (st < NST - 1), behind>(smem + cur * FG::STAGE_BYTES, smem + nxt * FG::STAGE_BYTES,
                                                      smem + fill * FG::STAGE_BYTES, a_ptr + (int64_t)kf * FG::KB,
                                                      b_ptr + kf * b_step, acc, a0, b0, a1, b1);
  });

  // no wave reads fragments any more (the last stage's barrier came after its
  // final fragment reads), so the stage buffers can be overwritten
  if constexpr (SPLIT) {
    // f32 partial sums of the rows that exist, 16 bytes per lane (4 consecutive n of one m)
    float *part = p.partial + (int64_t)slice * p.M * p.N;
    static_for<0, WJ>([&](auto jc) {
      constexpr int j = decltype(jc)::value;
      static_for<0, 4>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        const int64_t m = m0 + wm * 128 + i * 32 + l32;
        if (m < p.M) {
#pragma unroll
          for (int q = 0; q < 4; q++) {
            const int64_t n = n0 + wn * (32 * WJ) + j * 32 + 8 * q + 4 * lh;
            f32x4_t v = {(float)acc[j][i][4 * q], (float)acc[j][i][4 * q + 1], (float)acc[j][i][4 * q + 2],
                         (float)acc[j][i][4 * q + 3]};
            *reinterpret_cast<f32x4_t *>(part + m * p.N + n) = v;
          }
        }
      });
    });
    return; // the sum over slices and the epilogue are the second kernel's (a kernel boundary is the cheapest
            // way to make partial sums visible across XCDs: device-scope fences write back and invalidate whole L2s)
  }
  if constexpr (!SPLIT) {
    if (p.out_dt == DT_BF16)
      gemm_epilogue<ES, false, true, WJ, true>(p, acc, m0, n0, wm, wn, l32, lh, smem + wave * (128 * (64 * WJ + 16)), colp);
    else
      gemm_epilogue<ES, false, false, WJ, true>(p, acc, m0, n0, wm, wn, l32, lh, nullptr, colp);
  }
}

// ---------------------------------------------------------------------------
// The whole-tile kernel on v_mfma_f32_16x16x32_bf16 / v_mfma_i32_16x16x64_i8 (B stored [K,N], no K slices).  Same
// tile, ring, DMA and epilogue as gemm_tile256_fast_kernel<ES, 2, 2>; what differs is the MFMA shape.  The board holds a power limit by
// lowering the clock, and per multiply-accumulate the 16x16x32 form moves less register-file data (0.25 B of
// accumulator + 0.25 B of operands against 0.5 B + 0.125 B): a loop of nothing but MFMAs sustains 2.13 PFLOP/s at
// 2.29 GHz with it and 1.89 PFLOP/s at 2.11 GHz with 32x32x16.
// One ring stage (64 bytes of K per row) is exactly one k-step of 32.  A wave's 128 x 64 tile is 8 x 4 tiles of
// 16 x 16; the stage is computed in two halves of 16 MFMAs (row tiles 0-3, then 4-7).  Register fragments: the
// A tiles of the half being computed and of the half to come (2 x 16 registers) and one set of B tiles (16).
// First half: read the A tiles of the second half (and B tile 3).  Barrier (next stage published).  Second half:
// read the next stage's first-half A tiles, and B tiles 0-2 as soon as their last MFMAs of this stage are issued.
#ifndef G_FAST_MI16
#define G_FAST_MI16 1
#endif
#ifndef G_MI16_SPLIT
#define G_MI16_SPLIT 3
#endif
// TB: B stored [N,K]; its tile is staged and read like the A tile (plain 16-byte fragment reads).
template <int ES, bool TB = false> __global__ __launch_bounds__(512, 1) void gemm_tile256_mi16_kernel(GemmParams p) {
  static_assert(!TB || ES == 2, "B stored [N,K]: bf16 only");
  typedef FastGemm<ES, 2, 2, false, TB> FG;
  typedef typename std::conditional<ES == 2, f32x4_t, i32x4_t>::type acc4_t;
  constexpr int NST = FG::NST;
  // one array: the ring / epilogue staging, then the column parameters (see gemm_tile256_fast_kernel)
  __shared__ __align__(1024) char smem[8 * G_STG_WAVE_BYTES + 3 * G_BN * 4];
  float *colp = reinterpret_cast<float *>(smem + 8 * G_STG_WAVE_BYTES);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 2, wn = wave & 3;
  const int l32 = lane & 31, lh = lane >> 5;
  const int r16 = lane & 15, g16 = lane >> 4;

  const int tiles_m = (int)(p.M / G_BM), tiles_n = (int)(p.N / G_BN);
  int tm, tn;
  tile_of_block(blockIdx.x, gridDim.x, tiles_m, tiles_n, p.group_m, tm, tn);
  const int64_t m0 = (int64_t)tm * G_BM, n0 = (int64_t)tn * G_BN;
  const int64_t lda_b = p.lda * ES, ldb_b = p.ldb * ES;
  {
    const int64_t bz = blockIdx.y; // strided batch
    p.A = reinterpret_cast<const char *>(p.A) + bz * p.a_bs * ES;
    p.B = reinterpret_cast<const char *>(p.B) + bz * p.b_bs * ES;
    p.C = reinterpret_cast<char *>(p.C) + bz * p.c_bs * (p.out_dt == DT_BF16 ? 2 : 4);
    if (p.residual)
      p.residual = reinterpret_cast<const char *>(p.residual) + bz * p.c_bs * (p.residual_dt == DT_BF16 ? 2 : 4);
  }

  FG g;
  g.wave_u = wave;
  g.a_xor = p.a_xor;
#pragma unroll
  for (int i = 0; i < FG::NDMA; i++) { // as in gemm_tile256_fast_kernel
    const int row = (wave * FG::NDMA + i) * FG::A_ROWS_PER_DMA + lane / FG::A_CPR;
    const int c = (lane % FG::A_CPR) ^ FG::a_swz(row);
    g.a_src[i] = (uint32_t)(row * lda_b + c * 16);
    const int krow = (wave * FG::NDMA + i) * FG::B_ROWS_PER_DMA + lane / FG::B_CPR;
    const int cb = (lane % FG::B_CPR) ^ ((krow % FG::RG) * FG::CW);
    g.b_src[i] = TB ? (uint32_t)(row * ldb_b + c * 16) : (uint32_t)(krow * ldb_b + cb * 16);
  }
  // A tile `it` (16 rows): lane -> row lane%16, logical 16-byte chunk lane/16 of the row's 64 bytes (8 bf16 or
  // 16 int8 of k)
  const int row_a = wm * 128 + r16; // + 16*it: leaves the swizzle unchanged
  const uint32_t a_ld = (uint32_t)(row_a * FG::KB + ((g16 ^ FG::a_swz(row_a)) << 4));
  // B tile `jt` (16 columns): the 16 lanes of a group hand the transposing read an RG (k) x 16 (n) block of 8-byte
  // pieces (bf16: k row lane%16/4, columns 4*(lane%4)..+3; int8: k row lane%16/2, columns 8*(lane%2)..+7) and get
  // back column lane%16 of those RG k rows; group lane/16 takes k rows 2*RG*(lane/16)..+RG-1 and, 2048 bytes (RG
  // k rows) on, the RG after them
  uint32_t b_ld[4];
  {
    const int kk = ES == 2 ? (r16 >> 2) : (r16 >> 1);
    const int cc = ES == 2 ? (r16 & 3) : (r16 & 1);
#pragma unroll
    for (int jt = 0; jt < 4; jt++) {
      const int chunk = ES == 2 ? (wn * 4 + jt) * 2 + (cc >> 1) : (wn * 4 + jt);
      const int sub = ES == 2 ? (cc & 1) * 8 : cc * 8;
      b_ld[jt] = (uint32_t)(FG::A_BYTES + (2 * FG::RG * g16 + kk) * FG::B_ROW_BYTES + ((chunk ^ (kk * FG::CW)) << 4) + sub);
      if (TB) { // row of the [N,K] tile = column of C; chunk and swizzle as for A
        const int row_b = wn * 64 + jt * 16 + r16;
        b_ld[jt] = (uint32_t)(FG::A_BYTES + row_b * FG::KB + ((g16 ^ FG::a_swz(row_b)) << 4));
      }
    }
  }

  acc4_t acc4[2][4][4]; // [j][i][q]: the 16 x 16 tile at columns 16*(q/2), rows 16*(q%2) of the 32 x 32 block (j, i)
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
      for (int q = 0; q < 4; q++)
        acc4[j][i][q] = acc4_t{0, 0, 0, 0};

  const int64_t b_step = TB ? (int64_t)FG::KB : (int64_t)FG::BK * ldb_b;
  const int KT = (int)(p.K / FG::BK); // a positive multiple of NST (checked by the launcher)
  const char *a_ptr = reinterpret_cast<const char *>(p.A) + m0 * lda_b;
  const char *b_ptr = reinterpret_cast<const char *>(p.B) + (TB ? n0 * ldb_b : n0 * ES);

  uint4 a_lo[4], a_hi[4], bb[4];
  auto load_a = [&](const char *__restrict__ st, int half, uint4(&a)[4]) {
#pragma unroll
    for (int ii = 0; ii < 4; ii++) {
      uint4 v = *reinterpret_cast<const uint4 *>(st + a_ld + (half * 4 + ii) * (16 * FG::KB));
      if (ES == 1) // u8 activations: a - 128 as s8 == a ^ 0x80
        v = make_uint4(v.x ^ g.a_xor, v.y ^ g.a_xor, v.z ^ g.a_xor, v.w ^ g.a_xor);
      a[ii] = v;
    }
  };
  auto load_b_tile = [&](const char *__restrict__ st, int jt) -> uint4 {
    if constexpr (TB) {
      return *reinterpret_cast<const uint4 *>(st + b_ld[jt]);
    } else {
      const uint2 lo = MfmaOp<ES>::tr_read(st + b_ld[jt]);
      const uint2 hi = MfmaOp<ES>::tr_read(st + b_ld[jt] + FG::RG * FG::B_ROW_BYTES);
      return make_uint4(lo.x, lo.y, hi.x, hi.y);
    }
  };
  auto load_b = [&](const char *__restrict__ st, uint4(&b)[4]) {
#pragma unroll
    for (int jt = 0; jt < 4; jt++)
      b[jt] = load_b_tile(st, jt);
  };
  // 16 MFMAs: row tiles 4*HALF..+3 against the 4 column tiles; operand roles swapped as in the 32x32 kernels
  // (first operand = B fragment), so a lane ends up with 4 consecutive columns of one row
  auto mfma_half = [&](auto halfc, auto jt0c, auto jt1c, const uint4(&a)[4], const uint4(&b)[4]) {
    constexpr int HALF = decltype(halfc)::value, JT0 = decltype(jt0c)::value, JT1 = decltype(jt1c)::value;
    static_for<JT0, JT1>([&](auto jtc) {
      constexpr int jt = decltype(jtc)::value;
      static_for<0, 4>([&](auto iic) {
        constexpr int it = HALF * 4 + decltype(iic)::value;
        constexpr int j = jt >> 1, i = it >> 1, q = 2 * (jt & 1) + (it & 1);
        if constexpr (ES == 2)
          acc4[j][i][q] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, b[jt]),
                                                                  __builtin_bit_cast(bf16x8_t, a[it & 3]), acc4[j][i][q], 0, 0, 0);
        else
          acc4[j][i][q] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(i32x4_t, b[jt]),
                                                                __builtin_bit_cast(i32x4_t, a[it & 3]), acc4[j][i][q], 0, 0, 0);
      });
    });
  };
  // MFMA, two LDS reads, MFMA, two LDS reads ... until the group's reads are out, then the remaining MFMAs
  auto hint = [&](auto ndsc, auto nmc) {
    constexpr int N_DS = decltype(ndsc)::value, N_MFMA = decltype(nmc)::value;
    static_for<0, N_MFMA>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      constexpr int left = N_DS - 2 * i;
      if constexpr (left > 0)
        __builtin_amdgcn_sched_group_barrier(0x100, left < 2 ? left : 2, 0);
    });
  };
  // One stage (see FastGemm::stage for the ring).  MFMAs run column tile by column tile; a column tile's B fragment
  // is dead after its four MFMAs of the second half and is reloaded from the next stage on the spot, so B needs one
  // set of registers.
  auto stage = [&](auto has_fill, auto has_next, auto behindc, char *__restrict__ cur, char *__restrict__ nxt,
                   char *__restrict__ fill, const char *a_fill, const char *b_fill) {
    constexpr bool HAS_FILL = decltype(has_fill)::value, HAS_NEXT = decltype(has_next)::value;
    constexpr int BEHIND = decltype(behindc)::value;
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, 1> I1;
    typedef std::integral_constant<int, G_MI16_SPLIT> I3; // column tiles of the first half in front of the barrier
    typedef std::integral_constant<int, 4> I4;
    if constexpr (HAS_FILL)
      g.issue_loads(fill, a_fill, b_fill);
    load_a(cur, 1, a_hi);
    // the last column tile's B fragment is first read behind the barrier: fetched here rather than at the very end
    // of the previous stage, where the (full) LDS wait in front of this half would have to sit it out
    bb[3] = load_b_tile(cur, 3);
    mfma_half(I0{}, I0{}, I3{}, a_lo, bb); // 12 of the first half's 16
    hint(std::integral_constant<int, TB ? 5 : 6>{}, std::integral_constant<int, 4 * G_MI16_SPLIT>{});
    // The barrier sits three quarters into the first half: the reads above have returned by then (its wait covers
    // them), and the four MFMAs left over cover the barrier's own latency.  Nothing may move across it.
    __builtin_amdgcn_sched_barrier(0);
    FG::template wait_dma<BEHIND>();
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    mfma_half(I0{}, I3{}, I4{}, a_lo, bb); // the last readers of a_lo
    if constexpr (HAS_NEXT)
      load_a(nxt, 0, a_lo);
    static_for<0, 4>([&](auto jtc) {
      constexpr int jt = decltype(jtc)::value;
      mfma_half(I1{}, jtc, std::integral_constant<int, jt + 1>{}, a_hi, bb);
      if constexpr (HAS_NEXT && jt < 3)
        bb[jt] = load_b_tile(nxt, jt);
    });
    // issue order after the barrier: the four MFMAs left of the first half; the next stage's first-half A tiles
    // between the MFMAs of column tile 0; after each column tile its B fragment of the next stage
    if constexpr (G_MI16_SPLIT < 4)
      __builtin_amdgcn_sched_group_barrier(0x008, 4 * (4 - G_MI16_SPLIT), 0);
    static_for<0, 4>([&](auto ic) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if constexpr (HAS_NEXT)
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    });
    static_for<0, 4>([&](auto jtc) {
      if constexpr (decltype(jtc)::value > 0)
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
      if constexpr (HAS_NEXT && decltype(jtc)::value < 3)
        __builtin_amdgcn_sched_group_barrier(0x100, TB ? 1 : 2, 0);
    });
  };

  // column parameters of this tile (see gemm_tile256_fast_kernel)
  float cp_bias = -0.0f, cp_scale = 1.0f;
  int cp_cs = 0;
  if (tid < G_BN) {
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
    g.issue_loads(smem + d * FG::STAGE_BYTES, a_ptr + d * FG::KB, b_ptr + d * b_step);
  if (tid < G_BN) {
    colp[tid] = cp_bias;
    colp[G_BN + tid] = cp_scale;
    reinterpret_cast<int *>(colp)[2 * G_BN + tid] = cp_cs;
  }
  FG::template wait_dma<NST - 2>();
  __builtin_amdgcn_s_barrier();
  load_a(smem, 0, a_lo);
  load_b(smem, bb);

  typedef std::integral_constant<bool, true> T;
  typedef std::integral_constant<bool, false> F;
  int kt0 = 0;
  for (; kt0 + 2 * NST <= KT; kt0 += NST) {
    static_for<0, NST>([&](auto sc) {
      constexpr int st = decltype(sc)::value;
      constexpr int cur = st, nxt = (st + 1) % NST, fill = (st + NST - 1) % NST;
      const int kf = kt0 + st + NST - 1;
      stage(T{}, T{}, std::integral_constant<int, NST - 2>{}, smem + cur * FG::STAGE_BYTES, smem + nxt * FG::STAGE_BYTES, smem + fill * FG::STAGE_BYTES,
            a_ptr + (int64_t)kf * FG::KB, b_ptr + kf * b_step);
    });
  }
  static_for<0, NST>([&](auto sc) { // last group: only its first stage requests a block; the ring drains
    constexpr int st = decltype(sc)::value;
    constexpr int cur = st, nxt = (st + 1) % NST, fill = (st + NST - 1) % NST;
    constexpr int behind = NST - 2 - st > 0 ? NST - 2 - st : 0;
    const int kf = kt0 + st + NST - 1;
    stage(std::integral_constant<bool, st == 0>{}, std::integral_constant<bool, (st < NST - 1)>{},
          std::integral_constant<int, behind>{}, smem + cur * FG::STAGE_BYTES,
          smem + nxt * FG::STAGE_BYTES, smem + fill * FG::STAGE_BYTES, a_ptr + (int64_t)kf * FG::KB, b_ptr + kf * b_step);
  });

  // the accumulators in the shape the epilogue takes: element 4q+e of block (j, i)
  typename MfmaOp<ES>::acc_t acc[2][4];
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
      for (int q = 0; q < 4; q++)
#pragma unroll
        for (int e = 0; e < 4; e++)
          acc[j][i][4 * q + e] = acc4[j][i][q][e];
  if (p.out_dt == DT_BF16)
    gemm_epilogue<ES, false, true, 2, true, true>(p, acc, m0, n0, wm, wn, l32, lh, smem + wave * G_STG_WAVE_BYTES, colp);
  else
    gemm_epilogue<ES, false, false, 2, true, true>(p, acc, m0, n0, wm, wn, l32, lh, nullptr, colp);
}

// ---------------------------------------------------------------------------
// The whole-tile kernel with one wave per SIMD: 4 waves as 2 x 2, each owning 128 x 128 of the 256 x 256 tile as
// 8 x 8 tiles of 16 x 16 (v_mfma_f32_16x16x32_bf16 / v_mfma_i32_16x16x64_i8), 256 accumulator registers.  Against
// the 8-wave kernel a multiply-accumulate costs a third less LDS read traffic (per k-step a wave reads 8 KiB of A
// and 8 KiB of B for 64 MFMAs, not 8 + 4 KiB for 32), which is what counts on a board that holds its power limit
// by lowering the clock.  With a single wave per SIMD nothing hides a stall, so every fragment is fetched a whole
// stage ahead:
//   stage s computes k-block s entirely from registers: A tiles in one of two register sets, B tiles in one set;
//   its MFMAs run column tile by column tile, and between them the wave reads k-block s+1: one A tile per column
//   tile into the other A set, and the B tile of a column as soon as that column's MFMAs are issued (column 7's
//   goes to a spare register set, alternating by stage, so it can be fetched early as well).
// Because a k-block sits in registers for the whole of its stage, its LDS slot is free during the stage: the ring
// of 4 slots carries k-blocks s+1 .. s+4, and the DMA of block s+4 is issued at the start of stage s, three full
// stages (about 3000 cycles) before the barrier that publishes it.  One barrier per stage, at its start:
//   s_waitcnt vmcnt(2 stages) lgkmcnt(0)   own share of block s+1 has landed; own reads of block s have returned
//   s_barrier                              block s+1 is visible to all; slot s may be overwritten
// The main loop is assembly text written by gen_gemm_w4_mainloop.py (registers and issue order fixed by hand: the
// compiler's allocator does not hold 64 accumulator tiles and three fragment sets without copies and spills);
// set-up and epilogue are the C++ below.
#include "gemm_w4_mainloop.inc"
#if defined(GCMI_W4_EXPERIMENT_OPTS) && !defined(GCMI_W4_ALLOW_EXPERIMENT)
#error "gemm_w4_mainloop.inc was generated with experiment switches (some give wrong products): regenerate it without GCMI_W4_EXPERIMENT"
#endif

// Epilogue of gemm_tile256_w4_kernel.  The main loop's assembly ends by writing the raw accumulators of column
// tiles 0-3 (the left 64 columns of the wave's 128 x 128) to a wave-private LDS region, 128 rows of 256 bytes at a
// pitch of 272; a second, small assembly statement does the same for column tiles 4-7 once the first half has been
// consumed.  What is left for this code is a rolled loop over rows: a lane reads four consecutive columns of a row
// (16 bytes, 16 lanes per row, 4 rows per instruction), applies the epilogue and stores 8 (bf16) or 16 bytes, so a
// row leaves as one or two whole 128-byte lines.  Unrolled over the 64 accumulator tiles in place of the loop, the
// same work was ten times the code, all of it executed once per workgroup and fetched cold: 12 us of a 100 us
// kernel went into instruction-cache misses.
static constexpr int W4_DUMP_PITCH = 272;                   // 64 f32 / s32 + 16 bytes: conflict-free for the 16-byte writes
static constexpr int W4_DUMP_WAVE_BYTES = 128 * W4_DUMP_PITCH; // 34816 per wave, 139264 per workgroup

// Four results of one row: c = the raw accumulators of columns n .. n+3 of row m.  HAS_BIAS / HAS_RES are
// compile-time so that the eight rows of an unrolled group are straight-line code (their LDS reads go out together).
// NAN_FREE: the caller has shown that no result of this row can be a NaN, so the bf16 conversions need no fix-up.
// MASKED (a tile that sticks out of C): row_ok says whether row m exists; nothing of a missing row is read or stored.
template <int ES, int ACT, int OUT, bool HAS_BIAS, bool HAS_RES, bool MASKED, bool NAN_FREE = false, typename acc4_t>
__device__ __forceinline__ void w4_epilogue_row(const GemmParams &p, const acc4_t &c, int64_t m, int64_t n,
                                                const f32x4_t &bias4, const f32x4_t &scale4, const i32x4_t &cs4,
                                                bool row_ok = true) {
  if (MASKED && !row_ok)
    return;
  char *Cb = reinterpret_cast<char *>(p.C);
  float x[4];
  uint32_t p0 = 0, p1 = 0; // bf16 results, two per register
  if constexpr (ES == 1) {
    int ci[4];
#pragma unroll
    for (int e = 0; e < 4; e++)
      ci[e] = (int)c[e] + cs4[e]; // exact: the zero-point term in integer arithmetic
    if constexpr (OUT == DT_S32) {
      *reinterpret_cast<i32x4_t *>(Cb + (m * p.ldc + n) * 4) = i32x4_t{ci[0], ci[1], ci[2], ci[3]};
      return;
    }
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const float v = fmaf((float)ci[e], scale4[e], bias4[e]); // an absent bias is -0.0: the product itself
#ifndef GCMI_GELU_BF16_PRECISE // (measurement builds define it to time the f32-grade erf in this place)
      if constexpr (OUT == DT_BF16 && NAN_FREE && ACT == ACT_GELU_ERF)
        x[e] = gelu_erf_bf16_result(v); // v is finite here and the result is rounded to bf16 below
      else
#endif
        x[e] = act_const<ACT>(v);
    }
    if constexpr (OUT == DT_F32) {
      *reinterpret_cast<f32x4_t *>(Cb + (m * p.ldc + n) * 4) = f32x4_t{x[0], x[1], x[2], x[3]};
      return;
    }
    // v_cvt_pk_bf16_f32 rounds to nearest even but keeps a NaN's sign and payload; a NaN among the four (their
    // sum is one; so is the sum of opposite infinities) sends them through the scalar rule: NaN -> 0x7FC0
    const float any_nan = NAN_FREE ? 0.0f : (x[0] + x[1]) + (x[2] + x[3]);
    if (__builtin_expect(any_nan != any_nan, 0)) {
      p0 = f32_to_bf16_bits(x[0]) | ((uint32_t)f32_to_bf16_bits(x[1]) << 16);
      p1 = f32_to_bf16_bits(x[2]) | ((uint32_t)f32_to_bf16_bits(x[3]) << 16);
    } else {
      p0 = pack_bf16x2(x[0], x[1]), p1 = pack_bf16x2(x[2], x[3]);
    }
  } else {
#pragma unroll
    for (int e = 0; e < 4; e++)
      x[e] = (float)c[e];
    float res4[4] = {0.f, 0.f, 0.f, 0.f};
    if constexpr (HAS_RES) { // 16-byte aligned rows (checked by the launcher)
      const int64_t at = m * p.ldr + n;
      if (p.residual_dt == DT_BF16) {
        const uint2 v = *reinterpret_cast<const uint2 *>(reinterpret_cast<const uint16_t *>(p.residual) + at);
        res4[0] = __uint_as_float(v.x << 16), res4[1] = __uint_as_float(v.x & 0xffff0000u);
        res4[2] = __uint_as_float(v.y << 16), res4[3] = __uint_as_float(v.y & 0xffff0000u);
      } else {
        const f32x4_t v = *reinterpret_cast<const f32x4_t *>(reinterpret_cast<const float *>(p.residual) + at);
        res4[0] = v[0], res4[1] = v[1], res4[2] = v[2], res4[3] = v[3];
      }
    }
    if constexpr (OUT == DT_F32) { // no intermediate rounding
#pragma unroll
      for (int e = 0; e < 4; e++) {
        if constexpr (HAS_BIAS)
          x[e] = x[e] + bias4[e];
        x[e] = act_const<ACT>(x[e]);
        if constexpr (HAS_RES) { // kept apart from the activation's last multiply: the sum equals a separate add
#pragma clang fp contract(off)
          x[e] = x[e] + res4[e];
        }
      }
      *reinterpret_cast<f32x4_t *>(Cb + (m * p.ldc + n) * 4) = f32x4_t{x[0], x[1], x[2], x[3]};
      return;
    }
    // bf16 graph: rounded after the matmul and after every bf16 op (lib/gc/Transforms/Pipeline.cpp:79-95), in
    // pairs.  A NaN stays a NaN through the ops that follow, so only the last conversion gives it 0x7FC0.
    auto rnd = [&]() {
      p0 = pack_bf16x2(x[0], x[1]), p1 = pack_bf16x2(x[2], x[3]);
      x[0] = __uint_as_float(p0 << 16), x[1] = __uint_as_float(p0 & 0xffff0000u);
      x[2] = __uint_as_float(p1 << 16), x[3] = __uint_as_float(p1 & 0xffff0000u);
    };
    constexpr bool LAST_IS_MATMUL = !HAS_BIAS && ACT == ACT_NONE && !HAS_RES;
    if constexpr (LAST_IS_MATMUL) { // nothing follows the first rounding: no need to widen again
      p0 = pack_bf16x2(x[0], x[1]), p1 = pack_bf16x2(x[2], x[3]);
    } else {
      rnd();
    }
    if constexpr (HAS_BIAS) {
#pragma unroll
      for (int e = 0; e < 4; e++)
        x[e] = x[e] + bias4[e];
      rnd();
    }
    if constexpr (ACT != ACT_NONE) {
#pragma unroll
      for (int e = 0; e < 4; e++)
        x[e] = act_const<ACT>(x[e]);
      if constexpr (ACT == ACT_RELU) { // max(x, 0) of a bf16 value is a bf16 value: nothing to round
        p0 = (__float_as_uint(x[0]) >> 16) | (__float_as_uint(x[1]) & 0xffff0000u);
        p1 = (__float_as_uint(x[2]) >> 16) | (__float_as_uint(x[3]) & 0xffff0000u);
      } else {
        rnd();
      }
    }
    if constexpr (HAS_RES) {
#pragma unroll
      for (int e = 0; e < 4; e++)
        x[e] = x[e] + res4[e];
      rnd();
    }
    const float any_nan = NAN_FREE ? 0.0f : (x[0] + x[1]) + (x[2] + x[3]);
    if (__builtin_expect(any_nan != any_nan, 0)) {
      if (x[0] != x[0]) p0 = (p0 & 0xffff0000u) | 0x7FC0u;
      if (x[1] != x[1]) p0 = (p0 & 0x0000ffffu) | 0x7FC00000u;
      if (x[2] != x[2]) p1 = (p1 & 0xffff0000u) | 0x7FC0u;
      if (x[3] != x[3]) p1 = (p1 & 0x0000ffffu) | 0x7FC00000u;
    }
  }
  typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
  const u32x2_t vv = {p0, p1};
  __builtin_nontemporal_store(vv, reinterpret_cast<u32x2_t *>(Cb + (m * p.ldc + n) * 2));
}

// One half (64 columns) of the wave tile.  OUT = DT_BF16 / DT_F32 / DT_S32.
// MASKED: rows_in / cols_in of the tile's 256 x 256 lie inside C (cols_in is a multiple of 4).
// WR x WC: the wave's tile (128 x 128 in the 256 x 256 kernel, 64 x 64 in the 128 x 128 one); rows_in / cols_in count
// from the workgroup tile's corner whatever its size.
template <int ES, int ACT, int OUT, bool MASKED, int WR = 128, int WC = 128>
__device__ __forceinline__ void w4_epilogue_half(const GemmParams &p, int half, int64_t m0, int64_t n0, int wm, int wn,
                                                 int lane, const char *dump, const float *colp, int rows_in, int cols_in) {
  typedef typename std::conditional<ES == 2, float, int>::type acc_e;
  typedef acc_e acc4_t __attribute__((ext_vector_type(4)));
  const int rr = lane >> 4, cc = lane & 15;
  const int col = wn * WC + half * 64 + 4 * cc; // this lane's four columns inside the workgroup tile
  const int64_t n = n0 + col;
  if (MASKED && col >= cols_in)
    return;
  const int row0 = wm * WR + rr; // + 4 * (i0 + u)
  const f32x4_t bias4 = *reinterpret_cast<const f32x4_t *>(colp + col); // -0.0 where there is no bias
  f32x4_t scale4 = {1.f, 1.f, 1.f, 1.f};
  i32x4_t cs4 = {0, 0, 0, 0}; // comp * colsum
  if constexpr (ES == 1) {
    scale4 = *reinterpret_cast<const f32x4_t *>(colp + 256 + col);
    cs4 = *reinterpret_cast<const i32x4_t *>(colp + 512 + col);
  }
  const bool has_bias = ES == 2 && p.bias != nullptr, has_res = ES == 2 && p.residual != nullptr;
  const bool bias_finite = fabsf((bias4[0] + bias4[1]) + (bias4[2] + bias4[3])) < __builtin_inff() || // the usual case
                           (fabsf(bias4[0]) < __builtin_inff() && fabsf(bias4[1]) < __builtin_inff() &&
                            fabsf(bias4[2]) < __builtin_inff() && fabsf(bias4[3]) < __builtin_inff());
  bool cols_tame = true;
  if constexpr (ES == 1) {
#pragma unroll
    for (int e = 0; e < 4; e++)
      cols_tame = cols_tame && fabsf(scale4[e]) < 0x1p90f && fabsf(bias4[e]) < 0x1p120f;
  }
  constexpr int U = 8; // rows in flight per lane
#pragma unroll 1
  for (int i0 = 0; i0 < WR / 4; i0 += U) {
    acc4_t c[U];
#pragma unroll
    for (int u = 0; u < U; u++)
      c[u] = *reinterpret_cast<const acc4_t *>(dump + ((i0 + u) * 4 + rr) * W4_DUMP_PITCH + cc * 16);
    auto rows = [&](auto hb, auto hr) {
      constexpr bool HB = decltype(hb)::value, HR = decltype(hr)::value;
      // bf16 results of finite accumulators and finite biases through nothing but an add and a ReLU are no NaNs:
      // one sum over the group's 32 accumulators (a NaN or an infinity among them makes it non-finite) replaces
      // the check of every row
      if constexpr (ES == 2 && OUT == DT_BF16 && !HR && (ACT == ACT_NONE || ACT == ACT_RELU)) {
        float t = 0.0f;
#pragma unroll
        for (int u = 0; u < U; u++)
          t += ((float)c[u][0] + (float)c[u][1]) + ((float)c[u][2] + (float)c[u][3]);
        if (__builtin_expect(bias_finite && fabsf(t) < __builtin_inff(), 1)) {
#pragma unroll
          for (int u = 0; u < U; u++)
            w4_epilogue_row<ES, ACT, OUT, HB, HR, MASKED, true>(p, c[u], m0 + row0 + (i0 + u) * 4, n, bias4, scale4, cs4,
                                                                row0 + (i0 + u) * 4 < rows_in);
          return;
        }
      }
#pragma unroll
      for (int u = 0; u < U; u++)
        w4_epilogue_row<ES, ACT, OUT, HB, HR, MASKED>(p, c[u], m0 + row0 + (i0 + u) * 4, n, bias4, scale4, cs4,
                                                      row0 + (i0 + u) * 4 < rows_in);
    };
    typedef std::integral_constant<bool, true> T;
    typedef std::integral_constant<bool, false> F;
    if constexpr (ES == 1) {
      // |acc| < 2^31: with scales below 2^90 and biases below 2^120 in magnitude the dequantised value is finite, and
      // so is every activation of it: no NaN to look for
      if (__builtin_expect(cols_tame, 1)) {
#pragma unroll
        for (int u = 0; u < U; u++)
          w4_epilogue_row<ES, ACT, OUT, false, false, MASKED, true>(p, c[u], m0 + row0 + (i0 + u) * 4, n, bias4, scale4, cs4,
                                                                    row0 + (i0 + u) * 4 < rows_in);
      } else {
        rows(F{}, F{});
      }
    } else {
      if (has_bias) {
        if (has_res)
          rows(T{}, T{});
        else
          rows(T{}, F{});
      } else {
        if (has_res)
          rows(F{}, T{});
        else
          rows(F{}, F{});
      }
    }
  }
}

// kind = act + 8 * (0: bf16, 1: f32, 2: s32)
template <int ES, bool MASKED, int WR = 128, int WC = 128>
__device__ __forceinline__ void w4_epilogue_half_any(const GemmParams &p, int kind, int half, int64_t m0, int64_t n0,
                                                     int wm, int wn, int lane, const char *dump, const float *colp,
                                                     int rows_in, int cols_in) {
#define GCMI_W4_CASE(ACT, OUT, K)                                                                                     \
  case (int)ACT + 8 * K:                                                                                              \
    w4_epilogue_half<ES, ACT, OUT, MASKED, WR, WC>(p, half, m0, n0, wm, wn, lane, dump, colp, rows_in, cols_in);      \
    break;
  switch (kind) {
    GCMI_W4_CASE(ACT_RELU, DT_BF16, 0)
    GCMI_W4_CASE(ACT_GELU_ERF, DT_BF16, 0)
    GCMI_W4_CASE(ACT_GELU_TANH, DT_BF16, 0)
    GCMI_W4_CASE(ACT_SIGMOID, DT_BF16, 0)
    GCMI_W4_CASE(ACT_NONE, DT_F32, 1)
    GCMI_W4_CASE(ACT_RELU, DT_F32, 1)
    GCMI_W4_CASE(ACT_GELU_ERF, DT_F32, 1)
    GCMI_W4_CASE(ACT_GELU_TANH, DT_F32, 1)
    GCMI_W4_CASE(ACT_SIGMOID, DT_F32, 1)
    GCMI_W4_CASE(ACT_NONE, DT_S32, 2)
  default:
    w4_epilogue_half<ES, ACT_NONE, DT_BF16, MASKED, WR, WC>(p, half, m0, n0, wm, wn, lane, dump, colp, rows_in, cols_in);
    break;
  }
#undef GCMI_W4_CASE
}

template <int ES, bool TB = false> __global__ __launch_bounds__(256, 1) void gemm_tile256_w4_kernel(GemmParams p) {
  // B stored [N,K]: bf16 only.  (The same loop for 8-bit operands -- plain 16-byte fragment reads in place of the
  // transposing ones -- was measured against [K,N] on one board and is no faster: 166.9-168.9 against 167.2-168.6 us
  // for the 4096 x 4096 x 11008 layer; an 8-bit weight stored [N,K] is copied once instead.)
  static_assert(!TB || ES == 2, "B stored [N,K]: bf16 only");
  typedef FastGemm<ES, 2, 4, false, TB> FG; // 4 waves: 4 DMA instructions per operand, wave and stage
  static_assert(FG::NST == 4 && FG::NDMA == 4 && FG::STAGE_BYTES == 32768 && FG::A_BYTES == 16384, "the assembly's ring");
#ifdef GCMI_W4_TIMING
  const long long wall_entry = wall_clock64();
  float *const timing_out = p.partial;
#endif
  // one array: the ring (128 KiB; the epilogue's 4 x 34 KiB of accumulators afterwards), then the column parameters
  __shared__ __align__(1024) char smem[8 * G_STG_WAVE_BYTES + 3 * G_BN * 4];
  static_assert(4 * W4_DUMP_WAVE_BYTES <= 8 * G_STG_WAVE_BYTES, "accumulator regions overlap the column parameters");
  float *colp = reinterpret_cast<float *>(smem + 8 * G_STG_WAVE_BYTES);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int r16 = lane & 15, g16 = lane >> 4;

  const int tiles_m = (int)((p.M + G_BM - 1) / G_BM), tiles_n = (int)((p.N + G_BN - 1) / G_BN); // edge tiles stick out
  int tm, tn;
  tile_of_block(blockIdx.x, gridDim.x, tiles_m, tiles_n, p.group_m, tm, tn);
  // integer division runs on the vector unit; the operand addresses below must be in scalar registers
  tm = __builtin_amdgcn_readfirstlane(tm), tn = __builtin_amdgcn_readfirstlane(tn);
  const int64_t m0 = (int64_t)tm * G_BM, n0 = (int64_t)tn * G_BN;
  const int64_t lda_b = p.lda * ES, ldb_b = p.ldb * ES;
  {
    const int64_t bz = blockIdx.y; // strided batch
    p.A = reinterpret_cast<const char *>(p.A) + bz * p.a_bs * ES;
    p.B = reinterpret_cast<const char *>(p.B) + bz * p.b_bs * ES;
    p.C = reinterpret_cast<char *>(p.C) + bz * p.c_bs * (p.out_dt == DT_BF16 ? 2 : 4);
    if (p.residual)
      p.residual = reinterpret_cast<const char *>(p.residual) + bz * p.c_bs * (p.residual_dt == DT_BF16 ? 2 : 4);
  }

  // per-lane source offsets of the wave's DMA instructions, as in gemm_tile256_fast_kernel.  An edge tile's rows past
  // M and columns past N are fetched from the last row / the last 16-byte chunk inside (N is a multiple of the
  // chunk's columns): their products land in accumulators that the epilogue never stores.
  const int rows_in = (int)min((int64_t)G_BM, p.M - m0), cols_in = (int)min((int64_t)G_BN, p.N - n0);
  i32x4_t a_off, b_off;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int row = (wave * 4 + i) * FG::A_ROWS_PER_DMA + lane / FG::A_CPR;
    const int c = (lane % FG::A_CPR) ^ FG::a_swz(row);
    a_off[i] = (int)(min(row, rows_in - 1) * lda_b + c * 16);
    const int krow = (wave * 4 + i) * FG::B_ROWS_PER_DMA + lane / FG::B_CPR;
    const int cb = min((lane % FG::B_CPR) ^ ((krow % FG::RG) * FG::CW), cols_in * ES / 16 - 1);
    b_off[i] = TB ? (int)(min(row, cols_in - 1) * ldb_b + c * 16) : (int)(krow * ldb_b + cb * 16);
  }
  // fragment addresses as in gemm_tile256_mi16_kernel: A tile `it` = rows wm*128 + 16*it .., B tile `jt` = columns
  // wn*128 + 16*jt ..; slots 2 and 3 through a second base (an instruction's offset field has 16 bits)
  const uint32_t lds0 = (uint32_t)(uintptr_t)(GCMI_LDS char *)smem;
  typedef int i32x8_t __attribute__((ext_vector_type(8)));
  i32x2_t a_ld;
  i32x8_t b_ld0, b_ld2;
  {
    const int row_a = wm * 128 + r16;
    a_ld[0] = (int)(lds0 + row_a * FG::KB + ((g16 ^ FG::a_swz(row_a)) << 4));
    a_ld[1] = a_ld[0] + 65536;
    const int kk = ES == 2 ? (r16 >> 2) : (r16 >> 1);
    const int cc = ES == 2 ? (r16 & 3) : (r16 & 1);
#pragma unroll
    for (int jt = 0; jt < 8; jt++) {
      const int chunk = ES == 2 ? (wn * 8 + jt) * 2 + (cc >> 1) : (wn * 8 + jt);
      const int sub = ES == 2 ? (cc & 1) * 8 : cc * 8;
      int at = FG::A_BYTES + (2 * FG::RG * g16 + kk) * FG::B_ROW_BYTES + ((chunk ^ (kk * FG::CW)) << 4) + sub;
      if (TB) {
        const int row_b = wn * 128 + jt * 16 + r16;
        at = FG::A_BYTES + row_b * FG::KB + ((g16 ^ FG::a_swz(row_b)) << 4);
      }
      b_ld0[jt] = (int)(lds0 + at);
      b_ld2[jt] = (int)(lds0 + at + 65536);
    }
  }

  // column parameters of this tile (see gemm_tile256_fast_kernel): 256 threads, one column each
  float cp_bias = -0.0f, cp_scale = 1.0f;
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

  uint64_t a_ptr = (uint64_t)(reinterpret_cast<const char *>(p.A) + m0 * lda_b);
  uint64_t b_ptr = (uint64_t)(reinterpret_cast<const char *>(p.B) + (TB ? n0 * ldb_b : n0 * ES));
  uint64_t b_step = TB ? (uint64_t)FG::KB : (uint64_t)(FG::BK * ldb_b);
  int trips = (int)(p.K / FG::BK) / 4 - 1; // k-blocks: a positive multiple of 4 (checked by the launcher)
  const uint32_t dma_lds = lds0 + (uint32_t)wave * 4096u;
  const uint32_t a_xor = p.a_xor;
  // where this lane writes its accumulators for the epilogue: row lane%16 (+ 16*it), 16-byte chunk lane/16 (+ 4*jt)
  // of the wave's region
  const uint32_t dump_ld = lds0 + (uint32_t)wave * W4_DUMP_WAVE_BYTES + (uint32_t)(r16 * W4_DUMP_PITCH + g16 * 16);

#define GCMI_W4_OPERANDS                                                                                              \
  : "+{s[40:41]}"(a_ptr), "+{s[42:43]}"(b_ptr), "+{s46}"(trips)                                                       \
  : "{v[0:3]}"(a_off), "{v[4:7]}"(b_off), "{v[8:9]}"(a_ld), "{v[10:17]}"(b_ld0), "{v[18:25]}"(b_ld2),                \
    "{s[44:45]}"(b_step), "{s47}"(dma_lds), "{s48}"(a_xor), "{v26}"(dump_ld)                                        \
  : "memory", "scc", "s49", GCMI_W4_CLOBBERS
#ifdef GCMI_W4_TIMING // measurement builds: core clock cycles and 100 MHz ticks spent in the main loop
  const long long tick0 = clock64(), wall0 = wall_clock64();
#endif
  if constexpr (ES == 1)
    asm volatile(GCMI_W4_ASM_I8 GCMI_W4_OPERANDS);
  else if constexpr (TB)
    asm volatile(GCMI_W4_ASM_BF16_TB GCMI_W4_OPERANDS);
  else
    asm volatile(GCMI_W4_ASM_BF16 GCMI_W4_OPERANDS);
#undef GCMI_W4_OPERANDS
#ifdef GCMI_W4_TIMING
  const long long tick1 = clock64(), wall1 = wall_clock64();
#endif
  // the column parameters were requested before the main loop and are first needed here
  colp[tid] = cp_bias;
  colp[G_BN + tid] = cp_scale;
  reinterpret_cast<int *>(colp)[2 * G_BN + tid] = cp_cs;
  __syncthreads();

  const int out_kind = p.out_dt == DT_BF16 ? 0 : ((ES == 1 && p.out_dt == DT_S32) ? 2 : 1);
  const int kind = (out_kind == 2 ? (int)ACT_NONE : p.act) + 8 * out_kind;
  const char *dump = smem + wave * W4_DUMP_WAVE_BYTES;
  // a tile that sticks out of C takes the same code with every row and lane tested against the edge
  const int rows_c = (int)min((int64_t)G_BM, p.M - m0), cols_c = (int)min((int64_t)G_BN, p.N - n0);
  const bool edge_tile = rows_c < G_BM || cols_c < G_BN; // the same for the whole workgroup
  if (edge_tile)
    w4_epilogue_half_any<ES, true>(p, kind, 0, m0, n0, wm, wn, lane, dump, colp, rows_c, cols_c);
  else
    w4_epilogue_half_any<ES, false>(p, kind, 0, m0, n0, wm, wn, lane, dump, colp, G_BM, G_BN);
  // the right half: the accumulators of column tiles 4-7 are still where the main loop left them
  asm volatile(GCMI_W4_ASM_DUMP_HI : : "{v26}"(dump_ld) : "memory");
  if (edge_tile)
    w4_epilogue_half_any<ES, true>(p, kind, 1, m0, n0, wm, wn, lane, dump, colp, rows_c, cols_c);
  else
    w4_epilogue_half_any<ES, false>(p, kind, 1, m0, n0, wm, wn, lane, dump, colp, G_BM, G_BN);
#ifdef GCMI_W4_TIMING
  const long long wall_issued = wall_clock64();
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if (timing_out && tid == 0 && blockIdx.x < 256) {
    long long *t = reinterpret_cast<long long *>(timing_out) + 8 * blockIdx.x;
    t[0] = tick1 - tick0, t[1] = wall1 - wall0, t[2] = wall0 - wall_entry, t[3] = wall_issued - wall1, t[4] = wall_clock64() - wall_issued;
    t[5] = wall_entry;
  }
#endif
}

#include "gemm_tile128.hpp"

// Second pass of split-K: out = epilogue(sum over slices of the f32 partials), slices added in ascending
// order (deterministic), the same rounding points as the fused epilogue.  One thread per 4 columns; the
// loads of eight slices are in flight together.
template <int ACT> __global__ __launch_bounds__(256) void gemm_splitk_reduce_kernel(GemmParams p) {
  const int64_t n4 = p.N / 4, idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= p.M * n4)
    return;
  const int64_t m = idx / n4, n = (idx % n4) * 4, sl = p.M * p.N;
  const float *src = p.partial + m * p.N + n;
  f32x4_t a = {0.f, 0.f, 0.f, 0.f};
  for (int s0 = 0; s0 < p.splits; s0 += 8) {
    f32x4_t b[8];
#pragma unroll
    for (int u = 0; u < 8; u++)
      b[u] = s0 + u < p.splits ? *reinterpret_cast<const f32x4_t *>(src + (s0 + u) * sl) : f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < 8; u++)
      if (s0 + u < p.splits) {
        if (s0 + u == 0)
          a = b[u];
        else
          a[0] += b[u][0], a[1] += b[u][1], a[2] += b[u][2], a[3] += b[u][3];
      }
  }
  float bias4[4] = {0.f, 0.f, 0.f, 0.f};
  if (p.bias) {
#pragma unroll
    for (int e = 0; e < 4; e++)
      bias4[e] = p.bias_dt == DT_BF16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t *>(p.bias)[n + e])
                                      : reinterpret_cast<const float *>(p.bias)[n + e];
  }
  uint16_t o16[4];
  float o32[4];
#pragma unroll
  for (int e = 0; e < 4; e++) {
    float x = a[e], r = 0.0f;
    if (p.residual)
      r = p.residual_dt == DT_BF16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t *>(p.residual)[m * p.ldr + n + e])
                                   : reinterpret_cast<const float *>(p.residual)[m * p.ldr + n + e];
    if (p.out_dt == DT_BF16) { // bf16 graph: round after the matmul and after every bf16 op
      x = round_bf16(x);
      if (p.bias)
        x = round_bf16(x + bias4[e]);
      if (ACT != ACT_NONE)
        x = round_bf16(act_const<ACT>(x));
      if (p.residual)
        x = round_bf16(x + r);
    } else {
      if (p.bias)
        x = x + bias4[e];
      x = act_const<ACT>(x);
      if (p.residual) { // kept apart from the activation's last multiply: the sum equals a separate add
#pragma clang fp contract(off)
        x = x + r;
      }
    }
    o32[e] = x;
    o16[e] = f32_to_bf16_bits(x);
  }
  if (p.out_dt == DT_BF16)
    *reinterpret_cast<uint2 *>(reinterpret_cast<uint16_t *>(p.C) + m * p.ldc + n) =
        make_uint2(o16[0] | ((uint32_t)o16[1] << 16), o16[2] | ((uint32_t)o16[3] << 16));
  else
    *reinterpret_cast<f32x4_t *>(reinterpret_cast<float *>(p.C) + m * p.ldc + n) = f32x4_t{o32[0], o32[1], o32[2], o32[3]};
}

// second pass of every K-sliced GEMM: one thread per four outputs, the activation as a template argument
static void launch_splitk_reduce(const GemmParams &p, hipStream_t stream) {
  const dim3 grid((unsigned)((p.M * (p.N / 4) + 255) / 256)), block(256);
  switch (p.act) {
  case ACT_RELU:
    hipLaunchKernelGGL(gemm_splitk_reduce_kernel<ACT_RELU>, grid, block, 0, stream, p);
    break;
  case ACT_GELU_ERF:
    hipLaunchKernelGGL(gemm_splitk_reduce_kernel<ACT_GELU_ERF>, grid, block, 0, stream, p);
    break;
  case ACT_GELU_TANH:
    hipLaunchKernelGGL(gemm_splitk_reduce_kernel<ACT_GELU_TANH>, grid, block, 0, stream, p);
    break;
  case ACT_SIGMOID:
    hipLaunchKernelGGL(gemm_splitk_reduce_kernel<ACT_SIGMOID>, grid, block, 0, stream, p);
    break;
  default:
    hipLaunchKernelGGL(gemm_splitk_reduce_kernel<ACT_NONE>, grid, block, 0, stream, p);
    break;
  }
}

// Host-side launch of the 256x256 tile kernels for one element size.
// want != null: nothing is launched; *want receives the floats of workspace this call would use if it had them.
// cfg != null: receives what was (or would be) chosen.
// Estimates behind the choice of tile and K slices for bf16 problems that do not fill the GPU with 256 x 256 tiles,
// in microseconds, fitted to graph-replayed timings on a 256-CU board (load = workgroups / compute units).  One ring
// group = 128 elements of K.  The rates grow with the load because the board lowers its clock as more of it works.
static inline double gcmi_us_per_group_256(double load) { // one workgroup per compute unit
  if (load <= 0.25)
    return 1.94;
  if (load <= 0.5)
    return 1.94 + 0.16 * (load - 0.25) / 0.25;
  if (load <= 1.0)
    return 2.1 + 0.65 * (load - 0.5) / 0.5;
  return 2.75;
}
static inline double gcmi_us_per_group_128(double load) { // up to two workgroups per compute unit
  if (load <= 0.25)
    return 0.85;
  if (load <= 1.0)
    return 0.85 + 0.27 * (load - 0.25) / 0.75;
  if (load <= 2.0) // as soon as some compute units hold two workgroups, those set the pace
    return 1.9 + 0.27 * (load - 1.0);
  return 2.17;
}
static constexpr double GCMI_US_FIXED_256 = 8.0, GCMI_US_FIXED_128 = 3.7; // launch, ring fill, epilogue
static constexpr double GCMI_US_SECOND_PASS = 3.0;     // the second kernel of a K-sliced product
static constexpr double GCMI_US_PER_SLICE_MOUT = 1.7;  // partial sums written and read back, per slice and 2^20 outputs
static constexpr double GCMI_ONE_PASS_MARGIN = 0.9;    // slices must win by this factor
enum GemmPlan { PLAN_TILE256 = 0, PLAN_TILE128, PLAN_SLICES_SHORT_A, PLAN_SLICES_TILE256, PLAN_SLICES_TILE128 };
template <int ES>
static int launch_tile256(const GemmParams *pp, hipStream_t stream, int64_t *want = nullptr, GemmTileConfig *cfg = nullptr) {
  GemmParams p = *pp;
  if (want)
    *want = 0;
  const bool dry = want != nullptr || (cfg != nullptr && stream == (hipStream_t)-1);
  const int64_t ws_cap = want ? INT64_MAX : (p.partial ? p.partial_cap : 0);
  float *const ws = p.partial;
  const int tiles_m = (int)((p.M + G_BM - 1) / G_BM), tiles_n = (int)((p.N + G_BN - 1) / G_BN);
  const int64_t nblk = (int64_t)tiles_m * tiles_n;
  if (nblk <= 0 || nblk > 0x7fffffff)
    return 2;
  const int out_es = p.out_dt == DT_BF16 ? 2 : 4;
  auto al16 = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  const int BK = G_KBYTES / ES;
  // fast path: whole tiles, 16-byte aligned rows, and a tile's rows reachable with 32-bit byte offsets
  const int KGROUP = 256 / ES; // K elements of one trip round the LDS ring
  const int res_es = p.residual_dt == DT_BF16 ? 2 : 4;
  // the kernels for whole tiles read four residual elements with one load
  const bool res_vec = !p.residual || (al16(p.residual) && (p.ldr * res_es) % 16 == 0);
  const bool aligned = p.K % KGROUP == 0 && p.K > 0 && al16(p.A) && al16(p.B) && al16(p.C) && res_vec &&
                       (p.lda * ES) % 16 == 0 && (p.ldb * ES) % 16 == 0 && (p.ldc * out_es) % 16 == 0 &&
                       p.lda * ES * G_BM < (int64_t)1 << 31 && p.ldb * ES * (p.trans_b ? G_BN : BK) < (int64_t)1 << 31;
  const bool fast_but_m = aligned && p.N % G_BN == 0;
  if (p.trans_b && ES != 2)
    return 3;
  if (p.residual && (ES != 2 || (p.residual_dt != DT_BF16 && p.residual_dt != DT_F32) || p.out_dt == DT_S32))
    return 3;
  bool fast = fast_but_m && p.M % G_BM == 0;
  p.splits = 0;
  p.partial = nullptr;
  const int64_t nbatch = p.batch > 1 ? p.batch : 1;
  if (nbatch > 65535)
    return 2;
  if (nbatch == 1)
    p.a_bs = p.b_bs = p.c_bs = 0;
  else if (!((p.a_bs * ES) % 16 == 0 && (p.b_bs * ES) % 16 == 0 && (p.c_bs * out_es) % 16 == 0 &&
             (!p.residual || (p.c_bs * res_es) % 16 == 0)))
    fast = false; // every batch's operands must keep the alignment the fast path loads with
  // Any M, N a whole number of 16-byte chunks: the 4-wave kernel still takes it; its edge tiles clamp their loads
  // and store what lies inside C.
  const bool ragged = !fast && aligned && p.N % (16 / ES) == 0 && (p.M % G_BM != 0 || p.N % G_BN != 0) &&
                      (nbatch == 1 || ((p.a_bs * ES) % 16 == 0 && (p.b_bs * ES) % 16 == 0 && (p.c_bs * out_es) % 16 == 0 &&
                                       (!p.residual || (p.c_bs * res_es) % 16 == 0)));
  if (p.group_m <= 0)
    p.group_m = 4;
  GemmTileConfig c{};
  c.bm = G_BM, c.bn = G_BN, c.split_k = 1, c.group_m = p.group_m, c.workgroups = (int32_t)nblk;
  c.from_attrs = (p.cfg_waves || p.cfg_split_k || p.cfg_tile == 256) ? 1 : 0;

  // What runs.  bf16 problems that fill the GPU with 256 x 256 tiles take those; smaller ones are given to more
  // workgroups, either by 128 x 128 tiles (two workgroups per compute unit: four times the workgroups), or by cutting
  // K into slices (one workgroup per tile and slice; f32 partial sums through the workspace and a small second
  // kernel; the slice count plays the part of the reference's KThreads, lib/gc/Analysis/MatmulConfigAnalysis.cpp:149-166),
  // or both; the estimates above decide.  A short A (M <= 128: decode-style shapes such as 32 x 4096 x 4096, whose
  // weights have to stream from HBM through all compute units) keeps the kernel that skips the empty 32-row blocks
  // of its tile and takes slices of unequal length, unless the 128 x 128 tiles are estimated faster (from 32 rows
  // on they are).  The 128 x 128 kernel cuts K itself (blockIdx.y = slice, whole ring groups, lengths differing by at
  // most one); the 256 x 256 kernel runs equal slices as a strided batch: batch = K slice, results f32 with
  // c_bs = M * N.  A caller's MatmulConfig replaces the choice.
  const bool batch_ok = nbatch == 1 || ((p.a_bs * ES) % 16 == 0 && (p.b_bs * ES) % 16 == 0 && (p.c_bs * out_es) % 16 == 0 &&
                                        (!p.residual || (p.c_bs * res_es) % 16 == 0));
  const bool t128_can = aligned && p.N % (16 / ES) == 0 && (ES == 2 ? p.out_dt != DT_S32 : !p.trans_b) && batch_ok;
  const bool slices_can = ES == 2 && fast_but_m && p.out_dt != DT_S32 && nbatch == 1; // the 256-wide kernels: whole column tiles
  const int64_t nblk128 = ((p.M + 127) / 128) * ((p.N + 127) / 128);
  const int n_cu = gcmi_num_cus();
  const int groups = (int)(p.K / KGROUP);
  int plan = PLAN_TILE256, splits = 1;
  if (p.cfg_tile == 128) {
    if (t128_can && nblk128 <= 0x7fffffff)
      plan = PLAN_TILE128, c.from_attrs = 1;
  } else if (p.cfg_tile == 256) {
    if (slices_can && p.cfg_split_k > 1) {
      splits = p.cfg_split_k < groups ? p.cfg_split_k : groups;
      plan = p.M > 128 && groups % splits == 0 ? PLAN_SLICES_TILE256 : PLAN_SLICES_SHORT_A;
    }
  } else if (aligned && nblk * nbatch < n_cu) { // (8-bit operands: the small tile in one pass is the only alternative)
    const double mn = (double)p.M * (double)p.N / 1048576.0;
    const double w256 = (double)(nblk * nbatch) / n_cu, w128 = (double)(nblk128 * nbatch) / n_cu;
    double best = GCMI_US_FIXED_256 + gcmi_us_per_group_256(w256) * groups; // one pass, less than one round
    const bool small_tile = p.M >= 32 && t128_can; // shorter: most of a 128-row tile would be padding
    if (small_tile) {
      const double t = GCMI_US_FIXED_128 + gcmi_us_per_group_128(w128) * groups * (double)((nblk128 * nbatch + 2 * n_cu - 1) / (2 * n_cu));
      if (t < best)
        best = t, plan = PLAN_TILE128;
    }
    best *= GCMI_ONE_PASS_MARGIN;
    if (ES == 2 && nbatch == 1 && (small_tile || p.M > 128)) {
      for (int s = 2; s <= groups; s++) {
        const double through_memory = GCMI_US_SECOND_PASS + GCMI_US_PER_SLICE_MOUT * s * mn;
        if (slices_can && p.M > 128 && groups % s == 0 && nblk * s <= n_cu) {
          const double t = GCMI_US_FIXED_256 + gcmi_us_per_group_256(w256 * s) * (groups / s) + through_memory;
          if (t < best)
            best = t, plan = PLAN_SLICES_TILE256, splits = s;
        }
        if (small_tile && nblk128 * s <= 2 * n_cu) {
          const double t = GCMI_US_FIXED_128 + gcmi_us_per_group_128(w128 * s) * ((groups + s - 1) / s) + through_memory;
          if (t < best)
            best = t, plan = PLAN_SLICES_TILE128, splits = s;
        }
      }
    }
    if (nbatch == 1 && p.M <= 128 && slices_can && nblk * 2 <= n_cu) { // a short A: 1.35 (32 rows) to 2 us (128) per group
      const double per_group = 1.35 + 0.65 * (double)((p.M + 31) / 32 - 1) / 3.0;
      const int smax = n_cu / (int)nblk < groups ? n_cu / (int)nblk : groups;
      for (int s = 2; s <= smax; s++) {
        const double t = 7.0 + per_group * ((groups + s - 1) / s) + GCMI_US_PER_SLICE_MOUT * s * mn;
        if (t < best)
          best = t, plan = PLAN_SLICES_SHORT_A, splits = s;
      }
    }
  }
  if (splits > 1) {
    if (want)
      *want = (int64_t)splits * p.M * p.N;
    // less workspace than that: fewer slices, or none
    while (splits > 1 && ((int64_t)splits * p.M * p.N > ws_cap || (plan == PLAN_SLICES_TILE256 && groups % splits != 0)))
      splits--;
    if (splits == 1)
      plan = plan == PLAN_SLICES_TILE128 ? PLAN_TILE128 : PLAN_TILE256;
  }
  if (want && !cfg)
    return 0;
  if (splits > 1) {
    const bool by128 = plan == PLAN_SLICES_TILE128, by256 = plan == PLAN_SLICES_TILE256;
    const int tiles = (int)(by128 ? nblk128 : nblk);
    c.kernel = GK_SPLITK, c.split_k = splits, c.workgroups = tiles * splits;
    if (by128) {
      c.bm = c.bn = 128, c.kbytes = T128_KB, c.stages = T128_NST;
      c.waves_m = c.waves_n = 2, c.wave_m = c.wave_n = 64, c.mfma_m = c.mfma_n = 16, c.mfma_k = 32;
    } else if (by256) {
      c.kbytes = 64, c.stages = 4, c.waves_m = 2, c.waves_n = 2, c.wave_m = 128, c.wave_n = 128;
      c.mfma_m = c.mfma_n = 16, c.mfma_k = 64 / ES;
    } else {
      c.kbytes = FastGemm<ES, G_FAST_KS, G_FAST_WJ, true>::KB, c.stages = FastGemm<ES, G_FAST_KS, G_FAST_WJ, true>::NST;
      c.waves_m = 2, c.waves_n = 8 / G_FAST_WJ, c.wave_m = 128, c.wave_n = 32 * G_FAST_WJ;
      c.mfma_m = c.mfma_n = 32, c.mfma_k = 32 / ES;
    }
    if (cfg)
      *cfg = c;
    if (dry)
      return 0;
    p.splits = splits;
    p.partial = ws;
    if constexpr (ES == 2) {
      if (by128) { // the kernel cuts K itself: blockIdx.y = slice
        const dim3 grid((unsigned)tiles, (unsigned)splits);
        if (p.trans_b)
          hipLaunchKernelGGL(gemm_tile128_kernel<true>, grid, dim3(256), 0, stream, p);
        else
          hipLaunchKernelGGL(gemm_tile128_kernel<false>, grid, dim3(256), 0, stream, p);
      } else if (by256) { // equal slices as a strided batch with f32 results
        GemmParams q = p;
        q.K = p.K / splits, q.batch = splits;
        q.a_bs = q.K, q.b_bs = p.trans_b ? q.K : q.K * p.ldb, q.c_bs = p.M * p.N;
        q.C = ws, q.ldc = p.N, q.out_dt = DT_F32;
        q.bias = nullptr, q.act = ACT_NONE, q.residual = nullptr, q.partial = nullptr, q.splits = 0;
        const dim3 grid((unsigned)tiles, (unsigned)splits);
        if (p.trans_b)
          hipLaunchKernelGGL((gemm_tile256_w4_kernel<ES, true>), grid, dim3(256), 0, stream, q);
        else
          hipLaunchKernelGGL(gemm_tile256_w4_kernel<ES>, grid, dim3(256), 0, stream, q);
      } else if (p.trans_b)
        hipLaunchKernelGGL((gemm_tile256_fast_kernel<ES, G_FAST_KS, G_FAST_WJ, true, true>),
                           dim3((unsigned)(tiles * splits)), dim3(1024 / G_FAST_WJ), 0, stream, p);
      else
        hipLaunchKernelGGL((gemm_tile256_fast_kernel<ES, G_FAST_KS, G_FAST_WJ, true>), dim3((unsigned)(tiles * splits)),
                           dim3(1024 / G_FAST_WJ), 0, stream, p);
    }
    launch_splitk_reduce(p, stream);
    return hipGetLastError() == hipSuccess ? 0 : 5;
  }
  if (plan == PLAN_TILE128) {
    c.kernel = GK_TILE128, c.bm = c.bn = 128, c.kbytes = T128_KB, c.stages = T128_NST;
    c.waves_m = c.waves_n = 2, c.wave_m = c.wave_n = 64, c.mfma_m = c.mfma_n = 16, c.mfma_k = 64 / ES;
    c.workgroups = (int32_t)nblk128;
    if (cfg)
      *cfg = c;
    if (dry)
      return 0;
    const dim3 grid((unsigned)nblk128, (unsigned)nbatch);
    if (p.trans_b) {
      if constexpr (ES == 2)
        hipLaunchKernelGGL((gemm_tile128_kernel<true, 2>), grid, dim3(256), 0, stream, p);
    } else {
      hipLaunchKernelGGL((gemm_tile128_kernel<false, ES>), grid, dim3(256), 0, stream, p);
    }
    return hipGetLastError() == hipSuccess ? 0 : 5;
  }
  // Whole tiles: 4 waves of 128 x 128 unless the caller asks for 8 waves of 128 x 64.  Results of 8-bit operands
  // leave the 4-wave kernel as bf16, f32 or as the raw s32 accumulators (same main loop, the epilogue is a plain
  // store).  Tiles that stick out of C (`ragged`): the 4-wave kernel.  Anything else (a K tail, unaligned rows): the
  // bounds-checked kernel.
  const bool w4_can = fast || ragged;
  const bool use_w4 = w4_can && (p.cfg_waves != 8 || !fast);
  const bool tiled = fast || use_w4; // one of the kernels with the LDS ring
  c.kernel = !tiled ? GK_EDGE : (use_w4 ? GK_WAVES4 : GK_WAVES8);
  c.kbytes = tiled ? 64 : G_KBYTES, c.stages = tiled ? 4 : 2;
  c.waves_m = 2, c.waves_n = use_w4 ? 2 : 4, c.wave_m = 128, c.wave_n = use_w4 ? 128 : 64;
  c.mfma_m = c.mfma_n = tiled ? 16 : 32, c.mfma_k = (tiled ? 64 : 32) / ES;
  // More than a round of whole tiles with a poorly filled last round: the tiles of the last round are a block of
  // columns (or rows) of C; where 128 x 128 tiles are estimated to finish that block clearly sooner than the large
  // ones (up to about 40 % of a round), it becomes a launch of its own behind the whole rounds.  Both kernels add
  // the products of an element in the same order, so C has the same bits either way.
  int64_t tail_cols = 0, tail_rows = 0;
  if (use_w4 && fast && nbatch == 1 && p.cfg_tile == 0 && t128_can && nblk > n_cu && nblk % n_cu != 0) {
    const int64_t tail = nblk % n_cu;
    const double t256 = GCMI_US_FIXED_256 + gcmi_us_per_group_256((double)tail / n_cu) * groups;
    const double t128 = GCMI_US_FIXED_128 + 2.0 + gcmi_us_per_group_128(4.0 * tail / n_cu) * groups * (double)((4 * tail + 2 * n_cu - 1) / (2 * n_cu));
    if (t128 < GCMI_ONE_PASS_MARGIN * t256) {
      if (tail % tiles_m == 0)
        tail_cols = tail / tiles_m * G_BN;
      else if (tail % tiles_n == 0)
        tail_rows = tail / tiles_n * G_BM;
    }
  }
  if (tail_cols || tail_rows)
    c.workgroups = (int32_t)(nblk - nblk % n_cu + 4 * (nblk % n_cu));
  if (cfg)
    *cfg = c;
  if (dry)
    return 0;
  if (tail_cols || tail_rows) {
    GemmParams head = p, rest = p;
    const int bias_es = p.bias_dt == DT_BF16 ? 2 : 4;
    if (tail_cols) {
      const int64_t n1 = p.N - tail_cols;
      head.N = n1, rest.N = tail_cols;
      rest.B = reinterpret_cast<const char *>(p.B) + (p.trans_b ? n1 * p.ldb : n1) * ES;
      rest.C = reinterpret_cast<char *>(p.C) + n1 * out_es;
      if (p.bias)
        rest.bias = reinterpret_cast<const char *>(p.bias) + n1 * bias_es;
      if (p.scale)
        rest.scale = p.scale + n1;
      if (p.colsum)
        rest.colsum = p.colsum + n1;
      if (p.residual)
        rest.residual = reinterpret_cast<const char *>(p.residual) + n1 * res_es;
    } else {
      const int64_t m1 = p.M - tail_rows;
      head.M = m1, rest.M = tail_rows;
      rest.A = reinterpret_cast<const char *>(p.A) + m1 * p.lda * ES;
      rest.C = reinterpret_cast<char *>(p.C) + m1 * p.ldc * out_es;
      if (p.residual)
        rest.residual = reinterpret_cast<const char *>(p.residual) + m1 * p.ldr * res_es;
    }
    const dim3 hgrid((unsigned)(nblk - nblk % n_cu)), tgrid((unsigned)(4 * (nblk % n_cu)));
    if (p.trans_b) {
      if constexpr (ES == 2) {
        hipLaunchKernelGGL((gemm_tile256_w4_kernel<ES, true>), hgrid, dim3(256), 0, stream, head);
        hipLaunchKernelGGL((gemm_tile128_kernel<true, 2>), tgrid, dim3(256), 0, stream, rest);
      }
    } else {
      hipLaunchKernelGGL(gemm_tile256_w4_kernel<ES>, hgrid, dim3(256), 0, stream, head);
      hipLaunchKernelGGL((gemm_tile128_kernel<false, ES>), tgrid, dim3(256), 0, stream, rest);
    }
    return hipGetLastError() == hipSuccess ? 0 : 5;
  }
  dim3 grid((unsigned)nblk, (unsigned)nbatch), block(G_THREADS);
  if (use_w4) {
    if constexpr (ES == 2) {
      if (p.trans_b) {
        hipLaunchKernelGGL((gemm_tile256_w4_kernel<ES, true>), grid, dim3(256), 0, stream, p);
        return hipGetLastError() == hipSuccess ? 0 : 5;
      }
    }
    hipLaunchKernelGGL(gemm_tile256_w4_kernel<ES>, grid, dim3(256), 0, stream, p);
    return hipGetLastError() == hipSuccess ? 0 : 5;
  }
  if constexpr (ES == 2) {
    if (p.trans_b) {
      if (fast)
        hipLaunchKernelGGL((gemm_tile256_mi16_kernel<ES, true>), grid, dim3(512), 0, stream, p);
      else
        hipLaunchKernelGGL((gemm_tile256_kernel<ES, true, true>), grid, block, 0, stream, p);
      return hipGetLastError() == hipSuccess ? 0 : 5;
    }
  }
  if (fast)
    hipLaunchKernelGGL(gemm_tile256_mi16_kernel<ES>, grid, dim3(512), 0, stream, p);
  else
    hipLaunchKernelGGL((gemm_tile256_kernel<ES, true>), grid, block, 0, stream, p);
  return hipGetLastError() == hipSuccess ? 0 : 5;
}

} // namespace gcmi
