// Fused multi-head attention forward for gfx950 (bf16, head_dim 128):
//   O = softmax(Q K^T * scale + mask) V
// i.e. the composition batch_matmul_transpose_b -> scale -> +mask -> softmax ->
// batch_matmul that the reference would run as separate ops
// (lib/gc/Transforms/DecomposeAggregatedOps.cpp:24-38 for the softmax;
// test/benchgc/src/benchgc/linalg/matmul.py:29-32,65-68 for the two batch
// matmuls), computed in one pass with an online softmax so the [Sq,Sk] score
// matrix never leaves registers.
//
// Work split: one workgroup = 128 query rows of one (batch, head); 4 waves x 32
// rows.  Keys/values stream through LDS in blocks of 64 (K 16 KiB + V 16 KiB,
// double buffered = 64 KiB, two workgroups per CU).
//
// Everything is kept TRANSPOSED in the accumulators:
//   S^T[key, q] = K . Q^T      MFMA 32x32x16: first operand = K rows (d is
//                              contiguous in memory -> ds_read_b128), second =
//                              Q rows held in registers for the whole kernel
//   O^T[d, q]  += V^T . P^T    first operand = V^T, read from the row-major V
//                              tile with ds_read_b64_tr_b16; second = P^T taken
//                              straight from the S^T accumulator registers
// In the 32x32 accumulator layout a lane owns ONE query column and 16 of the 32
// keys of a tile, so row max / row sum are in-lane reductions plus a single
// exchange with lane^32, and the softmax weights feed the second MFMA without
// any cross-lane movement: the contraction index of that MFMA is simply
// enumerated in the order the accumulator registers hold the keys
// (lane half h, register e -> key 16*j + 8*(e/4) + 4*h + e%4), and the V^T
// fragment is fetched in the same order.
//
// Workgroup order: query block is the fast index, (batch, head) the slow one.
// Consecutive workgroup ids go to different XCDs, so XCD x only ever touches
// the mask rows of query blocks congruent to x mod 8: a few MiB that stay
// resident in its L2 while K/V of successive heads stream through.
#include "common.hpp"
#include "gemm_params.h"

namespace gcmi {

static constexpr int FA_BQ = 128, FA_BK = 64, FA_D = 128, FA_THREADS = 256;
static constexpr int FA_TILE_BYTES = FA_BK * FA_D * 2; // 16 KiB

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  f32x2_t v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

template <bool HAS_MASK, bool EDGE> __global__ __launch_bounds__(FA_THREADS, 2) void mha_fwd_kernel(MhaParams p) {
  __shared__ __align__(16) char smem[2][2][FA_TILE_BYTES]; // [stage][0=K,1=V]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, lh = lane >> 5;
  const int nqb = (p.Sq + FA_BQ - 1) / FA_BQ;
  const int qb = blockIdx.x % nqb, bh = blockIdx.x / nqb;
  const int q_lane = qb * FA_BQ + wave * 32 + l32; // the query row this lane owns
  const bool q_ok = !EDGE || q_lane < p.Sq;

  const char *Qb = reinterpret_cast<const char *>(p.Q) + (int64_t)bh * p.Sq * FA_D * 2;
  const char *Kb = reinterpret_cast<const char *>(p.K) + (int64_t)bh * p.Sk * FA_D * 2;
  const char *Vb = reinterpret_cast<const char *>(p.V) + (int64_t)bh * p.Sk * FA_D * 2;

  // Q^T fragments (second MFMA operand): lane = query, 8 consecutive d per 16-step
  uint4 qf[8];
#pragma unroll
  for (int ds = 0; ds < 8; ds++)
    qf[ds] = q_ok ? *reinterpret_cast<const uint4 *>(Qb + (int64_t)q_lane * FA_D * 2 + ds * 32 + lh * 16)
                  : make_uint4(0, 0, 0, 0);

  // global -> LDS staging: 4 chunks of K and 4 of V per thread per block
  const int st_key0 = tid >> 4, st_c = tid & 15; // keys st_key0 + 16*i
  uint32_t k_st[4], v_st[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    int key = st_key0 + 16 * i;
    k_st[i] = key * 256 + ((st_c ^ (key & 15)) << 4);
    v_st[i] = key * 256 + ((st_c ^ ((key & 3) << 2)) << 4);
  }
  // LDS fragment offsets
  uint32_t k_ld[8]; // + kt*8192
#pragma unroll
  for (int ds = 0; ds < 8; ds++)
    k_ld[ds] = l32 * 256 + (((ds * 2 + lh) ^ (l32 & 15)) << 4);
  uint32_t v_ld[4]; // + (kt*32 + 16*h2 + 8*rd)*256
  {
    const int g = lane >> 4, i16 = lane & 15, kk = i16 >> 2, cc = i16 & 3;
#pragma unroll
    for (int dt = 0; dt < 4; dt++)
      v_ld[dt] = (4 * lh + kk) * 256 + (((dt * 4 + 2 * (g & 1) + (cc >> 1)) ^ (kk << 2)) << 4) + (cc & 1) * 8;
  }

  f32x16_t o[4];
#pragma unroll
  for (int dt = 0; dt < 4; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++)
      o[dt][r] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;

  const float LOG2E = 1.4426950408889634f;
  const float sl2 = p.scale * LOG2E;
  const int nkb = (p.Sk + FA_BK - 1) / FA_BK;
  uint4 rk[4], rv[4];

  auto gload = [&](int kb) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      int key = kb * FA_BK + st_key0 + 16 * i;
      if (!EDGE || key < p.Sk) {
        rk[i] = *reinterpret_cast<const uint4 *>(Kb + (int64_t)key * FA_D * 2 + st_c * 16);
        rv[i] = *reinterpret_cast<const uint4 *>(Vb + (int64_t)key * FA_D * 2 + st_c * 16);
      } else {
        rk[i] = make_uint4(0, 0, 0, 0);
        rv[i] = make_uint4(0, 0, 0, 0);
      }
    }
  };
  auto lstore = [&](int stage) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      *reinterpret_cast<uint4 *>(&smem[stage][0][k_st[i]]) = rk[i];
      *reinterpret_cast<uint4 *>(&smem[stage][1][v_st[i]]) = rv[i];
    }
  };

  gload(0);
  lstore(0);
  __syncthreads();

  for (int kb = 0; kb < nkb; kb++) {
    const int cur = kb & 1;
    if (kb + 1 < nkb)
      gload(kb + 1);
    const char *sK = &smem[cur][0][0];
    const char *sV = &smem[cur][1][0];

    // ---- S^T = K . Q^T for 64 keys x 32 queries
    f32x16_t s[2];
#pragma unroll
    for (int kt = 0; kt < 2; kt++) {
#pragma unroll
      for (int r = 0; r < 16; r++)
        s[kt][r] = 0.0f;
#pragma unroll
      for (int ds = 0; ds < 8; ds++) {
        uint4 kf = *reinterpret_cast<const uint4 *>(sK + k_ld[ds] + kt * 8192);
        s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, kf),
                                                        __builtin_bit_cast(bf16x8_t, qf[ds]), s[kt], 0, 0, 0);
      }
    }

    // ---- scale, additive mask, to log2 domain; block max
    float m_blk = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < 2; kt++) {
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) {
        const int key = kb * FA_BK + kt * 32 + 8 * q4 + 4 * lh;
        float mk[4] = {0.f, 0.f, 0.f, 0.f};
        if (HAS_MASK) {
          if (!EDGE) {
            f32x4_t mv = *reinterpret_cast<const f32x4_t *>(p.mask + (int64_t)q_lane * p.mask_ld + key);
            mk[0] = mv[0];
            mk[1] = mv[1];
            mk[2] = mv[2];
            mk[3] = mv[3];
          } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
              mk[e] = (q_ok && key + e < p.Sk) ? p.mask[(int64_t)q_lane * p.mask_ld + key + e] : 0.0f;
          }
        }
#pragma unroll
        for (int e = 0; e < 4; e++) {
          float v = s[kt][4 * q4 + e] * sl2;
          if (HAS_MASK)
            v = v + mk[e] * LOG2E;
          if (EDGE && key + e >= p.Sk)
            v = -INFINITY;
          s[kt][4 * q4 + e] = v;
          m_blk = fmaxf(m_blk, v);
        }
      }
    }
    m_blk = fmaxf(m_blk, __shfl_xor(m_blk, 32));

    // ---- online softmax update
    const float m_new = fmaxf(m_run, m_blk);
    const float m_use = (m_new == -INFINITY) ? 0.0f : m_new; // fully masked so far: keep exp2 finite
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
    m_run = m_new;
    float l_blk = 0.0f;
    uint32_t pk[2][8]; // bf16 pairs: pk[kt][e2] = (p[2*e2], p[2*e2+1])
#pragma unroll
    for (int kt = 0; kt < 2; kt++) {
#pragma unroll
      for (int r = 0; r < 16; r += 2) {
        float p0 = __builtin_amdgcn_exp2f(s[kt][r] - m_use);
        float p1 = __builtin_amdgcn_exp2f(s[kt][r + 1] - m_use);
        l_blk += p0 + p1;
        pk[kt][r >> 1] = pack_bf16x2(p0, p1);
      }
    }
    l_run = l_run * alpha + l_blk;
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int dt = 0; dt < 4; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++)
          o[dt][r] *= alpha;
    }

    // ---- O^T += V^T . P^T
#pragma unroll
    for (int kt = 0; kt < 2; kt++) {
#pragma unroll
      for (int h2 = 0; h2 < 2; h2++) {
        uint4 pf = make_uint4(pk[kt][4 * h2 + 0], pk[kt][4 * h2 + 1], pk[kt][4 * h2 + 2], pk[kt][4 * h2 + 3]);
#pragma unroll
        for (int dt = 0; dt < 4; dt++) {
          const char *vp = sV + v_ld[dt] + (kt * 32 + 16 * h2) * 256;
          bf16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((GCMI_LDS bf16x4_t *)vp);
          bf16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((GCMI_LDS bf16x4_t *)(vp + 8 * 256));
          uint2 lo2 = __builtin_bit_cast(uint2, lo), hi2 = __builtin_bit_cast(uint2, hi);
          uint4 vf = make_uint4(lo2.x, lo2.y, hi2.x, hi2.y);
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, vf),
                                                          __builtin_bit_cast(bf16x8_t, pf), o[dt], 0, 0, 0);
        }
      }
    }

    if (kb + 1 < nkb)
      lstore(cur ^ 1);
    __syncthreads();
  }

  // ---- normalise and store: lane owns query q_lane, d = dt*32 + 8*q4 + 4*lh + e
  const float l_tot = l_run + __shfl_xor(l_run, 32);
  const float inv = 1.0f / l_tot; // l_tot == 0 (row fully masked): 0 * inf = NaN, as softmax of all -inf
  if (q_ok) {
    char *Ob = reinterpret_cast<char *>(p.O) + ((int64_t)bh * p.Sq + q_lane) * FA_D * 2;
#pragma unroll
    for (int dt = 0; dt < 4; dt++)
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) {
        uint16_t h[4];
#pragma unroll
        for (int e = 0; e < 4; e++)
          h[e] = f32_to_bf16_bits(o[dt][4 * q4 + e] * inv);
        *reinterpret_cast<uint2 *>(Ob + (dt * 32 + 8 * q4 + 4 * lh) * 2) =
            make_uint2(h[0] | ((uint32_t)h[1] << 16), h[2] | ((uint32_t)h[3] << 16));
      }
  }
}

// ---------------------------------------------------------------------------
// Fast path (Sq % 128 == 0, Sk % 64 == 0, aligned): same tiling and register
// layout as above, restructured so that a wave never waits on memory inside an
// iteration:
//  * K/V blocks go global -> LDS with global_load_lds_dwordx4 (1 KiB per wave
//    instruction, swizzle applied on the global side), block kb+1 in flight
//    while block kb is computed; no staging registers, no ds_write.
//  * the additive mask tile of block kb+1 is loaded into registers while block
//    kb is computed (the loop is unrolled by two so the two register sets swap
//    roles without moves).
//  * S^T MFMAs alternate between the two 32-key tiles (independent
//    accumulators) with the K-fragment reads interleaved 1:1; the V^T
//    fragment reads are interleaved 2:1 with the PV MFMAs.
//  * softmax runs in the natural-log domain until the exponent:
//    t = s*scale + mask (one FMA), p = exp2(t*log2e - m*log2e) (one FMA + exp).
#define GCMI_GLB __attribute__((address_space(1)))

// Mask tile classes, found by one pass over the mask before the main kernel:
// a tile that is constant 0 or constant -inf needs no mask traffic in the main
// loop (the constant is put into the mask registers instead), and a -inf tile
// may be skipped altogether: it contributes exp(-inf) = 0 to every sum and
// leaves the running maximum unchanged.
enum : uint8_t { FA_TILE_GENERAL = 0, FA_TILE_ZERO = 1, FA_TILE_NEG_INF = 2 };
// The classes live in a buffer the caller brings (MhaParams::tile_class, one byte per tile); without one every tile
// is read from the mask and nothing is skipped.
static constexpr int FA_MAX_TILES = 1 << 20;

__global__ __launch_bounds__(64) void mha_classify_mask_kernel(const float *mask, int64_t mask_ld, int n_kb, uint8_t *cls) {
  const int qt = blockIdx.y, kb = blockIdx.x, lane = threadIdx.x;
  // 32 rows x 64 floats: lane -> (row = it*4 + lane/16, 16 B chunk lane%16)
  bool all_zero = true, all_ninf = true;
#pragma unroll
  for (int it = 0; it < 8; it++) {
    f32x4_t v = *reinterpret_cast<const f32x4_t *>(mask + (int64_t)(qt * 32 + it * 4 + (lane >> 4)) * mask_ld + kb * 64 +
                                                   (lane & 15) * 4);
#pragma unroll
    for (int e = 0; e < 4; e++) {
      all_zero = all_zero && (__float_as_uint(v[e]) << 1) == 0; // +0 or -0
      all_ninf = all_ninf && v[e] == -INFINITY;
    }
  }
  all_zero = __all(all_zero);
  all_ninf = __all(all_ninf);
  if (lane == 0)
    cls[qt * n_kb + kb] = all_zero ? FA_TILE_ZERO : (all_ninf ? FA_TILE_NEG_INF : FA_TILE_GENERAL);
}

// how far (natural-log units) a block maximum may exceed the softmax reference
// before the reference is moved: p stays below e^5 = 148
constexpr float FA_REF_SLACK = 5.0f;
// K fragment reads kept in flight ahead of the S MFMAs
constexpr int FA_K_AHEAD = 6;
// the set of visited key blocks is kept for up to 64 * FA_MAX_GROUPS blocks (65536 keys)
constexpr int FA_MAX_GROUPS = 16;

// NW waves per workgroup (4 or 8); each takes 32 query rows and 16/NW of the 16 DMA
// instructions that bring a K (or V) tile in.
template <int NW> struct FaFast {
  static constexpr int NDMA = 16 / NW;
  uint32_t k_src[NDMA], v_src[NDMA]; // per-lane global byte offsets of this wave's DMA instructions (within a 64-key block)
  uint32_t k_ld[8], v_ld[4];   // LDS fragment offsets
  int wave_u;

  // One 1 KiB piece: lane l's 16 bytes land at lds_addr + 16*l.  For the three-stage
  // ring (NW == 8) written as inline
  // assembly (M0 = LDS destination, as the instruction wants it) so that these
  // requests stay outside the compiler's own memory-counter bookkeeping: it would
  // otherwise make every later LDS read wait for all of them, and the point is to
  // keep them in flight across one or two key blocks.  The waits are the explicit
  // s_waitcnt vmcnt(..) in the main loop; nothing else in this kernel uses M0.
  static __device__ __forceinline__ void dma_1k(const char *src, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(lds_addr)
                 : "memory", "m0");
  }
  __device__ __forceinline__ void issue_kv(char *__restrict__ stage, const char *kb_ptr, const char *vb_ptr) const {
    if constexpr (NW == 8) {
      const uint32_t base = (uint32_t)(uintptr_t)(GCMI_LDS char *)stage + (uint32_t)(wave_u * NDMA) * 1024u;
#pragma unroll
      for (int i = 0; i < NDMA; i++)
        dma_1k(kb_ptr + k_src[i], base + i * 1024u);
#pragma unroll
      for (int i = 0; i < NDMA; i++)
        dma_1k(vb_ptr + v_src[i], base + FA_TILE_BYTES + i * 1024u);
    } else {
      // two stages, one block ahead: the compiler's own counting is exact enough here,
      // and it may spread these requests between the MFMAs
#pragma unroll
      for (int i = 0; i < NDMA; i++)
        __builtin_amdgcn_global_load_lds((GCMI_GLB const void *)(kb_ptr + k_src[i]),
                                         (GCMI_LDS void *)(stage + (wave_u * NDMA + i) * 1024), 16, 0, 0);
#pragma unroll
      for (int i = 0; i < NDMA; i++)
        __builtin_amdgcn_global_load_lds((GCMI_GLB const void *)(vb_ptr + v_src[i]),
                                         (GCMI_LDS void *)(stage + FA_TILE_BYTES + (wave_u * NDMA + i) * 1024), 16, 0, 0);
    }
  }

  // One 64-key block.  kind (wave-uniform): 0 the mask tile adds nothing, 1 read it
  // (mtile: this lane's 8 x 16 B pieces of it), 2 it is -inf throughout.  The mask joins the raw
  // scores as s + mask/scale, so that one code path (maximum of the raw scores,
  // scale folded into the exponent's multiplier) serves both cases; scale > 0.
  template <bool HAS_MASK>
  __device__ __forceinline__ void block(const char *__restrict__ st, const uint4 (&qf)[8], int kind, const float *mtile,
                                        float scale, float inv_scale, f32x16_t (&o)[4], float &m_run,
                                        float &l_run) const {
    const char *sK = st, *sV = st + FA_TILE_BYTES;
    // ---- S^T = K . Q^T, the two key tiles alternate
    f32x16_t s[2];
#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
      for (int r = 0; r < 16; r++)
        s[kt][r] = 0.0f;
#pragma unroll
    for (int ds = 0; ds < 8; ds++) {
#pragma unroll
      for (int kt = 0; kt < 2; kt++) {
        uint4 kf = *reinterpret_cast<const uint4 *>(sK + k_ld[ds] + kt * 8192);
        s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, kf),
                                                        __builtin_bit_cast(bf16x8_t, qf[ds]), s[kt], 0, 0, 0);
      }
    }
    // fragments of V for the first 16 keys are requested here, long before the
    // first PV MFMA needs them
    auto load_v = [&](int chunk, uint4 (&vf)[4]) {
#pragma unroll
      for (int dt = 0; dt < 4; dt++) {
        const char *vp = sV + v_ld[dt] + chunk * 16 * 256;
        bf16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((GCMI_LDS bf16x4_t *)vp);
        bf16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((GCMI_LDS bf16x4_t *)(vp + 8 * 256));
        uint2 lo2 = __builtin_bit_cast(uint2, lo), hi2 = __builtin_bit_cast(uint2, hi);
        vf[dt] = make_uint4(lo2.x, lo2.y, hi2.x, hi2.y);
      }
    };
    uint4 vcur[4];
    load_v(0, vcur);
    // issue order of the S phase: K fragments run FA_K_AHEAD reads ahead of the MFMAs
    __builtin_amdgcn_sched_group_barrier(0x100, FA_K_AHEAD, 0);
#pragma unroll
    for (int i = 0; i < 16 - FA_K_AHEAD; i++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, FA_K_AHEAD, 0);
    __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
    if (HAS_MASK && kind == 2) {
#pragma unroll
      for (int kt = 0; kt < 2; kt++)
#pragma unroll
        for (int r = 0; r < 16; r++)
          s[kt][r] = -INFINITY;
    } else if (HAS_MASK && kind == 1) {
#pragma unroll
      for (int t = 0; t < 8; t++) { // t = kt*4 + q4 -> keys kt*32 + 8*q4 + 4*(lane/32) .. +3
        const f32x4_t mk = *reinterpret_cast<const f32x4_t *>(mtile + (t >> 2) * 32 + (t & 3) * 8);
#pragma unroll
        for (int e = 0; e < 4; e++)
          s[t >> 2][4 * (t & 3) + e] = fmaf(mk[e], inv_scale, s[t >> 2][4 * (t & 3) + e]);
      }
    }
    const float LOG2E = 1.4426950408889634f;
    float m_blk = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
      for (int r = 0; r < 16; r += 2)
        m_blk = fmaxf(fmaxf(m_blk, s[kt][r]), s[kt][r + 1]);
    m_blk *= scale;
    m_blk = fmaxf(m_blk, __shfl_xor(m_blk, 32));
    // ---- online softmax with a lazily moved reference.  m_run is the value
    // subtracted in the exponent; it only moves (and O, l are only rescaled) when
    // the block maximum exceeds it by more than FA_REF_SLACK, so p <= e^FA_REF_SLACK
    // and after the first blocks of a row the rescale branch is hardly taken.
    const bool grow = m_blk > m_run + FA_REF_SLACK;
    if (__any(grow)) {
      const float m_new = grow ? m_blk : m_run;
      const float alpha = grow ? __builtin_amdgcn_exp2f((m_run - m_new) * LOG2E) : 1.0f;
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int dt = 0; dt < 4; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++)
          o[dt][r] *= alpha;
    }
    const float m_use = (m_run == -INFINITY) ? 0.0f : m_run; // fully masked so far: keep exp2 finite
    const float nm = -m_use * LOG2E;
    const float c = scale * LOG2E;
    // ---- p = exp2(t*log2e - m*log2e), O^T += V^T . P^T, 16 keys at a time: the
    // exponentials of one chunk are independent of the MFMAs of the previous one
    float l_blk = 0.0f;
#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
      for (int h2 = 0; h2 < 2; h2++) {
        uint32_t pk[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const int r = 8 * h2 + 2 * j;
          float p0 = __builtin_amdgcn_exp2f(fmaf(s[kt][r], c, nm));
          float p1 = __builtin_amdgcn_exp2f(fmaf(s[kt][r + 1], c, nm));
          l_blk += p0 + p1;
          pk[j] = pack_bf16x2(p0, p1);
        }
        uint4 pf = make_uint4(pk[0], pk[1], pk[2], pk[3]);
        uint4 vnext[4];
        if (kt * 2 + h2 < 3)
          load_v(kt * 2 + h2 + 1, vnext);
#pragma unroll
        for (int dt = 0; dt < 4; dt++)
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, vcur[dt]),
                                                          __builtin_bit_cast(bf16x8_t, pf), o[dt], 0, 0, 0);
        if (kt * 2 + h2 < 3) {
#pragma unroll
          for (int dt = 0; dt < 4; dt++)
            vcur[dt] = vnext[dt];
        }
      }
    l_run += l_blk;
    // issue order for the region above: the first chunk's exponentials, then every
    // MFMA followed by its share of the next chunk's VALU work, so that the vector
    // ALU runs in the shadow of the matrix pipe (0x2 VALU, 0x400 transcendental, 0x8 MFMA)
    __builtin_amdgcn_sched_group_barrier(0x002, 28, 0);
#pragma unroll
    for (int i = 0; i < 12; i++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 7, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
  }
};

// NW = 4: 128 query rows per workgroup, two workgroups per compute unit.
// NW = 8: 256 query rows, one workgroup per compute unit -- every K/V tile then
// serves twice as many rows, which halves the DMA traffic into LDS.
template <bool HAS_MASK, int NW>
__global__ __launch_bounds__(NW * 64, NW == 4 ? 2 : 1) void mha_fwd_fast_kernel(MhaParams p) {
  constexpr int BQ = NW * 32;
  __shared__ __align__(1024) char smem0[2 * FA_TILE_BYTES];
  __shared__ __align__(1024) char smem1[2 * FA_TILE_BYTES];
  // the 8-wave kernel (one workgroup per compute unit) has room for a third stage:
  // the DMA then runs two key blocks ahead
  constexpr int NST = NW == 8 ? 3 : 2;
  __shared__ __align__(1024) char smem2[NST == 3 ? 2 * FA_TILE_BYTES : 1024];
  __shared__ uint64_t s_zero[NW][FA_MAX_GROUPS], s_ninf[NW][FA_MAX_GROUPS]; // per wave and group of 64 key blocks: tile classes
         // per wave: -inf classes of the current group of 64 key blocks
  __shared__ uint64_t s_live[FA_MAX_GROUPS]; // per group of 64 key blocks: the ones the workgroup visits

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, lh = lane >> 5;
  const int nqb = p.Sq / BQ;
  // Workgroup -> (head, query block).  Consecutive workgroup ids are dealt
  // round-robin to the 8 XCDs; all query blocks of one (batch, head) are given to
  // ONE XCD so that its K/V (Sk x 512 B) is fetched once and then served from that
  // XCD's L2.  An XCD works on four heads at a time (4 MiB of K and V at 2048
  // keys) and takes their long (late) query blocks first, so that under a
  // triangular mask with skipping the short blocks fill the gaps at the end.
  int qb, bh;
  if ((p.BH & 7) == 0) {
    const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
    if (((p.BH >> 3) & 3) == 0) {
      const int grp = idx / (4 * nqb), r = idx % (4 * nqb);
      bh = (grp * 4 + (r & 3)) * 8 + xcd;
      qb = nqb - 1 - (r >> 2);
    } else {
      bh = (idx / nqb) * 8 + xcd;
      qb = nqb - 1 - idx % nqb;
    }
  } else {
    qb = nqb - 1 - blockIdx.x % nqb;
    bh = blockIdx.x / nqb;
  }
  const int q_lane = qb * BQ + wave * 32 + l32;

  const char *Qb = reinterpret_cast<const char *>(p.Q) + (int64_t)bh * p.Sq * FA_D * 2;
  const char *Kb = reinterpret_cast<const char *>(p.K) + (int64_t)bh * p.Sk * FA_D * 2;
  const char *Vb = reinterpret_cast<const char *>(p.V) + (int64_t)bh * p.Sk * FA_D * 2;

  uint4 qf[8];
#pragma unroll
  for (int ds = 0; ds < 8; ds++)
    qf[ds] = *reinterpret_cast<const uint4 *>(Qb + (int64_t)q_lane * FA_D * 2 + ds * 32 + lh * 16);

  FaFast<NW> g;
  g.wave_u = wave;
#pragma unroll
  for (int i = 0; i < FaFast<NW>::NDMA; i++) {
    int key = (wave * FaFast<NW>::NDMA + i) * 4 + (lane >> 4), ph = lane & 15;
    g.k_src[i] = (uint32_t)(key * 256 + ((ph ^ (key & 15)) << 4));
    g.v_src[i] = (uint32_t)(key * 256 + ((ph ^ ((key & 3) << 2)) << 4));
  }
#pragma unroll
  for (int ds = 0; ds < 8; ds++)
    g.k_ld[ds] = l32 * 256 + (((ds * 2 + lh) ^ (l32 & 15)) << 4);
  {
    const int gq = lane >> 4, i16 = lane & 15, kk = i16 >> 2, cc = i16 & 3;
#pragma unroll
    for (int dt = 0; dt < 4; dt++)
      g.v_ld[dt] = (4 * lh + kk) * 256 + (((dt * 4 + 2 * (gq & 1) + (cc >> 1)) ^ (kk << 2)) << 4) + (cc & 1) * 8;
  }

  f32x16_t o[4];
#pragma unroll
  for (int dt = 0; dt < 4; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++)
      o[dt][r] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;
  const int nkb = p.Sk / FA_BK;
  const int64_t blk_bytes = (int64_t)FA_BK * FA_D * 2;
  const float *mrow = HAS_MASK ? p.mask + (int64_t)q_lane * p.mask_ld + 4 * lh : nullptr;

  // Classes of this wave's mask tiles, one bit per key block in groups of 64,
  // read from memory once and kept in LDS: the main loop must not issue vector
  // memory loads of its own next to the K/V DMA it counts.
  const bool have_cls = HAS_MASK && p.tile_class && nkb <= 64 * FA_MAX_GROUPS;
  const int n_groups = (nkb + 63) >> 6;
  if (have_cls) {
    const uint8_t *cls_row = p.tile_class + (int64_t)(qb * NW + wave) * nkb;
    for (int group = 0; group < n_groups; group++) {
      uint8_t c = FA_TILE_GENERAL;
      if (group * 64 + lane < nkb)
        c = cls_row[group * 64 + lane];
      const uint64_t zb = __ballot(c == FA_TILE_ZERO), nb = __ballot(c == FA_TILE_NEG_INF);
      if (lane == 0) {
        s_zero[wave][group] = zb;
        s_ninf[wave][group] = nb;
      }
    }
  }
  __syncthreads();
  uint64_t zero_bits = 0, ninf_bits = 0;
  int cls_group = -1;
  auto bcast64 = [](uint64_t v) -> uint64_t {
    // readfirstlane returns int: widen through uint32_t, or bit 31 smears over the upper half
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)v);
    return ((uint64_t)hi << 32) | lo;
  };
  auto load_classes = [&](int group) {
    if (have_cls) {
      zero_bits = bcast64(s_zero[wave][group]);
      ninf_bits = bcast64(s_ninf[wave][group]);
    }
    cls_group = group;
  };
  // Key blocks whose tiles are -inf for all waves of the workgroup are left out: their set is
  // built once (one bit per block), and the main loop walks its bits, so there is
  // no branch around a block.  A wave whose own tile is -inf inside a visited
  // block fills its scores with -inf (every weight comes out 0).
  const bool use_list = have_cls && p.skip_masked;
  int n_live = nkb;
  if (use_list) {
    n_live = 0;
    for (int group = 0; group < n_groups; group++) {
      const int left = nkb - group * 64;
      uint64_t all_ninf = s_ninf[0][group];
#pragma unroll
      for (int w = 1; w < NW; w++)
        all_ninf &= s_ninf[w][group];
      const uint64_t live = bcast64(~all_ninf & (left >= 64 ? ~0ull : ((1ull << left) - 1)));
      if (tid == 0)
        s_live[group] = live;
      n_live += __builtin_popcountll(live);
    }
    __syncthreads();
    n_live = min(n_live, nkb);
  }
  // walks the visited blocks in order (all scalar); called at most n_live times
  int walk_group = -1;
  uint64_t walk_bits = 0;
  auto next_block = [&](int ordinal) -> int {
    if (!use_list)
      return ordinal;
    while (walk_bits == 0 && walk_group + 1 < n_groups) {
      walk_group++;
      walk_bits = bcast64(s_live[walk_group]);
    }
    if (walk_bits == 0)
      return nkb - 1; // not reached: next_block is called once per visited block
    const int kb = walk_group * 64 + __builtin_ctzll(walk_bits);
    walk_bits &= walk_bits - 1;
    return min(kb, nkb - 1); // the set only holds blocks below nkb; the clamp keeps every K/V address in range regardless
  };

  // kb_q[0] is the block being computed, kb_q[1..] the ones already requested
  int kb_q[NST - 1] = {};
  if (n_live > 0) {
    kb_q[0] = next_block(0);
    g.issue_kv(smem0, Kb + kb_q[0] * blk_bytes, Vb + kb_q[0] * blk_bytes);
    if (NST == 3) {
      kb_q[NST - 2] = n_live > 1 ? next_block(1) : kb_q[0];
      g.issue_kv(smem1, Kb + kb_q[NST - 2] * blk_bytes, Vb + kb_q[NST - 2] * blk_bytes);
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * FaFast<NW>::NDMA) : "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __builtin_amdgcn_s_barrier();
  }
  if constexpr (NW == 8) {
    // Make the compiler place its wait for the Q loads here.  Their first readers are the MFMAs inside the loop,
    // and it knows nothing of the hand-written requests above and in the loop: left alone it puts
    // "s_waitcnt vmcnt(7) .. vmcnt(0)" in front of those MFMAs in every trip, which in the real counter means
    // "until the K/V blocks requested a moment ago have landed" and takes the ring's lead away.
#pragma unroll
    for (int ds = 0; ds < 8; ds++) {
      i32x4_t t = {(int)qf[ds].x, (int)qf[ds].y, (int)qf[ds].z, (int)qf[ds].w};
      asm volatile("" : "+v"(t));
      qf[ds] = make_uint4((uint32_t)t[0], (uint32_t)t[1], (uint32_t)t[2], (uint32_t)t[3]);
    }
  }

  const float inv_scale = 1.0f / p.scale;
  // One visited key block: request the block NST-1 ahead into the stage that was
  // computed from last (past the end the last block is fetched again: the order
  // of requests stays unconditional), compute, wait for the next block only.
  auto step = [&](const char *cur, char *fill, int i) {
    const int kb = kb_q[0];
    const int kbf = i + NST - 1 < n_live ? next_block(i + NST - 1) : kb_q[NST - 2];
    if (NST == 3)
      kb_q[0] = kb_q[1];
    kb_q[NST - 2] = kbf;
    if (HAS_MASK && (kb >> 6) != cls_group)
      load_classes(kb >> 6);
    // 0: the tile adds nothing, 1: read it, 2: -inf throughout
    const int kind = !HAS_MASK ? 0 : ((zero_bits >> (kb & 63)) & 1) ? 0 : ((ninf_bits >> (kb & 63)) & 1) ? 2 : 1;
    g.issue_kv(fill, Kb + kbf * blk_bytes, Vb + kbf * blk_bytes);
    g.template block<HAS_MASK>(cur, qf, kind, mrow + kb * FA_BK, p.scale, inv_scale, o, m_run, l_run);
    if (NST == 3)
      asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(2 * FaFast<NW>::NDMA) : "memory");
    else
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
  };
  if (NST == 3) {
    for (int i = 0; i < n_live; i += 3) {
      step(smem0, smem2, i);
      if (i + 1 < n_live)
        step(smem1, smem0, i + 1);
      if (i + 2 < n_live)
        step(smem2, smem1, i + 2);
    }
  } else {
    for (int i = 0; i < n_live; i += 2) {
      step(smem0, smem1, i);
      if (i + 1 < n_live)
        step(smem1, smem0, i + 1);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // requests past the end have landed before the stages go away

  const float l_tot = l_run + __shfl_xor(l_run, 32);
  const float inv = 1.0f / l_tot;
  char *Ob = reinterpret_cast<char *>(p.O) + ((int64_t)bh * p.Sq + q_lane) * FA_D * 2;
#pragma unroll
  for (int dt = 0; dt < 4; dt++)
#pragma unroll
    for (int q4 = 0; q4 < 4; q4++) {
      uint16_t h[4];
#pragma unroll
      for (int e = 0; e < 4; e++)
        h[e] = f32_to_bf16_bits(o[dt][4 * q4 + e] * inv);
      *reinterpret_cast<uint2 *>(Ob + (dt * 32 + 8 * q4 + 4 * lh) * 2) =
          make_uint2(h[0] | ((uint32_t)h[1] << 16), h[2] | ((uint32_t)h[3] << 16));
    }
}

} // namespace gcmi

using namespace gcmi;

// bytes of workspace (MhaParams::tile_class) a masked call of this shape can use; 0: none
extern "C" int64_t gcmi_launch_mha_workspace(const MhaParams *p) {
  if (!p->mask || p->D != FA_D || p->Sq <= 0 || p->Sk <= 0 || p->Sq % FA_BQ != 0 || p->Sk % FA_BK != 0)
    return 0;
  const int64_t n_qt = p->Sq / 32, n_kb = p->Sk / FA_BK;
  return (n_qt * n_kb <= FA_MAX_TILES && n_qt <= 65535) ? n_qt * n_kb : 0;
}

extern "C" int gcmi_launch_mha_fwd(const MhaParams *pp, hipStream_t stream) {
  MhaParams p = *pp;
  if (p.D != FA_D)
    return 3;
  if (p.BH <= 0 || p.Sq <= 0 || p.Sk <= 0)
    return 0;
  int nqb = (p.Sq + FA_BQ - 1) / FA_BQ;
  int64_t nblk = (int64_t)nqb * p.BH;
  if (nblk > 0x7fffffff)
    return 2;
  auto al16 = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  // the fast kernel takes max(s*scale) as scale*max(s): it needs scale > 0
  bool fast = p.scale > 0.0f && p.Sq % FA_BQ == 0 && p.Sk % FA_BK == 0 && al16(p.Q) && al16(p.K) && al16(p.V) && al16(p.O) &&
              (!p.mask || (al16(p.mask) && p.mask_ld % 4 == 0));
  if (!(al16(p.Q) && al16(p.K) && al16(p.V) && al16(p.O)))
    return 2; // rows are 256 bytes: a 16-byte aligned base is required
  uint8_t *const ws = p.tile_class;
  p.tile_class = nullptr;
  if (p.mask && fast && ws) {
    const int64_t n_qt = p.Sq / 32, n_kb = p.Sk / FA_BK;
    if (n_qt * n_kb <= FA_MAX_TILES && n_qt <= 65535 && n_qt * n_kb <= p.tile_class_cap) {
      hipLaunchKernelGGL(mha_classify_mask_kernel, dim3((unsigned)n_kb, (unsigned)n_qt), dim3(64), 0, stream, p.mask,
                         p.mask_ld, (int)n_kb, ws);
      p.tile_class = ws;
    }
  }
  // 256-row workgroups when they still fill the GPU.  Measured at 4 x 32 heads, 2048 x 2048: 2-3 % faster
  // without a mask, slower with a triangular mask (block skipping is coarser, fewer workgroups
  // to even out), so masked calls keep the 128-row kernel.
  const bool wide = fast && !p.mask && p.Sq % 256 == 0 && (int64_t)(p.Sq / 256) * p.BH >= gcmi_num_cus();
  if (wide) {
    nqb = p.Sq / 256;
    nblk = (int64_t)nqb * p.BH;
  }
  dim3 grid((unsigned)nblk), block(wide ? 512 : FA_THREADS);
  if (p.mask) {
    if (wide)
      hipLaunchKernelGGL((mha_fwd_fast_kernel<true, 8>), grid, block, 0, stream, p);
    else if (fast)
      hipLaunchKernelGGL((mha_fwd_fast_kernel<true, 4>), grid, block, 0, stream, p);
    else
      hipLaunchKernelGGL((mha_fwd_kernel<true, true>), grid, block, 0, stream, p);
  } else {
    if (wide)
      hipLaunchKernelGGL((mha_fwd_fast_kernel<false, 8>), grid, block, 0, stream, p);
    else if (fast)
      hipLaunchKernelGGL((mha_fwd_fast_kernel<false, 4>), grid, block, 0, stream, p);
    else
      hipLaunchKernelGGL((mha_fwd_kernel<false, true>), grid, block, 0, stream, p);
  }
  return hipGetLastError() == hipSuccess ? 0 : 5;
}
