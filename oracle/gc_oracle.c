/*
 * gc_oracle.c -- CPU restatement of the reference's contraction hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the GPU path is compared
 * against and the "port" CPU baseline that the benchmark times.  Nothing in the
 * shipped library links, loads or calls it; the product path has no CPU
 * fallback.
 *
 * Every function cites the reference file:line whose arithmetic it restates
 * (paths relative to the reference tree).  Parity status of each function:
 *
 *   gco_f32_to_bf16 / gco_bf16_to_f32   pinned  (bit formula; checked against
 *                                               torch's RNE cast on all 2^16
 *                                               bf16 patterns and random f32)
 *   gco_brgemm                          pinned  (vs the compiled reference
 *                                               BrgemmNaive.cpp in oracle/_ref,
 *                                               committed golden vectors, the
 *                                               closed forms of the lit tests
 *                                               brgemm-simple-for / multilevel,
 *                                               and int64 / f64 textbook GEMM)
 *   gco_vnni_pack                       pinned  (index formula vs the lit shapes
 *                                               and round trip through brgemm)
 *   gco_validate_config                 pinned  (truth table restated from the
 *                                               reference predicate; lit configs)
 *   gco_deep_tile_matmul                pinned  (result independent of config:
 *                                               integer exact vs int64 GEMM for
 *                                               every valid config tried; loop
 *                                               extents vs lit expectations)
 *   gco_bias_add / relu / sigmoid       pinned  (closed forms of TestApiOps)
 *   gco_gelu_erf / gco_gelu_tanh        pinned  (vs torch gelu none / tanh)
 *   gco_dequant_comp                    pinned  (algebraic identity in int64)
 *   gco_softmax_rows / gco_mha          pinned  (vs torch.softmax / composition
 *                                               in f64; row sums; causal and
 *                                               key-permutation invariants)
 *   gco_mha_f64                         pinned  (vs the torch composition in f64;
 *                                               with P rounded it reproduces
 *                                               gco_mha_bf16 up to the final
 *                                               rounding)
 *   gco_compare_p2p / gco_compare_norm  pinned  (hand-computed cases; the strict
 *                                               '<' of the norm rule; empty
 *                                               tensors pass)
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define GCO_API __attribute__((visibility("default")))

/* dnnl_data_type_t values the microkernel ABI uses literally
 * (test/mlir/unittests/ExecutionEngine/BrgemmRuntime.cpp:61-62,117-118). */
enum { GCO_BF16 = 2, GCO_F32 = 3, GCO_S8 = 5, GCO_U8 = 6 };

/* ------------------------------------------------------------------------- */
/* bf16 <-> f32: include/gc/ExecutionEngine/CPURuntime/Microkernel/
 * BrgemmInterface.h:72-76 (widen by <<16) and :83-92 (RNE, NaN -> 0x7FC0).   */
GCO_API uint16_t gco_f32_to_bf16(float v) {
  uint32_t bits;
  memcpy(&bits, &v, 4);
  if (v != v)
    return 0x7FC0u;
  uint32_t bias = ((bits >> 16) & 1u) + 0x7FFFu;
  return (uint16_t)((bits + bias) >> 16);
}

GCO_API float gco_bf16_to_f32(uint16_t h) {
  uint32_t bits = (uint32_t)h << 16;
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

GCO_API void gco_f32_to_bf16_array(const float *src, uint16_t *dst, int64_t n) {
  for (int64_t i = 0; i < n; i++)
    dst[i] = gco_f32_to_bf16(src[i]);
}

GCO_API void gco_bf16_to_f32_array(const uint16_t *src, float *dst, int64_t n) {
  for (int64_t i = 0; i < n; i++)
    dst[i] = gco_bf16_to_f32(src[i]);
}

/* round every element to the nearest bf16 value, keep f32 storage: the effect
 * of ArithEmulateUnsupportedFloats{bf16->f32} after each bf16 elementwise op
 * (lib/gc/Transforms/Pipeline.cpp:79-95). */
GCO_API void gco_round_bf16_inplace(float *x, int64_t n) {
  for (int64_t i = 0; i < n; i++)
    x[i] = gco_bf16_to_f32(gco_f32_to_bf16(x[i]));
}

/* ------------------------------------------------------------------------- */
/* Batch-reduce GEMM microkernel:
 * lib/gc/ExecutionEngine/CPURuntime/Microkernel/BrgemmNaive.cpp:46-69 (f32),
 * :71-100 (bf16, B in VNNI-2), :102-140 (8-bit, B in VNNI-4), :158-209
 * (beta==0 zero-fills the M*N *dense* C block first, then dtype switch).
 * All offsets/strides in elements.  Per output element the accumulation order
 * is batch-major then k ascending, exactly as in the reference; the loop nest
 * here is (i, m, k, n) so the n loop vectorises without reordering any sum.
 * Returns 0, or -1 for an unsupported dtype pair (the reference asserts).    */
static int is_fp(int dt) { return dt == GCO_F32 || dt == GCO_BF16; }
static int is_i8(int dt) { return dt == GCO_S8 || dt == GCO_U8; }

GCO_API int gco_brgemm(int64_t M, int64_t N, int64_t K, int64_t LDA,
                       int64_t LDB, int64_t LDC, int64_t stride_a,
                       int64_t stride_b, float beta, int64_t dtA, int64_t dtB,
                       const void *A, uint64_t A_off, const void *B,
                       uint64_t B_off, void *C, uint64_t C_off, int num) {
  if (!((dtA == GCO_F32 && dtB == GCO_F32) ||
        (dtA == GCO_BF16 && dtB == GCO_BF16) || (is_i8(dtA) && is_i8(dtB))))
    return -1;

  if (beta == 0.0f) {
    /* BrgemmNaive.cpp:36-44: the init writes M*N contiguous elements starting
     * at C+C_off, not an LDC-strided block. */
    if (is_fp(dtA)) {
      float *c = (float *)C + C_off;
      for (int64_t i = 0; i < M * N; i++)
        c[i] = 0.0f;
    } else {
      int32_t *c = (int32_t *)C + C_off;
      for (int64_t i = 0; i < M * N; i++)
        c[i] = 0;
    }
  }

  if (dtA == GCO_F32) {
    const float *a = (const float *)A + A_off;
    const float *b = (const float *)B + B_off;
    float *c = (float *)C + C_off;
    for (int i = 0; i < num; i++) {
      for (int64_t m = 0; m < M; m++)
        for (int64_t k = 0; k < K; k++) {
          float av = a[m * LDA + k];
          const float *brow = b + k * LDB;
          float *crow = c + m * LDC;
          for (int64_t n = 0; n < N; n++)
            crow[n] += av * brow[n];
        }
      a += stride_a;
      b += stride_b;
    }
  } else if (dtA == GCO_BF16) {
    const uint16_t *a = (const uint16_t *)A + A_off;
    const uint16_t *b = (const uint16_t *)B + B_off;
    float *c = (float *)C + C_off;
    for (int i = 0; i < num; i++) {
      for (int64_t m = 0; m < M; m++)
        for (int64_t k = 0; k < K; k++) {
          /* element (k,n) of B lives at (k - k%2)*LDB + 2n + k%2; a K that is
           * odd simply stops, i.e. the VNNI pad reads as zero (:89-93). */
          float av = gco_bf16_to_f32(a[m * LDA + k]);
          const uint16_t *brow = b + (k & ~(int64_t)1) * LDB + (k & 1);
          float *crow = c + m * LDC;
          for (int64_t n = 0; n < N; n++)
            crow[n] += av * gco_bf16_to_f32(brow[2 * n]);
        }
      a += stride_a;
      b += stride_b;
    }
  } else {
    const uint8_t *a = (const uint8_t *)A + A_off;
    const uint8_t *b = (const uint8_t *)B + B_off;
    int32_t *c = (int32_t *)C + C_off;
    for (int i = 0; i < num; i++) {
      for (int64_t m = 0; m < M; m++)
        for (int64_t k = 0; k < K; k++) {
          uint8_t ar = a[m * LDA + k];
          int32_t av = dtA == GCO_S8 ? (int32_t)(int8_t)ar : (int32_t)ar;
          const uint8_t *brow = b + (k & ~(int64_t)3) * LDB + (k & 3);
          int32_t *crow = c + m * LDC;
          if (dtB == GCO_S8) {
            for (int64_t n = 0; n < N; n++)
              crow[n] += av * (int32_t)(int8_t)brow[4 * n];
          } else {
            for (int64_t n = 0; n < N; n++)
              crow[n] += av * (int32_t)brow[4 * n];
          }
        }
      a += stride_a;
      b += stride_b;
    }
  }
  return 0;
}

/* ------------------------------------------------------------------------- */
/* VNNI blocked packing of a logical row-major W[K,N] (row stride ldw, element
 * size es bytes, v = 2 for 16-bit / 4 for 8-bit) into
 *   B5[N/nb][K/kb][kb/v][nb][v],  B5[no,ko,ki,ni,vi] = W[ko*kb+ki*v+vi, no*nb+ni]
 * (lib/gc/Dialect/Linalgx/Utils.cpp:335-371, the VNNI_MM2D operand; lit type
 * tensor<128x128x16x32x2xbf16> for 4096x4096 with 32x32 blocks,
 * test/mlir/test/gc/Transforms/deepTileContractionNamedOp.mlir:100).
 * K and N need not divide: the tail is zero padded, kb is rounded up to v.   */
GCO_API int gco_vnni_pack(const void *W, int64_t K, int64_t N, int64_t ldw,
                          int es, int64_t kb, int64_t nb, void *out) {
  int v = es == 2 ? 2 : (es == 1 ? 4 : 0);
  if (!v || kb % v)
    return -1;
  int64_t KO = (K + kb - 1) / kb, NO = (N + nb - 1) / nb;
  const uint8_t *w = (const uint8_t *)W;
  uint8_t *o = (uint8_t *)out;
  memset(o, 0, (size_t)(NO * KO * kb * nb * es));
  for (int64_t no = 0; no < NO; no++)
    for (int64_t ko = 0; ko < KO; ko++)
      for (int64_t ki = 0; ki < kb / v; ki++)
        for (int64_t ni = 0; ni < nb; ni++)
          for (int vi = 0; vi < v; vi++) {
            int64_t k = ko * kb + ki * v + vi, n = no * nb + ni;
            if (k >= K || n >= N)
              continue;
            int64_t dst = ((((no * KO + ko) * (kb / v) + ki) * nb + ni) * v + vi);
            memcpy(o + dst * es, w + (k * ldw + n) * es, (size_t)es);
          }
  return 0;
}

/* ------------------------------------------------------------------------- */
/* MatmulConfig validity: lib/gc/Analysis/MatmulConfigAnalysis.cpp:40-65
 * (allowIndivisibleInnerblock=false, isVNNIMM2D=false) and the thread-product
 * rule :99-106.  cfg = {MThreads,NThreads,KThreads,MBlock,NBlock,KBlock,
 * innerMostMBlock,innerMostNBlock,innerMostKBlock}.                          */
GCO_API int gco_validate_config(const int64_t *cfg, int64_t M, int64_t N,
                                int64_t K, int64_t num_threads) {
  for (int i = 0; i < 9; i++)
    if (cfg[i] <= 0)
      return 0;
  int64_t MT = cfg[0], NT = cfg[1], KT = cfg[2], MB = cfg[3], NB = cfg[4],
          KB = cfg[5], iM = cfg[6], iN = cfg[7], iK = cfg[8];
  if (MB % iM || M % iM)
    return 0;
  if (NB % iN || N % iN)
    return 0;
  if (KB % iK || (K / KT) % KB || (K / KT) % iK)
    return 0;
  if ((K + KB - 1) / KB < KT)
    return 0;
  if (num_threads > 0 && MT * NT * KT != num_threads)
    return 0;
  return 1;
}

/* Default config when no attribute overrides and no cost model runs:
 * innermost = 32 when it divides the dimension else the whole dimension
 * (lib/gc/Analysis/MatmulConfigAnalysis.cpp:465-468); blocks = innermost;
 * all threads on M. */
GCO_API void gco_default_config(int64_t M, int64_t N, int64_t K,
                                int64_t num_threads, int64_t *cfg) {
  int64_t iM = M % 32 == 0 ? 32 : M, iN = N % 32 == 0 ? 32 : N,
          iK = K % 32 == 0 ? 32 : K;
  cfg[0] = num_threads > 0 ? num_threads : 1;
  cfg[1] = 1;
  cfg[2] = 1;
  cfg[3] = iM;
  cfg[4] = iN;
  cfg[5] = iK;
  cfg[6] = iM;
  cfg[7] = iN;
  cfg[8] = iK;
}

static int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
static int64_t min64(int64_t a, int64_t b) { return a < b ? a : b; }

/* per-thread extents of the three forall loops:
 * lib/gc/Transforms/DeepTileContractionOp.cpp:562-581.  out = {KPar,MPar,NPar},
 * KPar = 0 when KThreads == 1 (no K split). */
GCO_API void gco_deep_tile_extents(const int64_t *cfg, int64_t M, int64_t N,
                                   int64_t K, int64_t *out) {
  out[0] = cfg[2] == 1 ? 0 : ceil_div(ceil_div(K, cfg[5]), cfg[2]) * cfg[5];
  out[1] = ceil_div(ceil_div(M, cfg[3]), cfg[0]) * cfg[3];
  out[2] = ceil_div(ceil_div(N, cfg[4]), cfg[1]) * cfg[4];
}

/* Deep-tiled matmul: the loop nest of
 * lib/gc/Transforms/DeepTileContractionOp.cpp:506-540 / docs/
 * deep_tile_matmul_design.md:291-322:
 *   forall (pk, pm, pn) over thread grid
 *     for om, on, ok over MBlock / NBlock / KBlock
 *       for im, in over innermost blocks
 *         brgemm(bs = KBlock/iK, iM, iN, iK, beta = ok==0 ? 0 : 1)
 * A is plain row-major [M,K]; B is plain row-major [K,N] for f32 and is packed
 * here into the VNNI_MM2D layout with (iK,iN) blocks for 16/8-bit, which is the
 * only B layout the reference's brgemm accepts for those types
 * (lib/gc/Dialect/Microkernel/MicrokernelOps.cpp:380-389).
 * C is the accumulator-typed result (f32 / s32) [M,N] row stride ldc.  With
 * KThreads > 1 each pk accumulates into its own [M,N] partial and the partials
 * are summed in pk order (DeepTileContractionOp.cpp:988-996).
 * The innermost C tile is computed in a dense iM*iN scratch and copied out,
 * as the bufferised reference does with its thread-local tile.
 * Returns 0, -1 bad dtype, -2 invalid config.                               */
GCO_API int gco_deep_tile_matmul(const int64_t *cfg, int64_t M, int64_t N,
                                 int64_t K, int64_t dtA, int64_t dtB,
                                 const void *A, int64_t lda, const void *B,
                                 int64_t ldb, void *C, int64_t ldc) {
  if (!gco_validate_config(cfg, M, N, K, 0))
    return -2;
  if (!((dtA == GCO_F32 && dtB == GCO_F32) ||
        (dtA == GCO_BF16 && dtB == GCO_BF16) || (is_i8(dtA) && is_i8(dtB))))
    return -1;
  int64_t MT = cfg[0], NT = cfg[1], KT = cfg[2], MB = cfg[3], NB = cfg[4],
          KB = cfg[5], iM = cfg[6], iN = cfg[7], iK = cfg[8];
  int es = dtA == GCO_F32 ? 4 : (dtA == GCO_BF16 ? 2 : 1);
  int v = es == 4 ? 1 : (es == 2 ? 2 : 4);
  int64_t iKp = ceil_div(iK, v) * v; /* VNNI-padded innermost K */
  int64_t ext[3];
  gco_deep_tile_extents(cfg, M, N, K, ext);
  int64_t KPar = KT == 1 ? K : ext[0], MPar = ext[1], NPar = ext[2];

  void *Bp = NULL;
  int64_t KO = ceil_div(K, iK);
  if (es != 4) {
    Bp = malloc((size_t)(ceil_div(N, iN) * KO * iKp * iN * es));
    if (!Bp)
      return -3;
    /* gco_vnni_pack blocks K by iKp.  iK == iKp whenever iK % v == 0; an
     * innermost K that is not a multiple of the VNNI factor is only usable as
     * the single whole-K block (the default when K % 32 != 0), where the pad
     * rows read as zero (BrgemmNaive.cpp:89-93,121-132). */
    if (iKp != iK && iK != K) {
      free(Bp);
      return -2;
    }
    gco_vnni_pack(B, K, N, ldb, es, iKp, iN, Bp);
  }
  void *partial = NULL;
  if (KT > 1) {
    partial = calloc((size_t)(KT * M * N), 4);
    if (!partial)
      return -3;
  }

  int64_t nthreads = MT * NT * KT;
#pragma omp parallel for schedule(static)
  for (int64_t t = 0; t < nthreads; t++) {
    int64_t pk = t / (MT * NT), pm = (t / NT) % MT, pn = t % NT;
    int64_t m_lo = pm * MPar, m_hi = min64(M, m_lo + MPar);
    int64_t n_lo = pn * NPar, n_hi = min64(N, n_lo + NPar);
    int64_t k_lo = pk * KPar, k_hi = min64(K, k_lo + KPar);
    void *tile = malloc((size_t)(iM * iN * 4));
    char *Cdst = KT > 1 ? (char *)partial + (size_t)pk * M * N * 4 : (char *)C;
    int64_t ldcd = KT > 1 ? N : ldc;
    for (int64_t om = m_lo; om < m_hi; om += MB)
      for (int64_t on = n_lo; on < n_hi; on += NB)
        for (int64_t ok = k_lo; ok < k_hi; ok += KB) {
          int64_t kb_cur = min64(KB, k_hi - ok);
          int bs = (int)(kb_cur / iK);
          for (int64_t im = om; im < min64(om + MB, m_hi); im += iM)
            for (int64_t in = on; in < min64(on + NB, n_hi); in += iN) {
              /* load the running C tile (beta = 1 path) or let brgemm zero it */
              float beta = ok == k_lo ? 0.0f : 1.0f;
              if (beta != 0.0f)
                for (int64_t r = 0; r < iM; r++)
                  memcpy((char *)tile + r * iN * 4,
                         Cdst + ((im + r) * ldcd + in) * 4, (size_t)iN * 4);
              if (es == 4) {
                gco_brgemm(iM, iN, iK, lda, ldb, iN, iK, iK * ldb, beta, dtA,
                           dtB, A, (uint64_t)(im * lda + ok), B,
                           (uint64_t)(ok * ldb + in), tile, 0, bs);
              } else {
                int64_t nb_idx = in / iN, kb_idx = ok / iK;
                uint64_t boff =
                    (uint64_t)((nb_idx * KO + kb_idx) * iKp * iN);
                gco_brgemm(iM, iN, iK, lda, iN, iN, iK, iKp * iN, beta, dtA, dtB,
                           A, (uint64_t)(im * lda + ok), Bp, boff, tile, 0, bs);
              }
              for (int64_t r = 0; r < iM; r++)
                memcpy(Cdst + ((im + r) * ldcd + in) * 4,
                       (char *)tile + r * iN * 4, (size_t)iN * 4);
            }
        }
    free(tile);
  }

  if (KT > 1) {
    /* final linalg.reduce over the KThreads axis, pk ascending */
    if (is_fp(dtA)) {
      float *c = (float *)C;
      const float *p = (const float *)partial;
#pragma omp parallel for schedule(static)
      for (int64_t m = 0; m < M; m++)
        for (int64_t n = 0; n < N; n++) {
          float s = 0.0f;
          for (int64_t q = 0; q < KT; q++)
            s += p[(q * M + m) * N + n];
          c[m * ldc + n] = s;
        }
    } else {
      int32_t *c = (int32_t *)C;
      const int32_t *p = (const int32_t *)partial;
      for (int64_t m = 0; m < M; m++)
        for (int64_t n = 0; n < N; n++) {
          int32_t s = 0;
          for (int64_t q = 0; q < KT; q++)
            s += p[(q * M + m) * N + n];
          c[m * ldc + n] = s;
        }
    }
    free(partial);
  }
  free(Bp);
  return 0;
}

/* ------------------------------------------------------------------------- */
/* Post-ops on an f32-stored [M,N] tile.  For a bf16 graph the caller inserts
 * gco_round_bf16_inplace after every op (Pipeline.cpp:79-95).               */

/* bias broadcast along rows + add: lib/gc/Transforms/OneDNNGraphToLinalg.cpp:
 * 64-118 (broadcast), :421-499 (matmul bias). */
GCO_API void gco_bias_add(float *x, const float *bias, int64_t M, int64_t N,
                          int64_t ldx) {
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; m++)
    for (int64_t n = 0; n < N; n++)
      x[m * ldx + n] = x[m * ldx + n] + bias[n];
}

/* ReLU = linalg.max(x, 0): OneDNNGraphToLinalg.cpp:355-358.  arith.maximumf
 * propagates NaN. */
GCO_API void gco_relu(float *x, int64_t n) {
  for (int64_t i = 0; i < n; i++)
    x[i] = x[i] != x[i] ? x[i] : (x[i] > 0.0f ? x[i] : 0.0f);
}

/* linalgx.sigmoid = 1/(1+exp(-x)): lib/gc/Dialect/Linalgx/LinalgxOps.cpp:42-61 */
GCO_API void gco_sigmoid(float *x, int64_t n) {
  for (int64_t i = 0; i < n; i++)
    x[i] = 1.0f / (1.0f + expf(-x[i]));
}

/* GELU, erf form: legacy/core/src/ops/gelu.cpp:110-131 -- op order
 * mul(x,c) -> erf -> add 1 -> mul x -> mul 0.5, c = bits 0x3f3504f3. */
GCO_API void gco_gelu_erf(float *x, int64_t n) {
  uint32_t cb = 0x3f3504f3u;
  float c;
  memcpy(&c, &cb, 4);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; i++) {
    float v = x[i];
    float e = erff(v * c);
    x[i] = ((e + 1.0f) * v) * 0.5f;
  }
}

/* GELU, tanh form: legacy/core/src/ops/gelu.cpp:78-108 -- op order
 * ((x*x)*0.044715 + 1) * x * 0.79788458 -> tanh -> +1 -> *x -> *0.5 */
GCO_API void gco_gelu_tanh(float *x, int64_t n) {
  for (int64_t i = 0; i < n; i++) {
    float v = x[i];
    float t = (((v * v) * 0.044715f + 1.0f) * v) * 0.79788458f;
    x[i] = (v * (tanhf(t) + 1.0f)) * 0.5f;
  }
}

/* column sums of an s8 weight [K,N] in s32: the weight-only term of the
 * asymmetric-activation compensation,
 * legacy/core/src/ops/matmul_core.cpp:546-557, 673-735. */
GCO_API void gco_colsum_s8(const int8_t *W, int64_t K, int64_t N, int64_t ldw,
                           int32_t *out) {
  for (int64_t n = 0; n < N; n++)
    out[n] = 0;
  for (int64_t k = 0; k < K; k++)
    for (int64_t n = 0; n < N; n++)
      out[n] += (int32_t)W[k * ldw + n];
}

/* quantised matmul epilogue: s32 compensation then dequantise
 *   y = f32(acc - zpA*colsum[n]) * scale[n]
 * (matmul_core.cpp:529-571 "sub" of the data compensation in s32;
 * legacy/core/src/compiler/ir/graph/quantization/quantize_op.cpp:259-277
 * cast -> mul scale; graph_reschedule.cpp:220-235 puts the dequantize right
 * after the s32 matmul). */
GCO_API void gco_dequant_comp(const int32_t *acc, int64_t M, int64_t N,
                              int64_t ldacc, int32_t zpA, const int32_t *colsum,
                              const float *scale, float *out, int64_t ldo) {
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; m++)
    for (int64_t n = 0; n < N; n++) {
      int32_t c = acc[m * ldacc + n] - zpA * colsum[n];
      out[m * ldo + n] = (float)c * scale[n];
    }
}

/* ------------------------------------------------------------------------- */
/* Row softmax in f32, numerically stable: max-reduce, sub, exp, add-reduce,
 * div (lib/gc/Transforms/DecomposeAggregatedOps.cpp:24-38 -> upstream
 * linalg.softmax decomposition; legacy/core/src/ops/softmax.cpp:50-123).
 * A row whose maximum is -inf yields NaN (inf - inf), as torch.softmax does. */
GCO_API void gco_softmax_rows(float *x, int64_t rows, int64_t cols,
                              int64_t ldx) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; r++) {
    float *p = x + r * ldx;
    float mx = -INFINITY;
    for (int64_t c = 0; c < cols; c++)
      mx = p[c] > mx ? p[c] : mx;
    float s = 0.0f;
    for (int64_t c = 0; c < cols; c++) {
      p[c] = expf(p[c] - mx);
      s += p[c];
    }
    for (int64_t c = 0; c < cols; c++)
      p[c] = p[c] / s;
  }
}

/* Multi-head attention as the composition the reference can express:
 *   S = batch_matmul_transpose_b(Q, K)    bf16 in, f32 accumulate
 *       (test/benchgc/src/benchgc/linalg/matmul.py:65-68)
 *   S = S * scale ; S = S + mask          f32 elementwise, mask [Sq,Sk]
 *       broadcast over (batch, head); mask may be NULL
 *   P = softmax(S, -1) in f32             (gco_softmax_rows)
 *   Pb = bf16(P)                          (RNE, gco_f32_to_bf16)
 *   O = batch_matmul(Pb, V)               f32 accumulate, then bf16
 * Q,K,V,O are bf16 [BH, S, D] contiguous.  k ascending accumulation.        */
GCO_API int gco_mha_bf16(const uint16_t *Q, const uint16_t *Kt,
                         const uint16_t *V, const float *mask, float scale,
                         int64_t BH, int64_t Sq, int64_t Sk, int64_t D,
                         uint16_t *O) {
  int fail = 0;
#pragma omp parallel for schedule(dynamic, 1)
  for (int64_t bh = 0; bh < BH; bh++) {
    float *S = (float *)malloc((size_t)Sk * 4);
    float *kf = (float *)malloc((size_t)Sk * D * 4);
    float *vf = (float *)malloc((size_t)Sk * D * 4);
    float *acc = (float *)malloc((size_t)D * 4);
    if (!S || !kf || !vf || !acc) {
      fail = 1;
    } else {
      gco_bf16_to_f32_array(Kt + bh * Sk * D, kf, Sk * D);
      gco_bf16_to_f32_array(V + bh * Sk * D, vf, Sk * D);
      for (int64_t q = 0; q < Sq; q++) {
        const uint16_t *qr = Q + (bh * Sq + q) * D;
        for (int64_t j = 0; j < Sk; j++) {
          float s = 0.0f;
          for (int64_t d = 0; d < D; d++)
            s += gco_bf16_to_f32(qr[d]) * kf[j * D + d];
          s = s * scale;
          if (mask)
            s = s + mask[q * Sk + j];
          S[j] = s;
        }
        gco_softmax_rows(S, 1, Sk, Sk);
        for (int64_t d = 0; d < D; d++)
          acc[d] = 0.0f;
        for (int64_t j = 0; j < Sk; j++) {
          float p = gco_bf16_to_f32(gco_f32_to_bf16(S[j]));
          for (int64_t d = 0; d < D; d++)
            acc[d] += p * vf[j * D + d];
        }
        for (int64_t d = 0; d < D; d++)
          O[(bh * Sq + q) * D + d] = gco_f32_to_bf16(acc[d]);
      }
    }
    free(S);
    free(kf);
    free(vf);
    free(acc);
  }
  return fail ? -3 : 0;
}

/* ------------------------------------------------------------------------- */
/* Point-to-point comparison rule of the reference harness
 * (test/benchgc/src/benchgc/arg/compare.py:60-137): an element passes when
 * both are NaN, or both the same infinity, or
 *   d = |ref| > 1e-5 ? |ref-res|/|ref| : |ref-res|,  d <= thr.
 * Returns the number of failing elements; *max_d receives the largest d.     */
GCO_API int64_t gco_compare_p2p(const float *ref, const float *res, int64_t n,
                                float thr, float *max_d) {
  int64_t bad = 0;
  float md = 0.0f;
  for (int64_t i = 0; i < n; i++) {
    float r = ref[i], s = res[i];
    if (r != r && s != s)
      continue;
    if (isinf(r) && isinf(s) && ((r > 0) == (s > 0)))
      continue;
    float a = fabsf(r);
    float d = a > 1e-5f ? fabsf(r - s) / a : fabsf(r - s);
    if (!(d <= thr))
      bad++;
    if (d > md || d != d)
      md = d;
  }
  if (max_d)
    *max_d = md;
  return bad;
}

/* Norm comparison rule of the reference harness
 * (test/benchgc/src/benchgc/arg/compare.py:41-57): pass iff
 *   sqrt( sum (ref-res)^2 / sum ref^2 ) < thr      (strictly less),
 * an empty tensor passes.  The harness sums in f32 with torch; here the two
 * sums are formed in f64 and the quotient and root in f32, which agrees with
 * any f32 summation order to a few 1e-7 relative.  *l2 receives the value.   */
GCO_API int gco_compare_norm(const float *ref, const float *res, int64_t n,
                             float thr, float *l2) {
  if (n == 0) {
    if (l2)
      *l2 = 0.0f;
    return 1;
  }
  double dd = 0.0, rr = 0.0;
  for (int64_t i = 0; i < n; i++) {
    double d = (double)ref[i] - (double)res[i];
    dd += d * d;
    rr += (double)ref[i] * (double)ref[i];
  }
  float v = sqrtf((float)dd / (float)rr);
  if (l2)
    *l2 = v;
  return v < thr ? 1 : 0;
}

/* The same rule applied to every row of a [rows, cols] tensor: returns the
 * number of rows that fail; l2_rows (optional, [rows]) receives each value.
 * A row of zeros in ref with zeros in res is 0/0 = NaN and fails, as the rule
 * above would.                                                              */
GCO_API int64_t gco_compare_norm_rows(const float *ref, const float *res,
                                      int64_t rows, int64_t cols, float thr,
                                      float *l2_rows) {
  int64_t bad = 0;
  for (int64_t r = 0; r < rows; r++) {
    float v;
    if (!gco_compare_norm(ref + r * cols, res + r * cols, cols, thr, &v))
      bad++;
    if (l2_rows)
      l2_rows[r] = v;
  }
  return bad;
}

/* The attention composition of gco_mha_bf16 evaluated in f64, for error
 * attribution: scores, scale, mask, softmax and both matmuls in double.
 * round_p != 0: the softmax weights are rounded to bf16 where the reference
 * graph rounds them (P is a bf16 tensor between the softmax and the second
 * batch_matmul); 0: no rounding anywhere.  The result is NOT rounded.
 * Q,K,V bf16 [BH,S,D]; O double [BH,Sq,D].                                   */
GCO_API int gco_mha_f64(const uint16_t *Q, const uint16_t *Kt, const uint16_t *V,
                        const float *mask, double scale, int64_t BH, int64_t Sq,
                        int64_t Sk, int64_t D, int round_p, double *O) {
  int fail = 0;
#pragma omp parallel for schedule(dynamic, 1)
  for (int64_t bh = 0; bh < BH; bh++) {
    double *S = (double *)malloc((size_t)Sk * 8);
    double *kf = (double *)malloc((size_t)Sk * D * 8);
    double *vf = (double *)malloc((size_t)Sk * D * 8);
    if (!S || !kf || !vf) {
      fail = 1;
    } else {
      for (int64_t i = 0; i < Sk * D; i++) {
        kf[i] = (double)gco_bf16_to_f32(Kt[bh * Sk * D + i]);
        vf[i] = (double)gco_bf16_to_f32(V[bh * Sk * D + i]);
      }
      for (int64_t q = 0; q < Sq; q++) {
        const uint16_t *qr = Q + (bh * Sq + q) * D;
        double mx = -INFINITY;
        for (int64_t j = 0; j < Sk; j++) {
          double s = 0.0;
          for (int64_t d = 0; d < D; d++)
            s += (double)gco_bf16_to_f32(qr[d]) * kf[j * D + d];
          s = s * scale;
          if (mask)
            s = s + (double)mask[q * Sk + j];
          S[j] = s;
          mx = s > mx ? s : mx;
        }
        double sum = 0.0;
        for (int64_t j = 0; j < Sk; j++) {
          S[j] = exp(S[j] - mx);
          sum += S[j];
        }
        double *o = O + (bh * Sq + q) * D;
        for (int64_t d = 0; d < D; d++)
          o[d] = 0.0;
        for (int64_t j = 0; j < Sk; j++) {
          double p = S[j] / sum;
          if (round_p)
            p = (double)gco_bf16_to_f32(gco_f32_to_bf16((float)p));
          for (int64_t d = 0; d < D; d++)
            o[d] += p * vf[j * D + d];
        }
      }
    }
    free(S);
    free(kf);
    free(vf);
  }
  return fail ? -3 : 0;
}

GCO_API int gco_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
