// Plain-data argument blocks passed by value to the GEMM / attention kernels.
#pragma once
#include <stdint.h>

namespace gcmi {

struct GemmParams {
  const void *A;   // [M,K] row-major, lda elements between rows
  const void *B;   // [K,N] row-major, ldb elements between rows
  void *C;         // [M,N] row-major, ldc elements between rows
  int64_t M, N, K;
  int64_t lda, ldb, ldc;
  const void *bias;      // [N] or null; dtype bias_dt (bf16 or f32)
  const float *scale;    // int8 only: per-output-channel dequant scale [N] or null
  const int32_t *colsum; // int8 only: sum_k W[k,n] in s32, [N] or null
  int32_t comp;          // int8 only: integer factor of colsum added to the accumulator
  uint32_t a_xor;        // int8 only: 0x80808080 when A is u8, else 0
  int32_t act;           // gcmi::Act
  int32_t out_dt;        // gcmi::DType of C
  int32_t bias_dt;       // gcmi::DType of bias
  int32_t group_m;       // tile-order group height (XCD/L2 locality), 0 = default
  // split-K (set by the launcher; one tile row, M <= 256): workgroup b takes tile b % tiles and K slice b / tiles,
  // and writes its f32 partial sums [M x N] to partial + slice * M * N; a second kernel sums the slices and
  // runs the epilogue
  int32_t splits;        // 0 or 1: off
  // workspace of the f32 partial sums: brought by the caller (partial_cap floats; without one K is not sliced)
  float *partial;
  int64_t partial_cap;
  int32_t trans_b;       // bf16 only: B is stored [N,K] (k contiguous), ldb elements between its rows
  // strided batch (bf16 tile kernels): blockIdx.y is the batch index, operands advance by these element strides
  // (0 = the operand is shared by all batches).  batch <= 1: a single GEMM.
  int64_t batch, a_bs, b_bs, c_bs;
  // bf16 GEMMs: a tensor of the shape of C that is added last, after bias and activation (a residual connection);
  // with bf16 output the sum is rounded like every other op of a bf16 graph.  Batches advance it like C.
  const void *residual; // null: none
  int64_t ldr;          // elements between its rows
  int32_t residual_dt;  // DT_BF16 or DT_F32
  // wishes of the caller (the op's MatmulConfig attributes, translated): 0 = the launcher's own choice
  int32_t cfg_waves;    // 4 or 8 waves per workgroup on whole tiles
  int32_t cfg_split_k;  // number of K slices (1: none) where the shape can be sliced
  int32_t cfg_tile;     // 128: the 128 x 128 tile kernel where the shape allows it; 256: never that kernel
};

// What the launcher decides for one GEMM call: the GPU's counterpart of the reference's MatmulConfig
// (include/gc/Analysis/MatmulConfigAnalysis.h:25-34: thread split, L2 block, innermost block per dim), chosen per
// (M, N, K, element type, layout) instead of by the CPU cost model.  Reported by dnnl_graph_compiler_explain.
struct GemmTileConfig {
  int32_t kernel;          // GemmKernel
  int32_t bm, bn;          // workgroup tile (the reference's MBlock / NBlock)
  int32_t kbytes;          // bytes of K per LDS stage and row (KBlock * element size)
  int32_t stages;          // slots of the LDS ring
  int32_t waves_m, waves_n; // waves of a workgroup along m and n
  int32_t wave_m, wave_n;  // tile of one wave (the reference's innermost block: what one microkernel call covers)
  int32_t mfma_m, mfma_n, mfma_k; // shape of the matrix instruction
  int32_t split_k;         // K slices (the reference's KThreads); 1: none
  int32_t group_m;         // tile rows an XCD walks before moving on (L2 locality)
  int32_t workgroups;      // launched
  int32_t from_attrs;      // 1: MatmulConfig attributes of the op were applied
};
enum GemmKernel : int32_t {
  GK_EDGE = 0,    // bounds-checked 256x256 tile, 8 waves, 32x32 MFMAs: any shape and alignment
  GK_WAVES8 = 1,  // whole tiles, 8 waves of 128 x 64, 16x16 MFMAs
  GK_WAVES4 = 2,  // whole tiles, 4 waves of 128 x 128 (one per SIMD), 16x16 MFMAs, hand-placed main loop
  GK_SPLITK = 3,  // too few tiles for the GPU: K slices over workgroups + second pass
  GK_STREAM = 4,  // a short A against wide weights: weight-streaming kernel (+ second pass where K is sliced)
  GK_TILE128 = 5, // 128 x 128 tiles, 4 waves of 64 x 64, two workgroups per compute unit: problems of few 256 x 256 tiles
};

struct F32GemmParams {
  const float *A, *B;
  float *C;
  int64_t M, N, K;
  int64_t a_rs, a_cs; // element strides of A along m and k (transposes fold in here)
  int64_t b_rs, b_cs; // element strides of B along k and n
  int64_t ldc;
  const float *bias;
  int32_t act;
  float beta; // 0: overwrite, 1: accumulate into C before the epilogue
  int64_t batch, a_bs, b_bs, c_bs; // strided batch in blockIdx.z (0 stride = shared operand); batch <= 1: single GEMM
};

struct MhaParams {
  const void *Q, *K, *V; // bf16 [B*H, S, D] contiguous
  void *O;               // bf16 [B*H, Sq, D]
  const float *mask;     // f32 [Sq, Sk] additive, shared by every (batch, head); or null
  int64_t mask_ld;
  int32_t BH, Sq, Sk, D;
  float scale;
  // fast path only: class of every (32 query rows x 64 keys) mask tile, [Sq/32][Sk/64].  The caller brings the
  // buffer (tile_class_cap bytes); the launcher fills it with a classification pass.  Null: no classes (every tile is
  // read from the mask, nothing is skipped)
  uint8_t *tile_class;
  int64_t tile_class_cap;
  int32_t skip_masked; // 1: tiles whose mask is all -inf are not computed (the result is the same)
  // 1: tile_class already holds the classes of this mask (an earlier call's classification pass for the same mask,
  // shape and buffer): the pass is not launched again.  2: launch the pass only, no attention kernel.
  int32_t classes_mode;
};

} // namespace gcmi
