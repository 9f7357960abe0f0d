/*
 * gc_hip_kernels.h -- C ABI of the MI355X (gfx950) kernels behind the graph
 * compiler's contraction hot path.  Every pointer is a DEVICE pointer unless
 * stated otherwise; sizes and leading dimensions are in elements; `stream` is a
 * hipStream_t passed as void* (NULL = the default stream).  Calls are
 * asynchronous on `stream`.
 *
 * Scratch memory.  Two kinds of call need device memory beyond their operands:
 * K-sliced GEMMs (too few 256 x 256 tiles for the GPU, e.g. a short A against
 * wide weights or 1024 x 1024 x 8192: f32 partial sums) and masked
 * attention (one byte per mask tile).  Each entry point says where it comes
 * from:
 *   - plain entry points (gcmi_gemm_bf16, gcmi_mha_fwd_bf16, ...): a workspace
 *     the library allocates per device at the first call that needs one and
 *     grows on demand (hipMalloc under a lock).  Calls that use it are put in
 *     order across streams (an event behind each, waited for by the next call
 *     on another stream), so they are safe from any number of host threads;
 *   - *_ws entry points: a workspace the caller brings (size from the
 *     *_workspace_bytes query).  Nothing is shared: calls with different
 *     workspaces may overlap on different streams.  This is what a compiled
 *     partition uses (its arena holds the workspace);
 *   - gcmi_gemm_bf16_noalloc: a static device array; allocates nothing.
 * Everything else needs no scratch and allocates nothing.
 *
 * Return value: a dnnl_status_t-compatible int (0 success, 2 invalid
 * arguments, 3 unimplemented, 5 runtime error); gcmi_last_error() gives text.
 *
 * Each entry point names the reference interface whose work it takes over
 * (paths relative to the intel/graph-compiler tree).
 */
#ifndef GC_HIP_KERNELS_H
#define GC_HIP_KERNELS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
#pragma GCC visibility push(default)

/* dnnl_data_type_t values, as the reference passes them across its microkernel
 * ABI (test/mlir/unittests/ExecutionEngine/BrgemmRuntime.cpp:61-62,117-118). */
enum { GCMI_F16 = 1, GCMI_BF16 = 2, GCMI_F32 = 3, GCMI_S32 = 4, GCMI_S8 = 5, GCMI_U8 = 6 };

/* fused post-op of a GEMM epilogue */
enum { GCMI_ACT_NONE = 0, GCMI_ACT_RELU = 1, GCMI_ACT_GELU_ERF = 2, GCMI_ACT_GELU_TANH = 3, GCMI_ACT_SIGMOID = 4 };

/* Library / device set-up.  Selects `device`, checks it is a gfx950 part and
 * returns 0.  Optional: every entry point works on the current device. */
int gcmi_init(int device);
const char *gcmi_last_error(void);

/*
 * bf16 matmul with fused epilogue:  C = act( (A.B) [+ bias] ).
 * Takes over: linalg.matmul lowered by DeepTileMatmul to a loop nest of
 * dnnl_brgemm_execute calls plus the fused consumers
 * (lib/gc/Transforms/DeepTileContractionOp.cpp:958-1014,
 *  lib/gc/Transforms/IterativeTilingAndFusion.cpp:585-611,
 *  include/gc/ExecutionEngine/CPURuntime/Microkernel/BrgemmInterface.h:31-63).
 * A [M,K] and B [K,N] row-major bf16 (B is NOT VNNI packed).  f32 accumulate
 * over all of K.  out_dtype GCMI_BF16: bf16 graph semantics, the value is
 * rounded to bf16 after the matmul, after the bias add and after the
 * activation (lib/gc/Transforms/Pipeline.cpp:79-95).  out_dtype GCMI_F32: no
 * intermediate rounding.  bias: [N] of bias_dtype (GCMI_BF16 or GCMI_F32) or
 * NULL.
 * When A has at most 256 rows and N is narrow (fewer column tiles than half the
 * compute units), K is cut into slices over workgroups and a second kernel adds
 * the f32 partial sums in a fixed order (results do not vary from run to run).
 * The partial sums go through the library workspace (see "Scratch memory").
 */
int gcmi_gemm_bf16(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                   int64_t ldc, const void *bias, int bias_dtype, int act, int out_dtype, void *stream);

/*
 * The same with B stored transposed: Bt [N,K] row-major (k contiguous, ldb
 * elements between its rows), C = epilogue(A . Bt^T).  Takes over
 * linalg.matmul_transpose_b / onednn_graph.matmul{transpose_b} on bf16
 * (lib/gc/Transforms/OneDNNGraphToLinalg.cpp:421-499; the weights of
 * test/benchgc/cases/llama2.mlir are stored this way).  No transposed copy is
 * made: the tile of Bt is staged and read like the tile of A.
 */
int gcmi_gemm_bf16_nt(const void *A, const void *Bt, void *C, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                      int64_t ldc, const void *bias, int bias_dtype, int act, int out_dtype, void *stream);

/*
 * Strided batches of the same GEMM in one launch: batch b reads A + b*stride_a,
 * B + b*stride_b and writes C + b*stride_c (element strides; 0 shares the
 * operand between batches; at most 65535 batches).  trans_b as in
 * gcmi_gemm_bf16_nt.  Takes over linalg.batch_matmul{,_transpose_b} and the
 * batch dims of onednn_graph.matmul (lib/gc/Dialect/OneDNNGraph/
 * OneDNNGraphOps.cpp:204-310; the reference tiles the batch as the outermost
 * parallel loop, lib/gc/Transforms/DeepTileContractionOp.cpp:570-575).
 */
int gcmi_gemm_bf16_batched(const void *A, const void *B, void *C, int64_t batch, int64_t M, int64_t N, int64_t K,
                           int64_t lda, int64_t ldb, int64_t ldc, int64_t stride_a, int64_t stride_b, int64_t stride_c,
                           int trans_b, const void *bias, int bias_dtype, int act, int out_dtype, void *stream);

/*
 * gcmi_gemm_bf16_batched with a residual connection in the epilogue:
 * C = act(A.B + bias) + R, R a tensor of the shape of C (residual_dtype
 * GCMI_BF16 or GCMI_F32, ldr elements between its rows, batch b at
 * R + b*stride_c; NULL: none).  With out_dtype GCMI_BF16 the sum is rounded
 * to bf16 like every other op of a bf16 graph, so the result equals a matmul
 * followed by a separate add bit for bit.  Takes over the add that the
 * reference fuses into the matmul's innermost loop nest as a consumer
 * (tileAndFuseConsumerOfOpResult, lib/gc/Transforms/
 * IterativeTilingAndFusion.cpp:505-560; the matmuls of
 * test/benchgc/cases/llama2.mlir:10 and :75 end in one).
 * R may be C itself (every element is read before it is written), but must not
 * overlap it otherwise.
 */
int gcmi_gemm_bf16_residual(const void *A, const void *B, void *C, int64_t batch, int64_t M, int64_t N, int64_t K,
                            int64_t lda, int64_t ldb, int64_t ldc, int64_t stride_a, int64_t stride_b, int64_t stride_c,
                            int trans_b, const void *bias, int bias_dtype, int act, const void *residual, int64_t ldr,
                            int residual_dtype, int out_dtype, void *stream);

/*
 * gcmi_gemm_bf16_residual with the workspace as an argument: `workspace`
 * (16-byte aligned, workspace_bytes long; NULL / 0: K is not sliced) holds the
 * partial sums of a K-sliced call.  gcmi_gemm_bf16_workspace_bytes gives the
 * size the shape can use (0: the shape is never sliced); with less, fewer
 * slices are cut.  The result does not depend on the workspace's address, and
 * for a given size it does not vary from run to run.  No counterpart in the
 * reference, whose K-sliced partial sums live in a buffer its generated code
 * allocates (lib/gc/Transforms/DeepTileContractionOp.cpp:988-996).
 */
size_t gcmi_gemm_bf16_workspace_bytes(int64_t M, int64_t N, int64_t K, int trans_b);
/* The same for a call that passes `matmul_config` (nine MatmulConfig integers, or NULL): a KThreads that names more
 * slices than the shape would get by default needs a workspace where the default needs none. */
size_t gcmi_gemm_bf16_workspace_bytes_cfg(int64_t M, int64_t N, int64_t K, int trans_b, const int64_t *matmul_config);
int gcmi_gemm_bf16_ws(const void *A, const void *B, void *C, int64_t batch, int64_t M, int64_t N, int64_t K,
                      int64_t lda, int64_t ldb, int64_t ldc, int64_t stride_a, int64_t stride_b, int64_t stride_c,
                      int trans_b, const void *bias, int bias_dtype, int act, const void *residual, int64_t ldr,
                      int residual_dtype, int out_dtype, void *workspace, size_t workspace_bytes,
                      const int64_t *matmul_config, void *stream);

/*
 * The tile descriptor: what the launcher chooses for a GEMM call, the GPU's
 * counterpart of the reference's MatmulConfig (include/gc/Analysis/
 * MatmulConfigAnalysis.h:25-34; chosen there by a CPU cost model,
 * lib/gc/Analysis/MatmulConfigAnalysis.cpp:435-552, here per shape, element
 * type and layout).  `kernel`: 0 bounds-checked tile (any shape), 1 whole
 * tiles with 8 waves of 128 x 64, 2 tiles with 4 waves of 128 x 128 (any M,
 * N a multiple of 16 bytes of columns: edge tiles store what lies inside C),
 * 3 K slices over workgroups + second pass (tiles on less than half of the
 * compute units), 4 weight-streaming
 * kernel (up to 128 rows of A against wide weights in either layout; bn = 64:
 * the 8-wave kernel with the LDS ring, with split_k > 1 followed by the second
 * pass), 5 tiles of 128 x 128 with 4 waves
 * of 64 x 64 (problems of few 256 x 256 tiles; with split_k > 1 kind 3 is
 * reported and bm = bn = 128 tells).
 *
 * matmul_config (may be NULL) is the reference's per-op override: the nine
 * integers {MThreads, NThreads, KThreads, MBlock, NBlock, KBlock,
 * innermostMBlock, innermostNBlock, innermostKBlock} of the op's attributes
 * (readConfigFromAttrs, MatmulConfigAnalysis.cpp:368-404: all nine or none;
 * validateConfig, :40-65).  On the GPU they steer: MBlock x NBlock = the
 * workgroup tile (256 x 256 and 128 x 128 are built),
 * innermostMBlock x innermostNBlock = the tile of one wave (128 x 128: 4 waves
 * per workgroup; 128 x 64: 8 waves; 64 x 64 with the 128 x 128 tile), KThreads
 * = the number of K slices where the shape is sliced (1 with the 128 x 128 tile).  A config that
 * is invalid or names a tile that is not built is ignored, like an invalid one
 * in the reference; gcmi_gemm_tile_config_query says why in `note`.
 * gcmi_gemm_bf16_ws and gcmi_gemm_int8_cfg take the same nine integers.
 */
typedef struct gcmi_gemm_tile_config {
  int32_t kernel;
  int32_t bm, bn;           /* workgroup tile */
  int32_t kbytes;           /* bytes of K per LDS stage and row */
  int32_t stages;           /* slots of the LDS ring */
  int32_t waves_m, waves_n; /* waves of a workgroup */
  int32_t wave_m, wave_n;   /* tile of one wave */
  int32_t mfma_m, mfma_n, mfma_k;
  int32_t split_k;          /* K slices; 1: none */
  int32_t group_m;          /* tile rows an XCD walks before moving on */
  int32_t workgroups;
  int32_t from_attrs;       /* 1: matmul_config was applied */
} gcmi_gemm_tile_config;
int gcmi_gemm_tile_config_query(int a_dtype, int64_t M, int64_t N, int64_t K, int trans_b, int out_dtype,
                                const int64_t *matmul_config, gcmi_gemm_tile_config *out, char *note, size_t note_len);

/*
 * gcmi_gemm_bf16 / gcmi_gemm_bf16_nt (trans_b) for callers that cannot
 * allocate device memory: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  No counterpart in the reference.  The
 * partial sums of a K-sliced call go to a static device array of
 * gcmi_noalloc_scratch_bytes() = 32 MiB that every device the library runs on
 * holds until the process ends; the call allocates nothing and frees nothing.
 * A shape whose K slices need more than that (gcmi_gemm_bf16_workspace_bytes)
 * is refused with status 2 and a message; shapes that are not K-sliced need no
 * scratch and are never refused.  Every call on a device shares that device's
 * array: calls that overlap in time on one device (different streams) race;
 * calls on one stream are safe.  Results equal gcmi_gemm_bf16's bit for bit.
 */
size_t gcmi_noalloc_scratch_bytes(void);
int gcmi_gemm_bf16_noalloc(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K, int64_t lda,
                           int64_t ldb, int64_t ldc, int trans_b, const void *bias, int bias_dtype, int act,
                           int out_dtype, void *stream);

/*
 * 8-bit matmul with s32 accumulation and fused dequantise epilogue.
 * Takes over: the u8/s8 brgemm (lib/gc/ExecutionEngine/CPURuntime/Microkernel/
 * BrgemmNaive.cpp:102-140) under the deep-tile nest, the asymmetric-activation
 * compensation (legacy/core/src/ops/matmul_core.cpp:529-571), Dequantize
 * (legacy/core/src/compiler/ir/graph/quantization/quantize_op.cpp:230-277) and
 * GELU (legacy/core/src/ops/gelu.cpp:72-133).
 * A [M,K] of a_dtype (GCMI_U8 or GCMI_S8), W [K,N] s8, both row-major.
 *   acc[m,n]  = sum_k A[m,k]*W[k,n]                       (s32, exact)
 *   out_dtype GCMI_S32 : C = acc                          (raw accumulators)
 *   otherwise          : x = f32(acc - zp_a*colsum[n]) * scale[n] (+ bias[n]);
 *                        C = act(x) as GCMI_F32 or GCMI_BF16 (one RNE rounding)
 * colsum [N] s32 = sum_k W[k,n] (gcmi_colsum_s8); required when a_dtype is
 * GCMI_U8 or zp_a != 0.  scale, bias: f32 [N] or NULL (scale 1, no bias).
 */
int gcmi_gemm_int8(const void *A, int a_dtype, const void *W, void *C, int64_t M, int64_t N, int64_t K, int64_t lda,
                   int64_t ldb, int64_t ldc, const int32_t *colsum, int32_t zp_a, const float *scale,
                   const float *bias, int act, int out_dtype, void *stream);

/* gcmi_gemm_int8 with the op's MatmulConfig attributes (see gcmi_gemm_tile_config_query; NULL: none). */
int gcmi_gemm_int8_cfg(const void *A, int a_dtype, const void *W, void *C, int64_t M, int64_t N, int64_t K, int64_t lda,
                       int64_t ldb, int64_t ldc, const int32_t *colsum, int32_t zp_a, const float *scale,
                       const float *bias, int act, int out_dtype, const int64_t *matmul_config, void *stream);

/* Column sums of an s8 weight [K,N] into s32 [N]: the weight-only constant of
 * the compensation term (legacy/core/src/ops/matmul_core.cpp:546-557). */
int gcmi_colsum_s8(const void *W, int64_t K, int64_t N, int64_t ldw, int32_t *colsum, void *stream);

/*
 * f32 matmul (+bias, +activation), transposes folded into strides.
 * Takes over: onednn_graph.matmul{transpose_a,transpose_b} + bias + ReLU on
 * f32 (lib/gc/Transforms/OneDNNGraphToLinalg.cpp:421-499, :355-358).
 * Logical A is [M,K], logical B is [K,N]; when trans_a the stored A is [K,M]
 * with leading dimension lda, likewise trans_b.  Plain f32 FMA arithmetic.
 */
int gcmi_gemm_f32(const float *A, const float *B, float *C, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                  int64_t ldc, int trans_a, int trans_b, const float *bias, int act, void *stream);

/* The f32 GEMM over strided batches (see gcmi_gemm_bf16_batched). */
int gcmi_gemm_f32_batched(const float *A, const float *B, float *C, int64_t batch, int64_t M, int64_t N, int64_t K,
                          int64_t lda, int64_t ldb, int64_t ldc, int64_t stride_a, int64_t stride_b, int64_t stride_c,
                          int trans_a, int trans_b, const float *bias, int act, void *stream);

/*
 * Fused multi-head attention forward, bf16, head_dim D = 128 or 64 (any other: status unimplemented):
 *   O = softmax(Q K^T * scale + mask) V,  softmax over keys in f32.
 * Takes over the composition batch_matmul_transpose_b -> mul -> add -> softmax
 * -> batch_matmul (lib/gc/Transforms/DecomposeAggregatedOps.cpp:24-38;
 * test/benchgc/src/benchgc/linalg/matmul.py:29-32,65-68).
 * Q [BH,Sq,D], K and V [BH,Sk,D], O [BH,Sq,D], contiguous bf16; mask f32
 * [Sq,Sk] with row stride mask_ld, added to every (batch, head), or NULL.
 * A query row whose keys are all masked with -inf yields NaN.
 */
int gcmi_mha_fwd_bf16(const void *Q, const void *K, const void *V, const float *mask, int64_t mask_ld, void *O,
                      int64_t BH, int64_t Sq, int64_t Sk, int64_t D, float scale, void *stream);

/*
 * The same with the block-skipping switch exposed.  When a mask is given, one
 * pass over it classifies every (32 query rows x 64 keys) tile as all 0, all
 * -inf or general; constant tiles cost no mask traffic in the main kernel.
 * skip_masked != 0 (what gcmi_mha_fwd_bf16 uses): a block of 64 keys whose
 * tiles are -inf for all 128 query rows of a workgroup is not visited at all --
 * it contributes exp(-inf) = 0 to every sum, so the result is bit-identical.
 * skip_masked == 0: every block is computed (the dense 4*BH*Sq*Sk*D operation
 * count).  scale must be > 0 for the fast kernel (otherwise a slower, general
 * kernel runs).  The tile classes go through the library workspace (see
 * "Scratch memory").
 * No counterpart in the reference.
 */
int gcmi_mha_fwd_bf16_opt(const void *Q, const void *K, const void *V, const float *mask, int64_t mask_ld, void *O,
                          int64_t BH, int64_t Sq, int64_t Sk, int64_t D, float scale, int skip_masked, void *stream);

/*
 * The same with the workspace as an argument: one byte per (32 query rows x 64
 * keys) mask tile, gcmi_mha_fwd_workspace_bytes in all (0: the shape has no
 * use for one).  With NULL or too small a workspace every tile is read from
 * the mask and nothing is skipped; the result is the same.
 *
 * A mask that does not change between calls (a constant of the partition, the
 * counterpart of the reference's constant-tensor cache, src/dnnl/JsonParser.cpp:
 * 295-299) need not be classified by every call: gcmi_mha_classify_mask runs the
 * pass alone into `workspace`, and calls that pass skip_masked |
 * GCMI_MHA_CLASSES_VALID with the same mask, mask_ld, Sq, Sk, D and workspace
 * launch the attention kernel only.  The caller vouches that the mask's contents
 * are still what was classified; the result is otherwise undefined.
 */
#define GCMI_MHA_SKIP_MASKED 1
#define GCMI_MHA_CLASSES_VALID 2
size_t gcmi_mha_fwd_workspace_bytes(int64_t Sq, int64_t Sk, int64_t D, int has_mask);
int gcmi_mha_classify_mask(const float *mask, int64_t mask_ld, int64_t Sq, int64_t Sk, int64_t D, void *workspace,
                           size_t workspace_bytes, void *stream);
int gcmi_mha_fwd_bf16_ws(const void *Q, const void *K, const void *V, const float *mask, int64_t mask_ld, void *O,
                         int64_t BH, int64_t Sq, int64_t Sk, int64_t D, float scale, int skip_masked, void *workspace,
                         size_t workspace_bytes, void *stream);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif
#endif /* GC_HIP_KERNELS_H */
