/*
 * dnnl_graph_compiler.h -- the oneDNN-Graph compiler-backend C API of
 * intel/graph-compiler, served by MI355X (gfx950) kernels.
 *
 * The reference implements these six entry points in
 * src/dnnl/dnnl_graph_compiler.cpp:157-226 against a header that lives in a
 * oneDNN fork (graph/backend/elyzor/include/dnnl_graph_compiler.h) and is not
 * part of the reference tree.  This header re-declares the same functions and
 * structures as recovered from every use site:
 *   context  {num_threads}                      test/dnnl/TestApiBasic.cpp:28
 *   tensor   {id, ndims, dims, data}            test/dnnl/TestApiOps.cpp:46-48,
 *                                               src/dnnl/dnnl_graph_compiler.cpp:76-77,121-133
 *   version  {api_version, gc_version} x {major, minor, patch, hash}
 *                                               src/dnnl/dnnl_graph_compiler.cpp:159-166
 * The integer widths of the fork's header are not pinned by the reference
 * tree; the widths below are the ones its call sites are consistent with.
 *
 * Behaviour kept from the reference: JSON partition in, tensors matched by id
 * (any order), caller-owned buffers, no exception crosses the ABI, statuses
 * are dnnl_status_t values, an executable must not outlive its compiler.
 * `data` may be a host pointer (the reference's only mode: inputs are copied
 * to the GPU and outputs copied back) or a device pointer (used in place).
 * execute() returns after the work has completed.
 */
#ifndef DNNL_GRAPH_COMPILER_H
#define DNNL_GRAPH_COMPILER_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
#pragma GCC visibility push(default)

#define DNNL_GC_API_V_MAJOR 0
#define DNNL_GC_API_V_MINOR 1
#define DNNL_GC_API_V_PATCH 0
#define DNNL_GC_API_V_HASH "N/A"

#ifndef DNNL_MAX_NDIMS
#define DNNL_MAX_NDIMS 12
#endif

/* dnnl_status_t values of oneDNN (oneapi/dnnl/dnnl_common_types.h) */
#ifndef DNNL_COMMON_TYPES_H
typedef enum {
  dnnl_success = 0,
  dnnl_out_of_memory = 1,
  dnnl_invalid_arguments = 2,
  dnnl_unimplemented = 3,
  dnnl_last_impl_reached = 4,
  dnnl_runtime_error = 5,
  dnnl_not_required = 6,
  dnnl_invalid_graph = 7,
  dnnl_invalid_graph_op = 8,
  dnnl_invalid_shape = 9,
  dnnl_invalid_data_type = 10
} dnnl_status_t;
#endif

struct dnnl_graph_compiler;
struct dnnl_graph_compiler_executable;

struct dnnl_graph_compiler_version {
  struct version {
    uint8_t major;
    uint8_t minor;
    uint8_t patch;
    const char *hash;
  } api_version, gc_version;
};

struct dnnl_graph_compiler_context {
  uint32_t num_threads; /* kept for source compatibility; the GPU path ignores it */
};

struct dnnl_graph_compiler_tensor {
  size_t id;
  uint8_t ndims;
  int64_t *dims;
  void *data;
};

/* src/dnnl/dnnl_graph_compiler.cpp:157-167 */
const struct dnnl_graph_compiler_version *dnnl_graph_compiler_get_version(void);
/* :169-183 -- ctx may be NULL */
dnnl_status_t dnnl_graph_compiler_create(const struct dnnl_graph_compiler_context *ctx,
                                         const struct dnnl_graph_compiler **gc);
/* :185-188 */
void dnnl_graph_compiler_destroy(const struct dnnl_graph_compiler *gc);
/* :190-207 -- malformed graph: dnnl_invalid_graph; unsupported op, dtype,
 * engine or attribute type: dnnl_unimplemented; failed verification or device
 * error: dnnl_runtime_error */
dnnl_status_t dnnl_graph_compiler_compile(const struct dnnl_graph_compiler *gc, const char *graph_json,
                                          const struct dnnl_graph_compiler_executable **exe);
/* :209-212 */
void dnnl_graph_compiler_destroy_executable(const struct dnnl_graph_compiler_executable *exe);
/* :214-226 -- inputs/outputs hold as many entries as the graph has inputs and
 * outputs; a missing id or ndims > DNNL_MAX_NDIMS: dnnl_runtime_error */
dnnl_status_t dnnl_graph_compiler_execute(const struct dnnl_graph_compiler_executable *exe,
                                          struct dnnl_graph_compiler_tensor *inputs,
                                          struct dnnl_graph_compiler_tensor *outputs);

/* No counterpart in the reference, whose execute runs on CPU threads and returns
 * when they are done.  For callers that keep their tensors on the GPU (a serving
 * loop, a framework with its own streams): the launches of execute on `stream`
 * (a hipStream_t; NULL is the default stream), ordered with the caller's other
 * work there, without waiting for them.  Every tensor's data must be a device
 * pointer (a host pointer: dnnl_invalid_arguments, and nothing is launched).
 * An executable keeps its intermediates in one
 * arena: calls on one executable must follow one another on one stream, or be
 * ordered by the caller with events. */
dnnl_status_t dnnl_graph_compiler_execute_async(const struct dnnl_graph_compiler_executable *exe,
                                                struct dnnl_graph_compiler_tensor *inputs,
                                                struct dnnl_graph_compiler_tensor *outputs, void *stream);

/* Host-side stages only (parse, verify, fuse, plan): writes the kernel launch
 * plan of the partition, one line per launch, into buf (NUL terminated,
 * truncated to len) and returns the status compile would return for these
 * stages.  Needs no GPU.  No counterpart in the reference, whose equivalent is
 * printing the IR after the pass pipeline (gc-opt --gc-cpu-pipeline). */
dnnl_status_t dnnl_graph_compiler_explain(const char *graph_json, char *buf, size_t len);

/* compile / explain for a module in MLIR's textual form: one func.func over
 * ranked tensors made of tensor.empty, arith.constant, linalg.{fill, matmul,
 * matmul_transpose_a/b, batch_matmul, batch_matmul_transpose_a/b, matvec,
 * vecmat, dot, batch_matvec, batch_vecmat, batch_reduce_matmul, add, sub, mul,
 * div, max, min, powf, negf, exp, copy, abs, ceil, floor, erf, log, round,
 * rsqrt, sqrt, square, tanh, reciprocal, broadcast, transpose, softmax,
 * reduce(addf), generic (a contraction or a single point-wise op)} and
 * tensor.{collapse,expand}_shape -- the subset of the reference's benchgc
 * cases (test/benchgc/cases/{llama2,generic}.mlir), its MLP pattern
 * (test/benchgc/src/benchgc/pattern/mlp.py) and the element-wise, binary and
 * matmul cases of its linalg driver (test/benchgc/src/benchgc/linalg/); and
 * the ops of the reference's front-end dialect, onednn_graph.{matmul, add, mul,
 * sub, div, relu, sigmoid, pow, type_cast, reduce_sum, reduce_mean}
 * (test/mlir/test/gc/Dialect/OneDNNGraph/).  The first function of the text is
 * compiled.  Takes over what gc-cpu-runner /
 * benchgc `--driver mlir` do with such a module on the CPU
 * (src/gc-cpu-runner/gc-cpu-runner.cpp, test/benchgc/src/benchgc/runner.py).
 * Tensor ids for execute: function argument i has id i, result j has id
 * (number of arguments) + j.  Anything outside the subset: dnnl_unimplemented. */
dnnl_status_t dnnl_graph_compiler_compile_mlir(const struct dnnl_graph_compiler *gc, const char *module_text,
                                               const struct dnnl_graph_compiler_executable **exe);
dnnl_status_t dnnl_graph_compiler_explain_mlir(const char *module_text, char *buf, size_t len);

/* Groups of point-wise ops (with an optional row sum inside) that the plan runs
 * as one launch get a kernel of their own when the partition is compiled: HIP
 * source written for the group's exact shapes, strides, types and ops, and
 * compiled with hiprtc -- the counterpart of the reference lowering each fused
 * group to its own loop nest and compiling it with LLVM
 * (lib/gc/Transforms/Pipeline.cpp:152-194,
 * lib/gc/ExecutionEngine/Driver/Driver.cpp:63-82).  The generated kernels give
 * the same bits as the library's generic kernels for such groups, which stay
 * in place when hiprtc is missing, when GCMI_NO_GENERATED_KERNELS=1 is set, or
 * when an operand is not 16-byte aligned.
 * ..._generated_source_mlir writes that source for a module (as accepted by
 * compile_mlir) into buf without touching a GPU; with check_arch (for example
 * "gfx950") it also compiles it and returns dnnl_runtime_error with the
 * compiler's log as last error if that fails.
 * ..._generated_kernel_launches counts the launches of generated kernels in
 * this process so far. */
dnnl_status_t dnnl_graph_compiler_generated_source_mlir(const char *module_text, const char *check_arch, char *buf, size_t len);
long dnnl_graph_compiler_generated_kernel_launches(void);

/* Text of the last error raised on the calling thread by the functions above
 * (no counterpart in the reference, which prints to stderr in debug builds). */
const char *dnnl_graph_compiler_last_error(void);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif
#endif /* DNNL_GRAPH_COMPILER_H */
