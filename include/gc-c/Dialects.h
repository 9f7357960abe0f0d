/*
 * gc-c/Dialects.h -- symbol-compatible shims of the reference's MLIR-C dialect
 * registration hooks (include/gc-c/Dialects.h:28-31 of intel/graph-compiler:
 * MLIR_DECLARE_CAPI_DIALECT_REGISTRATION(OneDNNGraph, onednn_graph) and
 * (CPURuntime, cpuruntime)).  There is no MLIR in this library: the handles
 * are null and registering them is a no-op.  They exist so that a host that
 * links these names still links; they are not a compile/execute path (that is
 * dnnl_graph_compiler.h).
 */
#ifndef GC_C_DIALECTS_H
#define GC_C_DIALECTS_H
#ifdef __cplusplus
extern "C" {
#endif
#pragma GCC visibility push(default)
typedef struct MlirDialectHandle {
  const void *ptr;
} MlirDialectHandle;
MlirDialectHandle mlirGetDialectHandle__onednn_graph__(void);
MlirDialectHandle mlirGetDialectHandle__cpuruntime__(void);
#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif
#endif
