/*
 * gc-c/Passes.h -- shim of mlirRegisterAllGCPassesAndPipelines
 * (include/gc-c/Passes.h:29, lib/gc/CAPI/Passes.cpp:30-34 of
 * intel/graph-compiler).  The pass pipeline has no counterpart here -- tile
 * selection and fusion happen when a partition is compiled -- so this does
 * nothing.
 */
#ifndef GC_C_PASSES_H
#define GC_C_PASSES_H
#ifdef __cplusplus
extern "C" {
#endif
#pragma GCC visibility push(default)
void mlirRegisterAllGCPassesAndPipelines(void);
#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif
#endif
