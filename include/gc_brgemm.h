/*
 * gc_brgemm.h -- the reference's runtime microkernel ABI, device-pointer
 * edition.  Same four symbols, argument meaning and handle protocol as
 * include/gc/ExecutionEngine/CPURuntime/Microkernel/BrgemmInterface.h:31-63 of
 * the intel/graph-compiler tree, so generated code and the reference's own
 * runtime unit test (test/mlir/unittests/ExecutionEngine/BrgemmRuntime.cpp)
 * translate one to one.  A, B and C are DEVICE pointers here.
 *
 *   C[m*LDC+n] = (beta == 0 ? 0 : C[m*LDC+n])
 *              + sum_{i<num} sum_{k<K} A[A_off + i*stride_a + m*LDA + k] * b(i,k,n)
 *   f32 : b = B[B_off + i*stride_b + k*LDB + n]
 *   bf16: b = B[B_off + i*stride_b + (k-k%2)*LDB + 2n + k%2]   (VNNI-2)
 *   8bit: b = B[B_off + i*stride_b + (k-k%4)*LDB + 4n + k%4]   (VNNI-4)
 * C is f32 for f32/bf16 inputs and s32 for 8-bit inputs; all offsets, leading
 * dimensions and batch strides are in elements; dtypes are dnnl_data_type_t
 * values (bf16 2, f32 3, s8 5, u8 6).  With beta == 0 the LDC-strided M x N
 * block is overwritten (the behaviour of the reference's oneDNN back-end,
 * lib/gc/ExecutionEngine/CPURuntime/Microkernel/BrgemmOnednn.cpp:94-98).  The
 * reference's naive fallback runtime differs when LDC > N: its beta == 0 clears
 * the first M*N elements of C densely (BrgemmNaive.cpp:36-44), so rows past
 * M*N/LDC are accumulated into and the padding in front of them is cleared; that
 * is not reproduced here (tests/golden holds both results for such cases).
 *
 * Handles are small dense integers from a process-wide table that is never
 * freed; dispatch is thread safe and may run from static constructors.  An
 * invalid handle or unsupported dtype pair makes dispatch return -1 and
 * execute do nothing (the reference asserts).  execute launches on the HIP
 * default stream and returns without waiting.
 */
#ifndef GC_BRGEMM_H
#define GC_BRGEMM_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
#pragma GCC visibility push(default)

/* BrgemmInterface.h:31-35 */
int64_t dnnl_brgemm_dispatch(int64_t M, int64_t N, int64_t K, int64_t LDA, int64_t LDB, int64_t LDC, int64_t stride_a,
                             int64_t stride_b, float beta, int64_t dtypeA, int64_t dtypeB);
/* BrgemmInterface.h:42 -- AMX tile state has no GPU counterpart: no-op */
void dnnl_brgemm_tileconfig(int64_t kernel);
/* BrgemmInterface.h:49 -- no-op */
void dnnl_brgemm_tilerelease(void);
/* BrgemmInterface.h:60-63 */
void dnnl_brgemm_execute(int64_t kernel, void *A, uint64_t A_offset, void *B, uint64_t B_offset, void *C,
                         uint64_t C_offset, int num);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif
#endif /* GC_BRGEMM_H */
