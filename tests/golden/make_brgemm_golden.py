"""Writes tests/golden/brgemm_golden.npz: input/output vectors of the reference's
own naive brgemm (lib/gc/ExecutionEngine/CPURuntime/Microkernel/BrgemmNaive.cpp),
compiled from the reference tree into oracle/_ref/ by oracle/Makefile.

Run in a container that has /root/reference:  python tests/golden/make_brgemm_golden.py
The fixture holds data only (operands, parameters, results); the oracle and the
GPU microkernel are both checked against it.
"""
import ctypes as C
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import gc_oracle as orc  # noqa: E402

BF16, F32, S8, U8 = 2, 3, 5, 6
NP = {F32: np.float32, BF16: np.uint16, S8: np.int8, U8: np.uint8}


def gen(rng, dt, n):
    if dt == F32:
        return (rng.random(n, dtype=np.float32) * 10 - 10).astype(np.float32)
    if dt == BF16:
        return orc.f32_to_bf16((rng.random(n, dtype=np.float32) * 10 - 10).astype(np.float32))
    if dt == S8:
        return rng.integers(-128, 128, n).astype(np.int8)
    return rng.integers(0, 256, n).astype(np.uint8)


def main():
    ref = orc.ref_lib()
    if ref is None:
        raise SystemExit("oracle/_ref/libbrgemm_naive_ref.so missing: run `make -C oracle ref` where the reference tree exists")
    rng = np.random.default_rng(20240607)
    cases = []
    # (M, N, K, LDA_pad, LDB_pad, LDC_pad, num, a_off, b_off, c_off)
    shapes = [
        (32, 32, 32, 0, 0, 0, 4, 0, 0, 0),      # the reference unit-test shape
        (8, 16, 32, 0, 0, 0, 1, 0, 0, 0),
        (5, 7, 9, 3, 2, 0, 3, 11, 8, 0),        # K tail, padded leading dims, offsets
        (4, 8, 30, 2, 0, 0, 2, 0, 4, 0),        # K % 4 == 2
        (3, 5, 31, 0, 1, 0, 2, 5, 0, 0),        # K % 4 == 3, K % 2 == 1
        (6, 4, 33, 1, 1, 0, 2, 0, 0, 0),        # K % 4 == 1
        (16, 16, 16, 0, 0, 0, 5, 0, 0, 7),      # C offset
    ]
    pairs = [(F32, F32), (BF16, BF16), (U8, S8), (S8, S8), (U8, U8), (S8, U8)]
    for (dtA, dtB) in pairs:
        v = 1 if dtA == F32 else (2 if dtA == BF16 else 4)
        for (M, N, K, pa, pb, pc, num, ao, bo, co) in shapes:
            for beta in (0.0, 1.0):
                LDA, LDB, LDC = K + pa, N + pb, N + pc
                Kp = -(-K // v) * v
                stride_a = M * LDA + 3
                stride_b = (Kp // v) * LDB * v + 2 * v if v > 1 else K * LDB + 1
                A = gen(rng, dtA, ao + num * stride_a + 8)
                B = gen(rng, dtB, bo + num * stride_b + 8)
                cdt = np.float32 if dtA in (F32, BF16) else np.int32
                if cdt == np.float32:
                    C0 = (rng.random(co + M * LDC + 8, dtype=np.float32) * 10 - 10).astype(np.float32)
                else:
                    C0 = rng.integers(-500, 500, co + M * LDC + 8).astype(np.int32)
                Cr = C0.copy()
                h = ref.dnnl_brgemm_dispatch(M, N, K, LDA, LDB, LDC, stride_a, stride_b, C.c_float(beta), dtA, dtB)
                ref.dnnl_brgemm_execute(h, A.ctypes.data_as(C.c_void_p), ao, B.ctypes.data_as(C.c_void_p), bo,
                                        Cr.ctypes.data_as(C.c_void_p), co, num)
                cases.append(dict(params=np.array([M, N, K, LDA, LDB, LDC, stride_a, stride_b, dtA, dtB, num, ao, bo, co],
                                                  np.int64), beta=np.float32(beta), A=A, B=B, C0=C0, C=Cr))
    # LDC > N (a C window inside a wider buffer).  With beta == 0 the naive runtime clears the first M*N elements of
    # the buffer DENSELY (BrgemmNaive.cpp:36-44), not the LDC-strided window: rows past M*N/LDC keep their old values
    # and are accumulated into, and the padding in front of them is cleared.  `C` holds that result (what the oracle
    # restates); `Cwin` holds the result of overwriting exactly the M x N window, which is what the reference's
    # oneDNN back end computes and what the GPU microkernel does: made by the same compiled reference with beta = 1
    # on a buffer whose window was cleared beforehand, so its sums are the reference's own, in its order.
    rng = np.random.default_rng(20240608)
    wide = [(5, 7, 9, 3, 2, 4, 3, 11, 8, 0), (16, 16, 16, 0, 0, 5, 2, 0, 0, 7)]
    for (dtA, dtB) in pairs:
        v = 1 if dtA == F32 else (2 if dtA == BF16 else 4)
        for (M, N, K, pa, pb, pc, num, ao, bo, co) in wide:
            for beta in (0.0, 1.0):
                LDA, LDB, LDC = K + pa, N + pb, N + pc
                Kp = -(-K // v) * v
                stride_a = M * LDA + 3
                stride_b = (Kp // v) * LDB * v + 2 * v if v > 1 else K * LDB + 1
                A = gen(rng, dtA, ao + num * stride_a + 8)
                B = gen(rng, dtB, bo + num * stride_b + 8)
                if dtA in (F32, BF16):
                    C0 = (rng.random(co + M * LDC + 8, dtype=np.float32) * 10 - 10).astype(np.float32)
                else:
                    C0 = rng.integers(-500, 500, co + M * LDC + 8).astype(np.int32)
                Cr, Cw = C0.copy(), C0.copy()
                h = ref.dnnl_brgemm_dispatch(M, N, K, LDA, LDB, LDC, stride_a, stride_b, C.c_float(beta), dtA, dtB)
                ref.dnnl_brgemm_execute(h, A.ctypes.data_as(C.c_void_p), ao, B.ctypes.data_as(C.c_void_p), bo,
                                        Cr.ctypes.data_as(C.c_void_p), co, num)
                if beta == 0.0:
                    for m in range(M):
                        Cw[co + m * LDC:co + m * LDC + N] = 0
                h1 = ref.dnnl_brgemm_dispatch(M, N, K, LDA, LDB, LDC, stride_a, stride_b, C.c_float(1.0), dtA, dtB)
                ref.dnnl_brgemm_execute(h1, A.ctypes.data_as(C.c_void_p), ao, B.ctypes.data_as(C.c_void_p), bo,
                                        Cw.ctypes.data_as(C.c_void_p), co, num)
                cases.append(dict(params=np.array([M, N, K, LDA, LDB, LDC, stride_a, stride_b, dtA, dtB, num, ao, bo, co],
                                                  np.int64), beta=np.float32(beta), A=A, B=B, C0=C0, C=Cr, Cwin=Cw))
    out = {}
    for i, c in enumerate(cases):
        for k, vv in c.items():
            out["c%03d_%s" % (i, k)] = vv
    out["n_cases"] = np.int64(len(cases))
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "brgemm_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, len(cases), "cases", os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
