"""CPU: the oracle's batch-reduce GEMM against (1) golden vectors produced by the
reference's own BrgemmNaive.cpp, (2) that compiled reference live when
oracle/_ref exists, (3) the closed forms of the reference's lit execution tests
and (4) textbook GEMM in f64 / int64 on unpacked operands."""
import ctypes as C
import os

import numpy as np
import pytest

from conftest import ROOT

BF16, F32, S8, U8 = 2, 3, 5, 6
GOLDEN = os.path.join(ROOT, "tests", "golden", "brgemm_golden.npz")


def _cases():
    z = np.load(GOLDEN)
    for i in range(int(z["n_cases"])):
        k = "c%03d_" % i
        yield i, z[k + "params"], float(z[k + "beta"]), z[k + "A"], z[k + "B"], z[k + "C0"], z[k + "C"]


def test_golden_vectors_bit_exact(orc):
    n = 0
    for i, p, beta, A, B, C0, Cref in _cases():
        M, N, K, LDA, LDB, LDC, sa, sb, dtA, dtB, num, ao, bo, co = (int(v) for v in p)
        Cb = C0.copy()
        orc.brgemm(M, N, K, LDA, LDB, LDC, sa, sb, beta, dtA, dtB, A, ao, B, bo, Cb, co, num)
        assert Cb.tobytes() == Cref.tobytes(), "golden case %d (dt %d,%d M%d N%d K%d beta %g)" % (i, dtA, dtB, M, N, K, beta)
        n += 1
    assert n == 108  # 84 with LDC == N, 24 with LDC > N (beta == 0 there: the naive runtime's dense M*N clear)


def test_matches_compiled_reference_live(orc):
    ref = orc.ref_lib()
    if ref is None:
        pytest.skip("oracle/_ref not built (reference tree absent on this machine)")
    rng = np.random.default_rng(7)
    NP = {F32: np.float32, BF16: np.uint16, S8: np.int8, U8: np.uint8}
    for dtA, dtB in [(F32, F32), (BF16, BF16), (U8, S8), (S8, S8), (U8, U8), (S8, U8)]:
        v = 1 if dtA == F32 else (2 if dtA == BF16 else 4)
        for _ in range(6):
            M, N, K = (int(x) for x in rng.integers(1, 40, 3))
            num = int(rng.integers(1, 5))
            LDA, LDB, LDC = K + int(rng.integers(0, 3)), N + int(rng.integers(0, 3)), N
            Kp = -(-K // v) * v
            sa, sb = M * LDA, (Kp // v) * LDB * v
            beta = float(rng.integers(0, 2))

            def gen(dt, n):
                if dt == F32:
                    return rng.standard_normal(n).astype(np.float32)
                if dt == BF16:
                    return orc.f32_to_bf16(rng.standard_normal(n).astype(np.float32))
                lo, hi = (-128, 128) if dt == S8 else (0, 256)
                return rng.integers(lo, hi, n).astype(NP[dt])

            A, B = gen(dtA, num * sa + 4), gen(dtB, num * sb + 4)
            C0 = rng.standard_normal(M * LDC).astype(np.float32) if v <= 2 else rng.integers(-9, 9, M * LDC).astype(np.int32)
            mine, theirs = C0.copy(), C0.copy()
            orc.brgemm(M, N, K, LDA, LDB, LDC, sa, sb, beta, dtA, dtB, A, 0, B, 0, mine, 0, num)
            h = ref.dnnl_brgemm_dispatch(M, N, K, LDA, LDB, LDC, sa, sb, C.c_float(beta), dtA, dtB)
            ref.dnnl_brgemm_execute(h, A.ctypes.data_as(C.c_void_p), 0, B.ctypes.data_as(C.c_void_p), 0,
                                    theirs.ctypes.data_as(C.c_void_p), 0, num)
            assert mine.tobytes() == theirs.tobytes()


def test_lit_closed_form_f32(orc):
    """test/mlir/test/gc/cpu-runner/brgemm-simple-for.mlir:17-60: A == 1, B == 2,
    C starts at -64*i*j, batch 16 of 32x32x32, then +3 and ReLU:
    value(i,j) = max(0, 1027 - 64*i*j)."""
    A = np.ones(4 * 16 * 32 * 32, np.float32)
    B = np.full(8 * 16 * 32 * 32, 2.0, np.float32)
    for i in range(4):
        for j in range(8):
            Cb = np.full(32 * 32, -64.0 * i * j, np.float32)
            orc.brgemm(32, 32, 32, 32, 32, 32, 1024, 1024, 1.0, F32, F32, A, i * 16 * 1024, B, j * 16 * 1024, Cb, 0, 16)
            out = np.maximum(Cb + 3.0, 0.0)
            assert (out == max(0.0, 1027.0 - 64.0 * i * j)).all()
    # first CHECK lines of the file: 1027, 963, 899 on row i=1
    assert [max(0.0, 1027.0 - 64.0 * j) for j in range(3)] == [1027.0, 963.0, 899.0]


def test_lit_closed_form_bf16_vnni(orc):
    """test/mlir/test/gc/cpu-runner/brgemm-multilevel-for.mlir:17-41: the same
    with bf16 operands, B as memref<8x16x16x32x2xbf16> (VNNI-2)."""
    one, two = orc.f32_to_bf16(np.float32(1.0)), orc.f32_to_bf16(np.float32(2.0))
    A = np.full(4 * 16 * 32 * 32, one, np.uint16)
    B = np.full(8 * 16 * 16 * 32 * 2, two, np.uint16)
    for i in (0, 1, 3):
        for j in (0, 2, 7):
            Cb = np.full(32 * 32, -64.0 * i * j, np.float32)
            orc.brgemm(32, 32, 32, 32, 32, 32, 1024, 1024, 1.0, BF16, BF16, A, i * 16 * 1024, B, j * 16 * 1024, Cb, 0, 16)
            assert (np.maximum(Cb + 3.0, 0.0) == max(0.0, 1027.0 - 64.0 * i * j)).all()


def _unpack_vnni(Bv, K, N, LDB, v):
    """logical (k,n) from the VNNI formula of BrgemmNaive.cpp:71-140."""
    out = np.zeros((K, N), Bv.dtype)
    for k in range(K):
        for n in range(N):
            out[k, n] = Bv[(k - k % v) * LDB + v * n + k % v]
    return out


@pytest.mark.parametrize("dtA,dtB", [(U8, S8), (S8, S8), (U8, U8), (S8, U8)])
@pytest.mark.parametrize("K", [32, 29, 7])
def test_int8_equals_int64_textbook(orc, dtA, dtB, K):
    rng = np.random.default_rng(K * 10 + dtA + dtB)
    NP = {S8: np.int8, U8: np.uint8}
    M, N, num, LDA, LDB, LDC = 9, 11, 3, K + 2, 13, 11
    Kp = -(-K // 4) * 4
    sa, sb = M * LDA + 1, (Kp // 4) * LDB * 4
    A = rng.integers(*((-128, 128) if dtA == S8 else (0, 256)), num * sa).astype(NP[dtA])
    B = rng.integers(*((-128, 128) if dtB == S8 else (0, 256)), num * sb).astype(NP[dtB])
    C0 = rng.integers(-100, 100, M * LDC).astype(np.int32)
    for beta in (0.0, 1.0):
        Cb = C0.copy()
        orc.brgemm(M, N, K, LDA, LDB, LDC, sa, sb, beta, dtA, dtB, A, 0, B, 0, Cb, 0, num)
        want = np.zeros((M, N), np.int64) if beta == 0 else C0.reshape(M, LDC)[:, :N].astype(np.int64)
        for i in range(num):
            a = A[i * sa:i * sa + M * LDA].reshape(M, LDA)[:, :K].astype(np.int64)
            b = _unpack_vnni(B[i * sb:i * sb + sb], K, N, LDB, 4).astype(np.int64)
            want = want + a @ b
        assert (Cb.reshape(M, LDC)[:, :N] == want).all()


@pytest.mark.parametrize("dt", [F32, BF16])
def test_fp_close_to_f64_textbook(orc, dt):
    rng = np.random.default_rng(3)
    M, N, K, num = 17, 19, 33, 4
    v = 1 if dt == F32 else 2
    LDA, LDB, LDC = K, N, N
    Kp = -(-K // v) * v
    sa, sb = M * LDA, (Kp // v) * LDB * v
    if dt == F32:
        A = rng.standard_normal(num * sa).astype(np.float32)
        B = rng.standard_normal(num * sb).astype(np.float32)
        Af, Bf = A, B
    else:
        A = orc.f32_to_bf16(rng.standard_normal(num * sa).astype(np.float32))
        B = orc.f32_to_bf16(rng.standard_normal(num * sb).astype(np.float32))
        Af, Bf = orc.bf16_to_f32(A), orc.bf16_to_f32(B)
    Cb = np.zeros(M * LDC, np.float32)
    orc.brgemm(M, N, K, LDA, LDB, LDC, sa, sb, 0.0, dt, dt, A, 0, B, 0, Cb, 0, num)
    want = np.zeros((M, N))
    for i in range(num):
        a = Af[i * sa:(i + 1) * sa].reshape(M, LDA).astype(np.float64)
        b = _unpack_vnni(Bf[i * sb:(i + 1) * sb], K, N, LDB, v).astype(np.float64) if v > 1 else \
            Bf[i * sb:(i + 1) * sb].reshape(K, LDB).astype(np.float64)
        want += a @ b
    assert np.allclose(Cb.reshape(M, N), want, rtol=1e-5, atol=1e-4)


def test_unsupported_pair_is_an_error(orc):
    z = np.zeros(16, np.float32)
    with pytest.raises(ValueError):
        orc.brgemm(2, 2, 2, 2, 2, 2, 4, 4, 0.0, F32, BF16, z, 0, z, 0, z, 0, 1)
