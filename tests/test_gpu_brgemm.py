"""GPU parity of the microkernel ABI (dnnl_brgemm_*, device pointers) against
the golden vectors of the reference's naive brgemm and against the oracle on the
shapes of the reference's runtime unit test
(test/mlir/unittests/ExecutionEngine/BrgemmRuntime.cpp:146-206)."""
import ctypes as C
import os

import numpy as np
import pytest
import torch

from conftest import ROOT

pytestmark = pytest.mark.gpu
BF16, F32, S8, U8 = 2, 3, 5, 6


def _run(gc, dev, p, beta, A, B, C0):
    M, N, K, LDA, LDB, LDC, sa, sb, dtA, dtB, num, ao, bo, co = (int(v) for v in p)
    L = gc.lib()

    def up(a):
        return torch.from_numpy(a.view(np.uint8).copy()).to(dev)

    Ad, Bd, Cd = up(A), up(B), up(C0)
    h = L.dnnl_brgemm_dispatch(M, N, K, LDA, LDB, LDC, sa, sb, beta, dtA, dtB)
    assert h >= 0
    L.dnnl_brgemm_tileconfig(h)
    L.dnnl_brgemm_execute(h, C.c_void_p(Ad.data_ptr()), ao, C.c_void_p(Bd.data_ptr()), bo, C.c_void_p(Cd.data_ptr()), co, num)
    L.dnnl_brgemm_tilerelease()
    torch.cuda.synchronize()
    return Cd.cpu().numpy().view(C0.dtype)


def test_golden_vectors(gc, dev):
    z = np.load(os.path.join(ROOT, "tests", "golden", "brgemm_golden.npz"))
    for i in range(int(z["n_cases"])):
        k = "c%03d_" % i
        p, beta = z[k + "params"], float(z[k + "beta"])
        got = _run(gc, dev, p, beta, z[k + "A"], z[k + "B"], z[k + "C0"])
        # LDC > N: `Cwin` = exactly the M x N window overwritten (beta == 0) or accumulated into, the sums in the
        # reference's order.  That is the documented contract of include/gc_brgemm.h and what the reference's oneDNN
        # back end does; the naive runtime's beta == 0 clears M*N elements densely instead
        # (BrgemmNaive.cpp:36-44), a result the oracle restates (`C`) and the GPU deliberately does not.
        want = z[k + "Cwin"] if (k + "Cwin") in z.files else z[k + "C"]
        # bit for bit, floats included (the reference's own test allows rtol 1e-4 / atol 1e-6,
        # BrgemmRuntime.cpp:38-39): the kernel sums in the reference's order without fused multiply-adds
        assert (got.view(np.uint32) == want.view(np.uint32)).all(), "golden case %d" % i
        if (k + "Cwin") in z.files:  # nothing outside the window is touched
            M, N, LDC, co = int(p[0]), int(p[1]), int(p[5]), int(p[13])
            outside = np.ones(got.shape, bool)
            for m in range(M):
                outside[co + m * LDC:co + m * LDC + N] = False
            assert (got.view(np.uint32)[outside] == z[k + "C0"].view(np.uint32)[outside]).all(), "golden case %d padding" % i


@pytest.mark.parametrize("dtA,dtB", [(F32, F32), (BF16, BF16), (U8, S8)])
@pytest.mark.parametrize("beta", [0.0, 1.0])
def test_reference_unit_test_shapes(gc, orc, dev, dtA, dtB, beta):
    rng = np.random.default_rng(4)
    batch, M, N, K = 4, 32, 32, 32
    if dtA == F32:
        A = (rng.random(batch * M * K) * 10 - 10).astype(np.float32)
        B = (rng.random(batch * K * N) * 10 - 10).astype(np.float32)
    elif dtA == BF16:
        A = orc.f32_to_bf16((rng.random(batch * M * K) * 10 - 10).astype(np.float32))
        B = orc.f32_to_bf16((rng.random(batch * K * N) * 10 - 10).astype(np.float32))
    else:
        A = rng.integers(0, 100, batch * M * K).astype(np.uint8)
        B = rng.integers(-100, 0, batch * K * N).astype(np.int8)
    C0 = (rng.random(M * N) * 10 - 10).astype(np.float32) if dtA != U8 else rng.integers(-500, 0, M * N).astype(np.int32)
    p = [M, N, K, 32, 32, 32, 1024, 1024, dtA, dtB, batch, 0, 0, 0]
    want = C0.copy()
    orc.brgemm(M, N, K, 32, 32, 32, 1024, 1024, beta, dtA, dtB, A, 0, B, 0, want, 0, batch)
    got = _run(gc, dev, p, beta, A, B, C0)
    assert (got.view(np.uint32) == want.view(np.uint32)).all()
