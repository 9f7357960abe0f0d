"""The reference harness's matmul-driver fill and compare rule, restated (CPU tests).
test/benchgc/src/benchgc/arg/matmul.py:104-173, test/benchgc/src/benchgc/arg/compare.py:60-137."""
import numpy as np
import pytest
import torch

from conftest import mistrusted, strict_failures


@pytest.mark.parametrize("dtype,K", [(torch.float32, 512), (torch.float32, 4096), (torch.bfloat16, 64),
                                     (torch.bfloat16, 4096)])
def test_fill_is_integer_valued_and_sums_are_exact(wl, orc, dtype, K):
    M, N = 48, 40
    A = wl.benchgc_matmul_fill("src", (M, K), dtype, dtype, K)
    B = wl.benchgc_matmul_fill("wei", (K, N), dtype, dtype, K)
    assert A.dtype == dtype and B.dtype == dtype
    Ad, Bd = A.double(), B.double()
    assert (Ad == Ad.round()).all() and (Bd == Bd.round()).all()
    lim_a, lim_b = (64, 128) if dtype == torch.float32 else (4, 8)
    assert Ad.min() >= -lim_a and Ad.max() < lim_a + 1 and Bd.min() >= -lim_b and Bd.max() < lim_b + 1
    assert A.flatten()[0] > 0 and B.flatten()[0] > 0  # matmul.py:144-146
    # weight density min(2^digits / (max_src * max_wei) / K, 1): 2048/K for f32, 8/K for bf16
    want = min((2048 if dtype == torch.float32 else 8) / K, 1.0) * (1 - 1 / (2 * lim_b))  # randint draws 0 too
    got = float((Bd != 0).double().mean())
    assert abs(got - want) < 0.25 * want + 0.01
    exact = (Ad @ Bd).numpy()
    if dtype == torch.float32:
        ref = orc.matmul_f32(A.numpy(), B.numpy())
    else:
        ref = orc.bf16_to_f32(orc.matmul_bf16(wl.bf16_bits(A), wl.bf16_bits(B)))
    assert np.array_equal(ref, exact)  # what the density rule is for: no rounding anywhere
    thr = 1e-6 if dtype == torch.float32 else 2.0 ** -7
    assert not strict_failures(orc, ref, exact.astype(np.float32), thr).any()
    assert not mistrusted(ref, 90.0)


def test_fill_is_seeded_like_the_driver(wl):
    a1 = wl.benchgc_matmul_fill("src", (8, 16), torch.float32, torch.float32, 16)
    a2 = wl.benchgc_matmul_fill("src", (8, 16), torch.float32, torch.float32, 16)
    b1 = wl.benchgc_matmul_fill("wei", (16, 8), torch.float32, torch.float32, 16)
    assert torch.equal(a1, a2) and not torch.equal(a1, b1.t())
    torch.manual_seed(0)  # src: seed 0, bernoulli(1.0) * randint(-64, 64)
    want = torch.bernoulli(torch.full((8, 16), 1.0)) * torch.randint(-64, 64, (8, 16))
    assert torch.equal(a1.flatten()[1:], want.flatten()[1:].float())


def test_strict_rule_and_mistrust(orc):
    ref = np.array([1.0, -2.0, 1e-6, 0.0, np.inf, np.nan, 100.0, 5e-6], np.float32)
    res = np.array([1.0 + 5e-7, -2.0, 2e-6, 1e-7, np.inf, np.nan, 100.1, -5e-6], np.float32)
    bad = strict_failures(orc, ref, res, 1e-6)
    # 1e-6 vs 2e-6: |ref| <= 1e-5 -> absolute 1e-6 passes; 100 vs 100.1 fails; 5e-6 vs -5e-6: absolute 1e-5 fails
    assert bad.tolist() == [False, False, False, False, False, False, True, True]
    assert strict_failures(orc, np.array([np.inf], np.float32), np.array([-np.inf], np.float32), 1.0).all()
    z = np.zeros(100, np.float32)
    z[:9] = 1
    assert mistrusted(z, 90.0) and not mistrusted(np.ones(100, np.float32), 90.0)
    assert not mistrusted(np.zeros(5, np.float32), 90.0)  # fewer than 10 elements: never mistrusted
