"""CPU: post-op semantics and the composite partition oracles."""
import math

import numpy as np
import torch


def test_gelu_erf_matches_torch_and_constant_bits(orc):
    x = np.linspace(-8, 8, 20001).astype(np.float32)
    got = orc.gelu(x, "erf")
    want = torch.nn.functional.gelu(torch.from_numpy(x).double(), approximate="none").numpy()
    assert np.abs(got - want).max() < 5e-7
    assert np.array([0x3f3504f3], np.uint32).view(np.float32)[0] == np.float32(0.70710677)  # gelu.cpp:113
    assert orc.gelu(np.array([0.0], np.float32))[0] == 0.0


def test_gelu_tanh_matches_torch(orc):
    x = np.linspace(-8, 8, 20001).astype(np.float32)
    got = orc.gelu(x, "tanh")
    want = torch.nn.functional.gelu(torch.from_numpy(x).double(), approximate="tanh").numpy()
    assert np.abs(got - want).max() < 2e-6


def test_sigmoid_relu_closed_forms_of_reference_api_tests(orc):
    """test/dnnl/TestApiOps.cpp:183-201 (relu on i-64) and :278-297 (sigmoid)."""
    x = (np.arange(128) - 64).astype(np.float32)
    assert (orc.relu(x) == np.where(x < 0, 0, x)).all()
    want = (1.0 / (1.0 + np.exp(-x.astype(np.float32)))).astype(np.float32)
    assert np.allclose(orc.sigmoid(x), want, rtol=1e-6, atol=0)
    assert np.isnan(orc.relu(np.array([np.nan], np.float32))[0])  # maximumf propagates NaN


def test_matmul_transpose_a_bias_closed_form(orc):
    """test/dnnl/TestApiOps.cpp:69-119: A[i][j]=i+j (128x512, transpose_a),
    B[i][j]=i-j (128x64), bias[j]=j; every product and sum is an exact integer."""
    i, j = np.meshgrid(np.arange(128), np.arange(512), indexing="ij")
    A = (i + j).astype(np.float32)
    i, j = np.meshgrid(np.arange(128), np.arange(64), indexing="ij")
    B = (i - j).astype(np.float32)
    bias = np.arange(64).astype(np.float32)
    got = orc.matmul_f32(A, B, bias, None, transpose_a=True)
    want = A.astype(np.int64).T @ B.astype(np.int64) + np.arange(64)
    assert np.abs(want).max() < 2 ** 24
    assert (got.astype(np.int64) == want).all() and got.shape == (512, 64)


def test_dequant_compensation_identity_in_int64(orc):
    """sum_k (a - zp) w == sum_k a w - zp * sum_k w (legacy/core/src/ops/
    matmul_core.cpp:546-557)."""
    rng = np.random.default_rng(2)
    M, K, N, zp = 48, 160, 96, 128
    A = rng.integers(0, 256, (M, K)).astype(np.uint8)
    W = rng.integers(-127, 128, (K, N)).astype(np.int8)
    scale = (rng.random(N) * 0.009 + 0.001).astype(np.float32)
    acc = orc.matmul_u8s8_acc(A, W)
    cs = orc.colsum_s8(W)
    assert (cs == W.astype(np.int64).sum(0)).all()
    got = orc.dequant_comp(acc, zp, cs, scale)
    centred = (A.astype(np.int64) - zp) @ W.astype(np.int64)
    want = centred.astype(np.float32) * scale[None, :]
    assert (got == want).all()


def test_int8_layer_composition(orc):
    rng = np.random.default_rng(3)
    M, K, N = 64, 128, 96
    A = rng.integers(0, 256, (M, K)).astype(np.uint8)
    W = rng.integers(-127, 128, (K, N)).astype(np.int8)
    scale = (rng.random(N) * 0.009 + 0.001).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    acc, y = orc.int8_layer(A, W, scale, bias, 128, "gelu_erf")
    assert (acc == A.astype(np.int64) @ W.astype(np.int64)).all()
    x = ((A.astype(np.float64) - 128) @ W.astype(np.float64)) * scale + bias
    want = torch.nn.functional.gelu(torch.from_numpy(x), approximate="none").to(torch.bfloat16).float().numpy()
    got = orc.bf16_to_f32(y)
    assert np.abs(got - want).max() <= np.abs(want).max() * 2 ** -7  # at most one bf16 ulp apart


def test_bf16_matmul_rounding_points_match_torch_bf16_ops(orc):
    """bf16 graph: round after matmul, after bias add, after relu
    (lib/gc/Transforms/Pipeline.cpp:79-95).  torch's bf16 add/relu do exactly
    widen-op-round; the matmul is reproduced by f32 mm of the widened inputs."""
    torch.manual_seed(0)
    A = torch.randn(96, 160).to(torch.bfloat16)
    B = torch.randn(160, 64).to(torch.bfloat16)
    bias = torch.randn(64).to(torch.bfloat16)

    def bits(t):
        return t.view(torch.int16).numpy().view(np.uint16)

    got = orc.bf16_to_f32(orc.matmul_bf16(bits(A), bits(B), bits(bias), "relu"))
    mm = (A.double() @ B.double()).float().to(torch.bfloat16)
    want = torch.relu(mm + bias).float().numpy()
    # f64 vs f32 accumulation can flip a rounding: allow one bf16 ulp, require near-total agreement
    assert np.abs(got - want).max() <= 2 ** -7 * np.abs(want).max()
    assert (got == want).mean() > 0.99


def test_compare_p2p_rule(orc):
    """test/benchgc/src/benchgc/arg/compare.py:79-93"""
    ref = np.array([1.0, 1e-6, np.nan, np.inf, -np.inf, 2.0], np.float32)
    res = np.array([1.005, 2e-6, np.nan, np.inf, np.inf, 2.0], np.float32)
    bad, md = orc.compare_p2p(ref, res, 1e-2)
    assert bad == 1  # only the -inf vs +inf pair fails; 1e-6 -> absolute rule
    bad, _ = orc.compare_p2p(ref[:2], res[:2], 1e-3)
    assert bad == 1  # 0.5% relative error on the first element


def test_compare_norm_rule(orc):
    """test/benchgc/src/benchgc/arg/compare.py:41-57: sqrt(sum (ref-res)^2 / sum ref^2) < thr, strictly; an empty
    tensor passes.  Hand-computed: ref (3, 4), res (3, 4.5): sqrt(0.25 / 25) = 0.1."""
    ok, v = orc.compare_norm(np.array([3.0, 4.0], np.float32), np.array([3.0, 4.5], np.float32), 0.11)
    assert ok and abs(v - 0.1) < 1e-7
    ok, v = orc.compare_norm(np.array([3.0, 4.0], np.float32), np.array([3.0, 4.5], np.float32), np.float32(v))
    assert not ok                                   # equal to the threshold: '<' fails
    ok, v = orc.compare_norm(np.array([1.0, -2.0], np.float32), np.array([1.0, -2.0], np.float32), 1e-30)
    assert ok and v == 0.0
    ok, _ = orc.compare_norm(np.array([1.0, -2.0], np.float32), np.array([1.0, -2.0], np.float32), 0.0)
    assert not ok                                   # 0 < 0 is false
    assert orc.compare_norm(np.zeros(0, np.float32), np.zeros(0, np.float32), 0.0) == (True, 0.0)
    ok, v = orc.compare_norm(np.array([1.0, 2.0], np.float32), np.array([1.0, np.nan], np.float32), 1.0)
    assert not ok and np.isnan(v)
    # a sign error or a swapped pair is a large norm, unlike under a loose per-element tolerance
    ref = np.arange(1, 9, dtype=np.float32)
    swapped = ref.copy()
    swapped[[0, 1]] = swapped[[1, 0]]
    assert abs(orc.compare_norm(ref, swapped, 1.0)[1] - np.sqrt(2.0 / 204.0)) < 1e-7
    # per row: rows are judged one by one
    ref2 = np.array([[3.0, 4.0], [1.0, 0.0], [0.0, 0.0]], np.float32)
    res2 = np.array([[3.0, 4.5], [1.0, 0.0], [0.0, 0.0]], np.float32)
    bad, l2 = orc.compare_norm_rows(ref2, res2, 0.05)
    assert bad == 2 and abs(l2[0] - 0.1) < 1e-7 and l2[1] == 0.0 and np.isnan(l2[2])  # 0/0: not a pass
    # against torch in float32, the arithmetic the harness itself uses
    import torch
    rng = np.random.default_rng(3)
    a = rng.standard_normal(10000).astype(np.float32)
    b = (a + 1e-3 * rng.standard_normal(10000)).astype(np.float32)
    ta, tb = torch.from_numpy(a), torch.from_numpy(b)
    want = torch.sqrt(torch.square(ta - tb).sum() / torch.square(ta).sum()).item()
    assert abs(orc.compare_norm(a, b, 1.0)[1] - want) <= 1e-6 * want
