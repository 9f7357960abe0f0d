"""CPU: softmax and the MHA composition of the oracle against torch in f64 and
against invariants of attention."""
import numpy as np
import torch


def _bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def _inputs(B, H, Sq, Sk, D, seed=0):
    torch.manual_seed(seed)
    Q = torch.randn(B, H, Sq, D).to(torch.bfloat16)
    K = torch.randn(B, H, Sk, D).to(torch.bfloat16)
    V = torch.randn(B, H, Sk, D).to(torch.bfloat16)
    return Q, K, V


def _torch_ref(Q, K, V, mask, scale):
    S = Q.double() @ K.double().transpose(-1, -2) * scale
    if mask is not None:
        S = S + mask.double()
    P = torch.softmax(S, -1)
    return (P @ V.double()).numpy()


def test_softmax_rows_matches_torch_and_sums_to_one(orc):
    rng = np.random.default_rng(0)
    x = (rng.standard_normal((37, 301)) * 5).astype(np.float32)
    got = orc.softmax_rows(x)
    want = torch.softmax(torch.from_numpy(x).double(), -1).numpy()
    assert np.abs(got - want).max() < 1e-6
    assert np.abs(got.sum(-1) - 1).max() < 1e-5
    big = orc.softmax_rows(np.array([[1000.0, 1000.0, -1000.0]], np.float32))  # stable form: no overflow
    assert np.allclose(big, [[0.5, 0.5, 0.0]])
    assert np.isnan(orc.softmax_rows(np.full((1, 4), -np.inf, np.float32))).all()  # as torch.softmax


def test_mha_matches_f64_composition(orc):
    Q, K, V = _inputs(1, 2, 96, 80, 128)
    scale = 1 / np.sqrt(128)
    for mask in (None, torch.triu(torch.full((96, 80), float("-inf")), diagonal=1),
                 torch.randn(96, 80)):
        got = orc.bf16_to_f32(orc.mha_bf16(_bits(Q), _bits(K), _bits(V), None if mask is None else mask.numpy(), scale))
        want = _torch_ref(Q, K, V, mask, scale)
        # two bf16 roundings (P and O): a couple of 2^-8 steps relative to the row scale
        assert np.abs(got - want).max() < 2 ** -6 * max(1.0, np.abs(want).max())
        assert np.sqrt(np.mean((got - want) ** 2)) < 3e-3


def test_causal_rows_ignore_future_keys(orc):
    Q, K, V = _inputs(1, 1, 64, 64, 128, seed=3)
    mask = torch.triu(torch.full((64, 64), float("-inf")), diagonal=1).numpy()
    scale = 1 / np.sqrt(128)
    base = orc.mha_bf16(_bits(Q), _bits(K), _bits(V), mask, scale)
    K2, V2 = K.clone(), V.clone()
    K2[:, :, 40:] = torch.randn(1, 1, 24, 128).to(torch.bfloat16) * 7
    V2[:, :, 40:] = torch.randn(1, 1, 24, 128).to(torch.bfloat16) * 7
    pert = orc.mha_bf16(_bits(Q), _bits(K2), _bits(V2), mask, scale)
    assert (base[:, :, :40] == pert[:, :, :40]).all()   # rows 0..39 never see keys >= 40
    assert (base[:, :, 41:] != pert[:, :, 41:]).any()
    # row 0 attends to key 0 only: output is V[0] exactly (softmax weight 1.0)
    assert (base[0, 0, 0] == _bits(V)[0, 0, 0]).all()


def test_key_permutation_leaves_output_unchanged_up_to_rounding(orc):
    Q, K, V = _inputs(1, 1, 32, 96, 128, seed=5)
    scale = 1 / np.sqrt(128)
    perm = torch.randperm(96)
    a = orc.bf16_to_f32(orc.mha_bf16(_bits(Q), _bits(K), _bits(V), None, scale))
    b = orc.bf16_to_f32(orc.mha_bf16(_bits(Q), _bits(K[:, :, perm]), _bits(V[:, :, perm]), None, scale))
    assert np.abs(a - b).max() <= 2 ** -7 * np.abs(a).max()


def test_fully_masked_row_is_nan(orc):
    Q, K, V = _inputs(1, 1, 4, 8, 128, seed=7)
    mask = np.zeros((4, 8), np.float32)
    mask[2, :] = -np.inf
    out = orc.bf16_to_f32(orc.mha_bf16(_bits(Q), _bits(K), _bits(V), mask, 0.1))
    assert np.isnan(out[0, 0, 2]).all() and not np.isnan(out[0, 0, [0, 1, 3]]).any()


def test_mha_f64_is_the_torch_composition_and_its_rounded_form_is_the_oracle(orc):
    """gco_mha_f64 without rounding equals the float64 torch composition to 1e-12; with the softmax weights rounded
    at the reference's point it reproduces gco_mha_bf16 once its result is rounded to bf16 (the f32 sums of the
    oracle differ from f64 by far less than a bf16 step: a handful of ties may fall the other way)."""
    Q, K, V = _inputs(1, 2, 96, 80, 128, seed=11)
    scale = 1 / np.sqrt(128)
    for mask in (None, torch.triu(torch.full((96, 80), float("-inf")), diagonal=1), torch.randn(96, 80)):
        m = None if mask is None else mask.numpy()
        exact = orc.mha_f64(_bits(Q), _bits(K), _bits(V), m, scale, False)
        assert np.abs(exact - _torch_ref(Q, K, V, mask, scale)).max() < 1e-12
        rounded = orc.mha_f64(_bits(Q), _bits(K), _bits(V), m, scale, True)
        got = orc.mha_bf16(_bits(Q), _bits(K), _bits(V), m, scale)
        want = orc.f32_to_bf16(rounded.astype(np.float32))
        differ = (got != want)
        assert differ.mean() < 5e-3
        S = Q.double() @ K.double().transpose(-1, -2) * scale + (0 if mask is None else mask.double())
        mag = (torch.softmax(S, -1) @ V.double().abs()).numpy()
        # where they differ: one bf16 step of the value, plus (a weight at a rounding tie that falls the other way in
        # f32 moves its whole row) one step of a weight times the terms' magnitude
        gap = np.abs(orc.bf16_to_f32(got).astype(np.float64) - orc.bf16_to_f32(want))
        assert (gap[differ] <= 2.0 ** -7 * np.abs(rounded[differ]) + 2.0 ** -8 * mag[differ]).all()
        # the rounding of P is what separates the two f64 forms: a few 2^-9 of the terms' magnitude
        assert (np.abs(rounded - exact) <= 2.0 ** -8 * mag).all() and np.abs(rounded - exact).max() > 0
