"""GPU parity under the reference harness's own acceptance rule.

Part 1: the matmul driver's fill (integer-valued, weight density chosen so every sum is exactly representable,
test/benchgc/src/benchgc/arg/matmul.py:104-148) and its STRICT point-to-point compare at its own thresholds
(1e-6 for f32, eps(bf16) = 2^-7 for bf16, mistrust above 90 % zeros, :160-173; compare.py:60-137), on whole-tile,
ragged, K-sliced and weight-streaming shapes.

Part 2: on the N(0,1) configurations the strict rule (threshold 1e-2, the stated bar) cannot hold for elements
that cancel to ~0: their f32 summation-order noise is relative to sum |a_i b_i|, not to the result.  The tests
count the strict failures, print the count, and assert that every one of them is such a cancellation: |ref| below
a stated fraction of sum |a_i b_i| (or of the magnitude that was rounded before a later op cancelled it)."""
import numpy as np
import pytest
import torch

from conftest import mistrusted, strict_failures

pytestmark = pytest.mark.gpu

EPS_BF16 = 2.0 ** -7
# |ref| of every strict failure must lie below this fraction of the element's sum |a_i b_i|
CANCEL_FRACTION = 1e-3


F32_SHAPES = [(128, 256, 512), (100, 130, 77), (512, 512, 2048), (64, 64, 4096), (1, 7, 5)]


@pytest.mark.parametrize("M,N,K", F32_SHAPES)
def test_f32_matmul_driver_fill_strict(gc, orc, wl, dev, M, N, K):
    A = wl.benchgc_matmul_fill("src", (M, K), torch.float32, torch.float32, K)
    B = wl.benchgc_matmul_fill("wei", (K, N), torch.float32, torch.float32, K)
    ref = orc.matmul_f32(A.numpy(), B.numpy())
    assert np.array_equal(ref, (A.double() @ B.double()).numpy())  # the fill makes every sum exact
    out = gc.gemm_f32(A.to(dev), B.to(dev)).cpu().numpy()
    bad = strict_failures(orc, ref, out, 1e-6)
    assert not bad.any(), "%d of %d beyond 1e-6" % (bad.sum(), bad.size)
    assert not mistrusted(out, 90.0)


# whole tiles (one-pass MFMA kernels), ragged (bounds-checked kernel), one tile row (K slices + second pass)
BF16_SHAPES = [(256, 256, 128), (512, 768, 1024), (1024, 1024, 4096), (300, 200, 100), (257, 511, 129),
               (32, 4096, 4096), (100, 2048, 1024), (256, 4096, 2048)]


@pytest.mark.parametrize("M,N,K", BF16_SHAPES)
@pytest.mark.parametrize("layout", ["kn", "nk"])
def test_bf16_matmul_driver_fill_strict(gc, orc, wl, dev, M, N, K, layout):
    A = wl.benchgc_matmul_fill("src", (M, K), torch.bfloat16, torch.bfloat16, K)
    B = wl.benchgc_matmul_fill("wei", (K, N), torch.bfloat16, torch.bfloat16, K)
    ref = orc.bf16_to_f32(orc.matmul_bf16(wl.bf16_bits(A), wl.bf16_bits(B)))
    assert np.array_equal(ref, (A.double() @ B.double()).numpy())  # exactly representable in bf16
    if layout == "kn":
        out = gc.gemm_bf16(A.to(dev), B.to(dev))
    else:  # the [N,K] layout: tile kernels with B staged like A, or the weight-streaming kernel for M <= 64
        out = gc.gemm_bf16_nt(A.to(dev), B.t().contiguous().to(dev))
    torch.cuda.synchronize()
    res = out.float().cpu().numpy()
    bad = strict_failures(orc, ref, res, EPS_BF16)
    assert not bad.any(), "%d of %d beyond eps(bf16)" % (bad.sum(), bad.size)
    assert np.array_equal(ref, res)  # stronger than the harness asks: exact
    assert not mistrusted(res, 90.0)


def test_bf16_matmul_driver_fill_strict_full_size(gc, orc, wl, dev):
    """Config 2's shape under the driver fill: all 16.7 M results against an exact f64 product."""
    n = 4096
    A = wl.benchgc_matmul_fill("src", (n, n), torch.bfloat16, torch.bfloat16, n)
    B = wl.benchgc_matmul_fill("wei", (n, n), torch.bfloat16, torch.bfloat16, n)
    out = gc.gemm_bf16(A.to(dev), B.to(dev))
    torch.cuda.synchronize()
    ref = (A.to(dev).double() @ B.to(dev).double()).float().cpu().numpy()  # integers below 2^8: exact in any order
    res = out.float().cpu().numpy()
    bad = strict_failures(orc, ref, res, EPS_BF16)
    assert not bad.any(), "%d of %d beyond eps(bf16)" % (bad.sum(), bad.size)
    assert not mistrusted(res, 90.0)
    rows = list(range(0, n, 300))
    assert np.array_equal(orc.bf16_to_f32(orc.matmul_bf16(wl.bf16_bits(A[rows]), wl.bf16_bits(B))), res[rows])


def _report(name, bad, ref, scale_sum):
    n = int(bad.sum())
    worst = float((np.abs(ref[bad]) / scale_sum[bad]).max()) if n else 0.0
    print("\n%s: strict rule (|ref-res|/|ref| <= 1e-2, absolute below 1e-5) fails on %d of %d elements; "
          "largest |ref| / sum|a_i b_i| among them %.2e" % (name, n, bad.size, worst))
    return worst


def test_config2_strict_failures_are_cancellations(gc, orc, wl, dev):
    """bf16 GEMM 4096^3, N(0, 0.1) data: 48 rows against the oracle under the strict rule."""
    A, B = wl.bf16_gemm()
    out = gc.gemm_bf16(A.to(dev), B.to(dev))
    torch.cuda.synchronize()
    rows = sorted(set(list(range(0, 4096, 256)) + list(range(255, 4096, 256)) + list(range(97, 4096, 331))))[:48]
    ref = orc.bf16_to_f32(orc.matmul_bf16(wl.bf16_bits(A[rows]), wl.bf16_bits(B)))
    res = out[rows].float().cpu().numpy()
    bad = strict_failures(orc, ref, res, 1e-2)
    scale_sum = (A[rows].double().abs() @ B.double().abs()).numpy()
    worst = _report("config 2", bad, ref, scale_sum)
    assert worst < CANCEL_FRACTION
    assert bad.sum() <= 0.01 * bad.size


def test_config3_strict_failures_are_gelu_tail_or_cancellations(gc, orc, wl, dev):
    """int8 MLP layer at full size (4096 x 4096 x 11008, dequantise + bias + GELU to bf16): 48 rows against the
    oracle under the strict rule at 1e-2, and under the harness's norm rule per row.  The accumulators are exact
    (tests/test_gpu_gemm.py), so whatever differs comes from the epilogue: the GPU forms acc * scale + bias as one
    fused multiply-add and evaluates GELU for a bf16 result as x * Phi(x) with Phi(-|x|) = 2^(-t q(t) - 1) (relative
    error below 2^-11.9 of the value, tail included).  A strict failure could only be (a) a pre-activation value x in
    the negative GELU tail, where the REFERENCE's gelu(x) = x/2 * (erf + 1) is a difference of nearly equal f32 numbers
    -- (erf + 1) < 2e-5 from x < -4.2 on; past x = -4.7 |gelu| < 1e-5 falls under the rule's absolute branch --, or
    (b) a cancellation of acc * scale against the bias.  (With the f32-grade erf this kernel used before, whose error
    is absolute, 6 of these 495,360 elements failed, all in that tail; with the relative form: none.)  Where the
    reference's erf has saturated (x < -5.5) it returns -0 and the GPU the tiny negative value GELU really has there
    (-5.9e-9 at x = -6, underflowing to -0 below x = -13): different bits, both zero to any tolerance."""
    A, W, scale, bias = wl.int8_mlp_layer()
    Ad, Wd = A.to(dev), W.to(dev)
    cs = gc.colsum_s8(Wd)
    out = gc.gemm_int8(Ad, Wd, cs, 128, scale.to(dev), bias.to(dev), "gelu_erf", gc.BF16)
    torch.cuda.synchronize()
    rows = sorted(set(list(range(0, 4096, 256)) + list(range(255, 4096, 256)) + list(range(97, 4096, 331))))[:48]
    acc, y = orc.int8_layer(A[rows].numpy(), W.numpy(), scale.numpy(), bias.numpy(), 128, "gelu_erf")
    ref = orc.bf16_to_f32(y)
    res = out[rows].float().cpu().numpy()
    bad = strict_failures(orc, ref, res, 1e-2)
    prod = (acc.astype(np.float64) - 128.0 * W.to(torch.int64).sum(0).numpy()[None, :]) * scale.double().numpy()[None, :]
    x = prod + bias.double().numpy()[None, :]                   # the pre-activation value, exact
    tail = (x < -4.0) & (x > -5.0)
    cancel = np.abs(x) < CANCEL_FRACTION * (np.abs(prod) + np.abs(bias.double().numpy())[None, :])
    n = int(bad.sum())
    print("\nconfig 3: strict rule fails on %d of %d elements (%d in the GELU tail -5 < x < -4, %d cancellations of "
          "acc*scale + bias); elements in that tail window: %d" % (n, bad.size, int((bad & tail).sum()),
                                                                   int((bad & cancel & ~tail).sum()), int(tail.sum())))
    assert (tail | cancel)[bad].all(), x[bad & ~(tail | cancel)][:8]
    assert n <= 1e-3 * bad.size
    # elsewhere the two agree to a bf16 step, and nearly always bit for bit (leaving out the saturated tail, see above)
    differ = (ref != res) & ((np.abs(ref) > 1e-7) | (np.abs(res) > 1e-7))
    assert differ.mean() < 1e-3
    # one bf16 step where GELU is not in its far tail; there (|gelu| < 1e-4, where the reference's own f32 (erf + 1)
    # has few correct digits left) an absolute 1e-6
    assert (np.abs(ref - res)[differ] <= np.where(np.abs(ref)[differ] > 1e-4, 2.0 ** -7 * np.abs(ref)[differ], 1e-6)).all()
    # the harness's norm rule (test/benchgc/src/benchgc/arg/compare.py:41-57), per sampled row
    nbad, l2 = orc.compare_norm_rows(ref, res, 1e-4)
    print("config 3: per-row norm of the difference: max %.2e, median %.2e" % (float(l2.max()), float(np.median(l2))))
    assert nbad == 0


def test_config4_full_size_and_strict_failures(gc, orc, wl, dev):
    """bf16 MLP chain at full size (4096 x 4096 x 11008 -> 4096): sampled rows of both layers against
    the oracle's chain, column checksums of both layers over all rows in f64, and the strict-rule count."""
    from conftest import assert_close
    x, W1, W2, b2 = wl.bf16_mlp_chain()
    xd, W1d, W2d, b2d = x.to(dev), W1.to(dev), W2.to(dev), b2.to(dev)
    h = gc.gemm_bf16(xd, W1d, None, "relu")
    y = gc.gemm_bf16(h, W2d, b2d, None)
    torch.cuda.synchronize()
    rows = sorted(set(list(range(0, 4096, 512)) + list(range(255, 4096, 512)) + [1, 2049, 3000]))[:16]
    href, yref = orc.mlp_chain_bf16(wl.bf16_bits(x[rows]), wl.bf16_bits(W1), wl.bf16_bits(W2), wl.bf16_bits(b2))
    hres = h[rows].float().cpu().numpy()
    yres = y[rows].float().cpu().numpy()
    assert_close(orc.bf16_to_f32(href), hres, 1e-2, "mlp hidden, full size")
    mm = orc.bf16_to_f32(orc.matmul_bf16(href, wl.bf16_bits(W2)))
    assert_close(orc.bf16_to_f32(yref), yres, 2e-2, "mlp out, full size (two rounding points)", mag=mm)
    # strict rule, layer 1: a ReLU output is 0 or a rounded sum; failures must be cancellations of x.W1
    hsum = (x[rows].double().abs() @ W1.double().abs()).numpy()
    bad_h = strict_failures(orc, orc.bf16_to_f32(href), hres, 1e-2)
    assert _report("config 4 hidden", bad_h, orc.bf16_to_f32(href), hsum) < CANCEL_FRACTION
    # layer 2 on the GPU's own hidden rows (isolates the second GEMM): bf16(bf16(h.W2) + b2)
    hg = h[rows].cpu()
    y2 = orc.bf16_to_f32(orc.matmul_bf16(wl.bf16_bits(hg), wl.bf16_bits(W2), wl.bf16_bits(b2)))
    ysum = (hg.double().abs() @ W2.double().abs()).numpy() + b2.double().abs().numpy()
    bad_y = strict_failures(orc, y2, yres, 1e-2)
    assert _report("config 4 output", bad_y, y2, ysum) < CANCEL_FRACTION
    assert bad_h.sum() <= 0.01 * bad_h.size and bad_y.sum() <= 0.02 * bad_y.size
    # every element of both layers takes part: column sums over all 4096 rows in f64
    want_y = (h.double().sum(0, keepdim=True) @ W2d.double()).squeeze(0) + 4096 * b2d.double()
    got_y = y.double().sum(0)
    scale_y = (h.double().abs().sum(0, keepdim=True) @ W2d.double().abs()).squeeze(0) + 4096 * b2d.double().abs()
    assert ((got_y - want_y).abs() <= 2 ** -7 * scale_y).all()
    # layer 1: ReLU is not linear, so the column sums run over the elements the GPU left non-zero, against an
    # exact f64 product (an element whose sign the GPU got wrong would show as a missing or extra term)
    exact = xd.double() @ W1d.double()
    want_h = ((h != 0).double() * exact).sum(0)
    got_h = h.double().sum(0)
    scale_h = (xd.double().abs() @ W1d.double().abs()).sum(0)
    assert ((got_h - want_h).abs() <= 2 ** -7 * scale_h).all()
    # and the sign pattern itself: zero where the exact sum is clearly negative, non-zero where clearly positive
    noise = 1e-5 * (xd.double().abs() @ W1d.double().abs())
    assert not ((h != 0) & (exact < -noise)).any() and not ((h == 0) & (exact > noise + 1e-30)).any()


def test_config5_strict_failures_are_cancellations(gc, orc, wl, dev):
    """Attention B4 H32 S2048 D128 with the causal mask as data: three heads against the oracle."""
    Q, K, V, mask, scale = wl.bf16_mha()
    out = gc.mha_fwd_bf16(Q.to(dev), K.to(dev), V.to(dev), mask.to(dev), scale)
    torch.cuda.synchronize()
    worst_all = 0.0
    n_bad = n_all = 0
    for (b, h) in [(0, 0), (1, 17), (3, 31)]:
        q, k, v = Q[b:b + 1, h:h + 1], K[b:b + 1, h:h + 1], V[b:b + 1, h:h + 1]
        ref = orc.bf16_to_f32(orc.mha_bf16(wl.bf16_bits(q), wl.bf16_bits(k), wl.bf16_bits(v), mask.numpy(), scale))[0, 0]
        res = out[b, h].float().cpu().numpy()
        bad = strict_failures(orc, ref, res, 1e-2)
        S = q[0, 0].double() @ k[0, 0].double().t() * scale + mask.double()
        mag = (torch.softmax(S, -1) @ v[0, 0].double().abs()).numpy()  # sum_j p_ij |v_jd|
        worst_all = max(worst_all, _report("config 5 head (%d,%d)" % (b, h), bad, ref, mag))
        n_bad += int(bad.sum())
        n_all += bad.size
        # P is a bf16 tensor in the reference graph: every term p_ij v_jd carries a rounding error of up to 2^-9 of
        # itself, and the GPU rounds P at another scale (running maximum), so the two sums differ by a random walk
        # of those errors -- bounded by 2^-8 sum_j p_ij |v_jd|, plus the result's own rounding
        err = np.abs(ref.astype(np.float64) - res)
        assert (err[bad] <= 2.0 ** -8 * mag[bad] + 2.0 ** -7 * np.abs(ref[bad])).all()
    # O_id is a sum of terms of random sign: |O| falls below 0.16 of its own standard deviation -- where that random
    # walk of rounding errors (~1.6e-3 sigma) exceeds 1e-2 |O| -- for about 13 % of the elements
    assert worst_all < 0.6
    assert n_bad <= 0.20 * n_all
