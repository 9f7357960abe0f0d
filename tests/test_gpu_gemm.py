"""GPU parity: MFMA GEMMs through the C ABI against the CPU oracle.
bf16/f32 outputs: max relative error (see conftest.close_report) <= 1e-2 / 1e-4;
s32 accumulators: bit exact."""
import numpy as np
import pytest
import torch

from conftest import assert_close

pytestmark = pytest.mark.gpu

BF16_SHAPES = [(256, 256, 64), (512, 512, 256), (256, 512, 1024), (300, 200, 100), (257, 511, 129), (1, 7, 5),
               (33, 1, 64), (128, 256, 8)]


@pytest.mark.parametrize("M,N,K", BF16_SHAPES)
@pytest.mark.parametrize("epi", ["none", "bias", "bias_relu", "gelu"])
def test_bf16_gemm_matches_oracle(gc, orc, wl, dev, M, N, K, epi):
    torch.manual_seed(0)
    A = (torch.randn(M, K) * 0.5).to(torch.bfloat16)
    torch.manual_seed(1)
    B = (torch.randn(K, N) * 0.5).to(torch.bfloat16)
    torch.manual_seed(2)
    bias = torch.randn(N).to(torch.bfloat16) if "bias" in epi else None
    act = {"none": None, "bias": None, "bias_relu": "relu", "gelu": "gelu_erf"}[epi]
    ref = orc.bf16_to_f32(orc.matmul_bf16(wl.bf16_bits(A), wl.bf16_bits(B),
                                          None if bias is None else wl.bf16_bits(bias), act))
    mm = orc.bf16_to_f32(orc.matmul_bf16(wl.bf16_bits(A), wl.bf16_bits(B))) if bias is not None else None
    out = gc.gemm_bf16(A.to(dev), B.to(dev), None if bias is None else bias.to(dev), act)
    torch.cuda.synchronize()
    # 1e-2 per bf16 rounding point of the reference graph: the matmul result is
    # rounded once; a bias add or activation after it rounds a second time, and
    # the two one-ulp (2^-7) differences of a different f32 summation order add.
    rtol = 1e-2 if epi == "none" else 2e-2
    assert_close(ref, out.float().cpu().numpy(), rtol, "bf16 %dx%dx%d %s" % (M, N, K, epi), mag=mm)


@pytest.mark.parametrize("epi", ["none", "bias", "bias_relu", "gelu"])
def test_bf16_gemm_special_values_whole_tiles(gc, orc, wl, dev, epi):
    """Whole tiles (the kernel that rounds to bf16 in pairs): NaNs of either sign in A, infinities in A and in the
    bias.  Where the reference has a NaN the result is its 0x7FC0
    (include/gc/ExecutionEngine/CPURuntime/Microkernel/BrgemmInterface.h:83-92), infinities agree bit for bit."""
    M, N, K = 256, 512, 256
    torch.manual_seed(0)
    A = wl.bf16_bits((torch.randn(M, K) * 0.5).to(torch.bfloat16)).copy()
    torch.manual_seed(1)
    B = (torch.randn(K, N) * 0.5).to(torch.bfloat16)
    A[3, 5], A[40, 7], A[41, 0] = 0xFFC1, 0x7FC0, 0x7F81       # NaNs: negative with payload, canonical, signalling
    A[100, 9], A[101, 9] = 0x7F80, 0xFF80                      # +inf, -inf: whole rows of +-inf
    A[102, 1], A[102, 2] = 0x7F80, 0xFF80                      # both in one row: inf - inf
    bias = None
    if "bias" in epi:
        torch.manual_seed(2)
        bias = wl.bf16_bits(torch.randn(N).to(torch.bfloat16)).copy()
        bias[17], bias[18], bias[300] = 0x7F80, 0xFF80, 0xFFFF
    act = {"none": None, "bias": None, "bias_relu": "relu", "gelu": "gelu_erf"}[epi]
    want = np.asarray(orc.matmul_bf16(A, wl.bf16_bits(B), bias, act)).view(np.uint16).reshape(M, N)
    At = torch.from_numpy(A.view(np.int16)).view(torch.bfloat16)
    bt = None if bias is None else torch.from_numpy(bias.view(np.int16)).view(torch.bfloat16).to(dev)
    out = gc.gemm_bf16(At.to(dev), B.to(dev), bt, act)
    torch.cuda.synchronize()
    got = out.view(torch.int16).cpu().numpy().view(np.uint16)
    special = (want & 0x7F80) == 0x7F80
    assert (want[special] == 0x7FC0).any() and (want[special] != 0x7FC0).any()
    bad = special & (got != want)
    assert not bad.any(), sorted({(int(r), int(c), hex(int(g)), hex(int(w))) for r, c, g, w in
                                  zip(*np.nonzero(bad), got[bad], want[bad])})[:12]
    assert_close(orc.bf16_to_f32(want[~special]), orc.bf16_to_f32(got[~special]), 2e-2, "finite part")


def test_bf16_gemm_f32_out_and_strided_operands(gc, orc, wl, dev):
    M, N, K = 260, 264, 200
    torch.manual_seed(0)
    Abig = torch.randn(M, K + 24).to(torch.bfloat16).to(dev)
    Bbig = torch.randn(K, N + 8).to(torch.bfloat16).to(dev)
    A, B = Abig[:, :K], Bbig[:, :N]
    Cbig = torch.full((M, N + 4), 7.0, device=dev)
    out = gc.gemm_bf16(A, B, None, None, gc.F32, out=Cbig[:, :N])
    torch.cuda.synchronize()
    ref = orc.deep_tile_matmul(wl.bf16_bits(A.cpu().contiguous()), wl.bf16_bits(B.cpu().contiguous()), orc.BF16, orc.BF16)
    assert_close(ref, out.cpu().numpy(), 1e-4, "bf16->f32 strided")
    assert (Cbig[:, N:] == 7.0).all()  # nothing written past the row


def test_bf16_identity_is_exact_at_full_size(gc, dev):
    """A . I == A bit for bit: every product is exact and every sum has one term."""
    n = 4096
    torch.manual_seed(3)
    A = torch.randn(n, n, device=dev).to(torch.bfloat16)
    eye = torch.eye(n, device=dev, dtype=torch.bfloat16)
    out = gc.gemm_bf16(A, eye)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), A.view(torch.int16))


def test_bf16_full_size_rows_against_oracle(gc, orc, wl, dev):
    """BASELINE config 2 (4096^3): 48 rows spread over every row tile."""
    A, B = wl.bf16_gemm()
    out = gc.gemm_bf16(A.to(dev), B.to(dev))
    torch.cuda.synchronize()
    rows = sorted(set(list(range(0, 4096, 256)) + list(range(255, 4096, 256)) + [1, 130, 2049, 3000] +
                      list(range(97, 4096, 331))))[:48]
    ref = orc.bf16_to_f32(orc.matmul_bf16(wl.bf16_bits(A[rows]), wl.bf16_bits(B)))
    assert_close(ref, out[rows].float().cpu().numpy(), 1e-2, "bf16 4096^3 sampled rows")
    # column checksum over all rows in f64 (every output element takes part)
    want = (A.double().sum(0, keepdim=True) @ B.double()).squeeze(0)
    got = out.double().sum(0).cpu()
    scale = (A.double().abs().sum(0, keepdim=True) @ B.double().abs()).squeeze(0)
    assert ((got - want).abs() <= 2 ** -8 * scale).all()


INT8_SHAPES = [(256, 256, 128), (512, 768, 384), (100, 130, 77), (1, 5, 3), (260, 40, 500)]


@pytest.mark.parametrize("M,N,K", INT8_SHAPES)
@pytest.mark.parametrize("a_signed", [False, True])
def test_int8_accumulators_bit_exact(gc, orc, dev, M, N, K, a_signed):
    torch.manual_seed(0)
    A = torch.randint(-128, 128, (M, K), dtype=torch.int32).to(torch.int8) if a_signed else \
        torch.randint(0, 256, (M, K), dtype=torch.int32).to(torch.uint8)
    torch.manual_seed(1)
    W = torch.randint(-128, 128, (K, N), dtype=torch.int32).to(torch.int8)
    ref = orc.deep_tile_matmul(A.numpy(), W.numpy(), orc.S8 if a_signed else orc.U8, orc.S8)
    Wd = W.to(dev)
    cs = gc.colsum_s8(Wd)
    torch.cuda.synchronize()
    assert (cs.cpu().numpy() == orc.colsum_s8(W.numpy())).all()
    raw = gc.gemm_int8(A.to(dev), Wd, cs, 0, None, None, None, gc.S32)
    torch.cuda.synchronize()
    assert (raw.cpu().numpy() == ref).all()


@pytest.mark.parametrize("M,N,K", INT8_SHAPES[:4])
@pytest.mark.parametrize("act,zp", [("gelu_erf", 128), ("relu", 3), (None, 0), ("gelu_tanh", 128)])
def test_int8_layer_matches_oracle(gc, orc, dev, M, N, K, act, zp):
    torch.manual_seed(0)
    A = torch.randint(0, 256, (M, K), dtype=torch.int32).to(torch.uint8)
    torch.manual_seed(1)
    W = torch.randint(-127, 128, (K, N), dtype=torch.int32).to(torch.int8)
    torch.manual_seed(2)
    sc = torch.rand(N) * 0.009 + 0.001
    torch.manual_seed(3)
    bs = torch.randn(N)
    _, y = orc.int8_layer(A.numpy(), W.numpy(), sc.numpy(), bs.numpy(), zp, act)
    Wd = W.to(dev)
    out = gc.gemm_int8(A.to(dev), Wd, gc.colsum_s8(Wd), zp, sc.to(dev), bs.to(dev), act, gc.BF16)
    torch.cuda.synchronize()
    assert_close(orc.bf16_to_f32(y), out.float().cpu().numpy(), 1e-2, "int8 layer")
    _, yf = orc.int8_layer(A.numpy(), W.numpy(), sc.numpy(), bs.numpy(), zp, act, out_bf16=False)
    outf = gc.gemm_int8(A.to(dev), Wd, gc.colsum_s8(Wd), zp, sc.to(dev), bs.to(dev), act, gc.F32)
    torch.cuda.synchronize()
    assert_close(yf, outf.cpu().numpy(), 1e-4, "int8 layer f32 out")


@pytest.mark.parametrize("act", ["gelu_erf", "relu", None])
def test_int8_layer_special_scales_and_biases(gc, orc, dev, act):
    """Whole-tile shape (the kernel that converts to bf16 in pairs): NaNs of either sign and any payload,
    infinities and overflowing products in scale and bias.  Every NaN of the result is the reference's 0x7FC0
    (include/gc/ExecutionEngine/CPURuntime/Microkernel/BrgemmInterface.h:83-92), infinities keep their sign."""
    M = N = K = 256
    torch.manual_seed(0)
    A = torch.randint(0, 256, (M, K), dtype=torch.int32).to(torch.uint8)
    torch.manual_seed(1)
    W = torch.randint(-127, 128, (K, N), dtype=torch.int32).to(torch.int8)
    sc = (torch.rand(N) * 0.009 + 0.001).numpy()
    bs = torch.randn(N).numpy()
    sc_bits, bs_bits = sc.view(np.uint32), bs.view(np.uint32)
    sc_bits[3], sc_bits[40] = 0xFFC12345, 0x7F800001          # negative quiet NaN with payload, signalling NaN
    sc[7], sc[64], sc[65], sc[130] = np.inf, -np.inf, 3e38, -3e38
    bs_bits[9], bs_bits[200] = 0xFFFFFFFF, 0x7FC00001
    bs[11], bs[12], bs[7], bs[64] = np.inf, -np.inf, -np.inf, np.inf
    _, y = orc.int8_layer(A.numpy(), W.numpy(), sc, bs, 128, act)
    Wd = W.to(dev)
    out = gc.gemm_int8(A.to(dev), Wd, gc.colsum_s8(Wd), 128, torch.from_numpy(sc).to(dev), torch.from_numpy(bs).to(dev),
                       act, gc.BF16)
    torch.cuda.synchronize()
    got = out.view(torch.int16).cpu().numpy().view(np.uint16)
    want = np.asarray(y).view(np.uint16).reshape(M, N)
    special = (want & 0x7F80) == 0x7F80
    assert special.any() and (want[special] == 0x7FC0).any() and (want[special] == 0x7F80).any()
    bad = special & (got != want)
    assert not bad.any(), sorted({(int(c), hex(int(g)), hex(int(w))) for c, g, w in
                                  zip(np.nonzero(bad)[1], got[bad], want[bad])})[:12]
    assert_close(orc.bf16_to_f32(want[~special]), orc.bf16_to_f32(got[~special]), 1e-2, "finite part")


@pytest.mark.parametrize("a_signed", [False, True])
def test_int8_full_size_exact_checksums_and_rows(gc, orc, wl, dev, a_signed):
    """BASELINE config 3 (4096 x 4096 x 11008), on the kernel the benchmark times (4 waves of 128 x 128, asserted
    through the tile descriptor): the raw s32 accumulators leave it through a plain store.  Exactness of all 45M
    accumulators through integer checksums (row sums and column sums of the s32 result against int64 products of the
    operand sums), exact rows against the oracle (lib/gc/ExecutionEngine/CPURuntime/Microkernel/BrgemmNaive.cpp:102-140
    is what it restates), the 8-wave kernel's accumulators bit for bit, and the fused epilogue against the oracle on
    those rows.  u8 activations (the config) and s8 activations (no byte flip, no zero-point term)."""
    A, W, scale, bias = wl.int8_mlp_layer()
    zp = 128
    if a_signed:
        A, zp = (A.to(torch.int16) - 128).to(torch.int8), 0
    c, _ = gc.tile_config(4096, 11008, 4096, a_dtype=gc.S8 if a_signed else gc.U8, out_dtype=gc.S32)
    assert (c.kernel, c.waves_m * c.waves_n, c.wave_m, c.wave_n) == (2, 4, 128, 128)
    Ad, Wd = A.to(dev), W.to(dev)
    cs = gc.colsum_s8(Wd)
    raw = gc.gemm_int8(Ad, Wd, cs, 0 if a_signed else 128, None, None, None, gc.S32)
    torch.cuda.synchronize()
    assert (cs.cpu() == W.to(torch.int64).sum(0)).all()
    raw64 = raw.to(torch.int64)
    col_want = (A.to(torch.int64).sum(0, keepdim=True) @ W.to(torch.int64)).squeeze(0)   # 1^T A W
    row_want = (A.to(torch.int64) @ W.to(torch.int64).sum(1, keepdim=True)).squeeze(1)   # A W 1
    assert (raw64.sum(0).cpu() == col_want).all()
    assert (raw64.sum(1).cpu() == row_want).all()
    # a second, position-dependent checksum: a swap of two accumulators inside a row or a column would keep the plain
    # sums; weights r_i = i + 1 and c_j = j + 1 catch it.  (r^T A) W c in int64.
    r = torch.arange(1, 4097, dtype=torch.int64)
    cw = torch.arange(1, 11009, dtype=torch.int64)
    want_rc = ((r.unsqueeze(0) @ A.to(torch.int64)) @ (W.to(torch.int64) @ cw.unsqueeze(1))).item()
    got_rc = int((raw64.cpu() * r.unsqueeze(1) * cw.unsqueeze(0)).sum().item())
    assert got_rc == want_rc
    rows = [0, 255, 256, 1027, 2048, 3333, 4095] + list(range(61, 4096, 449))
    acc = orc.deep_tile_matmul(A[rows].numpy(), W.numpy(), orc.S8 if a_signed else orc.U8, orc.S8)
    assert (raw[rows].cpu().numpy() == acc).all()
    eight = gc.gemm_int8(Ad, Wd, cs, 0 if a_signed else 128, None, None, None, gc.S32,
                         matmul_config=[1, 1, 1, 256, 256, 64, 128, 64, 32])
    torch.cuda.synchronize()
    assert torch.equal(raw, eight)
    del eight, raw64
    if a_signed:
        return
    _, y = orc.int8_layer(A[rows].numpy(), W.numpy(), scale.numpy(), bias.numpy(), zp, "gelu_erf")
    out = gc.gemm_int8(Ad, Wd, cs, zp, scale.to(dev), bias.to(dev), "gelu_erf", gc.BF16)
    torch.cuda.synchronize()
    assert_close(orc.bf16_to_f32(y), out[rows].float().cpu().numpy(), 1e-2, "int8 mlp rows")


@pytest.mark.parametrize("M,N,K,ta,tb", [(128, 256, 512, False, False), (512, 64, 128, True, False),
                                         (70, 33, 45, False, True), (65, 67, 19, True, True), (1, 1, 1, False, False),
                                         # 64 or more whole 128 x 128 tiles of row-major operands: the f32 matrix instruction
                                         (1024, 1024, 256, False, False), (1536, 768, 80, False, False)])
def test_f32_gemm_bias_relu(gc, orc, dev, M, N, K, ta, tb):
    torch.manual_seed(0)
    A = torch.rand((K, M) if ta else (M, K)) * 2 - 1
    torch.manual_seed(1)
    B = torch.rand((N, K) if tb else (K, N)) * 2 - 1
    torch.manual_seed(2)
    bias = torch.rand(N) * 2 - 1
    ref = orc.matmul_f32(A.numpy(), B.numpy(), bias.numpy(), "relu", ta, tb)
    out = gc.gemm_f32(A.to(dev), B.to(dev), bias.to(dev), "relu", ta, tb)
    torch.cuda.synchronize()
    assert_close(ref, out.cpu().numpy(), 1e-4, "f32 gemm")


def test_mlp_chain_bf16_reduced(gc, orc, wl, dev):
    """BASELINE config 4 at 1/8 size: x W1 -> ReLU -> W2 + bias, bf16 rounding
    points after the matmul, the add and the ReLU."""
    x, W1, W2, b2 = wl.bf16_mlp_chain(M=512, K=512, H=1376)
    h = gc.gemm_bf16(x.to(dev), W1.to(dev), None, "relu")
    y = gc.gemm_bf16(h, W2.to(dev), b2.to(dev), None)
    torch.cuda.synchronize()
    href, yref = orc.mlp_chain_bf16(wl.bf16_bits(x), wl.bf16_bits(W1), wl.bf16_bits(W2), wl.bf16_bits(b2))
    assert_close(orc.bf16_to_f32(href), h.float().cpu().numpy(), 1e-2, "mlp hidden")
    mm = orc.bf16_to_f32(orc.matmul_bf16(href, wl.bf16_bits(W2)))
    assert_close(orc.bf16_to_f32(yref), y.float().cpu().numpy(), 2e-2, "mlp out (two rounding points)", mag=mm)


def test_gelu_erf_epilogue_absolute_accuracy(gc, dev):
    """The epilogue's erf is 1 - 2^(-|x| q(|x|)) with a fitted polynomial q, absolute error < 2e-7
    (the reference's own erf is an approximation of that class): GELU over a
    dense grid of x, computed as a [M,1]x[1,1] matmul with the activation fused,
    against float64."""
    x = torch.linspace(-8, 8, 200001, dtype=torch.float32).reshape(-1, 1)
    one = torch.ones(1, 1, dtype=torch.float32)
    out = gc.gemm_f32(x.to(dev), one.to(dev), act="gelu_erf").cpu().numpy().astype(np.float64).ravel()
    xd = x.numpy().astype(np.float64).ravel()
    ref = 0.5 * xd * (1 + torch.special.erf(torch.from_numpy(xd) * 0.7071067811865476).numpy())  # float64
    assert np.abs(out - ref).max() <= 2e-6  # |x| <= 8: 0.5 * 8 * 2e-7 + f32 rounding
    # the argument of erf is clamped at 4.2 = 5.94 / sqrt 2, and from 3.9 on the result is exactly +-1, as libm's is
    assert (out[xd < -5.84] == 0).all() and (out[xd > 5.84] == xd[xd > 5.84]).all()


def test_gelu_of_the_int8_layer_with_bf16_result(gc, orc, dev):
    """The 8-bit tile kernels evaluate GELU for a bf16 result with a shorter polynomial (relative error below 2^-11.9
    of the value, a quarter of a bf16's last place; the f32-result path keeps the 1.5e-7 form).  A one-hot weight and
    per-column scales and biases put x = (a - 128) * scale + bias on a dense grid over [-9, 9]: every result against
    the float64 GELU -- within half a bf16 step of it plus that 2^-11.9 --, against the oracle at the stated 1e-2, and
    the share of results that are not the exactly rounded value."""
    M = N = K = 256
    A = torch.zeros(M, K, dtype=torch.uint8)
    A[:, 0] = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    W = torch.zeros(K, N, dtype=torch.int8)
    W[0, :] = 1
    scale = ((torch.arange(N, dtype=torch.float32) % 64 + 1) / 64 * 0.0625)          # up to 8 / 128 per count
    bias = ((torch.arange(N, dtype=torch.float32) // 64) - 1.5) * 0.37 + torch.arange(N, dtype=torch.float32) * 1e-3
    Wd = W.to(dev)
    out = gc.gemm_int8(A.to(dev), Wd, gc.colsum_s8(Wd), 128, scale.to(dev), bias.to(dev), "gelu_erf", gc.BF16)
    torch.cuda.synchronize()
    got = out.float().cpu().numpy().astype(np.float64)
    # the pre-activation value as the kernel forms it: one fused multiply-add, rounded to f32 once
    x = torch.addcmul(bias[None, :].double(), (A[:, :1].to(torch.float64) - 128), scale[None, :].double()).float().double()
    exact = (0.5 * x * (1 + torch.special.erf(x * 0.7071067811865476))).numpy()
    assert x.min() < -8 and x.max() > 8
    bits = np.abs(exact).astype(np.float32).view(np.uint32)
    step = (((bits >> 23) << 23).view(np.float32)).astype(np.float64) * 2.0 ** -7      # a bf16 step at |exact|
    assert (np.abs(got - exact) <= 0.5 * step + 2.0 ** -11.9 * np.abs(exact) + 1.2e-9).all()
    rounded = orc.bf16_to_f32(orc.f32_to_bf16(exact.astype(np.float32))).astype(np.float64)
    share = float((got != rounded).mean())
    assert share < 0.06, share
    _, y = orc.int8_layer(A.numpy(), W.numpy(), scale.numpy(), bias.numpy(), 128, "gelu_erf")
    assert_close(orc.bf16_to_f32(y), got, 1e-2, "int8 layer, GELU grid")
    # large |x|: x itself, or -0, as the reference's saturated erf gives
    big = torch.tensor([[255, 0]], dtype=torch.uint8).repeat(256, 128)
    Wb = torch.zeros(K, N, dtype=torch.int8)
    Wb[0, :] = 127
    Wb[1, :] = -127
    Wbd = Wb.to(dev)
    o2 = gc.gemm_int8(big.to(dev), Wbd, gc.colsum_s8(Wbd), 128, torch.full((N,), 0.01).to(dev), None, "gelu_erf", gc.BF16)
    torch.cuda.synchronize()
    _, y2 = orc.int8_layer(big.numpy(), Wb.numpy(), np.full(N, 0.01, np.float32), None, 128, "gelu_erf")
    assert (o2.view(torch.int16).cpu().numpy().view(np.uint16) == np.asarray(y2).reshape(M, N)).all()


@pytest.mark.parametrize("M,N", [(300, 264), (520, 256), (512, 520), (1000, 1000)])
@pytest.mark.parametrize("variant", ["plain", "bias_gelu_f32", "bias_relu_residual", "nt"])
@pytest.mark.parametrize("tile", [256, 128])
def test_bf16_edge_tiles_of_the_four_wave_kernels(gc, orc, wl, dev, M, N, variant, tile):
    """M any, N a multiple of 8, K a multiple of 128: the 4-wave kernels (256 x 256 and 128 x 128 tiles, each asked for
    by its MatmulConfig) take the shape; tiles on the lower and right edges clamp their loads and store what lies
    inside C.  Every element equals, bit for bit, the element of the same GEMM padded to whole tiles (same kernel,
    same sums), and the result matches the oracle."""
    K = 384
    how = 1 if tile == 256 else "tile128"
    cfg = [1, 1, 1, 256, 256, 64, 128, 128, 32] if tile == 256 else [1, 1, 1, 128, 128, 64, 64, 64, 32]
    c, _ = gc.tile_config(M, N, K, trans_b=(variant == "nt"), out_dtype=gc.F32 if variant == "bias_gelu_f32" else gc.BF16,
                          matmul_config=cfg)
    assert c.kernel == (2 if tile == 256 else 5) and c.workgroups == -(-M // tile) * -(-N // tile) and c.from_attrs == 1
    Mp, Np = -(-M // 256) * 256, -(-N // 256) * 256
    torch.manual_seed(0)
    Ap = (torch.randn(Mp, K) * 0.5).to(torch.bfloat16)
    torch.manual_seed(1)
    Bp = (torch.randn(K, Np) * 0.5).to(torch.bfloat16)
    torch.manual_seed(2)
    biasp = torch.randn(Np).to(torch.bfloat16)
    torch.manual_seed(3)
    resp = torch.randn(Mp, Np).to(torch.bfloat16)
    A, B, bias, res = Ap[:M].contiguous(), Bp[:, :N].contiguous(), biasp[:N].contiguous(), resp[:M, :N].contiguous()
    d = lambda t: t.to(dev)
    odt = torch.float32 if variant == "bias_gelu_f32" else torch.bfloat16
    guard = torch.full((M + 2, N), 7.0, dtype=odt, device=dev)
    out = guard[1:M + 1]
    full = torch.empty((Mp, Np), dtype=odt, device=dev)
    ref = None
    if variant == "plain":
        _gemm_ws(gc, d(A), d(B), False, out, how)
        _gemm_ws(gc, d(Ap), d(Bp), False, full, how)
        ref = orc.bf16_to_f32(orc.matmul_bf16(wl.bf16_bits(A), wl.bf16_bits(B)))
    elif variant == "bias_gelu_f32":
        _gemm_ws(gc, d(A), d(B), False, out, how, bias=d(bias), act="gelu_erf")
        _gemm_ws(gc, d(Ap), d(Bp), False, full, how, bias=d(biasp), act="gelu_erf")
    elif variant == "bias_relu_residual":
        _gemm_ws(gc, d(A), d(B), False, out, how, bias=d(bias), act="relu", residual=d(res))
        _gemm_ws(gc, d(Ap), d(Bp), False, full, how, bias=d(biasp), act="relu", residual=d(resp))
    else:
        _gemm_ws(gc, d(A), d(B.t().contiguous()), True, out, how)
        _gemm_ws(gc, d(Ap), d(Bp.t().contiguous()), True, full, how)
        ref = orc.bf16_to_f32(orc.matmul_bf16(wl.bf16_bits(A), wl.bf16_bits(B)))
    torch.cuda.synchronize()
    assert (guard[0] == 7).all() and (guard[M + 1] == 7).all()  # nothing written outside C
    bits = torch.int32 if out.dtype == torch.float32 else torch.int16
    assert (out.view(bits) == full[:M, :N].contiguous().view(bits)).all()
    if ref is not None:
        assert_close(ref, out.float().cpu().numpy(), 1e-2, "bf16 edge tiles %dx%d %s" % (M, N, variant))


@pytest.mark.parametrize("M,N", [(300, 272), (520, 256), (512, 528), (1000, 1008)])
@pytest.mark.parametrize("tile", [256, 128])
def test_int8_edge_tiles_of_the_four_wave_kernels(gc, orc, dev, M, N, tile):
    """The same for u8 x s8 with dequantisation, bias and GELU to bf16 (N a multiple of 16, K of 256), on the tile
    each MatmulConfig names; the two tiles give the same bits (integer sums are exact, the epilogue is one code)."""
    K = 512
    cfg = [1, 1, 1, 256, 256, 64, 128, 128, 32] if tile == 256 else [1, 1, 1, 128, 128, 64, 64, 64, 32]
    c, _ = gc.tile_config(M, N, K, a_dtype=gc.U8, matmul_config=cfg)
    assert c.kernel == (2 if tile == 256 else 5) and c.workgroups == -(-M // tile) * -(-N // tile) and c.from_attrs == 1
    torch.manual_seed(0)
    A = torch.randint(0, 256, (M, K), dtype=torch.int32).to(torch.uint8)
    torch.manual_seed(1)
    W = torch.randint(-127, 128, (K, N), dtype=torch.int32).to(torch.int8)
    torch.manual_seed(2)
    sc = torch.rand(N) * 0.009 + 0.001
    torch.manual_seed(3)
    bs = torch.randn(N)
    _, y = orc.int8_layer(A.numpy(), W.numpy(), sc.numpy(), bs.numpy(), 128, "gelu_erf")
    Wd = W.to(dev)
    guard = torch.full((M + 2, N), 7.0, dtype=torch.bfloat16, device=dev)
    gc.gemm_int8(A.to(dev), Wd, gc.colsum_s8(Wd), 128, sc.to(dev), bs.to(dev), "gelu_erf", gc.BF16, out=guard[1:M + 1], matmul_config=cfg)
    other = gc.gemm_int8(A.to(dev), Wd, gc.colsum_s8(Wd), 128, sc.to(dev), bs.to(dev), "gelu_erf", gc.BF16)  # the launcher's choice
    torch.cuda.synchronize()
    assert (guard[0] == 7).all() and (guard[M + 1] == 7).all()
    assert torch.equal(guard[1:M + 1].view(torch.int16), other.view(torch.int16))
    assert_close(orc.bf16_to_f32(y), guard[1:M + 1].float().cpu().numpy(), 1e-2, "int8 edge tiles")


@pytest.mark.parametrize("a_signed", [False, True])
def test_int8_few_tiles_take_the_small_tile(gc, dev, a_signed):
    """8-bit problems under one round of 256 x 256 tiles run on 128 x 128 tiles: raw accumulators against the integer
    product, and every output type bit for bit against the large tiles (asked for by name)."""
    big = [1, 1, 1, 256, 256, 64, 128, 128, 32]
    torch.manual_seed(5)
    for M, N, K in [(128, 128, 256), (512, 384, 1024), (129, 16, 256), (1024, 2048, 1024)]:
        c, _ = gc.tile_config(M, N, K, a_dtype=gc.S8 if a_signed else gc.U8)
        assert (c.kernel, c.bm, c.bn) == (5, 128, 128), (M, N, K, c.kernel)
        A = torch.randint(-128, 128, (M, K), dtype=torch.int8, device=dev) if a_signed else torch.randint(0, 256, (M, K), dtype=torch.uint8, device=dev)
        W = torch.randint(-127, 128, (K, N), dtype=torch.int8, device=dev)
        cs = gc.colsum_s8(W)
        zp = 3 if a_signed else 128
        scale = (torch.rand(N, device=dev) * 0.009 + 0.001).float()
        bias = torch.randn(N, device=dev).float()
        raw = gc.gemm_int8(A, W, cs, zp, out_dtype=gc.S32)
        assert torch.equal(raw.cpu().to(torch.int64), A.cpu().to(torch.int64) @ W.cpu().to(torch.int64))
        for odt, act, sc, bi in [(gc.BF16, "gelu_erf", scale, bias), (gc.F32, "relu", scale, bias), (gc.BF16, None, scale, None)]:
            got = gc.gemm_int8(A, W, cs, zp, sc, bi, act, odt)
            want = gc.gemm_int8(A, W, cs, zp, sc, bi, act, odt, matmul_config=big)
            torch.cuda.synchronize()
            v = torch.int16 if odt == gc.BF16 else torch.int32
            assert torch.equal(want.view(v), got.view(v)), (M, N, K, odt, act)


def test_gelu_tanh_epilogue_absolute_accuracy(gc, dev):
    """The tanh form of GELU (legacy/core/src/ops/gelu.cpp:78-108) over a dense grid of x against float64: the
    epilogue's tanh is 1 - 2 / (e^(2|t|) + 1), absolute error about 2e-7."""
    x = torch.linspace(-10, 10, 200001, dtype=torch.float32).reshape(-1, 1)
    one = torch.ones(1, 1, dtype=torch.float32)
    out = gc.gemm_f32(x.to(dev), one.to(dev), act="gelu_tanh").cpu().numpy().astype(np.float64).ravel()
    xd = x.numpy().astype(np.float64).ravel()
    ref = 0.5 * xd * (1 + np.tanh(0.79788458 * xd * (1 + 0.044715 * xd * xd)))
    assert np.abs(out - ref).max() <= 4e-6  # 0.5 * 10 * 2e-7 + f32 rounding of the argument and the product
    assert (out[xd > 6] == xd[xd > 6]).all() and (out[xd < -6] == 0).all()


@pytest.mark.parametrize("M,N,K,act,with_bias,out_f32", [(32, 4096, 4096, None, False, False), (1, 4096, 4096, "relu", True, False),
                                                         (100, 11008, 4096, "gelu_erf", True, False),
                                                         (32, 4096, 11008, None, True, True), (256, 2048, 1024, "sigmoid", False, False),
                                                         (7, 256, 128, None, False, False)])
def test_short_a_takes_split_k(gc, orc, wl, dev, M, N, K, act, with_bias, out_f32):
    """One tile row of A (M <= 256) against a wide weight: the K range is cut over workgroups and the f32
    partial sums are reduced by a second kernel.  Same rounding points as the one-pass kernel."""
    torch.manual_seed(M + N)
    A = (torch.randn(M, K) * 0.5).to(torch.bfloat16)
    torch.manual_seed(K)
    B = (torch.randn(K, N) * 0.05).to(torch.bfloat16)
    torch.manual_seed(3)
    bias = torch.randn(N).to(torch.bfloat16) if with_bias else None
    out = gc.gemm_bf16(A.to(dev), B.to(dev), None if bias is None else bias.to(dev), act,
                       out_dtype=gc.F32 if out_f32 else gc.BF16)
    torch.cuda.synchronize()
    if out_f32:
        ref = A.float().double() @ B.float().double()
        if bias is not None:
            ref = ref + bias.double()
        assert_close(ref.float().numpy(), out.cpu().numpy(), 1e-4, "split-k f32 out")
    else:
        ref = orc.bf16_to_f32(orc.matmul_bf16(wl.bf16_bits(A), wl.bf16_bits(B), None if bias is None else wl.bf16_bits(bias), act))
        mm = orc.bf16_to_f32(orc.matmul_bf16(wl.bf16_bits(A), wl.bf16_bits(B)))
        assert_close(ref, out.float().cpu().numpy(), 2e-2 if (with_bias or act) else 1e-2, "split-k", mag=mm)
    again = gc.gemm_bf16(A.to(dev), B.to(dev), None if bias is None else bias.to(dev), act,
                         out_dtype=gc.F32 if out_f32 else gc.BF16)
    torch.cuda.synchronize()
    assert torch.equal(out, again)  # fixed summation order: reruns agree bit for bit


def _gemm_ws(gc, A, B, trans_b, out, slices=None, bias=None, act=None, ws=None, residual=None):
    """gcmi_gemm_bf16_ws with a caller's workspace; slices: the KThreads of a full MatmulConfig attribute set with the
    256 x 256 tile, or "tile128": the set that names the 128 x 128 tile."""
    import ctypes as C
    M, K = A.shape
    N = B.shape[0] if trans_b else B.shape[1]
    if slices == "tile128":
        cfg = (C.c_int64 * 9)(1, 1, 1, 128, 128, 64, 64, 64, 32)
    else:
        cfg = None if slices is None else (C.c_int64 * 9)(1, 1, slices, 256, 256, 64, 128, 128, 32)
    st = gc.lib().gcmi_gemm_bf16_ws(A.data_ptr(), B.data_ptr(), out.data_ptr(), 1, M, N, K, K, B.shape[1], N, 0, 0, 0, int(trans_b),
                                    None if bias is None else bias.data_ptr(), gc.BF16, gc.ACT[act],
                                    None if residual is None else residual.data_ptr(), N, gc.BF16,
                                    gc.F32 if out.dtype == torch.float32 else gc.BF16,
                                    None if ws is None else ws.data_ptr(), 0 if ws is None else ws.numel() * ws.element_size(), cfg,
                                    C.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert st == 0, gc.lib().gcmi_last_error().decode()


@pytest.mark.parametrize("M,N,K,act,with_bias,out_f32", [(512, 512, 4096, "relu", True, False), (300, 1024, 2048, "gelu_erf", True, False),
                                                         (640, 768, 3072, None, True, True), (1024, 1024, 2048, None, False, False),
                                                         (257, 2048, 1024, "sigmoid", False, False)])
def test_few_tiles_and_a_deep_k_take_k_slices(gc, orc, wl, dev, M, N, K, act, with_bias, out_f32):
    """Several tile rows but too few 256 x 256 tiles for the GPU: 128 x 128 tiles, and where K is deep, equal K slices
    run as a strided batch of a tile kernel into f32 partial sums; the second kernel adds them and applies the
    epilogue.  Same rounding points as one pass."""
    c, _ = gc.tile_config(M, N, K, out_dtype=gc.F32 if out_f32 else gc.BF16)
    assert c.kernel in (3, 5) and c.workgroups <= 512, (c.kernel, c.split_k, c.workgroups)
    assert (c.kernel == 3) == (c.split_k > 1) and K // 128 % c.split_k == 0
    torch.manual_seed(M + N)
    A = (torch.randn(M, K) * 0.5).to(torch.bfloat16)
    torch.manual_seed(K)
    B = (torch.randn(K, N) * 0.05).to(torch.bfloat16)
    torch.manual_seed(3)
    bias = torch.randn(N).to(torch.bfloat16) if with_bias else None
    for trans_b in (False, True):
        Bd = B.t().contiguous().to(dev) if trans_b else B.to(dev)
        f = gc.gemm_bf16_nt if trans_b else gc.gemm_bf16
        out = f(A.to(dev), Bd, None if bias is None else bias.to(dev), act, out_dtype=gc.F32 if out_f32 else gc.BF16)
        again = f(A.to(dev), Bd, None if bias is None else bias.to(dev), act, out_dtype=gc.F32 if out_f32 else gc.BF16)
        torch.cuda.synchronize()
        assert torch.equal(out, again)  # fixed summation order: reruns agree bit for bit
        if out_f32:
            ref = A.float().double() @ B.float().double()
            if bias is not None:
                ref = ref + bias.double()
            assert_close(ref.float().numpy(), out.cpu().numpy(), 1e-4, "k slices f32 out")
        else:
            ref = orc.bf16_to_f32(orc.matmul_bf16(wl.bf16_bits(A), wl.bf16_bits(B), None if bias is None else wl.bf16_bits(bias), act))
            mm = orc.bf16_to_f32(orc.matmul_bf16(wl.bf16_bits(A), wl.bf16_bits(B)))
            assert_close(ref, out.float().cpu().numpy(), 2e-2 if (with_bias or act) else 1e-2, "k slices", mag=mm)


@pytest.mark.parametrize("trans_b", [False, True])
def test_k_slices_exact_on_integers_for_any_slice_count(gc, dev, trans_b):
    """Small integers make every partial sum exact, so each slice count must give the bits of the f32 product: the
    default, even counts (the 4-wave kernel as a batch), counts that do not divide K's ring groups (the kernel with
    slices of unequal length, here on two and three tile rows, the last one short), one slice (no second pass), a
    workspace too small for the count asked for or chosen (fewer slices), none at all, and the 128 x 128 tile by name."""
    torch.manual_seed(11)
    for M, N, K in [(512, 512, 2048), (600, 768, 1536), (257, 1024, 1024)]:
        A = torch.randint(-3, 4, (M, K), device=dev).to(torch.bfloat16)
        B = torch.randint(-3, 4, (K, N), device=dev).to(torch.bfloat16)
        want = A.float() @ B.float()
        Bd = B.t().contiguous() if trans_b else B
        ws = torch.empty(16 * M * N, dtype=torch.float32, device=dev)
        for slices, w in [(None, ws), (1, ws), (2, ws), (3, ws), (4, ws), (5, ws), (7, ws), (8, ws), (4, ws[:2 * M * N + 5]), (4, None),
                          ("tile128", ws), (None, ws[:2 * M * N]), (None, None)]:
            out = torch.full((M, N), 7.0, dtype=torch.float32, device=dev)
            _gemm_ws(gc, A, Bd, trans_b, out, slices, ws=w)
            torch.cuda.synchronize()
            assert torch.equal(out, want), (M, N, K, slices, None if w is None else w.numel())
        bias = torch.randint(-4, 5, (N,), device=dev).to(torch.bfloat16)
        out = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
        _gemm_ws(gc, A, Bd, trans_b, out, 3, bias=bias, act="relu", ws=ws)
        torch.cuda.synchronize()
        assert torch.equal(out, torch.relu((want.to(torch.bfloat16).float() + bias.float()).to(torch.bfloat16)))  # rounded after each op


@pytest.mark.parametrize("M,N,K", [(4096, 5120, 512), (4352, 4096, 256), (8192, 4352, 256)])
@pytest.mark.parametrize("trans_b", [False, True])
def test_a_thin_last_round_runs_on_small_tiles(gc, dev, M, N, K, trans_b):
    """Just over a round of 256 x 256 tiles (320, 272 and 544 of them on 256 compute units): the last round's block of
    columns or rows is a second launch on 128 x 128 tiles.  Exact on integers, and bit for bit the single launch of
    large tiles (asked for by name) with bias, GELU and a residual."""
    big = [1, 1, 1, 256, 256, 64, 128, 128, 32]
    tiles = (M // 256) * (N // 256)
    c, _ = gc.tile_config(M, N, K, trans_b=trans_b)
    assert c.kernel == 2 and c.workgroups == tiles - tiles % 256 + 4 * (tiles % 256), (c.kernel, c.workgroups)
    c, _ = gc.tile_config(M, N, K, trans_b=trans_b, matmul_config=big)
    assert c.kernel == 2 and c.workgroups == tiles
    torch.manual_seed(M + N)
    A = torch.randint(-3, 4, (M, K), device=dev).to(torch.bfloat16)
    B = torch.randint(-3, 4, (K, N), device=dev).to(torch.bfloat16)
    out = torch.full((M, N), 7.0, dtype=torch.float32, device=dev)
    _gemm_ws(gc, A, B.t().contiguous() if trans_b else B, trans_b, out)
    torch.cuda.synchronize()
    assert torch.equal(out, A.float() @ B.float())
    A = (torch.randn(M, K, device=dev) * 0.5).to(torch.bfloat16)
    B = (torch.randn(K, N, device=dev) * 0.5).to(torch.bfloat16)
    Bd = B.t().contiguous() if trans_b else B
    bias, res = torch.randn(N, device=dev).to(torch.bfloat16), torch.randn(M, N, device=dev).to(torch.bfloat16)
    o1, o2 = torch.empty(M, N, dtype=torch.bfloat16, device=dev), torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    _gemm_ws(gc, A, Bd, trans_b, o1, bias=bias, act="gelu_erf", residual=res)
    _gemm_ws(gc, A, Bd, trans_b, o2, 1, bias=bias, act="gelu_erf", residual=res)
    torch.cuda.synchronize()
    assert torch.equal(o1.view(torch.int16), o2.view(torch.int16))


def test_a_thin_last_round_of_the_int8_layer(gc, dev):
    big = [1, 1, 1, 256, 256, 64, 128, 128, 32]
    M, N, K = 4096, 5120, 512
    c, _ = gc.tile_config(M, N, K, a_dtype=gc.U8)
    assert c.kernel == 2 and c.workgroups == 256 + 4 * 64
    torch.manual_seed(9)
    A = torch.randint(0, 256, (M, K), dtype=torch.uint8, device=dev)
    W = torch.randint(-127, 128, (K, N), dtype=torch.int8, device=dev)
    cs = gc.colsum_s8(W)
    scale, bias = (torch.rand(N, device=dev) * 0.009 + 0.001).float(), torch.randn(N, device=dev).float()
    a = gc.gemm_int8(A, W, cs, 128, scale, bias, "gelu_erf", gc.BF16)
    b = gc.gemm_int8(A, W, cs, 128, scale, bias, "gelu_erf", gc.BF16, matmul_config=big)
    raw = gc.gemm_int8(A, W, cs, 128, out_dtype=gc.S32)  # s32 results: the same two launches, plain stores
    c, _ = gc.tile_config(M, N, K, a_dtype=gc.U8, out_dtype=gc.S32)
    assert c.kernel == 2 and c.workgroups == 256 + 4 * 64
    torch.cuda.synchronize()
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    assert torch.equal(raw.cpu().to(torch.int64), A.cpu().to(torch.int64) @ W.cpu().to(torch.int64))


NT_SHAPES = [(256, 256, 128), (512, 768, 256), (300, 200, 100), (257, 511, 129), (1, 7, 5), (33, 1, 64), (128, 256, 8),
             (32, 4096, 4096), (1, 1024, 2048), (32, 11008, 4096), (64, 512, 2048), (33, 1024, 1024), (17, 2048, 512),
             (32, 4096, 11008), (65, 1024, 1024), (32, 1056, 1088), (32, 8192, 1024), (64, 8192, 512)]


def _streams_weights(M, N, K):
    """Shapes the [N,K] entry point gives to one of the weight-streaming kernels (short A, enough weights): the
    8-wave kernel with the LDS ring, or the one that loads fragments straight into registers."""
    ring = M <= 128 and N % 4 == 0 and N >= 512 and K % 128 == 0 and K >= 512 and N * K >= 1 << 22
    return ring or (M <= 32 and N % 32 == 0 and K % 64 == 0 and K >= 256 and 1 << 20 <= N * K <= 3 << 23)


@pytest.mark.parametrize("M,N,K", NT_SHAPES)
def test_bf16_gemm_transposed_b(gc, orc, wl, dev, M, N, K):
    """B stored [N,K] (linalg.matmul_transpose_b): against the oracle on A . Bt^T, and against the [K,N] kernel on
    a transposed copy -- bit for bit where both run the tile kernels (same products, same order), to rounding
    where the short-A shapes take the weight-streaming kernel (another summation order).  Covers whole-tile,
    ragged, split-K and streaming shapes, one and two row tiles."""
    torch.manual_seed(4)
    A = (torch.randn(M, K) * 0.5).to(torch.bfloat16).to(dev)
    Bt = (torch.randn(N, K) * 0.5).to(torch.bfloat16).to(dev)
    bias = torch.randn(N).to(torch.bfloat16).to(dev)
    B = Bt.t().contiguous()
    for b, act, odt in [(None, None, gc.BF16), (bias, "relu", gc.BF16), (bias, "gelu_erf", gc.F32)]:
        nt = gc.gemm_bf16_nt(A, Bt, b, act, odt)
        nn = gc.gemm_bf16(A, B, b, act, odt)
        again = gc.gemm_bf16_nt(A, Bt, b, act, odt)
        torch.cuda.synchronize()
        assert torch.equal(nt, again), "two runs differ"
        if _streams_weights(M, N, K):
            pre = (A.float() @ Bt.float().t()).cpu().numpy()  # magnitude of the value that was rounded before the bias
            assert_close(nn.float().cpu().numpy(), nt.float().cpu().numpy(), 1e-2 if odt == gc.BF16 else 1e-4,
                         "NT against NN (%s)" % act, mag=pre)
        else:
            assert torch.equal(nt, nn), "NT differs from NN on the transposed copy (%s, %s)" % (act, odt)
    if M * N * K <= 1 << 24:
        ref = orc.bf16_to_f32(orc.matmul_bf16(wl.bf16_bits(A.cpu()), wl.bf16_bits(B.cpu())))
        out = gc.gemm_bf16_nt(A, Bt)
        torch.cuda.synchronize()
        assert_close(ref, out.float().cpu().numpy(), 1e-2, "bf16 NT %dx%dx%d" % (M, N, K))


def test_bf16_gemm_streaming_kernel_exact_on_integers(gc, dev):
    """Small integers: every product and partial sum is exact in f32, so any summation order gives the same bits.
    32 and 64 rows, K slices of unequal length (K/64 = 43 steps over 16 waves), and wide N where one slice per
    workgroup is enough and the epilogue runs inside the streaming kernel."""
    torch.manual_seed(8)
    for M, N, K in [(32, 1024, 2752), (64, 1024, 2752), (5, 4096, 256), (32, 8192, 1024), (40, 16384, 512)]:
        A = torch.randint(-3, 4, (M, K), device=dev).to(torch.bfloat16)
        Bt = torch.randint(-3, 4, (N, K), device=dev).to(torch.bfloat16)
        out = gc.gemm_bf16_nt(A, Bt, out_dtype=gc.F32)
        torch.cuda.synchronize()
        assert torch.equal(out, A.float() @ Bt.float().t())
        # left to itself the launcher keeps the streaming kernel for up to 32 rows; a slice count by name (KThreads)
        # selects it for every shape it can run, the 64-row instantiation included
        c, _ = gc.tile_config(M, N, K, trans_b=True, out_dtype=gc.F32, matmul_config=[1, 1, 16, 256, 256, 64, 128, 128, 32])
        if K >= 1024:  # 16 slices need 16 K blocks of 64 (the reference's validity rule), else the set is ignored
            assert c.kernel == 4, (M, N, K, c.kernel)
        ws = torch.empty(16 * M * N, dtype=torch.float32, device=dev)
        out2 = torch.full((M, N), 7.0, dtype=torch.float32, device=dev)
        _gemm_ws(gc, A, Bt, True, out2, 16, ws=ws)
        torch.cuda.synchronize()
        assert torch.equal(out2, out)


@pytest.mark.parametrize("M", [1, 7, 16, 32, 33, 50, 64, 65, 100, 128])
@pytest.mark.parametrize("N,K", [(4096, 1024), (4100, 4096), (520, 11008), (11008, 4096), (12352, 640)])
def test_short_a_streaming_kernel_exact_on_integers(gc, dev, M, N, K):
    """Up to 128 rows against [N,K] weights (the A tile of the ring holds 32, 64 or 128): 8-wave workgroups on panels of 64 columns (the last one 4 or 8 columns
    wide here), K in one piece where the panels fill the GPU and in slices with the second pass where they do not,
    slice lengths that differ (86 and 5 stages), rows past M.  Small integers: every sum is exact in f32, whatever
    the order.  The caller's slice count and a call without workspace (one slice, epilogue in the kernel) agree."""
    c, _ = gc.tile_config(M, N, K, trans_b=True, out_dtype=gc.F32)
    assert (c.kernel, c.bm, c.bn, c.waves_m * c.waves_n) == (4, 32 if M <= 32 else (64 if M <= 64 else 128), 64, 4) and c.workgroups == -(-N // 64) * c.split_k
    want_s = (256 + -(-N // 64) // 2) // -(-N // 64)
    if M > 32 and want_s * -(-N // 64) > 256:   # the 64-row ring: one workgroup per compute unit
        want_s = max(1, 256 // -(-N // 64))
    assert c.split_k == (1 if N > 10000 else min(K // 512, want_s))
    torch.manual_seed(M + N + K)
    A = torch.randint(-3, 4, (M, K), device=dev).to(torch.bfloat16)
    Bt = torch.randint(-3, 4, (N, K), device=dev).to(torch.bfloat16)
    want = A.float() @ Bt.float().t()
    guard = torch.full((M + 2, N), 7.0, dtype=torch.float32, device=dev)
    out = guard[1:M + 1]
    gc.gemm_bf16_nt(A, Bt, out_dtype=gc.F32, out=out)
    torch.cuda.synchronize()
    assert torch.equal(out, want)
    assert bool((guard[0] == 7.0).all()) and bool((guard[M + 1] == 7.0).all())
    # the same weights stored [K,N]: the same kernel with transposing fragment reads (N a multiple of 8), else tiles
    B = Bt.t().contiguous()
    ckn, _ = gc.tile_config(M, N, K, out_dtype=gc.F32)
    assert (ckn.kernel == 4) == (N % 8 == 0), (ckn.kernel, N)
    guard_kn = torch.full((M + 2, N), 7.0, dtype=torch.float32, device=dev)
    gc.gemm_bf16(A, B, out_dtype=gc.F32, out=guard_kn[1:M + 1])
    torch.cuda.synchronize()
    assert torch.equal(guard_kn[1:M + 1], want)
    assert bool((guard_kn[0] == 7.0).all()) and bool((guard_kn[M + 1] == 7.0).all())
    one = torch.full((M, N), 7.0, dtype=torch.float32, device=dev)
    _gemm_ws(gc, A, Bt, True, one)  # no workspace: K in one piece
    ws = torch.empty(3 * M * N, dtype=torch.float32, device=dev)
    three = torch.full((M, N), 7.0, dtype=torch.float32, device=dev)
    _gemm_ws(gc, A, Bt, True, three, 3, ws=ws)
    torch.cuda.synchronize()
    assert torch.equal(one, want) and torch.equal(three, want)


@pytest.mark.parametrize("M,N,K", [(32, 4096, 4096), (9, 11008, 4096), (32, 4096, 11008), (20, 1032, 4096), (64, 4096, 4096), (40, 11008, 4096), (128, 4096, 4096),
                                   (77, 11008, 4096)])
def test_short_a_streaming_kernel_rounding_points(gc, dev, M, N, K):
    """N(0,1) data through bias, GELU and a residual, bf16 and f32 results: against the same sums in float64 rounded
    at the reference's points (after the matmul and after each op for bf16 results), to one bf16 step of the larger of
    the value and the rounded intermediate; sliced and unsliced agree to the same bound."""
    torch.manual_seed(N + K)
    A = (torch.randn(M, K, device=dev) * 0.5).to(torch.bfloat16)
    Bt = (torch.randn(N, K, device=dev) * 0.05).to(torch.bfloat16)
    bias, res = torch.randn(N, device=dev).to(torch.bfloat16), torch.randn(M, N, device=dev).to(torch.bfloat16)
    acc = A.double() @ Bt.double().t()
    r = lambda t: t.to(torch.bfloat16).double()  # noqa: E731
    gelu = lambda t: 0.5 * t * (1.0 + torch.special.erf(t / 2.0 ** 0.5))  # noqa: E731
    want16 = r(r(gelu(r(r(acc) + bias.double()))) + res.double())
    want32 = gelu(acc + bias.double()) + res.double()
    o16 = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    o32 = torch.empty(M, N, dtype=torch.float32, device=dev)
    _gemm_ws(gc, A, Bt, True, o16, bias=bias, act="gelu_erf", residual=res)
    _gemm_ws(gc, A, Bt, True, o32, bias=bias, act="gelu_erf", residual=res)
    ws = torch.empty(4 * M * N, dtype=torch.float32, device=dev)
    s16 = torch.empty_like(o16)
    _gemm_ws(gc, A, Bt, True, s16, 4, bias=bias, act="gelu_erf", residual=res, ws=ws)
    torch.cuda.synchronize()
    mag = torch.maximum(acc.abs(), torch.maximum(want16.abs(), res.double().abs())) + 1.0
    # [K,N] weights: the same products in the same order, so the same bits
    k16 = torch.empty_like(o16)
    _gemm_ws(gc, A, Bt.t().contiguous(), False, k16, bias=bias, act="gelu_erf", residual=res)
    torch.cuda.synchronize()
    if N % 8 == 0:
        assert torch.equal(k16.view(torch.int16), o16.view(torch.int16))
    # a bias given as f32 holds the same values: the same bits come out
    assert torch.equal(gc.gemm_bf16_nt(A, Bt, bias.float(), "relu", gc.F32), gc.gemm_bf16_nt(A, Bt, bias, "relu", gc.F32))
    assert float(((o16.double() - want16).abs() / mag).max()) < 2.0 ** -7
    assert float(((s16.double() - want16).abs() / mag).max()) < 2.0 ** -7
    assert float(((o32.double() - want32).abs() / mag).max()) < 1e-5


def test_short_a_streaming_kernel_strided_operands(gc, dev):
    """Rows of A, of the weights and of the result further apart than their length (slices of wider tensors, start
    offsets of 16 bytes): exact on integers, and nothing written between the rows of the result."""
    M, N, K = 24, 2048, 2048
    c, _ = gc.tile_config(M, N, K, trans_b=True)
    assert c.kernel == 4 and c.bn == 64
    torch.manual_seed(12)
    wide_a = torch.randint(-3, 4, (M, K + 72), device=dev).to(torch.bfloat16)
    wide_w = torch.randint(-3, 4, (N, K + 136), device=dev).to(torch.bfloat16)
    wide_c = torch.full((M, N + 40), 7.0, dtype=torch.float32, device=dev)
    A, Bt, out = wide_a[:, 8:8 + K], wide_w[:, 16:16 + K], wide_c[:, 4:4 + N]
    gc.gemm_bf16_nt(A, Bt, out_dtype=gc.F32, out=out)
    torch.cuda.synchronize()
    assert torch.equal(out, A.float() @ Bt.float().t())
    assert bool((wide_c[:, :4] == 7.0).all()) and bool((wide_c[:, 4 + N:] == 7.0).all())


def test_bf16_gemm_transposed_b_strided_rows(gc, dev):
    """Rows of Bt further apart than K (a weight that is a slice of a wider one)."""
    torch.manual_seed(6)
    M, N, K = 256, 512, 256
    A = torch.randn(M, K, device=dev).bfloat16()
    wide = torch.randn(N, K + 64, device=dev).bfloat16()
    Bt = wide[:, 8:8 + K]  # row stride K+64, start offset 16 bytes
    out = gc.gemm_bf16_nt(A, Bt)
    ref = gc.gemm_bf16(A, Bt.t().contiguous())
    torch.cuda.synchronize()
    assert torch.equal(out, ref)


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("nb,M,N,K", [(6, 256, 256, 128), (3, 100, 72, 50), (16, 128, 64, 64), (2, 512, 768, 256)])
def test_batched_gemm_one_launch(gc, dev, dtype, nb, M, N, K):
    """Strided batches in one launch against the same GEMMs one at a time (bit for bit: the same kernel runs on
    each batch), with B per batch, B stored [N,K], and one B shared by all batches; and against torch."""
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    torch.manual_seed(31)
    A = (torch.randn(nb, M, K, device=dev) * 0.5).to(td)
    B = (torch.randn(nb, K, N, device=dev) * 0.5).to(td)
    bias = torch.randn(N, device=dev).to(td)
    one = gc.gemm_bf16 if dtype == "bf16" else gc.gemm_f32
    out = gc.gemm_batched(A, B, bias=bias, act="relu")
    ref = torch.stack([one(A[b], B[b], bias, "relu") for b in range(nb)])
    torch.cuda.synchronize()
    assert torch.equal(out, ref)
    exact = torch.relu(A.double() @ B.double() + bias.double())
    assert_close(exact.cpu().numpy(), out.double().cpu().numpy(), 2e-2 if dtype == "bf16" else 1e-4, "batched %s" % dtype,
                 mag=(A.double() @ B.double()).cpu().numpy())
    Bt = B.transpose(1, 2).contiguous()
    out_t = gc.gemm_batched(A, Bt, trans_b=True, bias=bias, act="relu")
    shared = gc.gemm_batched(A, B[0].contiguous())
    ref_s = torch.stack([one(A[b], B[0].contiguous()) for b in range(nb)])
    torch.cuda.synchronize()
    assert torch.equal(out_t, ref) if dtype == "bf16" else torch.allclose(out_t, ref, rtol=1e-5, atol=1e-5)
    assert torch.equal(shared, ref_s)


# every kernel that can finish a bf16 GEMM: whole tiles (staged bf16 stores / direct f32 stores), partial tiles,
# K sliced over workgroups with the second pass, weights stored [N,K] streamed by the short-A kernel with one
# slice (epilogue in the kernel) and with several (second pass), and [N,K] weights through the tile kernel
RESIDUAL_CASES = [(512, 512, 256, False), (256, 768, 512, True), (300, 200, 100, False), (257, 130, 96, True),
                  (64, 512, 2048, False), (32, 4096, 4096, True), (32, 11008, 4096, True), (48, 8192, 512, True),
                  (1, 7, 5, False)]


@pytest.mark.parametrize("M,N,K,nt", RESIDUAL_CASES)
@pytest.mark.parametrize("res_dtype,out_f32", [("bf16", False), ("f32", False), ("f32", True), ("bf16", True)])
@pytest.mark.parametrize("epi", ["none", "bias_gelu"])
def test_bf16_gemm_residual_equals_separate_add(gc, dev, M, N, K, nt, res_dtype, out_f32, epi):
    """act(A.B + bias) + R in the epilogue is, bit for bit, the same GEMM without R followed by an add that rounds
    once more when the result is bf16 (the rounding points of the reference's bf16 graphs)."""
    torch.manual_seed(M * 7 + N)
    A = (torch.randn(M, K) * 0.5).to(torch.bfloat16).to(dev)
    B = (torch.randn((N, K) if nt else (K, N)) * 0.5).to(torch.bfloat16).to(dev)
    R = torch.randn(M, N).to(torch.bfloat16 if res_dtype == "bf16" else torch.float32).to(dev)
    bias = torch.randn(N).to(torch.bfloat16).to(dev) if epi != "none" else None
    act = "gelu_erf" if epi != "none" else None
    odt = gc.F32 if out_f32 else gc.BF16
    plain = (gc.gemm_bf16_nt if nt else gc.gemm_bf16)(A, B, bias, act, out_dtype=odt)
    fused = gc.gemm_bf16_residual(A, B, R, trans_b=nt, bias=bias, act=act, out_dtype=odt)
    torch.cuda.synchronize()
    want = plain.float() + R.float()  # one f32 add, as in the kernel
    if not out_f32:
        want = want.to(torch.bfloat16)
    assert fused.dtype == want.dtype and torch.equal(fused, want), \
        "max diff " + str((fused.float() - want.float()).abs().max().item())


def test_bf16_gemm_residual_unaligned_and_strided(gc, dev):
    """A residual whose rows are not 16-byte aligned goes through the kernels that load element by element; row
    strides larger than the row are honoured."""
    M, N, K = 256, 256, 128
    torch.manual_seed(3)
    A = (torch.randn(M, K) * 0.5).to(torch.bfloat16).to(dev)
    B = (torch.randn(K, N) * 0.5).to(torch.bfloat16).to(dev)
    big = torch.randn(M, N + 3).to(torch.bfloat16).to(dev)
    plain = gc.gemm_bf16(A, B)
    for R in (big[:, 1:N + 1], big[:, :N]):
        fused = gc.gemm_bf16_residual(A, B, R)
        torch.cuda.synchronize()
        assert torch.equal(fused, (plain.float() + R.float()).to(torch.bfloat16))


def test_bf16_gemm_residual_in_place_and_errors(gc, dev):
    M, N, K = 512, 256, 192
    torch.manual_seed(4)
    A = (torch.randn(M, K) * 0.5).to(torch.bfloat16).to(dev)
    B = (torch.randn(K, N) * 0.5).to(torch.bfloat16).to(dev)
    R = torch.randn(M, N).to(torch.bfloat16).to(dev)
    want = (gc.gemm_bf16(A, B).float() + R.float()).to(torch.bfloat16)
    acc = R.clone()
    gc.gemm_bf16_residual(A, B, acc, out=acc)  # x += A.B: every element is read before it is written
    torch.cuda.synchronize()
    assert torch.equal(acc, want)
    L = gc.lib()
    import ctypes as C
    vp = lambda t: C.c_void_p(t.data_ptr())
    st = L.gcmi_gemm_bf16_residual(vp(A), vp(B), vp(acc), 1, M, N, K, K, N, N, 0, 0, 0, 0, None, gc.BF16, 0, vp(R), N - 1,
                                   gc.BF16, gc.BF16, None)
    assert st != 0 and b"ldr" in L.gcmi_last_error()
    st = L.gcmi_gemm_bf16_residual(vp(A), vp(B), vp(acc), 1, M, N, K, K, N, N, 0, 0, 0, 0, None, gc.BF16, 0, vp(R), N,
                                   gc.S32, gc.BF16, None)
    assert st != 0 and b"residual_dtype" in L.gcmi_last_error()
