"""GPU parity: fused attention through the C ABI against the oracle's
batch_matmul -> scale -> +mask -> softmax -> batch_matmul composition."""
import numpy as np
import pytest
import torch

from conftest import assert_close

pytestmark = pytest.mark.gpu

def _pv_mag(Q, K, V, mask, scale):
    """sum_j softmax(S)_ij |V_jd| in f64: the magnitude of the terms whose
    weights are rounded to bf16 before the second matmul (in the reference
    graph P is a bf16 tensor).  One half-ulp of each term, 2^-9 p|v|, is the
    error unit of an output element, however much the signed sum cancels."""
    S = Q.double() @ K.double().transpose(-1, -2) * scale
    if mask is not None:
        S = S + mask.double()
    return (torch.softmax(S, -1) @ V.double().abs()).numpy()


CASES = [(1, 2, 128, 128, "causal"), (1, 1, 256, 192, "none"), (2, 2, 100, 77, "causal"), (1, 2, 384, 384, "neg1e9"),
         (1, 1, 1, 1, "none"), (1, 3, 130, 64, "random"), (1, 1, 64, 300, "neg30000"),
         # the pipelined loop's ends: one key block (no steady state), two, an odd count with general mask tiles
         (1, 2, 128, 64, "causal"), (1, 2, 256, 64, "random"), (1, 1, 128, 320, "random"), (1, 2, 128, 128, "none"),
         # row and key counts off the tile sizes on the pipelined kernel: the last workgroup / key block overlaps its
         # predecessor (duplicate keys masked out); general, constant and absent masks, one and several blocks
         (1, 2, 200, 200, "causal"), (1, 2, 130, 68, "random"), (2, 2, 300, 1000, "causal"), (1, 1, 257, 321, "none"),
         (1, 2, 129, 127 + 1, "neg1e9"), (1, 1, 1000, 100, "random"), (1, 2, 1111, 1112, "causal"),
         # odd key counts with a mask: its rows start at any 4-byte aligned address
         (1, 2, 131, 129, "random"), (1, 1, 1001, 1001, "causal"), (2, 2, 257, 70, "neg30000")]


def _mask(kind, Sq, Sk):
    if kind == "none":
        return None
    if kind == "causal":
        return torch.triu(torch.full((Sq, Sk), float("-inf")), diagonal=1)
    if kind == "neg1e9":
        return torch.triu(torch.full((Sq, Sk), -1e9), diagonal=1)
    if kind == "neg30000":
        return torch.triu(torch.full((Sq, Sk), -30000.0), diagonal=1)
    torch.manual_seed(9)
    return torch.randn(Sq, Sk) * 2


@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("B,H,Sq,Sk,kind", CASES)
def test_mha_matches_oracle(gc, orc, wl, dev, B, H, Sq, Sk, kind, D):
    torch.manual_seed(0)
    Q = torch.randn(B, H, Sq, D).to(torch.bfloat16)
    torch.manual_seed(1)
    K = torch.randn(B, H, Sk, D).to(torch.bfloat16)
    torch.manual_seed(2)
    V = torch.randn(B, H, Sk, D).to(torch.bfloat16)
    mask = _mask(kind, Sq, Sk)
    scale = 1 / np.sqrt(D)
    ref = orc.bf16_to_f32(orc.mha_bf16(wl.bf16_bits(Q), wl.bf16_bits(K), wl.bf16_bits(V),
                                       None if mask is None else mask.numpy(), scale))
    out = gc.mha_fwd_bf16(Q.to(dev), K.to(dev), V.to(dev), None if mask is None else mask.to(dev), scale)
    torch.cuda.synchronize()
    assert_close(ref, out.float().cpu().numpy(), 1e-2, "mha %s D=%d" % (kind, D), mag=_pv_mag(Q, K, V, mask, scale))


def test_head_dims_not_built_are_refused(gc, dev):
    Q = torch.zeros(1, 1, 64, 96, dtype=torch.bfloat16, device=dev)
    with pytest.raises(Exception, match="head_dim 96"):
        gc.mha_fwd_bf16(Q, Q, Q)


def test_fully_masked_rows_are_nan_like_the_reference_softmax(gc, orc, wl, dev):
    torch.manual_seed(0)
    Q = torch.randn(1, 1, 128, 128).to(torch.bfloat16)
    K = torch.randn(1, 1, 128, 128).to(torch.bfloat16)
    V = torch.randn(1, 1, 128, 128).to(torch.bfloat16)
    mask = torch.zeros(128, 128)
    mask[5, :] = float("-inf")
    mask[70, :64] = float("-inf")  # first key block fully masked, second one live
    ref = orc.bf16_to_f32(orc.mha_bf16(wl.bf16_bits(Q), wl.bf16_bits(K), wl.bf16_bits(V), mask.numpy(), 0.1))
    out = gc.mha_fwd_bf16(Q.to(dev), K.to(dev), V.to(dev), mask.to(dev), 0.1).float().cpu().numpy()
    assert np.isnan(out[0, 0, 5]).all() and np.isnan(ref[0, 0, 5]).all()
    assert not np.isnan(np.delete(out[0, 0], 5, axis=0)).any()
    assert_close(ref, out, 1e-2, "mha masked rows", mag=_pv_mag(Q, K, V, mask, 0.1))


def test_mha_full_size_heads_and_invariants(gc, orc, wl, dev):
    """BASELINE config 5 (B4 H32 S2048 D128, additive causal mask): three
    (batch, head) slices against the oracle; first row equals V[0] exactly;
    V == 1 gives 1 (weights sum to one)."""
    Q, K, V, mask, scale = wl.bf16_mha()
    Qd, Kd, Vd, md = Q.to(dev), K.to(dev), V.to(dev), mask.to(dev)
    out = gc.mha_fwd_bf16(Qd, Kd, Vd, md, scale)
    torch.cuda.synchronize()
    assert torch.equal(out[:, :, 0].view(torch.int16), Vd[:, :, 0].view(torch.int16))
    for (b, h) in [(0, 0), (2, 17), (3, 31)]:
        ref = orc.bf16_to_f32(orc.mha_bf16(wl.bf16_bits(Q[b:b + 1, h:h + 1]), wl.bf16_bits(K[b:b + 1, h:h + 1]),
                                           wl.bf16_bits(V[b:b + 1, h:h + 1]), mask.numpy(), scale))
        mag = _pv_mag(Q[b:b + 1, h:h + 1], K[b:b + 1, h:h + 1], V[b:b + 1, h:h + 1], mask, scale)
        assert_close(ref, out[b:b + 1, h:h + 1].float().cpu().numpy(), 1e-2, "mha full size (%d,%d)" % (b, h), mag=mag)
    ones = gc.mha_fwd_bf16(Qd, Kd, torch.ones_like(Vd), md, scale)
    torch.cuda.synchronize()
    assert (ones.float() - 1).abs().max().item() <= 2 ** -7


@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("Sq,Sk,kind", [(512, 512, "causal"), (384, 640, "causal"), (256, 256, "neg1e9"), (300, 200, "random"),
                                        (1000, 1000, "causal"), (200, 1100, "causal")])
def test_skipping_masked_blocks_changes_no_bit(gc, dev, Sq, Sk, kind, D):
    """Key blocks whose mask tile is -inf for a whole query block carry softmax
    weight exactly 0: leaving them out must give the same bits as visiting them (both head dims of the pipelined
    kernel, also with row and key counts off the tile sizes)."""
    torch.manual_seed(4)
    Q = torch.randn(1, 8, Sq, D).to(torch.bfloat16).to(dev)
    K = torch.randn(1, 8, Sk, D).to(torch.bfloat16).to(dev)
    V = torch.randn(1, 8, Sk, D).to(torch.bfloat16).to(dev)
    mask = _mask(kind, Sq, Sk).to(dev)
    a = gc.mha_fwd_bf16(Q, K, V, mask, 0.088, skip_masked=True)
    b = gc.mha_fwd_bf16(Q, K, V, mask, 0.088, skip_masked=False)
    torch.cuda.synchronize()
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))


@pytest.mark.parametrize("skip", [True, False])
def test_band_mask_over_many_key_blocks(gc, orc, wl, dev, skip):
    """8192 keys = 128 key blocks (two groups of 64 in the kernel's bookkeeping).
    A band mask leaves -inf blocks before and after the band, and the band
    crosses the group boundary: the set of visited blocks has gaps on both
    sides and spans both groups."""
    torch.manual_seed(5)
    H, Sq, Sk, D = 8, 256, 8192, 128
    Q = torch.randn(1, H, Sq, D).to(torch.bfloat16)
    K = torch.randn(1, H, Sk, D).to(torch.bfloat16)
    V = torch.randn(1, H, Sk, D).to(torch.bfloat16)
    qi = torch.arange(Sq).reshape(-1, 1)
    kj = torch.arange(Sk).reshape(1, -1)
    lo = 3000 + 4 * qi            # band start moves with the query row
    mask = torch.where((kj >= lo) & (kj < lo + 1500), 0.0, float("-inf")).float()
    mask[:, 7000:7003] = -2.5      # a few finite entries far from the band: one more visited block
    scale = 1 / np.sqrt(D)
    out = gc.mha_fwd_bf16(Q.to(dev), K.to(dev), V.to(dev), mask.to(dev), scale, skip_masked=skip)
    torch.cuda.synchronize()
    for h in (0, 5):
        ref = orc.bf16_to_f32(orc.mha_bf16(wl.bf16_bits(Q[:, h:h + 1]), wl.bf16_bits(K[:, h:h + 1]),
                                           wl.bf16_bits(V[:, h:h + 1]), mask.numpy(), scale))
        assert_close(ref, out[:, h:h + 1].float().cpu().numpy(), 1e-2, "band mask head %d" % h,
                     mag=_pv_mag(Q[:, h:h + 1], K[:, h:h + 1], V[:, h:h + 1], mask, scale))


@pytest.mark.parametrize("kind", ["causal", "none"])
def test_head_dim_64_at_benchmark_size(gc, orc, wl, dev, kind):
    """B4 H32 S2048 at head dim 64 on the pipelined kernel: three heads against the oracle."""
    B, H, S, D = 4, 32, 2048, 64
    Q, K, V, mask, scale = wl.bf16_mha(B, H, S, D)
    if kind == "none":
        mask = None
    out = gc.mha_fwd_bf16(Q.to(dev), K.to(dev), V.to(dev), None if mask is None else mask.to(dev), scale)
    torch.cuda.synchronize()
    for (b, h) in [(0, 0), (2, 13), (3, 31)]:
        sl = (slice(b, b + 1), slice(h, h + 1))
        ref = orc.bf16_to_f32(orc.mha_bf16(wl.bf16_bits(Q[sl]), wl.bf16_bits(K[sl]), wl.bf16_bits(V[sl]),
                                           None if mask is None else mask.numpy(), scale))
        assert_close(ref, out[sl].float().cpu().numpy(), 1e-2, "D=64 head (%d,%d) %s" % (b, h, kind),
                     mag=_pv_mag(Q[sl], K[sl], V[sl], mask, scale))


def test_negative_scale_takes_the_general_kernel(gc, orc, wl, dev):
    """The fast kernel folds the scale into the maximum (needs scale > 0); a
    negative scale must still give the reference result."""
    torch.manual_seed(6)
    Q = torch.randn(1, 2, 128, 128).to(torch.bfloat16)
    K = torch.randn(1, 2, 128, 128).to(torch.bfloat16)
    V = torch.randn(1, 2, 128, 128).to(torch.bfloat16)
    mask = _mask("causal", 128, 128)
    ref = orc.bf16_to_f32(orc.mha_bf16(wl.bf16_bits(Q), wl.bf16_bits(K), wl.bf16_bits(V), mask.numpy(), -0.05))
    out = gc.mha_fwd_bf16(Q.to(dev), K.to(dev), V.to(dev), mask.to(dev), -0.05)
    torch.cuda.synchronize()
    assert_close(ref, out.float().cpu().numpy(), 1e-2, "negative scale", mag=_pv_mag(Q, K, V, mask, -0.05))


@pytest.mark.parametrize("kind", ["causal", "random", "none"])
def test_wide_workgroups_many_heads(gc, orc, wl, dev, kind):
    """256 (batch, head) pairs x 256 query rows: enough 256-row workgroups to fill
    the GPU, so the 8-wave kernel runs.  A few heads against the oracle, and the
    skip / no-skip modes against each other."""
    torch.manual_seed(7)
    B, H, Sq, Sk, D = 8, 32, 256, 320, 128
    Q = torch.randn(B, H, Sq, D).to(torch.bfloat16)
    K = torch.randn(B, H, Sk, D).to(torch.bfloat16)
    V = torch.randn(B, H, Sk, D).to(torch.bfloat16)
    mask = _mask(kind, Sq, Sk)
    md = None if mask is None else mask.to(dev)
    scale = 1 / np.sqrt(D)
    out = gc.mha_fwd_bf16(Q.to(dev), K.to(dev), V.to(dev), md, scale)
    out2 = gc.mha_fwd_bf16(Q.to(dev), K.to(dev), V.to(dev), md, scale, skip_masked=False)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), out2.view(torch.int16))
    for (b, h) in [(0, 0), (3, 17), (7, 31)]:
        sl = (slice(b, b + 1), slice(h, h + 1))
        ref = orc.bf16_to_f32(orc.mha_bf16(wl.bf16_bits(Q[sl]), wl.bf16_bits(K[sl]), wl.bf16_bits(V[sl]),
                                           None if mask is None else mask.numpy(), scale))
        assert_close(ref, out[sl].float().cpu().numpy(), 1e-2, "wide %s (%d,%d)" % (kind, b, h),
                     mag=_pv_mag(Q[sl], K[sl], V[sl], mask, scale))
