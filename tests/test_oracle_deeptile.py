"""CPU: deep-tile loop nest, config validity and VNNI packing of the oracle."""
import numpy as np
import pytest

BF16, F32, S8, U8 = 2, 3, 5, 6


def test_validate_config_truth_table(orc):
    """Predicate of lib/gc/Analysis/MatmulConfigAnalysis.cpp:40-65,99-106."""
    lit = [4, 2, 1, 256, 256, 256, 32, 32, 32]  # deepTileContractionNamedOp.mlir:33
    assert orc.validate_config(lit, 4096, 4096, 4096, 8)
    assert not orc.validate_config(lit, 4096, 4096, 4096, 16)        # thread product != num_threads
    assert orc.validate_config(lit, 4096, 4096, 4096, 0)             # 0: product not checked
    assert not orc.validate_config([4, 2, 1, 256, 256, 256, 0, 32, 32], 4096, 4096, 4096)   # non-positive
    assert not orc.validate_config([4, 2, 1, 250, 256, 256, 32, 32, 32], 4096, 4096, 4096)  # MBlock % iM
    assert not orc.validate_config([1, 1, 1, 32, 32, 32, 32, 32, 32], 4100, 4096, 4096)     # M % iM
    assert not orc.validate_config([1, 1, 1, 32, 32, 32, 32, 32, 32], 4096, 4100, 4096)     # N % iN
    assert not orc.validate_config([1, 1, 1, 32, 32, 96, 32, 32, 32], 4096, 4096, 4096)     # K % KBlock
    assert not orc.validate_config([1, 1, 1, 32, 32, 48, 32, 32, 32], 4096, 4096, 4096)     # KBlock % iK
    assert orc.validate_config([32, 2, 2, 256, 256, 256, 32, 32, 32], 4096, 4096, 4096, 128)  # :130 (KThreads 2)
    assert not orc.validate_config([1, 1, 8, 32, 32, 64, 32, 32, 32], 128, 128, 256)        # ceil(K/KBlock) < KThreads


def test_default_innermost_is_32_or_whole_dim(orc):
    """lib/gc/Analysis/MatmulConfigAnalysis.cpp:465-468"""
    assert orc.default_config(128, 256, 512).tolist()[6:] == [32, 32, 32]
    assert orc.default_config(100, 256, 77).tolist()[6:] == [100, 32, 77]


def test_extents_match_lit_expectations(orc):
    """forall steps FileChecked in test/mlir/test/gc/Transforms/
    deepTileContractionNamedOp.mlir:10-13 (M step 1024, N step 2048) and
    :108-109 (32 M-threads on 4096 rows -> step 256; KThreads 2 -> K halves)."""
    assert orc.deep_tile_extents([4, 2, 1, 256, 256, 256, 32, 32, 32], 4096, 4096, 4096) == (0, 1024, 2048)
    k, m, _ = orc.deep_tile_extents([32, 2, 2, 256, 256, 256, 32, 32, 32], 4096, 4096, 4096)
    assert (k, m) == (2048, 256)
    # rows that do not split evenly: ceil(ceil(M/MBlock)/MThreads)*MBlock
    assert orc.deep_tile_extents([3, 1, 1, 64, 32, 32, 32, 32, 32], 320, 64, 64)[1] == 128


CONFIGS = [
    [1, 1, 1, 32, 32, 32, 32, 32, 32],
    [4, 2, 1, 64, 64, 64, 32, 32, 32],
    [2, 2, 2, 64, 32, 32, 32, 32, 32],
    [3, 1, 1, 64, 128, 128, 32, 64, 32],   # uneven M split, tails inside blocks
    [1, 4, 4, 128, 32, 32, 64, 32, 16],
    [8, 1, 1, 32, 256, 256, 32, 128, 64],
]


@pytest.mark.parametrize("cfg", CONFIGS)
def test_int8_result_is_config_independent_and_exact(orc, cfg):
    rng = np.random.default_rng(11)
    M, N, K = 192, 256, 256
    A = rng.integers(0, 256, (M, K)).astype(np.uint8)
    W = rng.integers(-127, 128, (K, N)).astype(np.int8)
    assert orc.validate_config(cfg, M, N, K)
    got = orc.deep_tile_matmul(A, W, U8, S8, cfg)
    want = A.astype(np.int64) @ W.astype(np.int64)
    assert (got == want).all()


@pytest.mark.parametrize("cfg", CONFIGS[:4])
def test_fp_results_agree_across_configs(orc, cfg):
    rng = np.random.default_rng(12)
    M, N, K = 192, 256, 256
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.standard_normal((K, N)).astype(np.float32)
    want = A.astype(np.float64) @ B.astype(np.float64)
    got = orc.deep_tile_matmul(A, B, F32, F32, cfg)
    assert np.allclose(got, want, rtol=1e-5, atol=1e-4)
    A16, B16 = orc.f32_to_bf16(A), orc.f32_to_bf16(B)
    got16 = orc.deep_tile_matmul(A16, B16, BF16, BF16, cfg)
    want16 = orc.bf16_to_f32(A16).astype(np.float64) @ orc.bf16_to_f32(B16).astype(np.float64)
    assert np.allclose(got16, want16, rtol=1e-5, atol=1e-4)
    if cfg[2] == 1:
        # without a K split every element is one k-ascending f32 sum: identical bits for any tiling
        base = orc.deep_tile_matmul(A16, B16, BF16, BF16, CONFIGS[0])
        assert got16.tobytes() == base.tobytes()


def test_ragged_shapes_use_whole_dim_blocks(orc):
    rng = np.random.default_rng(13)
    M, N, K = 37, 50, 29  # nothing divides 32; K odd (VNNI pad row reads as zero)
    A = rng.integers(-128, 128, (M, K)).astype(np.int8)
    W = rng.integers(-128, 128, (K, N)).astype(np.int8)
    got = orc.deep_tile_matmul(A, W, S8, S8)
    assert (got == A.astype(np.int64) @ W.astype(np.int64)).all()


def test_invalid_config_is_rejected(orc):
    A = np.zeros((64, 64), np.float32)
    with pytest.raises(ValueError):
        orc.deep_tile_matmul(A, A, F32, F32, [1, 1, 1, 48, 32, 32, 32, 32, 32])


def test_vnni_pack_formula_and_lit_shapes(orc):
    """B5[no,ko,ki,ni,vi] = W[ko*kb+ki*v+vi, no*nb+ni] (lib/gc/Dialect/Linalgx/
    Utils.cpp:344-350); shapes of test/mlir/unittests/Linalgx/TestUtils.cpp:
    157-172 (int8 [16,2,8,32,4] for K=64,N=512) and :206-219 (bf16 [..,16,32,2])."""
    rng = np.random.default_rng(5)
    W = rng.integers(-128, 128, (64, 512)).astype(np.int8)
    P = orc.vnni_pack(W, 32, 32).reshape(16, 2, 8, 32, 4)
    for (no, ko, ki, ni, vi) in [(0, 0, 0, 0, 0), (15, 1, 7, 31, 3), (3, 1, 2, 5, 1), (9, 0, 6, 17, 2)]:
        assert P[no, ko, ki, ni, vi] == W[ko * 32 + ki * 4 + vi, no * 32 + ni]
    W16 = rng.integers(0, 65536, (128, 96)).astype(np.uint16)
    P16 = orc.vnni_pack(W16, 32, 32).reshape(3, 4, 16, 32, 2)
    for (no, ko, ki, ni, vi) in [(0, 0, 0, 0, 0), (2, 3, 15, 31, 1), (1, 2, 7, 9, 0)]:
        assert P16[no, ko, ki, ni, vi] == W16[ko * 32 + ki * 2 + vi, no * 32 + ni]
    # the 4096x4096 bf16 weight of deepTileContractionNamedOp.mlir:100 packs to 128x128x16x32x2
    assert 128 * 128 * 16 * 32 * 2 == 4096 * 4096
    # ragged: zero padded
    Wr = rng.integers(1, 100, (5, 3)).astype(np.int8)
    Pr = orc.vnni_pack(Wr, 8, 4).reshape(1, 1, 2, 4, 4)
    assert Pr[0, 0, 1, 2, 0] == Wr[4, 2] and Pr[0, 0, 1, 2, 1] == 0 and Pr[0, 0, 0, 3, 0] == 0
