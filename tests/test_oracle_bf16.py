"""CPU: the oracle's bf16 conversion against the reference bit formula
(include/gc/ExecutionEngine/CPURuntime/Microkernel/BrgemmInterface.h:72-92)
and against torch's round-to-nearest-even cast."""
import numpy as np
import torch


def test_all_bf16_patterns_round_trip(orc):
    h = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    f = orc.bf16_to_f32(h)
    assert (f.view(np.uint32) == (h.astype(np.uint32) << 16)).all()  # widen = <<16
    back = orc.f32_to_bf16(f)
    nan = np.isnan(f)
    assert (back[~nan] == h[~nan]).all()
    assert (back[nan] == 0x7FC0).all()  # every NaN collapses to the canonical quiet NaN


def test_rne_matches_torch_on_random_f32(orc):
    rng = np.random.default_rng(1)
    bits = rng.integers(0, 2 ** 32, 2_000_000, dtype=np.uint64).astype(np.uint32)
    x = bits.view(np.float32)
    x = x[~np.isnan(x)]
    got = orc.f32_to_bf16(x)
    want = torch.from_numpy(x.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert (got == want).all()


def test_ties_go_to_even_and_overflow_to_inf(orc):
    def f(bits):
        return np.array([bits], np.uint32).view(np.float32)

    assert orc.f32_to_bf16(f(0x3F808000))[0] == 0x3F80  # 1 + 2^-8: tie, even stays
    assert orc.f32_to_bf16(f(0x3F818000))[0] == 0x3F82  # tie above an odd mantissa rounds up
    assert orc.f32_to_bf16(f(0x3F808001))[0] == 0x3F81  # just above the tie
    assert orc.f32_to_bf16(f(0x7F7FFFFF))[0] == 0x7F80  # FLT_MAX rounds to +inf
    assert orc.f32_to_bf16(f(0x80000000))[0] == 0x8000  # -0 keeps its sign
    assert orc.f32_to_bf16(f(0xFFC00001))[0] == 0x7FC0  # negative NaN -> 0x7FC0 too
    assert orc.lib().gco_f32_to_bf16(1.0) == 0x3F80
