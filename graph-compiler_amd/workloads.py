"""Seeded synthetic inputs for the five benchmark configurations.

Seeding follows the reference harness: every argument of a case is drawn after
torch.manual_seed(seed + argument_index), in f32 (or int) on the CPU, then cast
to the tensor's dtype (test/benchgc/src/benchgc/arg/__init__.py:94-153,
test/benchgc/src/benchgc/util.py:163-171).
"""
import math

import torch


def _seeded(seed, idx):
    torch.manual_seed(seed + idx)


def f32_matmul_bias_relu(M=128, K=512, N=256, seed=0):
    """C1: A[MxK].B[KxN]+bias[N], U(-1,1), f32."""
    _seeded(seed, 0)
    A = torch.rand(M, K) * 2 - 1
    _seeded(seed, 1)
    B = torch.rand(K, N) * 2 - 1
    _seeded(seed, 2)
    bias = torch.rand(N) * 2 - 1
    return A, B, bias


def bf16_gemm(M=4096, N=4096, K=4096, seed=0):
    """C2: N(0,1)*0.1 rounded to bf16."""
    _seeded(seed, 0)
    A = (torch.randn(M, K) * 0.1).to(torch.bfloat16)
    _seeded(seed, 1)
    B = (torch.randn(K, N) * 0.1).to(torch.bfloat16)
    return A, B


def int8_mlp_layer(M=4096, K=4096, N=11008, seed=0):
    """C3: u8 activations U{0..255} (zero point 128), s8 weights U{-127..127},
    per-channel scales U(0.001,0.01), bias N(0,1) f32."""
    _seeded(seed, 0)
    A = torch.randint(0, 256, (M, K), dtype=torch.int32).to(torch.uint8)
    _seeded(seed, 1)
    W = torch.randint(-127, 128, (K, N), dtype=torch.int32).to(torch.int8)
    _seeded(seed, 2)
    scale = torch.rand(N) * 0.009 + 0.001
    _seeded(seed, 3)
    bias = torch.randn(N)
    return A, W, scale, bias


def bf16_mlp_chain(M=4096, K=4096, H=11008, seed=0):
    """C4: x N(0,1); W1 [K,H], W2 [H,K], bias2 [K] ~ N(0,0.02); all bf16."""
    _seeded(seed, 0)
    x = torch.randn(M, K).to(torch.bfloat16)
    _seeded(seed, 1)
    W1 = (torch.randn(K, H) * 0.02).to(torch.bfloat16)
    _seeded(seed, 2)
    W2 = (torch.randn(H, K) * 0.02).to(torch.bfloat16)
    _seeded(seed, 3)
    b2 = (torch.randn(K) * 0.02).to(torch.bfloat16)
    return x, W1, W2, b2


def benchgc_matmul_fill(name, shape, dtype, dst_dtype, amp):
    """Default fill of the reference harness's matmul driver
    (test/benchgc/src/benchgc/arg/matmul.py:104-148): integer-valued data, dense
    for the source, and for the weight of a density that keeps every sum exactly
    representable in the result type -- the fill under which its strict
    point-to-point compare (thresholds 1e-6 f32 / eps(bf16), :160-173) can be met.
    name "src" | "wei"; amp = the reduction length K (:64-102).  Ranges: src
    [-64,64) f32 / [-4,4) bf16,f16; wei [-128,128) f32 / [-8,8) bf16 / [-2,2) f16;
    seeds 0 (src) and 1 (wei) (:141, util.py:163-171 with the default --seed 0)."""
    rng = [{torch.float32: (-64, 64), torch.bfloat16: (-4, 4), torch.float16: (-4, 4)},
           {torch.float32: (-128, 128), torch.bfloat16: (-8, 8), torch.float16: (-2, 2)}]
    digits = {torch.float32: 24, torch.bfloat16: 8, torch.float16: 11}
    src_min, src_max = rng[0][dtype]
    wei_min, wei_max = rng[1][dtype]
    max_value = max(abs(src_min), abs(src_max)) * max(abs(wei_min), abs(wei_max))
    safe_n_acc = (1 << min(24, digits[dst_dtype])) // max_value
    if name == "src":
        lo, hi = src_min, src_max
        density = 1.0
    elif name == "wei":
        lo, hi = wei_min, wei_max
        density = min(safe_n_acc / int(amp), 1.0)
    else:
        raise ValueError(name)
    torch.manual_seed(0 if name == "src" else 1)
    value = torch.bernoulli(torch.full(tuple(shape), density)) * torch.randint(lo, hi, tuple(shape))
    while value.flatten()[0] <= 0:
        value.flatten()[0] = torch.randint(lo, hi + 1, size=[1])[0].item()
    return value.to(dtype)


def causal_mask(Sq, Sk, value=float("-inf")):
    """Additive mask: 0 on and below the diagonal, `value` above."""
    return torch.triu(torch.full((Sq, Sk), value, dtype=torch.float32), diagonal=1)


def bf16_mha(B=4, H=32, S=2048, D=128, seed=0, mask_value=float("-inf")):
    """C5: Q,K,V N(0,1) bf16 [B,H,S,D], scale 1/sqrt(D), additive causal mask f32 [S,S]."""
    _seeded(seed, 0)
    Q = torch.randn(B, H, S, D).to(torch.bfloat16)
    _seeded(seed, 1)
    K = torch.randn(B, H, S, D).to(torch.bfloat16)
    _seeded(seed, 2)
    V = torch.randn(B, H, S, D).to(torch.bfloat16)
    return Q, K, V, causal_mask(S, S, mask_value), 1.0 / math.sqrt(D)


# ---- bit-pattern helpers between torch.bfloat16 and the oracle's uint16 arrays
def bf16_bits(t):
    import numpy as np
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def bf16_from_bits(a):
    import numpy as np
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(torch.bfloat16)
