"""GPU: modules in MLIR's textual form through dnnl_graph_compiler_compile_mlir / execute, checked
against torch evaluating the same ops with the same rounding points (bf16 results round at every op
whose result type is bf16; the norms work in f32).  Shapes follow the reference's benchgc: the MLP
pattern (test/benchgc/src/benchgc/pattern/mlp.py, tolerance 1e-5 f32 / 5e-2 bf16 there),
test/benchgc/cases/llama2.mlir and test/benchgc/cases/generic.mlir."""
import importlib

import numpy as np
import pytest
import torch

from conftest import assert_close

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ga(gc, dev):
    return importlib.import_module("graph_compiler_amd.graph_api")


@pytest.fixture(scope="module")
def mm(gc):
    return importlib.import_module("graph_compiler_amd.mlir_modules")


def _run(ga, text, ins, outs):
    comp = ga.Compiler()
    try:
        st, exe = comp.compile_mlir(text)
        assert st == 0, "compile_mlir -> %d: %s" % (st, ga.api().dnnl_graph_compiler_last_error().decode())
        try:
            st = exe.execute(ins, outs)
            assert st == 0, "execute -> %d: %s" % (st, ga.api().dnnl_graph_compiler_last_error().decode())
            torch.cuda.synchronize()
        finally:
            exe.close()
    finally:
        comp.close()


@pytest.mark.parametrize("dtype,act,bias,hidden", [
    ("f32", "relu", [True, True], [512, 256, 64]), ("f32", "sigmoid", [True, False], [512, 256, 64]),
    ("bf16", "relu", [True], [512, 256]), ("bf16", "sigmoid", [False], [512, 256]),
    ("bf16", "relu", [True, False], [512, 256, 64]), ("bf16", "noop", [False, False], [512, 256, 64])])
def test_mlp_pattern(ga, mm, dev, dtype, act, bias, hidden):
    torch.manual_seed(5)
    td = torch.float32 if dtype == "f32" else torch.bfloat16
    batch, layers = 128, len(hidden) - 1
    x = torch.rand(batch, hidden[0], device=dev).to(td)  # benchgc fills this pattern with U(0, 1)
    ws = [(torch.rand(hidden[i], hidden[i + 1], device=dev) - 0.5).to(td) for i in range(layers)]
    bs = [torch.rand(hidden[i + 1], device=dev).to(td) for i in range(layers) if bias[i]]
    out = torch.zeros(batch, hidden[-1], device=dev, dtype=td)
    args = [x] + ws + bs
    _run(ga, mm.mlp(batch, hidden, bias, act, dtype), list(enumerate(args)), [(len(args), out)])
    ref, bi = x.double(), 0
    for i in range(layers):
        ref = ref @ ws[i].double()
        if bias[i]:
            ref = ref + bs[bi].double()
            bi += 1
        ref = torch.relu(ref) if act == "relu" else torch.sigmoid(ref) if act == "sigmoid" else ref
        ref = ref.to(td).double()  # the layer's result type
    # one bf16 layer: 1e-2.  Two: a hidden value that rounds the other way (2^-8 of it) shifts a whole output row by
    # about that much of a typical term, which is more than 1e-2 of the small outputs: 2e-2 (benchgc itself takes 5e-2)
    rtol = 1e-4 if dtype == "f32" else 1e-2 if layers == 1 else 2e-2
    assert_close(ref.cpu().numpy(), out.double().cpu().numpy(), rtol, "mlp %s %s" % (dtype, act))


@pytest.mark.parametrize("tb", [False, True])
def test_generic_matmul(ga, mm, dev, tb):
    rng = np.random.default_rng(3)
    A = rng.integers(-4, 5, (48, 40)).astype(np.float32)
    B = rng.integers(-4, 5, (24, 40) if tb else (40, 24)).astype(np.float32)
    out = np.zeros((48, 24), np.float32)
    _run(ga, mm.generic_matmul(48, 40, 24, "f32", transpose_b=tb), [(0, A), (1, B)], [(2, out)])
    assert (out == A @ (B.T if tb else B)).all()  # small integers: exact in f32


def _rmsnorm(x, eps, gamma):
    xf = x.float()
    ms = (xf * xf).sum(-1, keepdim=True) / x.shape[-1]
    return gamma * (xf * (ms + eps) ** -0.5).bfloat16()


def _block_ref(a, Wo, res, eps1, g1, Wg, Wu, Wd, eps2, g2):
    bf = torch.bfloat16
    mmf = lambda x, w: (x.float() @ w.float().t()).to(bf)  # noqa: E731  bf16 operands, f32 accumulation, bf16 result
    h = res + mmf(a, Wo)
    n1 = _rmsnorm(h, eps1, g1)
    gate = mmf(n1, Wg)
    silu = torch.sigmoid(gate.float()).to(bf) * gate
    out = h + mmf(silu * mmf(n1, Wu), Wd)
    return out, _rmsnorm(out, eps2, g2)


@pytest.mark.parametrize("T,H,F", [(32, 256, 512), (32, 4096, 11008)])
def test_decoder_mlp_block(ga, mm, dev, T, H, F):
    """The llama-2 block of the reference's benchgc case, at a small size and at the case's own."""
    torch.manual_seed(11)
    bf = torch.bfloat16
    r = lambda *s: torch.randn(*s, device=dev)  # noqa: E731
    a, res = r(1, T, H).to(bf), r(1, T, H).to(bf)
    Wo, Wg, Wu, Wd = (r(H, H) / H ** 0.5).to(bf), (r(F, H) / H ** 0.5).to(bf), (r(F, H) / H ** 0.5).to(bf), (r(H, F) / F ** 0.5).to(bf)
    g1, g2 = (1 + 0.1 * r(H)).to(bf), (1 + 0.1 * r(H)).to(bf)
    eps1 = torch.full((1,), 1e-5, device=dev)
    eps2 = torch.full((1,), 1e-6, device=dev)
    out, n2 = torch.zeros(1, T, H, device=dev, dtype=bf), torch.zeros(1, T, H, device=dev, dtype=bf)
    args = [a, Wo, res, eps1, g1, Wg, Wu, Wd, eps2, g2]
    _run(ga, mm.decoder_mlp_block(T, H, F), list(enumerate(args)), [(10, out), (11, n2)])
    ref_out, ref_n2 = _block_ref(a.view(T, H), Wo, res.view(T, H), eps1, g1, Wg, Wu, Wd, eps2, g2)
    # bf16 intermediates: one rounding step of an intermediate (2^-8) moves the result by about that much
    assert_close(ref_out.float().cpu().numpy(), out.view(T, H).float().cpu().numpy(), 2e-2, "block out")
    assert_close(ref_n2.float().cpu().numpy(), n2.view(T, H).float().cpu().numpy(), 2e-2, "block norm")


def test_attention_from_named_batch_ops(ga, mm, dev):
    """batch_matmul_transpose_b -> mul by a splat -> softmax -> batch_matmul lands on the fused attention kernel."""
    B, S, D = 8, 256, 128
    st, plan = ga.explain_mlir(mm.attention(B, S, D, 0.0884))
    assert st == 0 and plan.startswith("attention:"), plan
    torch.manual_seed(2)
    q, k, v = (torch.randn(B, S, D, device=dev).bfloat16() for _ in range(3))
    out = torch.zeros(B, S, D, device=dev, dtype=torch.bfloat16)
    _run(ga, mm.attention(B, S, D, 0.0884), [(0, q), (1, k), (2, v)], [(3, out)])
    p = torch.softmax(q.float() @ k.float().transpose(1, 2) * 0.0884, -1)
    ref = p @ v.float()
    # the probabilities are rounded to bf16 before P V: the error unit of an element is an ulp of sum_j p_ij |v_jd|
    assert_close(ref.cpu().numpy(), out.float().cpu().numpy(), 1e-2, "attention", mag=(p @ v.float().abs()).cpu().numpy())
    # head_dim 64 has no fused kernel: per-op kernels (batched GEMMs, softmax), f32
    B, S, D = 4, 64, 64
    q, k, v = (torch.randn(B, S, D, device=dev) for _ in range(3))
    out = torch.zeros(B, S, D, device=dev)
    _run(ga, mm.attention(B, S, D, 0.125, "f32"), [(0, q), (1, k), (2, v)], [(3, out)])
    ref = torch.softmax(q @ k.transpose(1, 2) * 0.125, -1) @ v
    assert_close(ref.cpu().numpy(), out.cpu().numpy(), 1e-4, "attention f32 unfused")


def test_results_that_are_arguments_or_constants(ga, dev):
    text = """func.func @f(%a: tensor<8x8xf32>) -> (tensor<8x8xf32>, tensor<8x8xf32>, tensor<8x8xf32>, tensor<8x8xf32>) {
      %e = tensor.empty() : tensor<8x8xf32>
      %c = arith.constant dense<2.500000e+00> : tensor<8x8xf32>
      %r = linalg.mul ins(%a, %c : tensor<8x8xf32>, tensor<8x8xf32>) outs(%e : tensor<8x8xf32>) -> tensor<8x8xf32>
      return %r, %r, %a, %c : tensor<8x8xf32>, tensor<8x8xf32>, tensor<8x8xf32>, tensor<8x8xf32>
    }"""
    a = np.arange(64, dtype=np.float32).reshape(8, 8)
    outs = [np.zeros((8, 8), np.float32) for _ in range(4)]
    _run(ga, text, [(0, a)], [(1 + j, o) for j, o in enumerate(outs)])
    assert (outs[0] == a * 2.5).all() and (outs[1] == a * 2.5).all() and (outs[2] == a).all() and (outs[3] == 2.5).all()
