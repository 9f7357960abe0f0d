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


@pytest.fixture(autouse=True, params=["generated", "library"])
def fused_kernels(request, monkeypatch):
    """Every test of this file runs twice: with the kernels that are generated for the fused groups when a module is
    compiled (a failure to generate or compile them is an error here, not a quiet return to the library's kernels),
    and with the library's generic kernels for such groups."""
    if request.param == "library":
        monkeypatch.setenv("GCMI_NO_GENERATED_KERNELS", "1")
    else:
        monkeypatch.setenv("GCMI_GENERATED_KERNELS_REQUIRED", "1")
    return request.param


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


def _block_outputs(ga, mm, dev, T, H, F, seed):
    torch.manual_seed(seed)
    bf = torch.bfloat16
    r = lambda *s: torch.randn(*s, device=dev)  # noqa: E731
    args = [r(1, T, H).to(bf), (r(H, H) / H ** 0.5).to(bf), r(1, T, H).to(bf), torch.full((1,), 1e-5, device=dev),
            (1 + 0.1 * r(H)).to(bf), (r(F, H) / H ** 0.5).to(bf), (r(F, H) / H ** 0.5).to(bf), (r(H, F) / F ** 0.5).to(bf),
            torch.full((1,), 1e-6, device=dev), (1 + 0.1 * r(H)).to(bf)]
    out, n2 = torch.zeros(1, T, H, device=dev, dtype=bf), torch.zeros(1, T, H, device=dev, dtype=bf)
    _run(ga, mm.decoder_mlp_block(T, H, F), list(enumerate(args)), [(10, out), (11, n2)])
    return out, n2


def test_fused_groups_compute_what_the_single_ops_compute(ga, mm, dev, monkeypatch):
    """Every instruction of a fused group rounds to its op's storage type, so fusing changes no bit: the decoder
    block with the fusion pass on (7 launches) and off (one launch per op)."""
    fused = _block_outputs(ga, mm, dev, 32, 512, 768, seed=3)
    fused_rows = _block_outputs(ga, mm, dev, 640, 256, 512, seed=4)  # rows enough for the one-launch normalisation
    monkeypatch.setenv("GCMI_NO_POINTWISE_FUSION", "1")
    single = _block_outputs(ga, mm, dev, 32, 512, 768, seed=3)
    single_rows = _block_outputs(ga, mm, dev, 640, 256, 512, seed=4)
    assert torch.equal(fused[0], single[0]) and torch.equal(fused[1], single[1])
    assert torch.equal(fused_rows[0], single_rows[0]) and torch.equal(fused_rows[1], single_rows[1])


def test_fused_broadcasts_views_and_reductions(ga, dev):
    """Row and column broadcasts, a middle-axis sum with a point-wise producer and consumer, a mean over two axes,
    and views between the ops, against numpy in f32."""
    text = """func.func @f(%x: tensor<6x40x24xf32>, %row: tensor<24xf32>, %col: tensor<6x40xf32>)
        -> (tensor<6x24xf32>, tensor<6x40x24xf32>, tensor<40xf32>) {
      %e3 = tensor.empty() : tensor<6x40x24xf32>
      %e2 = tensor.empty() : tensor<6x24xf32>
      %rb = linalg.broadcast ins(%row : tensor<24xf32>) outs(%e3 : tensor<6x40x24xf32>) dimensions = [0, 1]
      %cb = linalg.broadcast ins(%col : tensor<6x40xf32>) outs(%e3 : tensor<6x40x24xf32>) dimensions = [2]
      %0 = linalg.mul ins(%x, %rb : tensor<6x40x24xf32>, tensor<6x40x24xf32>) outs(%e3 : tensor<6x40x24xf32>) -> tensor<6x40x24xf32>
      %1 = linalg.add ins(%0, %cb : tensor<6x40x24xf32>, tensor<6x40x24xf32>) outs(%e3 : tensor<6x40x24xf32>) -> tensor<6x40x24xf32>
      %c0 = arith.constant 0.0 : f32
      %z = linalg.fill ins(%c0 : f32) outs(%e2 : tensor<6x24xf32>) -> tensor<6x24xf32>
      %s = linalg.reduce { arith.addf } ins(%1 : tensor<6x40x24xf32>) outs(%z : tensor<6x24xf32>) dimensions = [1]
      %half = arith.constant dense<5.000000e-01> : tensor<6x24xf32>
      %s2 = linalg.mul ins(%s, %half : tensor<6x24xf32>, tensor<6x24xf32>) outs(%e2 : tensor<6x24xf32>) -> tensor<6x24xf32>
      %v = tensor.expand_shape %s2 [[0], [1, 2]] output_shape [6, 1, 24] : tensor<6x24xf32> into tensor<6x1x24xf32>
      %vc = tensor.collapse_shape %v [[0], [1, 2]] : tensor<6x1x24xf32> into tensor<6x24xf32>
      %sb = linalg.broadcast ins(%vc : tensor<6x24xf32>) outs(%e3 : tensor<6x40x24xf32>) dimensions = [1]
      %2 = linalg.sub ins(%1, %sb : tensor<6x40x24xf32>, tensor<6x40x24xf32>) outs(%e3 : tensor<6x40x24xf32>) -> tensor<6x40x24xf32>
      %3 = linalg.exp ins(%2 : tensor<6x40x24xf32>) outs(%e3 : tensor<6x40x24xf32>) -> tensor<6x40x24xf32>
      %e1 = tensor.empty() : tensor<40xf32>
      %z1 = linalg.fill ins(%c0 : f32) outs(%e1 : tensor<40xf32>) -> tensor<40xf32>
      %m = linalg.reduce { arith.addf } ins(%0 : tensor<6x40x24xf32>) outs(%z1 : tensor<40xf32>) dimensions = [0, 2]
      return %s2, %3, %m : tensor<6x24xf32>, tensor<6x40x24xf32>, tensor<40xf32>
    }"""
    st, plan = ga.explain_mlir(text)
    assert st == 0, plan
    rng = np.random.default_rng(9)
    x = rng.standard_normal((6, 40, 24)).astype(np.float32) * 0.2
    row = rng.standard_normal(24).astype(np.float32)
    col = rng.standard_normal((6, 40)).astype(np.float32) * 0.1
    o1, o2, o3 = np.zeros((6, 24), np.float32), np.zeros((6, 40, 24), np.float32), np.zeros(40, np.float32)
    _run(ga, text, [(0, x), (1, row), (2, col)], [(3, o1), (4, o2), (5, o3)])
    t0 = x * row
    t1 = t0 + col[:, :, None]
    s2 = t1.sum(1, dtype=np.float64) * 0.5
    assert_close(s2, o1, 1e-5, "sum over the middle axis")
    assert_close(np.exp(t1 - s2[:, None, :]), o2, 1e-4, "exp(x - row statistic)")
    assert_close(t0.sum((0, 2), dtype=np.float64), o3, 1e-5, "sum over two axes")


def test_reduce_json_fixtures_use_the_row_kernel(ga, dev):
    """reduce_sum.json / reduce_mean.json style graphs at a size where one thread per output would crawl."""
    x = torch.randn(48, 8192, device=dev)
    for kind, ref in (("ReduceSum", x.double().sum(1)), ("ReduceMean", x.double().mean(1))):
        g = ga._graph([{"kind": kind, "attrs": {"axes": {"type": "s64[]", "value": [1]},
                                                 "keep_dims": {"type": "bool", "value": 0}},
                        "inputs": [ga._t(0, "f32", [48, 8192])], "outputs": [ga._t(1, "f32", [48])]}], [0], [1])
        out = torch.zeros(48, device=dev)
        comp = ga.Compiler()
        st, exe = comp.compile(g)
        assert st == 0, ga.api().dnnl_graph_compiler_last_error().decode()
        assert exe.execute([(0, x)], [(1, out)]) == 0
        torch.cuda.synchronize()
        exe.close()
        comp.close()
        assert_close(ref.cpu().numpy(), out.double().cpu().numpy(), 1e-5, kind)


UNARY = {"abs": torch.abs, "ceil": torch.ceil, "floor": torch.floor, "erf": torch.erf, "log": torch.log,
         "negf": torch.neg, "exp": torch.exp, "rsqrt": torch.rsqrt, "sqrt": torch.sqrt, "square": torch.square,
         "tanh": torch.tanh, "reciprocal": torch.reciprocal,
         "round": lambda x: torch.sign(x) * torch.floor(torch.abs(x) + 0.5)}  # math.round: halves away from zero
BINARY = {"add": torch.add, "sub": torch.sub, "mul": torch.mul, "div": torch.div, "max": torch.maximum,
          "min": torch.minimum}


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_linalg_driver_elementwise_ops(ga, mm, dev, dtype):
    """Every named unary and binary op of benchgc's linalg driver (test/benchgc/src/benchgc/linalg/{eltwise,binary}.py
    hold the torch references used here), f32 to 1e-4 (libm-grade device functions) and bf16 to one rounding."""
    td = torch.float32 if dtype == "f32" else torch.bfloat16
    torch.manual_seed(12)
    shape = [3, 50, 40]
    pos = (torch.rand(shape, device=dev) * 4 + 0.25).to(td)            # log, sqrt, rsqrt, reciprocal
    any_ = ((torch.rand(shape, device=dev) - 0.5) * 6.3).to(td)
    any_[0, 0, :6] = torch.tensor([0.5, -0.5, 1.5, -1.5, 2.5, -2.5]).to(td)  # ties of round
    other = ((torch.rand(shape, device=dev) - 0.5) * 4 + 0.01).to(td)
    for op, fn in UNARY.items():
        x = pos if op in ("log", "sqrt", "rsqrt", "reciprocal") else any_
        out = torch.zeros(shape, device=dev, dtype=td)
        _run(ga, mm.linalg_op(op, [shape], shape, dtype), [(0, x)], [(1, out)])
        ref = fn(x.double()).to(td)
        assert_close(ref.double().cpu().numpy(), out.double().cpu().numpy(), 1e-4 if dtype == "f32" else 1e-2, op)
    for op, fn in BINARY.items():
        out = torch.zeros(shape, device=dev, dtype=td)
        _run(ga, mm.linalg_op(op, [shape, shape], shape, dtype), [(0, any_), (1, other)], [(2, out)])
        ref = fn(any_.double(), other.double()).to(td)
        assert_close(ref.double().cpu().numpy(), out.double().cpu().numpy(), 1e-6 if dtype == "f32" else 1e-2, op)


def test_linalg_driver_contractions(ga, mm, dev):
    """matmul.py of the same driver: every 2-D, batched and vector form, on small integers (exact in f32)."""
    rng = np.random.default_rng(4)
    r = lambda *s: rng.integers(-3, 4, s).astype(np.float32)  # noqa: E731
    B, M, K, N = 3, 24, 40, 16
    cases = [("matmul", [r(M, K), r(K, N)], lambda a, b: a @ b),
             ("matmul_transpose_a", [r(K, M), r(K, N)], lambda a, b: a.T @ b),
             ("matmul_transpose_b", [r(M, K), r(N, K)], lambda a, b: a @ b.T),
             ("batch_matmul", [r(B, M, K), r(B, K, N)], lambda a, b: a @ b),
             ("batch_matmul_transpose_a", [r(B, K, M), r(B, K, N)], lambda a, b: a.transpose(0, 2, 1) @ b),
             ("batch_matmul_transpose_b", [r(B, M, K), r(B, N, K)], lambda a, b: a @ b.transpose(0, 2, 1)),
             ("matvec", [r(M, K), r(K)], lambda a, b: a @ b), ("vecmat", [r(K), r(K, N)], lambda a, b: a @ b),
             ("dot", [r(K), r(K)], lambda a, b: np.array(a @ b, np.float32)),
             ("batch_matvec", [r(B, M, K), r(B, K)], lambda a, b: np.einsum("bmk,bk->bm", a, b)),
             ("batch_vecmat", [r(B, K), r(B, K, N)], lambda a, b: np.einsum("bk,bkn->bn", a, b)),
             ("batch_reduce_matmul", [r(B, M, K), r(B, K, N)], lambda a, b: np.einsum("bmk,bkn->mn", a, b))]
    for op, ins, fn in cases:
        ref = fn(*ins)
        out = np.full(ref.shape, -7.0, np.float32)
        _run(ga, mm.linalg_op(op, [list(a.shape) for a in ins], list(ref.shape)), list(enumerate(ins)), [(2, out)])
        assert (out == ref).all(), op


def test_row_statistic_and_scaling_in_one_launch(ga, dev):
    """y = x / sum over the MIDDLE axis of x^2 (a normalisation whose rows are strided in memory): the statistic and
    the scaling are one kernel, the second pass writes through the output's own strides."""
    text = """func.func @f(%x: tensor<36x40x24xf32>, %g: tensor<24xf32>) -> tensor<36x40x24xf32> {
      %e3 = tensor.empty() : tensor<36x40x24xf32>
      %e2 = tensor.empty() : tensor<36x24xf32>
      %c0 = arith.constant 0.0 : f32
      %z = linalg.fill ins(%c0 : f32) outs(%e2 : tensor<36x24xf32>) -> tensor<36x24xf32>
      %sq = linalg.square ins(%x : tensor<36x40x24xf32>) outs(%e3 : tensor<36x40x24xf32>) -> tensor<36x40x24xf32>
      %s = linalg.reduce { arith.addf } ins(%sq : tensor<36x40x24xf32>) outs(%z : tensor<36x24xf32>) dimensions = [1]
      %rs = linalg.rsqrt ins(%s : tensor<36x24xf32>) outs(%e2 : tensor<36x24xf32>) -> tensor<36x24xf32>
      %sb = linalg.broadcast ins(%rs : tensor<36x24xf32>) outs(%e3 : tensor<36x40x24xf32>) dimensions = [1]
      %gb = linalg.broadcast ins(%g : tensor<24xf32>) outs(%e3 : tensor<36x40x24xf32>) dimensions = [0, 1]
      %n = linalg.mul ins(%x, %sb : tensor<36x40x24xf32>, tensor<36x40x24xf32>) outs(%e3 : tensor<36x40x24xf32>) -> tensor<36x40x24xf32>
      %y = linalg.mul ins(%n, %gb : tensor<36x40x24xf32>, tensor<36x40x24xf32>) outs(%e3 : tensor<36x40x24xf32>) -> tensor<36x40x24xf32>
      return %y : tensor<36x40x24xf32>
    }"""
    st, plan = ga.explain_mlir(text)
    assert st == 0 and plan.startswith("reduce: Multiply+Multiply after Rsqrt of ReduceSum of Square\narena"), plan
    rng = np.random.default_rng(10)
    x = rng.standard_normal((36, 40, 24)).astype(np.float32)
    g = rng.standard_normal(24).astype(np.float32)
    out = np.zeros((36, 40, 24), np.float32)
    _run(ga, text, [(0, x), (1, g)], [(2, out)])
    ref = x / np.sqrt((x.astype(np.float64) ** 2).sum(1, keepdims=True)) * g
    assert_close(ref, out, 1e-5, "normalisation over the middle axis")


def test_transpose_and_unfolded_broadcast(ga, dev):
    """linalg.transpose is a strided copy; a linalg.broadcast whose result is returned (nothing to fold it into) is a
    stride-0 copy."""
    text = """func.func @f(%x: tensor<8x16x4xf32>, %v: tensor<16xf32>) -> (tensor<4x8x16xf32>, tensor<8x16xf32>) {
      %e = tensor.empty() : tensor<4x8x16xf32>
      %t = linalg.transpose ins(%x : tensor<8x16x4xf32>) outs(%e : tensor<4x8x16xf32>) permutation = [2, 0, 1]
      %c = arith.constant dense<1.500000e+00> : tensor<4x8x16xf32>
      %y = linalg.mul ins(%t, %c : tensor<4x8x16xf32>, tensor<4x8x16xf32>) outs(%e : tensor<4x8x16xf32>) -> tensor<4x8x16xf32>
      %e2 = tensor.empty() : tensor<8x16xf32>
      %b = linalg.broadcast ins(%v : tensor<16xf32>) outs(%e2 : tensor<8x16xf32>) dimensions = [0]
      return %y, %b : tensor<4x8x16xf32>, tensor<8x16xf32>
    }"""
    rng = np.random.default_rng(14)
    x = rng.standard_normal((8, 16, 4)).astype(np.float32)
    v = rng.standard_normal(16).astype(np.float32)
    y, b = np.zeros((4, 8, 16), np.float32), np.zeros((8, 16), np.float32)
    _run(ga, text, [(0, x), (1, v)], [(2, y), (3, b)])
    assert (y == x.transpose(2, 0, 1) * np.float32(1.5)).all()
    assert (b == np.broadcast_to(v, (8, 16))).all()


def test_linear_layer_spelled_with_a_transpose(ga, dev):
    text = """func.func @f(%x: tensor<64x256xbf16>, %w: tensor<512x256xbf16>) -> tensor<64x512xbf16> {
      %et = tensor.empty() : tensor<256x512xbf16>
      %wt = linalg.transpose ins(%w : tensor<512x256xbf16>) outs(%et : tensor<256x512xbf16>) permutation = [1, 0]
      %c0 = arith.constant 0.0 : bf16
      %e = tensor.empty() : tensor<64x512xbf16>
      %z = linalg.fill ins(%c0 : bf16) outs(%e : tensor<64x512xbf16>) -> tensor<64x512xbf16>
      %y = linalg.matmul ins(%x, %wt : tensor<64x256xbf16>, tensor<256x512xbf16>) outs(%z : tensor<64x512xbf16>) -> tensor<64x512xbf16>
      return %y : tensor<64x512xbf16>
    }"""
    torch.manual_seed(17)
    x = torch.randn(64, 256, device=dev).bfloat16()
    w = (torch.randn(512, 256, device=dev) * 0.1).bfloat16()
    y = torch.zeros(64, 512, device=dev, dtype=torch.bfloat16)
    _run(ga, text, [(0, x), (1, w)], [(2, y)])
    assert_close((x.double() @ w.double().t()).cpu().numpy(), y.double().cpu().numpy(), 1e-2, "linear with transpose")


def test_onednn_graph_dialect_module(ga, dev):
    """The reference's front-end dialect: matmul (+bias, transposed weight) -> sigmoid -> f32 -> square -> row mean."""
    text = """func.func @f(%x: tensor<64x128xbf16>, %w: tensor<256x128xbf16>, %b: tensor<256xbf16>) -> tensor<64x1xf32> {
      %0 = onednn_graph.matmul %x, %w, %b {transpose_b = true}
           : (tensor<64x128xbf16>, tensor<256x128xbf16>, tensor<256xbf16>) -> tensor<64x256xbf16>
      %1 = onednn_graph.sigmoid %0 : (tensor<64x256xbf16>) -> tensor<64x256xbf16>
      %2 = onednn_graph.type_cast %1 : (tensor<64x256xbf16>) -> tensor<64x256xf32>
      %3 = onednn_graph.pow %2 {beta = 2.0 : f32} : (tensor<64x256xf32>) -> tensor<64x256xf32>
      %4 = onednn_graph.reduce_mean %3 {axes = array<i64: -1>, keep_dims = true} : (tensor<64x256xf32>) -> tensor<64x1xf32>
      return %4 : tensor<64x1xf32>
    }"""
    torch.manual_seed(23)
    x = torch.randn(64, 128, device=dev).bfloat16()
    w = (torch.randn(256, 128, device=dev) * 0.1).bfloat16()
    b = torch.randn(256, device=dev).bfloat16()
    out = torch.zeros(64, 1, device=dev)
    _run(ga, text, [(0, x), (1, w), (2, b)], [(3, out)])
    h = torch.sigmoid(((x.float() @ w.float().t()).bfloat16() + b).float()).bfloat16().float()
    assert_close((h * h).mean(1, keepdim=True).cpu().numpy(), out.cpu().numpy(), 1e-2, "dialect module")


@pytest.mark.parametrize("shape,axis", [((5, 7, 3), 2), ((5, 7, 3), 0), ((9, 130), 1), ((3, 1030), 1), ((257, 6), 1),
                                        ((2, 3, 5, 7), 1)])
def test_fused_kernels_on_odd_shapes_f16(ga, dev, shape, axis):
    """Shapes whose innermost dim is not a multiple of four (one element at a time instead of quads), row counts that
    leave part of the last workgroup idle, one to many elements per thread, f16 storage: a point-wise chain, a sum
    over `axis` with a producer and an op on the row result, and the normalisation that uses it."""
    def t(s, dt="f16"):
        return "tensor<%s%s>" % ("".join("%dx" % d for d in s), dt)
    kept = [d for i, d in enumerate(shape) if i != axis]
    full, row = t(shape), t(kept)
    rowdims = ", ".join(str(i) for i in range(len(shape)) if i == axis)
    text = f"""func.func @f(%x: {full}, %y: {full}) -> ({full}, {row}, {full}) {{
      %e = tensor.empty() : {full}
      %er = tensor.empty() : {row}
      %two = arith.constant dense<2.000000e+00> : {full}
      %a = linalg.mul ins(%x, %two : {full}, {full}) outs(%e : {full}) -> {full}
      %b = linalg.add ins(%a, %y : {full}, {full}) outs(%e : {full}) -> {full}
      %zero = arith.constant dense<0.000000e+00> : {full}
      %c = linalg.max ins(%b, %zero : {full}, {full}) outs(%e : {full}) -> {full}
      %c0 = arith.constant 0.0 : f16
      %z = linalg.fill ins(%c0 : f16) outs(%er : {row}) -> {row}
      %s = linalg.reduce {{ arith.addf }} ins(%c : {full}) outs(%z : {row}) dimensions = [{rowdims}]
      %one = arith.constant dense<1.000000e+00> : {row}
      %s1 = linalg.add ins(%s, %one : {row}, {row}) outs(%er : {row}) -> {row}
      %sb = linalg.broadcast ins(%s1 : {row}) outs(%e : {full}) dimensions = [{rowdims}]
      %n = linalg.div ins(%c, %sb : {full}, {full}) outs(%e : {full}) -> {full}
      return %c, %s1, %n : {full}, {row}, {full}
    }}"""
    torch.manual_seed(3)
    x = (torch.rand(shape, device=dev) - 0.3).half()
    y = (torch.rand(shape, device=dev) - 0.5).half()
    c, s1, nrm = torch.zeros(shape, device=dev).half(), torch.zeros(kept, device=dev).half(), torch.zeros(shape, device=dev).half()
    _run(ga, text, [(0, x), (1, y)], [(2, c), (3, s1), (4, nrm)])
    rc = torch.relu(((x.float() * 2).half().float() + y.float()).half().float()).half()
    assert torch.equal(c, rc)
    rs = (rc.float().sum(axis).half().float() + 1).half()
    assert_close(rs.float().cpu().numpy(), s1.float().cpu().numpy(), 2e-3, "row sums f16")  # f16: 2^-11 per rounding
    rn = (rc.float() / s1.float().unsqueeze(axis)).half()
    assert_close(rn.float().cpu().numpy(), nrm.float().cpu().numpy(), 2e-3, "normalised f16")


@pytest.mark.parametrize("M,K,N,nt", [(32, 4096, 4096, True), (300, 96, 200, False), (512, 256, 768, False)])
def test_residual_connection_runs_in_the_matmul(ga, gc, dev, M, K, N, nt):
    """x + relu(a.W + b), the result viewed as [1,M,N] in between: one launch, and bit for bit what the matmul with
    bias and ReLU followed by a separate bf16 add gives."""
    mt, at_ = "tensor<%dx%dxbf16>" % (M, N), "tensor<%dx%dxbf16>" % (M, K)
    wt, t3, bt = "tensor<%dx%dxbf16>" % ((N, K) if nt else (K, N)), "tensor<1x%dx%dxbf16>" % (M, N), "tensor<%dxbf16>" % N
    text = ("func.func @f(%a: " + at_ + ", %w: " + wt + ", %b: " + bt + ", %x: " + t3 + ") -> " + t3 + " {\n"
            "  %z = arith.constant 0.0 : bf16\n"
            "  %e = tensor.empty() : " + mt + "\n"
            "  %f = linalg.fill ins(%z : bf16) outs(%e : " + mt + ") -> " + mt + "\n"
            "  %m = linalg." + ("matmul_transpose_b" if nt else "matmul") + " ins(%a, %w : " + at_ + ", " + wt + ") outs(%f : " + mt + ") -> " + mt + "\n"
            "  %bb = linalg.broadcast ins(%b : " + bt + ") outs(%e : " + mt + ") dimensions = [0]\n"
            "  %s = linalg.add ins(%m, %bb : " + mt + ", " + mt + ") outs(%e : " + mt + ") -> " + mt + "\n"
            "  %r = linalg.max ins(%s, %f : " + mt + ", " + mt + ") outs(%e : " + mt + ") -> " + mt + "\n"
            "  %v = tensor.expand_shape %r [[0, 1], [2]] output_shape [1, " + str(M) + ", " + str(N) + "] : " + mt + " into " + t3 + "\n"
            "  %e3 = tensor.empty() : " + t3 + "\n"
            "  %o = linalg.add ins(%x, %v : " + t3 + ", " + t3 + ") outs(%e3 : " + t3 + ") -> " + t3 + "\n"
            "  return %o : " + t3 + "\n}")
    st, plan = ga.explain_mlir(text)
    assert st == 0 and [l for l in plan.splitlines() if not l.startswith(("arena", "  tile:"))] == ["gemm_bf16: MatMul+bias+act+residual"], plan
    torch.manual_seed(11)
    a = (torch.randn(M, K) * 0.5).to(torch.bfloat16).to(dev)
    w = (torch.randn((N, K) if nt else (K, N)) * 0.1).to(torch.bfloat16).to(dev)
    b = torch.randn(N).to(torch.bfloat16).to(dev)
    x = torch.randn(1, M, N).to(torch.bfloat16).to(dev)
    o = torch.empty(1, M, N, dtype=torch.bfloat16, device=dev)
    _run(ga, text, [(0, a), (1, w), (2, b), (3, x)], [(4, o)])
    plain = (gc.gemm_bf16_nt if nt else gc.gemm_bf16)(a, w, b, "relu")
    torch.cuda.synchronize()
    assert torch.equal(o[0], (plain.float() + x[0].float()).to(torch.bfloat16))


def test_generated_kernels_give_the_bits_of_the_library_kernels(ga, mm, dev, monkeypatch, fused_kernels):
    """The kernels written out for a module's fused groups evaluate the library kernels' expressions in their order:
    the decoder block (row statistics, scalings, the gate) at three shapes gives the same bits either way, and the
    generated kernels are the ones that ran."""
    if fused_kernels == "library":
        pytest.skip("compares the two modes itself")
    shapes = [(32, 512, 768, 3), (640, 256, 512, 4), (1024, 1024, 256, 5), (7, 36, 40, 6)]
    before = ga.generated_kernel_launches()
    gen = [_block_outputs(ga, mm, dev, T, H, F, seed) for T, H, F, seed in shapes]
    ran = ga.generated_kernel_launches() - before
    assert ran >= 3 * len(shapes), ran
    monkeypatch.setenv("GCMI_NO_GENERATED_KERNELS", "1")
    before = ga.generated_kernel_launches()
    lib = [_block_outputs(ga, mm, dev, T, H, F, seed) for T, H, F, seed in shapes]
    assert ga.generated_kernel_launches() == before
    for (a0, a1), (b0, b1) in zip(gen, lib):
        assert torch.equal(a0, b0) and torch.equal(a1, b1)


def test_execute_async_captured_in_a_hip_graph(ga, mm, dev):
    """The launches of execute_async can be recorded into a HIP graph (no allocation, copy or memset is among them):
    the decoder block -- split-K GEMMs with their workspace, residual epilogues, normalisations, the gate -- replayed
    three times with new inputs, eager executes and synchronisations in between, gives the eager results bit for bit."""
    T, H, F = 32, 512, 1024
    bf = torch.bfloat16
    torch.manual_seed(31)
    r = lambda *s: torch.randn(*s, device=dev)  # noqa: E731
    args = [r(1, T, H).to(bf), (r(H, H) / H ** 0.5).to(bf), r(1, T, H).to(bf), torch.full((1,), 1e-5, device=dev),
            (1 + 0.1 * r(H)).to(bf), (r(F, H) / H ** 0.5).to(bf), (r(F, H) / H ** 0.5).to(bf), (r(H, F) / F ** 0.5).to(bf),
            torch.full((1,), 1e-6, device=dev), (1 + 0.1 * r(H)).to(bf)]
    o1 = torch.zeros(1, T, H, device=dev, dtype=bf)
    o2 = torch.zeros_like(o1)
    comp = ga.Compiler()
    st, exe = comp.compile_mlir(mm.decoder_mlp_block(T, H, F))
    assert st == 0, ga.api().dnnl_graph_compiler_last_error().decode()
    try:
        eager = exe.bind(list(enumerate(args)), [(10, o1), (11, o2)])
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            call = exe.bind(list(enumerate(args)), [(10, o1), (11, o2)], stream=side.cuda_stream)
            assert call() == 0  # once outside the capture: modules and static buffers are resolved
            side.synchronize()
            graph.capture_begin()
            rc = call()
            graph.capture_end()
            assert rc == 0
        side.synchronize()
        for k in range(3):
            args[0].copy_(r(1, T, H).to(bf))
            args[2].copy_(r(1, T, H).to(bf))
            torch.cuda.synchronize()
            assert eager() == 0
            want = (o1.clone(), o2.clone())
            o1.zero_()
            o2.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(o1, want[0]) and torch.equal(o2, want[1]), "replay %d" % k
        del graph
    finally:
        exe.close()
        comp.close()


@pytest.mark.parametrize("rows,hidden,dtype", [(512, 1024, "f32"), (37, 300, "f32"), (2048, 768, "bf16"), (8, 4096, "bf16")])
def test_layer_normalisation(ga, mm, dev, monkeypatch, rows, hidden, dtype):
    """Mean, variance of the centred values, scaling: two launches, against torch and bit for bit against one launch
    per op."""
    td = torch.float32 if dtype == "f32" else torch.bfloat16
    torch.manual_seed(rows + hidden)
    x = (torch.randn(rows, hidden, device=dev) * 2 + 0.5).to(td)
    g = (1 + 0.2 * torch.randn(hidden, device=dev)).to(td)
    b = torch.randn(hidden, device=dev).to(td)
    y = torch.zeros(rows, hidden, device=dev, dtype=td)
    _run(ga, mm.layernorm(rows, hidden, dtype), [(0, x), (1, g), (2, b)], [(3, y)])
    ref = torch.nn.functional.layer_norm(x.double(), (hidden,), g.double(), b.double(), 1e-5)
    # bf16: every op of the chain rounds (the centred values, their squares, the statistics)
    assert_close(ref.cpu().numpy(), y.double().cpu().numpy(), 1e-4 if dtype == "f32" else 5e-2, "layer norm " + dtype)
    monkeypatch.setenv("GCMI_NO_POINTWISE_FUSION", "1")
    y1 = torch.zeros_like(y)
    _run(ga, mm.layernorm(rows, hidden, dtype), [(0, x), (1, g), (2, b)], [(3, y1)])
    assert torch.equal(y, y1)


@pytest.mark.parametrize("shape,axis,dtype", [((1024, 4096), 1, "f32"), ((100, 37), 1, "f32"), ((512, 2048), 1, "bf16"),
                                              ((6, 50, 520), 2, "f16"), ((16, 10000), 1, "f32"), ((3, 40000), 1, "f32"),
                                              ((8, 96, 33), 1, "f32"), ((2, 3, 4, 64), 3, "bf16")])
def test_softmax_alone(ga, dev, fused_kernels, shape, axis, dtype):
    """linalg.softmax outside an attention pattern: rows of 33 to 40000 elements, innermost and middle axes, three
    storage types.  Innermost-axis rows of up to 32768 elements get a generated kernel (a row is read once and kept
    in registers); the rest run on the library's kernel."""
    td = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}[dtype]
    t = "tensor<" + "".join("%dx" % d for d in shape) + dtype + ">"
    text = ("func.func @f(%x: " + t + ") -> " + t + " {\n  %e = tensor.empty() : " + t + "\n"
            "  %y = linalg.softmax dimension(" + str(axis) + ") ins(%x : " + t + ") outs(%e : " + t + ") -> " + t + "\n"
            "  return %y : " + t + "\n}")
    torch.manual_seed(len(shape) * 100 + shape[-1])
    x = (torch.randn(shape, device=dev) * 3).to(td)
    x.view(-1)[5] = float("-inf")  # one masked element: weight exactly 0
    y = torch.full(shape, 7.0, device=dev, dtype=td)
    before = ga.generated_kernel_launches()
    _run(ga, text, [(0, x)], [(1, y)])
    generated = ga.generated_kernel_launches() > before
    assert generated == (fused_kernels == "generated" and axis == len(shape) - 1 and shape[axis] <= 32768)
    ref = torch.softmax(x.double(), axis)
    tol = {"f32": 1e-4, "bf16": 1e-2, "f16": 2e-3}[dtype]
    assert_close(ref.cpu().numpy(), y.double().cpu().numpy(), tol, "softmax " + dtype)
    assert y.view(-1)[5].item() == 0.0
    assert_close(np.ones(ref.sum(axis).shape), y.double().sum(axis).cpu().numpy(), 10 * tol, "rows sum to one")
