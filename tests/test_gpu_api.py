"""GPU: the oneDNN-Graph backend API end to end (create / compile / execute /
destroy) with host buffers, as the reference's own API tests drive it
(test/dnnl/TestApiBasic.cpp:25-58, test/dnnl/TestApiOps.cpp:27-320), plus the
benchmark partitions against the oracle, with host and with device tensors."""
import importlib
import json
import os

import numpy as np
import pytest
import torch

from conftest import ROOT, assert_close

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ga(gc, dev):
    return importlib.import_module("graph_compiler_amd.graph_api")


@pytest.fixture(autouse=True, params=["generated", "library"])
def fused_kernels(request, monkeypatch):
    """Every test of this file runs with the kernels generated for fused point-wise groups at compile time (a failure
    to generate or compile one is an error) and with the library's generic kernels for such groups."""
    if request.param == "library":
        monkeypatch.setenv("GCMI_NO_GENERATED_KERNELS", "1")
    else:
        monkeypatch.setenv("GCMI_GENERATED_KERNELS_REQUIRED", "1")
    return request.param


def _res(name):
    return open(os.path.join(ROOT, "tests", "golden", name)).read()


def _run(ga, js, ins, outs):
    cst, est = ga.run(js, ins, outs)
    assert cst == 0, "compile -> %d: %s" % (cst, ga.api().dnnl_graph_compiler_last_error().decode())
    assert est == 0, "execute -> %d: %s" % (est, ga.api().dnnl_graph_compiler_last_error().decode())


def test_basic_workflow_add(ga):
    """TestApiBasic.basicWorkflow: add.json on 128 floats, 4 threads requested."""
    a = np.arange(128, dtype=np.float32)
    b = np.arange(128, dtype=np.float32) * 2
    out = np.zeros(128, np.float32)
    gcomp = ga.Compiler(4)
    st, exe = gcomp.compile(_res("add.json"))
    assert st == 0
    assert exe.execute([(0, a), (1, b)], [(2, out)]) == 0
    assert (out == a + b).all()
    # tensors may come in any order: they are matched by id
    out[:] = 0
    assert exe.execute([(1, b), (0, a)], [(2, out)]) == 0
    assert (out == a + b).all()
    # an id the graph does not know is a runtime error
    assert exe.execute([(0, a), (7, b)], [(2, out)]) == ga.RUNTIME_ERROR
    exe.close()
    gcomp.close()


def test_ops_div_mul_sub_pow_relu_sigmoid(ga):
    i = np.arange(64 * 32 * 32, dtype=np.float32).reshape(64, 32, 32)
    o = np.zeros_like(i)
    _run(ga, _res("div.json"), [(0, i), (1, i + 1)], [(2, o)])
    assert np.allclose(o, i / (i + 1), rtol=1e-6, atol=0)
    x = np.arange(128, dtype=np.float32)
    o = np.zeros(128, np.float32)
    _run(ga, _res("mul.json"), [(0, x), (1, x)], [(2, o)])
    assert (o == x * x).all()
    _run(ga, _res("sub.json"), [(0, x), (1, x * x)], [(2, o)])
    assert (o == x - x * x).all()
    x64, o64 = np.arange(64, dtype=np.float32), np.zeros(64, np.float32)
    _run(ga, _res("pow.json"), [(0, x64)], [(1, o64)])
    assert (o64 == x64 * x64).all()
    xs = (np.arange(128) - 64).astype(np.float32)
    _run(ga, _res("relu.json"), [(0, xs)], [(1, o)])
    assert (o == np.maximum(xs, 0)).all()
    _run(ga, _res("sigmoid.json"), [(0, xs)], [(1, o)])
    assert np.allclose(o, 1 / (1 + np.exp(-xs)), rtol=2e-6, atol=1e-30)


def test_ops_matmul_transpose_a_bias_closed_form(ga):
    """TestApiOps.matMul: A[i][j]=i+j (128x512, transpose_a), B[i][j]=i-j, bias=j; exact integers."""
    i, j = np.meshgrid(np.arange(128), np.arange(512), indexing="ij")
    A = (i + j).astype(np.float32)
    i, j = np.meshgrid(np.arange(128), np.arange(64), indexing="ij")
    B = (i - j).astype(np.float32)
    bias = np.arange(64, dtype=np.float32)
    out = np.zeros((512, 64), np.float32)
    _run(ga, _res("matmul.json"), [(0, A), (1, B), (2, bias)], [(3, out)])
    want = A.astype(np.int64).T @ B.astype(np.int64) + np.arange(64)
    assert (out.astype(np.int64) == want).all()


def test_ops_reduce_and_typecast(ga):
    x = np.arange(16 * 64 * 32, dtype=np.float32).reshape(16, 64, 32)
    o = np.zeros((16, 1, 32), np.float32)
    _run(ga, _res("reduce_sum.json"), [(0, x)], [(1, o)])
    want = np.zeros((16, 1, 32), np.float32)
    for y in range(64):  # the reference test sums in this order, in f32
        want[:, 0, :] += x[:, y, :]
    assert np.allclose(o, want, rtol=1e-6)
    _run(ga, _res("reduce_mean.json"), [(0, x)], [(1, o)])
    assert np.allclose(o, want / 64, rtol=1e-6)
    # typecast f32 -> f16 must be round-to-nearest-even bit for bit (TestApiOps.typecast)
    v = np.array([(k - 64) / np.exp(-(k - 64)) for k in range(128)], np.float32)
    h = np.zeros(128, np.uint16)
    _run(ga, _res("typecast.json"), [(0, v)], [(1, h)])
    assert (h == v.astype(np.float16).view(np.uint16)).all()


def test_add_relu_strided_input(ga):
    """add_relu.json declares input 1 with explicit strides [1,2,3,4]."""
    g = json.loads(_res("add_relu.json"))
    shape = g["graph"][0]["inputs"][0]["shape"]
    stride = g["graph"][0]["inputs"][1]["stride"]
    span = 1 + sum((d - 1) * s for d, s in zip(shape, stride))
    torch.manual_seed(0)
    a = torch.randn(shape).to(torch.bfloat16)
    braw = torch.randn(span).to(torch.bfloat16)
    b = torch.as_strided(braw, shape, stride)
    out = torch.zeros(shape, dtype=torch.bfloat16)
    _run(ga, _res("add_relu.json"), [(0, a), (1, braw)], [(3, out)])
    assert torch.equal(out, torch.relu(a + b))


def test_reference_mlp_fixture_bf16(ga, orc, wl):
    """mpl.json: MatMul+bias -> ReLU -> MatMul -> Add -> ReLU, all bf16."""
    torch.manual_seed(0)
    x = torch.randn(128, 512).to(torch.bfloat16)
    w1 = (torch.randn(512, 64) * 0.05).to(torch.bfloat16)
    b1 = torch.randn(64).to(torch.bfloat16)
    w2 = (torch.randn(64, 256) * 0.1).to(torch.bfloat16)
    b2 = torch.randn(256).to(torch.bfloat16)
    out = torch.zeros(128, 256, dtype=torch.bfloat16)
    _run(ga, _res("mpl.json"), [(0, x), (1, w1), (2, b1), (5, w2), (7, b2)], [(9, out)])
    h = orc.matmul_bf16(wl.bf16_bits(x), wl.bf16_bits(w1), wl.bf16_bits(b1), "relu")
    y = orc.matmul_bf16(h, wl.bf16_bits(w2), wl.bf16_bits(b2), "relu")
    mm = orc.bf16_to_f32(orc.matmul_bf16(h, wl.bf16_bits(w2)))
    assert_close(orc.bf16_to_f32(y), out.float().numpy(), 2e-2, "mpl.json", mag=mm)


def test_config1_f32_matmul_bias_relu_through_the_api(ga, orc, wl):
    """BASELINE config 1, host buffers in and out (max relative error <= 1e-4)."""
    A, B, bias = wl.f32_matmul_bias_relu()
    out = np.zeros((128, 256), np.float32)
    _run(ga, ga.matmul_bias_relu_json(128, 512, 256), [(0, A.numpy()), (1, B.numpy()), (2, bias.numpy())], [(4, out)])
    ref = orc.matmul_f32(A.numpy(), B.numpy(), bias.numpy(), "relu")
    assert_close(ref, out, 1e-4, "config 1 via API")


def test_int8_partition_through_the_api_with_device_tensors(ga, gc, orc, wl, dev):
    M, K, N = 512, 256, 768
    A, W, scale, bias = wl.int8_mlp_layer(M, K, N)
    sA = 0.02
    js, out_id = ga.int8_mlp_json(M, K, N, sA, 128, scale.tolist())
    out = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    _run(ga, js, [(0, A.to(dev)), (1, W.to(dev)), (2, bias.to(dev))], [(out_id, out)])
    torch.cuda.synchronize()
    eff = (np.float32(sA) * scale.numpy().astype(np.float32)).astype(np.float32)  # data scale x weight scales, in f32
    _, y = orc.int8_layer(A.numpy(), W.numpy(), eff, bias.numpy(), 128, "gelu_erf")
    assert_close(orc.bf16_to_f32(y), out.float().cpu().numpy(), 1e-2, "int8 partition")
    # the same with host buffers and an f32 result, executed twice (constant-weight colsum is cached)
    js2, oid2 = ga.int8_mlp_json(M, K, N, sA, 128, scale.tolist(), out_dtype="f32")
    o2 = np.zeros((M, N), np.float32)
    c = ga.Compiler()
    st, exe = c.compile(js2)
    assert st == 0
    for _ in range(2):
        o2[:] = 0
        assert exe.execute([(0, A.numpy()), (1, W.numpy()), (2, bias.numpy())], [(oid2, o2)]) == 0
        _, yf = orc.int8_layer(A.numpy(), W.numpy(), eff, bias.numpy(), 128, "gelu_erf", out_bf16=False)
        assert_close(yf, o2, 1e-4, "int8 partition f32")
    exe.close()
    c.close()


@pytest.mark.parametrize("constant", [True, False])
def test_int8_partition_with_weights_stored_nk(ga, orc, wl, dev, constant):
    """transpose_b on the quantised MatMul (weights [N,K], per-channel scales along axis 0): the fused 8-bit GEMM
    runs on a transposed copy that is made once when the weights are a constant; the bits are those of the [K,N]
    partition."""
    M, K, N = 512, 256, 768
    A, W, scale, bias = wl.int8_mlp_layer(M, K, N)
    sA = 0.02
    js_kn, oid = ga.int8_mlp_json(M, K, N, sA, 128, scale.tolist())
    js_nk, oid2 = ga.int8_mlp_json(M, K, N, sA, 128, scale.tolist(), weights_nk=True, weights_constant=constant)
    st, plan = ga.explain(js_nk)
    assert st == 0 and "Dequantize x2 + MatMul" in plan and "transpose copy of W" in plan, plan
    assert ("once" in plan.split("transpose copy of W")[1].splitlines()[0]) == constant
    want = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    _run(ga, js_kn, [(0, A.to(dev)), (1, W.to(dev)), (2, bias.to(dev))], [(oid, want)])
    Wt = W.t().contiguous().to(dev)
    c = ga.Compiler()
    st, exe = c.compile(js_nk)
    assert st == 0
    for rep in range(2):
        a = A if rep == 0 else A.flip(0).contiguous()
        got = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
        assert exe.execute([(0, a.to(dev)), (1, Wt), (2, bias.to(dev))], [(oid2, got)]) == 0
        torch.cuda.synchronize()
        ref = want if rep == 0 else want.flip(0)
        assert torch.equal(got.view(torch.int16), ref.view(torch.int16)), rep
    exe.close()
    c.close()


def test_mlp_chain_partition(ga, orc, wl, dev):
    M, K, H = 512, 512, 1280
    x, W1, W2, b2 = wl.bf16_mlp_chain(M, K, H)
    out = torch.zeros(M, K, dtype=torch.bfloat16)
    _run(ga, ga.mlp_chain_json(M, K, H), [(0, x), (1, W1), (4, W2), (5, b2)], [(6, out)])
    h, y = orc.mlp_chain_bf16(wl.bf16_bits(x), wl.bf16_bits(W1), wl.bf16_bits(W2), wl.bf16_bits(b2))
    mm = orc.bf16_to_f32(orc.matmul_bf16(h, wl.bf16_bits(W2)))
    assert_close(orc.bf16_to_f32(y), out.float().numpy(), 2e-2, "mlp chain partition", mag=mm)


@pytest.mark.parametrize("D", [128, 64])
def test_attention_with_a_constant_mask_classifies_it_once(ga, gc, wl, dev, D):
    """A mask with property_type "constant": its tile classes are prepared in the first execute and kept.  Two
    executes (other Q the second time) give the bits of the partition whose mask is a variable, and of the raw entry
    points with and without prepared classes."""
    B, H, S = 1, 4, 512
    Q, K, V, mask, scale = wl.bf16_mha(B, H, S, D)
    sval = np.array([scale], np.float32)
    Qd, Kd, Vd, md = Q.to(dev), K.to(dev), V.to(dev), mask.to(dev)
    outs = {}
    for const in (True, False):
        comp = ga.Compiler()
        st, exe = comp.compile(ga.mha_json(B, H, S, S, D, True, "Multiply", mask_constant=const))
        assert st == 0
        res = []
        for rep in range(2):
            q = Qd if rep == 0 else Qd.flip(2).contiguous()
            o = torch.zeros(B, H, S, D, dtype=torch.bfloat16, device=dev)
            assert exe.execute([(0, q), (1, Kd), (2, torch.from_numpy(sval).to(dev)), (3, md), (4, Vd)], [(9, o)]) == 0
            res.append(o.clone())
        outs[const] = res
        exe.close()
        comp.close()
    for rep in range(2):
        assert torch.equal(outs[True][rep].view(torch.int16), outs[False][rep].view(torch.int16))
    cls = gc.mha_mask_classes(md, S, S, D)
    assert cls is not None
    for skip in (True, False):
        a = gc.mha_fwd_bf16_classified(Qd, Kd, Vd, md, cls, scale, skip_masked=skip)
        b = gc.mha_fwd_bf16(Qd, Kd, Vd, md, scale, skip_masked=skip)
        torch.cuda.synchronize()
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    assert torch.equal(outs[True][0].view(torch.int16), a.view(torch.int16))


@pytest.mark.parametrize("D,with_mask,scale_op", [(128, True, "Multiply"), (128, False, "Divide"), (64, True, "Multiply")])
def test_attention_partition(ga, orc, wl, dev, D, with_mask, scale_op):
    """head dims 128 and 64 both run the fused kernel (softmax weights rounded to bf16, as the graph's tensor is)."""
    B, H, S = 1, 2, 128
    Q, K, V, mask, scale = wl.bf16_mha(B, H, S, D)
    sval = np.array([scale if scale_op == "Multiply" else 1.0 / scale], np.float32)
    out = torch.zeros(B, H, S, D, dtype=torch.bfloat16)
    ins = [(0, Q), (1, K), (2, sval)] + ([(3, mask)] if with_mask else []) + [(4, V)]
    _run(ga, ga.mha_json(B, H, S, S, D, with_mask, scale_op), ins, [(9, out)])
    assert "attention" in ga.explain(ga.mha_json(B, H, S, S, D, with_mask, scale_op))[1]
    ref = orc.bf16_to_f32(orc.mha_bf16(wl.bf16_bits(Q), wl.bf16_bits(K), wl.bf16_bits(V),
                                       mask.numpy() if with_mask else None, scale))
    Sd = Q.double() @ K.double().transpose(-1, -2) * scale + (mask.double() if with_mask else 0)
    mag = (torch.softmax(Sd, -1) @ V.double().abs()).numpy()
    assert_close(ref, out.float().numpy(), 1e-2, "attention partition", mag=mag)


def test_constant_transposed_weight_is_prepared_once(ga, orc, wl, dev):
    """W^T . x with W stored [K,M] (transpose_a): the bf16 kernel reads its first operand row-major, so a
    transposed copy of W is made.  With property_type "constant" that happens in the first execute only: a second
    execute that is handed a different buffer under the same id still multiplies by the first contents.  Without
    the property the copy is redone every time."""
    M, K, N = 768, 512, 32
    torch.manual_seed(21)
    x = (torch.randn(K, N) * 0.5).to(torch.bfloat16)
    W = (torch.randn(K, M) * 0.05).to(torch.bfloat16)
    W2 = (torch.randn(K, M) * 0.05).to(torch.bfloat16)

    def graph(prop):
        return ga._graph([{"kind": "MatMul", "attrs": {"transpose_a": {"type": "bool", "value": 1}},
                           "inputs": [ga._t(0, "bf16", [K, M], property_type=prop), ga._t(1, "bf16", [K, N])],
                           "outputs": [ga._t(2, "bf16", [M, N])]}], [0, 1], [2])

    ref1 = orc.bf16_to_f32(orc.matmul_bf16(wl.bf16_bits(W.t().contiguous()), wl.bf16_bits(x)))
    ref2 = orc.bf16_to_f32(orc.matmul_bf16(wl.bf16_bits(W2.t().contiguous()), wl.bf16_bits(x)))
    for prop, second in (("constant", ref1), ("variable", ref2)):
        comp = ga.Compiler()
        st, exe = comp.compile(graph(prop))
        assert st == 0, ga.api().dnnl_graph_compiler_last_error().decode()
        st, plan = ga.explain(graph(prop))
        assert ("once" in plan) == (prop == "constant")
        out = torch.zeros(M, N, dtype=torch.bfloat16)
        for Wt, ref in ((W, ref1), (W2, second)):
            for pass_device in (False, True):
                ws, xs = (Wt.to(dev), x.to(dev)) if pass_device else (Wt, x)
                assert exe.execute([(0, ws), (1, xs)], [(2, out)]) == 0
                assert_close(ref, out.float().numpy(), 1e-2, "transpose_a %s" % prop)
        exe.close()
        comp.close()


def test_transposed_b_weight_needs_no_copy(ga, orc, wl, dev):
    """x[32,512] . W^T with W stored [N,K] (transpose_b, as the reference's llama2 case stores its weights):
    one GEMM launch that reads W as it lies."""
    M, K, N = 32, 512, 768
    torch.manual_seed(22)
    x = (torch.randn(M, K) * 0.5).to(torch.bfloat16)
    W = (torch.randn(N, K) * 0.05).to(torch.bfloat16)
    g = ga._graph([{"kind": "MatMul", "attrs": {"transpose_b": {"type": "bool", "value": 1}},
                    "inputs": [ga._t(0, "bf16", [M, K]), ga._t(1, "bf16", [N, K])],
                    "outputs": [ga._t(2, "bf16", [M, N])]}], [0, 1], [2])
    st, plan = ga.explain(g)
    assert st == 0 and [ln for ln in plan.splitlines() if not ln.startswith(("arena", "  tile:"))] == ["gemm_bf16: MatMul"]
    out = torch.zeros(M, N, dtype=torch.bfloat16)
    _run(ga, g, [(0, x), (1, W)], [(2, out)])
    ref = orc.bf16_to_f32(orc.matmul_bf16(wl.bf16_bits(x), wl.bf16_bits(W.t().contiguous())))
    assert_close(ref, out.float().numpy(), 1e-2, "transpose_b")


def test_chain_of_four_matmuls_with_shared_temporaries(ga, orc, wl, dev):
    """The third temporary lives in the first one's memory (lifetimes do not overlap): results must not care."""
    M = 256
    torch.manual_seed(31)
    x = (torch.randn(M, M) * 0.5).to(torch.bfloat16)
    Ws = [(torch.randn(M, M) * 0.08).to(torch.bfloat16) for _ in range(4)]
    ops = []
    for i in range(4):
        src = 0 if i == 0 else 10 + i - 1
        ops.append({"kind": "MatMul", "inputs": [ga._t(src, "bf16", [M, M]), ga._t(1 + i, "bf16", [M, M])],
                    "outputs": [ga._t(10 + i, "bf16", [M, M])]})
    js = ga._graph(ops, [0, 1, 2, 3, 4], [13])
    out = torch.zeros(M, M, dtype=torch.bfloat16)
    _run(ga, js, [(0, x)] + [(1 + i, Ws[i]) for i in range(4)], [(13, out)])
    cur = wl.bf16_bits(x)
    for W in Ws:
        cur = orc.matmul_bf16(cur, wl.bf16_bits(W))
    assert_close(orc.bf16_to_f32(cur), out.float().numpy(), 4e-2, "four chained matmuls (four rounding points)")


def test_reduce_without_axes_returns_its_operand(ga, dev):
    """lib/gc/Dialect/OneDNNGraph/OneDNNGraphOps.cpp:116-120: no reduce axes, no reduction."""
    x = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    out = np.zeros_like(x)
    g = ga._graph([{"kind": "ReduceSum", "inputs": [ga._t(0, "f32", [2, 3, 4])], "outputs": [ga._t(1, "f32", [2, 3, 4])]}],
                  [0], [1])
    _run(ga, g, [(0, x)], [(1, out)])
    assert (out == x).all()


def test_json_elementwise_extension_ops(ga, dev):
    """Element-wise ops of the oneDNN Graph specification beyond the reference's eleven, as JSON: a chain that the
    planner runs as one fused launch."""
    shape = [6, 50]
    ops, src = [], 0
    chain = ["Abs", "Sqrt", "Tanh", "Exp", "Log", "Square", "Reciprocal"]
    for i, kind in enumerate(chain):
        ops.append({"kind": kind, "inputs": [ga._t(src, "f32", shape)], "outputs": [ga._t(10 + i, "f32", shape)]})
        src = 10 + i
    ops.append({"kind": "Maximum", "inputs": [ga._t(src, "f32", shape), ga._t(1, "f32", shape)], "outputs": [ga._t(30, "f32", shape)]})
    ops.append({"kind": "Minimum", "inputs": [ga._t(30, "f32", shape), ga._t(2, "f32", [50])], "outputs": [ga._t(31, "f32", shape)]})
    g = ga._graph(ops, [0, 1, 2], [31])
    st, plan = ga.explain(g)
    assert st == 0 and plan.startswith("fused: Abs+Sqrt+Tanh+Exp+Log+Square+Reciprocal+Maximum+Minimum"), plan
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(shape) * 2).astype(np.float32)
    y = rng.standard_normal(shape).astype(np.float32) + 1
    z = rng.standard_normal(50).astype(np.float32) + 1.5
    out = np.zeros(shape, np.float32)
    _run(ga, g, [(0, x), (1, y), (2, z)], [(31, out)])
    t = np.tanh(np.sqrt(np.abs(x.astype(np.float64))))
    ref = np.minimum(np.maximum(1.0 / np.square(np.log(np.exp(t))), y), z)
    assert_close(ref, out, 1e-4, "element-wise extension ops")


def test_bound_tensor_lists_execute_repeatedly(ga, dev):
    """Executable.bind builds the tensor structs once; calling it is the C execute alone, any number of times, and
    sees the buffers' current contents."""
    gcomp = ga.Compiler()
    st, exe = gcomp.compile(_res("add.json"))
    assert st == 0
    a = torch.arange(128, dtype=torch.float32, device=dev)
    b = torch.ones(128, dtype=torch.float32, device=dev)
    out = torch.zeros(128, dtype=torch.float32, device=dev)
    call = exe.bind([(0, a), (1, b)], [(2, out)])
    for k in range(3):
        b.fill_(float(k))
        torch.cuda.synchronize()
        assert call() == 0
        assert torch.equal(out, a + k)
    exe.close()
    gcomp.close()


def test_execute_async_on_the_callers_stream(ga, dev):
    """execute_async launches on the stream it is given and does not wait: two calls with different inputs follow one
    another there, results are read after the caller's own synchronisation; host buffers are refused."""
    import ctypes as C
    M, K, N = 64, 96, 128
    g = ga._graph([{"kind": "MatMul", "inputs": [ga._t(0, "f32", [M, K]), ga._t(1, "f32", [K, N])], "outputs": [ga._t(2, "f32", [M, N])]},
                   {"kind": "ReLU", "inputs": [ga._t(2, "f32", [M, N])], "outputs": [ga._t(3, "f32", [M, N])]},
                   {"kind": "Exp", "inputs": [ga._t(3, "f32", [M, N])], "outputs": [ga._t(4, "f32", [M, N])]},
                   {"kind": "Multiply", "inputs": [ga._t(4, "f32", [M, N]), ga._t(3, "f32", [M, N])], "outputs": [ga._t(5, "f32", [M, N])]}],
                  [0, 1], [5])
    comp = ga.Compiler()
    st, exe = comp.compile(g)
    assert st == 0, ga.api().dnnl_graph_compiler_last_error().decode()
    torch.manual_seed(21)
    a = [torch.randn(M, K, device=dev) * 0.2 for _ in range(2)]
    w = torch.randn(K, N, device=dev) * 0.2
    outs = [torch.zeros(M, N, device=dev) for _ in range(2)]
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        calls = [exe.bind([(0, a[i]), (1, w)], [(5, outs[i])], stream=side.cuda_stream) for i in range(2)]
        assert calls[0]() == 0 and calls[1]() == 0
    side.synchronize()
    for i in range(2):
        r = torch.relu(a[i].double() @ w.double())
        assert_close((torch.exp(r) * r).cpu().numpy(), outs[i].double().cpu().numpy(), 1e-4, "async call %d" % i)
    host = np.zeros((M, N), np.float32)
    bad = exe.bind([(0, a[0]), (1, w)], [(5, host)], stream=side.cuda_stream)
    assert bad() == ga.INVALID_ARGUMENTS and b"device pointer" in ga.api().dnnl_graph_compiler_last_error()
    exe.close()
    comp.close()


@pytest.mark.parametrize("seed", range(16))
def test_random_attention_partitions_against_torch(ga, dev, seed):
    """Attention graphs with random sizes (also ones the fused kernel's fast path does not take), head dims 128, 64
    (fused) and 32 (no fused kernel: the ops run one by one), the scale as Multiply or Divide, and masks that are
    absent, shared ([Sq,Sk] / [1,1,Sq,Sk]: fused kernel) or per batch ([B,1,Sq,Sk]: the matcher declines and the ops
    run one by one): all against torch with P rounded to bf16 as in the graph."""
    rng = np.random.default_rng(7000 + seed)
    B, H = int(rng.integers(1, 3)), int(rng.integers(1, 4))
    Sq, Sk = int(rng.choice([64, 128, 200, 256])), int(rng.choice([64, 128, 192, 200]))
    D = [32, 128, 64, 128][seed % 4]
    scale_op = "Multiply" if rng.random() < 0.5 else "Divide"
    mask_kind = ["none", "2d", "4d_shared", "per_batch"][int(rng.integers(4))]
    s = [B, H, Sq, Sk]
    mshape = {"none": None, "2d": [Sq, Sk], "4d_shared": [1, 1, Sq, Sk], "per_batch": [B, 1, Sq, Sk]}[mask_kind]
    ops = [{"kind": "MatMul", "attrs": {"transpose_b": {"type": "bool", "value": 1}},
            "inputs": [ga._t(0, "bf16", [B, H, Sq, D]), ga._t(1, "bf16", [B, H, Sk, D])], "outputs": [ga._t(5, "f32", s)]},
           {"kind": scale_op, "inputs": [ga._t(5, "f32", s), ga._t(2, "f32", [1])], "outputs": [ga._t(6, "f32", s)]}]
    cur, ins = 6, [0, 1, 2]
    if mshape:
        ops.append({"kind": "Add", "inputs": [ga._t(6, "f32", s), ga._t(3, "f32", mshape)], "outputs": [ga._t(7, "f32", s)]})
        cur = 7
        ins.append(3)
    ops.append({"kind": "SoftMax", "attrs": {"axis": {"type": "s64", "value": -1}},
                "inputs": [ga._t(cur, "f32", s)], "outputs": [ga._t(8, "bf16", s)]})
    ops.append({"kind": "MatMul", "inputs": [ga._t(8, "bf16", s), ga._t(4, "bf16", [B, H, Sk, D])],
                "outputs": [ga._t(9, "bf16", [B, H, Sq, D])]})
    ins.append(4)
    g = ga._graph(ops, ins, [9])
    st, plan = ga.explain(g)
    assert st == 0, plan
    fused = plan.startswith("attention") or "\nattention" in plan
    assert fused == (D in (128, 64) and not (mask_kind == "per_batch" and B > 1)), plan
    torch.manual_seed(seed)
    Q = torch.randn(B, H, Sq, D).to(torch.bfloat16)
    K = torch.randn(B, H, Sk, D).to(torch.bfloat16)
    V = torch.randn(B, H, Sk, D).to(torch.bfloat16)
    scale = 1.0 / D ** 0.5
    sval = np.array([scale if scale_op == "Multiply" else 1.0 / scale], np.float32)
    mask = None
    if mshape:
        mask = torch.where(torch.rand(mshape) < 0.3, torch.tensor(-30000.0), torch.zeros(())).float()
        mask[..., 0] = 0  # no fully masked row
    out = torch.zeros(B, H, Sq, D, dtype=torch.bfloat16)
    tensors = [(0, Q), (1, K), (2, sval)] + ([(3, mask)] if mshape else []) + [(4, V)]
    _run(ga, g, tensors, [(9, out)])
    S = Q.double() @ K.double().transpose(-1, -2) * scale + (mask.double() if mshape else 0)
    P = torch.softmax(S, -1)
    ref = (P.to(torch.bfloat16).double() @ V.double()).to(torch.bfloat16).float().numpy()
    mag = (P @ V.double().abs()).numpy()
    assert_close(ref, out.float().numpy(), 1e-2, "attention %s D=%d mask=%s\n%s" % (s, D, mask_kind, plan), mag=mag)


def test_two_executables_interleaved_on_two_streams_match_serial_runs(ga, wl, dev):
    """The reference's execute is re-entrant (src/dnnl/dnnl_graph_compiler.cpp:214-226; scratch is thread-local,
    lib/gc/ExecutionEngine/CPURuntime/Microkernel/BrgemmOnednn.cpp:70).  Here the scratch of K-sliced GEMMs and of
    masked attention is part of each executable's arena: two executables launched alternately on two streams,
    with nothing ordering one stream against the other, give the bits of serial execution."""
    M, K, N = 32, 4096, 4096   # a short A against a wide weight: K-sliced, partial sums in the workspace
    B, H, S, D = 1, 8, 512, 128
    comp = ga.Compiler()
    g_mm = ga._graph([{"kind": "MatMul", "inputs": [ga._t(0, "bf16", [M, K]), ga._t(1, "bf16", [K, N])],
                       "outputs": [ga._t(2, "bf16", [M, N])]}], [0, 1], [2])
    exes = []
    for _ in range(2):
        st, e = comp.compile(g_mm)
        assert st == 0, ga.api().dnnl_graph_compiler_last_error().decode()
        exes.append(e)
    st, e_att = comp.compile(ga.mha_json(B, H, S, S, D, True, "Multiply"))
    assert st == 0, ga.api().dnnl_graph_compiler_last_error().decode()
    assert b"attention" in ga.explain(ga.mha_json(B, H, S, S, D, True, "Multiply"))[1].encode()
    torch.manual_seed(5)
    A = [(torch.randn(M, K) * 0.5).to(torch.bfloat16).to(dev) for _ in range(2)]
    W = [(torch.randn(K, N) * 0.05).to(torch.bfloat16).to(dev) for _ in range(2)]
    Q, Kt, V, mask, scale = wl.bf16_mha(B, H, S, D)
    Q, Kt, V, mask = Q.to(dev), Kt.to(dev), V.to(dev), mask.to(dev)
    sval = torch.tensor([scale], dtype=torch.float32)

    # serial: one executable after the other, each waited for
    want = [torch.zeros(M, N, dtype=torch.bfloat16, device=dev) for _ in range(2)]
    for i in range(2):
        assert exes[i].execute([(0, A[i]), (1, W[i])], [(2, want[i])]) == 0
    want_att = torch.zeros(B, H, S, D, dtype=torch.bfloat16, device=dev)
    assert e_att.execute([(0, Q), (1, Kt), (2, sval.numpy()), (3, mask), (4, V)], [(9, want_att)]) == 0

    # interleaved: stream i runs executable i, twenty rounds back to back; the raw attention entry point (library
    # workspace, ordered across streams by the library) alternates with them on both streams
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    got = [[torch.zeros(M, N, dtype=torch.bfloat16, device=dev) for _ in range(20)] for _ in range(2)]
    got_att = [torch.zeros(B, H, S, D, dtype=torch.bfloat16, device=dev) for _ in range(20)]
    calls = [[exes[i].bind([(0, A[i]), (1, W[i])], [(2, got[i][r])], stream=streams[i].cuda_stream) for r in range(20)]
             for i in range(2)]
    gcm = __import__("sys").modules["graph_compiler_amd"]
    torch.cuda.synchronize()
    for r in range(20):
        for i in range(2):
            assert calls[i][r]() == 0
        with torch.cuda.stream(streams[r % 2]):
            gcm.mha_fwd_bf16(Q, Kt, V, mask, scale, out=got_att[r])
    torch.cuda.synchronize()
    for i in range(2):
        for r in range(20):
            assert torch.equal(got[i][r].view(torch.int16), want[i].view(torch.int16)), (i, r)
    for r in range(20):
        assert torch.equal(got_att[r].view(torch.int16), want_att.view(torch.int16)), r
    for e in exes + [e_att]:
        e.close()
    comp.close()


def test_execute_from_two_host_threads_on_one_executable(ga, dev):
    """Calls on one executable take turns (they share its arena): two threads calling execute at once both get
    correct results."""
    import threading
    M, K, N = 32, 2048, 4096
    comp = ga.Compiler()
    g = ga._graph([{"kind": "MatMul", "inputs": [ga._t(0, "bf16", [M, K]), ga._t(1, "bf16", [K, N])],
                    "outputs": [ga._t(2, "bf16", [M, N])]},
                   {"kind": "ReLU", "inputs": [ga._t(2, "bf16", [M, N])], "outputs": [ga._t(3, "bf16", [M, N])]}], [0, 1], [3])
    st, exe = comp.compile(g)
    assert st == 0, ga.api().dnnl_graph_compiler_last_error().decode()
    torch.manual_seed(6)
    W = (torch.randn(K, N) * 0.05).to(torch.bfloat16).to(dev)
    A = [(torch.randn(M, K) * 0.5).to(torch.bfloat16).to(dev) for _ in range(2)]
    ref = [torch.relu((A[i].float() @ W.float()).to(torch.bfloat16)) for i in range(2)]
    errs = []

    def work(i):
        for _ in range(10):
            out = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
            if exe.execute([(0, A[i]), (1, W)], [(3, out)]) != 0:
                errs.append("status")
            d = (out.float() - ref[i].float()).abs().max().item()
            if d > 0.25:
                errs.append("thread %d off by %g" % (i, d))

    ts = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for t in ts:
        t.start()
    for t in ts:
        t.join()
    assert not errs, errs
    exe.close()
    comp.close()


def test_matmul_config_attributes_change_the_kernel_not_the_result(ga, gc, orc, wl, dev):
    """The op's nine MatmulConfig attributes (lib/gc/Analysis/MatmulConfigAnalysis.cpp:368-422) pick 8 waves of
    128 x 64 in place of 4 waves of 128 x 128 -- the same products in the same order, so the same bits -- and the
    number of K slices of a short A (another summation order: equal to rounding)."""
    names = gc.MATMUL_CONFIG_NAMES

    def run(M, K, N, cfg):
        op = {"kind": "MatMul", "inputs": [ga._t(0, "bf16", [M, K]), ga._t(1, "bf16", [K, N])], "outputs": [ga._t(2, "bf16", [M, N])]}
        if cfg:
            op["attrs"] = {k: {"type": "s64", "value": v} for k, v in zip(names, cfg)}
        torch.manual_seed(M + N)
        A = (torch.randn(M, K) * 0.5).to(torch.bfloat16).to(dev)
        B = (torch.randn(K, N) * 0.1).to(torch.bfloat16).to(dev)
        out = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
        _run(ga, ga._graph([op], [0, 1], [2]), [(0, A), (1, B)], [(2, out)])
        return A, B, out

    A, B, dflt = run(512, 1024, 768, None)  # six tiles: the default cuts K into slices
    _, _, w4 = run(512, 1024, 768, [2, 3, 1, 256, 256, 64, 128, 128, 32])
    _, _, w8 = run(512, 1024, 768, [2, 3, 1, 256, 256, 64, 128, 64, 32])
    assert torch.equal(w4.view(torch.int16), w8.view(torch.int16))
    assert (dflt.float() - w4.float()).abs().max().item() <= 0.0625
    ref = orc.bf16_to_f32(orc.matmul_bf16(wl.bf16_bits(A.cpu()), wl.bf16_bits(B.cpu())))
    assert_close(ref, dflt.float().cpu().numpy(), 1e-2, "default tile")
    A, B, s16 = run(32, 4096, 4096, None)
    _, _, s4 = run(32, 4096, 4096, [1, 16, 4, 256, 256, 64, 128, 128, 32])
    _, _, s1 = run(32, 4096, 4096, [1, 16, 1, 256, 256, 64, 128, 128, 32])
    ref = orc.bf16_to_f32(orc.matmul_bf16(wl.bf16_bits(A.cpu()), wl.bf16_bits(B.cpu())))
    for name, got in (("16 slices", s16), ("4 slices", s4), ("no slices", s1)):
        assert_close(ref, got.float().cpu().numpy(), 1e-2, name)
    assert not torch.equal(s16.view(torch.int16), s1.view(torch.int16))  # another summation order did run
