"""CPU: the textual-MLIR front end (dnnl_graph_compiler_explain_mlir runs parse -> verify -> fuse ->
plan without a GPU).  Modules follow what the reference's benchgc builds or holds: the MLP pattern
(test/benchgc/src/benchgc/pattern/mlp.py), test/benchgc/cases/llama2.mlir (a decoder MLP block) and
test/benchgc/cases/generic.mlir (a matmul spelled as linalg.generic)."""
import importlib
import os

import pytest

OK, UNIMPL, RUNTIME, INVALID_GRAPH = 0, 3, 5, 7
REF_CASES = "/root/reference/test/benchgc/cases"


@pytest.fixture(scope="module")
def ga(gc):
    return importlib.import_module("graph_compiler_amd.graph_api")


@pytest.fixture(scope="module")
def mm(gc):
    return importlib.import_module("graph_compiler_amd.mlir_modules")


def _steps(plan):
    return [ln for ln in plan.splitlines() if not ln.startswith(("arena:", "target hints", "  tile:"))]


def test_mlp_pattern_fuses_bias_and_activation_into_the_gemm(ga, mm):
    st, plan = ga.explain_mlir(mm.mlp(128, [512, 256, 64], [True, False], "relu", "bf16"))
    assert st == OK, plan
    assert _steps(plan) == ["gemm_bf16: MatMul+bias+act", "gemm_bf16: MatMul+act"]
    st, plan = ga.explain_mlir(mm.mlp(32, [64, 64], [True], "noop", "f32"))
    assert st == OK and _steps(plan) == ["gemm_f32: MatMul+bias"]
    # 1 / (1 + exp(-x)) written as four linalg ops is one sigmoid, which the GEMM epilogue takes
    st, plan = ga.explain_mlir(mm.mlp(32, [64, 64], [True], "sigmoid", "f32"))
    assert st == OK and _steps(plan) == ["gemm_f32: MatMul+bias+act"]


def test_generic_contraction_is_a_matmul(ga, mm):
    for tb in (False, True):
        st, plan = ga.explain_mlir(mm.generic_matmul(16, 8, 4, "f32", transpose_b=tb))
        assert st == OK, plan
        assert _steps(plan)[-1] == "gemm_f32: MatMul"
    # a body that is not multiply-accumulate is outside the subset
    bad = mm.generic_matmul(16, 8, 4).replace("arith.mulf", "arith.subf")
    assert ga.explain_mlir(bad)[0] == UNIMPL
    # map results must be plain dims
    bad = mm.generic_matmul(16, 8, 4).replace("-> (d0, d2)", "-> (d0 + d1, d2)")
    assert ga.explain_mlir(bad)[0] == UNIMPL


def test_decoder_block_plan(ga, mm, monkeypatch):
    """31 linalg/tensor ops become 7 launches: four GEMMs, the two that feed a residual connection with the add in
    their epilogue (through the tensor.expand_shape view between them); per RMSNorm one launch (x^2 summed, / H,
    + eps, ^-0.5, then the scaling as a second pass over the row); the gate.  With the library's generic kernels
    instead of generated ones, the scaling of a few long rows (32 tokens) stays a launch of its own that spreads
    over all compute units: 9 launches; from 512 rows on the plan is the same."""
    merged = [
        "gemm_bf16: MatMul+residual",
        "reduce: TypeCast+Multiply+TypeCast+Multiply after Divide+Add+Pow of ReduceSum of TypeCast+Pow",
        "gemm_bf16: MatMul",
        "gemm_bf16: MatMul",
        "fused: Sigmoid+Multiply+Multiply",  # 1/(1+exp(-x)) was recognised as one sigmoid first
        "gemm_bf16: MatMul+residual",
        "reduce: TypeCast+Multiply+TypeCast+Multiply after Divide+Add+Pow of ReduceSum of TypeCast+Pow"]
    for tokens in (32, 1024):
        st, plan = ga.explain_mlir(mm.decoder_mlp_block(tokens, 256, 512))
        assert st == OK, plan
        assert _steps(plan) == merged
    monkeypatch.setenv("GCMI_NO_GENERATED_KERNELS", "1")
    st, plan = ga.explain_mlir(mm.decoder_mlp_block(32, 256, 512))
    assert st == OK, plan
    assert _steps(plan) == [
        "gemm_bf16: MatMul+residual",
        "reduce: Divide+Add+Pow of ReduceSum of TypeCast+Pow",
        "fused: TypeCast+Multiply+TypeCast+Multiply",
        "gemm_bf16: MatMul",
        "gemm_bf16: MatMul",
        "fused: Sigmoid+Multiply+Multiply",
        "gemm_bf16: MatMul+residual",
        "reduce: Divide+Add+Pow of ReduceSum of TypeCast+Pow",
        "fused: TypeCast+Multiply+TypeCast+Multiply"]
    st, plan = ga.explain_mlir(mm.decoder_mlp_block(1024, 256, 512))
    assert st == OK and _steps(plan) == merged, plan


def test_pointwise_fusion_rules(ga, monkeypatch):
    t = "tensor<8x16xf32>"
    e = "%e = tensor.empty() : " + t + "\n"

    def fn(body, res=t, args="%a: " + t + ", %b: " + t):
        return "func.func @f(%s) -> %s {\n%s%s\n}" % (args, res, e, body)

    def bin(res, op, x, y):
        return "%s = linalg.%s ins(%s, %s : %s, %s) outs(%%e : %s) -> %s\n" % (res, op, x, y, t, t, t, t)

    # a chain is one launch; a value with two point-wise readers is not stored either
    chain = fn(bin("%0", "add", "%a", "%b") + bin("%1", "mul", "%0", "%0") + bin("%2", "sub", "%1", "%0") + "return %2 : " + t)
    assert _steps(ga.explain_mlir(chain)[1]) == ["fused: Add+Multiply+Subtract"]
    # a value that is also returned is stored: it ends its own group, and its readers load it
    two = fn(bin("%0", "add", "%a", "%b") + bin("%1", "mul", "%0", "%b") + bin("%2", "sub", "%1", "%a") +
             "return %0, %2 : " + t + ", " + t, res="(" + t + ", " + t + ")")
    assert _steps(ga.explain_mlir(two)[1]) == ["fused: Add", "fused: Multiply+Subtract"]  # a lone op is a group of one
    # a matmul operand is stored
    mmul = fn(bin("%0", "add", "%a", "%b") + bin("%1", "mul", "%0", "%b") +
              "%c0 = arith.constant 0.0 : f32\n%z = linalg.fill ins(%c0 : f32) outs(%e : " + t + ") -> " + t + "\n"
              "%2 = linalg.matmul_transpose_b ins(%1, %a : " + t + ", " + t + ") outs(%ez : tensor<8x8xf32>) -> tensor<8x8xf32>\n"
              "return %2 : tensor<8x8xf32>", res="tensor<8x8xf32>").replace(
                  "%c0 = arith", "%ez = tensor.empty() : tensor<8x8xf32>\n%c0 = arith")
    assert _steps(ga.explain_mlir(mmul)[1]) == ["fused: Add+Multiply", "gemm_f32: MatMul"]
    # the switch that turns the pass off: one launch per op
    monkeypatch.setenv("GCMI_NO_POINTWISE_FUSION", "1")
    assert _steps(ga.explain_mlir(chain)[1]) == ["eltwise: Add", "eltwise: Multiply", "eltwise: Subtract"]


@pytest.mark.skipif(not os.path.isdir(REF_CASES), reason="the reference tree is not on this machine")
def test_reference_benchgc_cases_parse_and_plan(ga, mm):
    st, plan = ga.explain_mlir(open(os.path.join(REF_CASES, "llama2.mlir")).read())
    assert st == OK, plan
    # same structure as the builder's block at the case's sizes
    st2, plan2 = ga.explain_mlir(mm.decoder_mlp_block(32, 4096, 11008))
    assert st2 == OK and _steps(plan) == _steps(plan2)
    st, plan = ga.explain_mlir(open(os.path.join(REF_CASES, "generic.mlir")).read())
    assert st == OK and _steps(plan) == ["gemm_f32: MatMul"]


def test_target_spec_of_the_module_is_read(ga, mm):
    """benchgc attaches the CPU's cache sizes and thread count (mlir/util.py:187-197)."""
    spec = ('module attributes {\n dlti.target_system_spec = #dlti.target_system_spec<\n'
            '  "CPU": #dlti.target_device_spec<\n'
            '   #dlti.dl_entry<"L1_cache_size_in_bytes", 49152 : ui32>,\n'
            '   #dlti.dl_entry<"L2_cache_size_in_bytes", 2097152 : ui64>,\n'
            '   #dlti.dl_entry<"L3_cache_size_in_bytes", 110100480 : ui64>,\n'
            '   #dlti.dl_entry<"num_threads", 56 : i32>,\n'
            '   #dlti.dl_entry<"max_vector_width", 512 : i64>>\n >} {')
    text = mm.mlp(32, [64, 64]).replace("module {", spec, 1)
    st, plan = ga.explain_mlir(text)
    assert st == OK, plan
    line = [ln for ln in plan.splitlines() if ln.startswith("target hints")]
    assert line and "num_threads=56" in line[0] and "L2_cache_size_in_bytes=2097152" in line[0]
    assert _steps(plan) == ["gemm_f32: MatMul"]


def _fn(body, args="%a: tensor<8x8xf32>, %b: tensor<8x8xf32>", res="tensor<8x8xf32>"):
    return "func.func @f(%s) -> %s {\n%s\n}" % (args, res, body)


def test_error_classes(ga):
    ex = ga.explain_mlir
    e = "%e = tensor.empty() : tensor<8x8xf32>\n"
    ok = _fn(e + "%r = linalg.add ins(%a, %b : tensor<8x8xf32>, tensor<8x8xf32>) outs(%e : tensor<8x8xf32>) -> tensor<8x8xf32>\n"
             "return %r : tensor<8x8xf32>")
    st, plan = ex(ok)  # a bare function, no module around it
    assert st == OK and _steps(plan) == ["fused: Add"]
    # malformed text, undefined values -> invalid_graph
    assert ex("module {")[0] == INVALID_GRAPH
    assert ex(ok.replace("ins(%a, %b", "ins(%a, %nope"))[0] == INVALID_GRAPH
    assert ex(ok.replace("return %r : tensor<8x8xf32>", ""))[0] == INVALID_GRAPH
    assert ex(_fn("return"))[0] == INVALID_GRAPH  # nothing returned
    # outside the subset -> unimplemented
    assert ex(ok.replace("linalg.add", "linalg.conv_2d"))[0] == UNIMPL
    assert ex(ok.replace("tensor<8x8xf32>", "tensor<?x8xf32>"))[0] == UNIMPL
    assert ex(ok.replace("f32", "f8E4M3"))[0] == UNIMPL
    assert ex(_fn("%r = scf.for %i = %a to %b : index {}\nreturn %r : tensor<8x8xf32>"))[0] == UNIMPL
    st, msg = ex(ok.replace("linalg.add", "linalg.conv_2d"))
    assert "linalg.conv_2d" in msg
    # parses but does not verify (result shape) -> runtime_error, like a failed pipeline run
    wrong = ok.replace("outs(%e : tensor<8x8xf32>) -> tensor<8x8xf32>", "outs(%e : tensor<8x8xf32>) -> tensor<8x4xf32>")
    assert ex(wrong)[0] == RUNTIME
    # accumulating matmul (init that is not zero) is not taken
    acc = _fn("%r = linalg.matmul ins(%a, %b : tensor<8x8xf32>, tensor<8x8xf32>) outs(%a : tensor<8x8xf32>) -> tensor<8x8xf32>\n"
              "return %r : tensor<8x8xf32>")
    assert ex(acc)[0] == UNIMPL


def test_returned_argument_constant_and_duplicate_are_copied(ga):
    e = "%e = tensor.empty() : tensor<8x8xf32>\n"
    body = (e + "%c = arith.constant dense<2.500000e+00> : tensor<8x8xf32>\n"
            "%r = linalg.mul ins(%a, %c : tensor<8x8xf32>, tensor<8x8xf32>) outs(%e : tensor<8x8xf32>) -> tensor<8x8xf32>\n"
            "return %r, %r, %a, %c : tensor<8x8xf32>, tensor<8x8xf32>, tensor<8x8xf32>, tensor<8x8xf32>")
    st, plan = ga.explain_mlir(_fn(body, res="(tensor<8x8xf32>, tensor<8x8xf32>, tensor<8x8xf32>, tensor<8x8xf32>)"))
    assert st == OK, plan
    assert len(_steps(plan)) == 4  # the product, its copy, the copy of %a and the filled constant


def test_linalg_driver_single_ops_plan(ga, mm):
    """The element-wise, binary and matmul cases of benchgc's linalg driver, one op per module."""
    for op in ("abs", "ceil", "floor", "erf", "log", "negf", "exp", "round", "rsqrt", "sqrt", "square", "tanh", "reciprocal"):
        st, plan = ga.explain_mlir(mm.linalg_op(op, [[4, 8]], [4, 8]))
        assert st == OK and len(_steps(plan)) == 1 and _steps(plan)[0].startswith("fused:"), (op, plan)
    for op in ("add", "sub", "mul", "div", "max", "min"):
        st, plan = ga.explain_mlir(mm.linalg_op(op, [[4, 8], [4, 8]], [4, 8]))
        assert st == OK and len(_steps(plan)) == 1, (op, plan)
    cases = [("matmul", [[8, 16], [16, 4]], [8, 4]), ("matmul_transpose_a", [[16, 8], [16, 4]], [8, 4]),
             ("matmul_transpose_b", [[8, 16], [4, 16]], [8, 4]), ("batch_matmul", [[3, 8, 16], [3, 16, 4]], [3, 8, 4]),
             ("batch_matmul_transpose_a", [[3, 16, 8], [3, 16, 4]], [3, 8, 4]),
             ("batch_matmul_transpose_b", [[3, 8, 16], [3, 4, 16]], [3, 8, 4]),
             ("matvec", [[8, 16], [16]], [8]), ("vecmat", [[16], [16, 4]], [4]), ("dot", [[16], [16]], []),
             ("batch_matvec", [[3, 8, 16], [3, 16]], [3, 8]), ("batch_vecmat", [[3, 16], [3, 16, 4]], [3, 4]),
             ("batch_reduce_matmul", [[3, 8, 16], [3, 16, 4]], [8, 4])]
    for op, ins, out in cases:
        st, plan = ga.explain_mlir(mm.linalg_op(op, ins, out))
        assert st == OK, (op, plan)
        assert any(s.startswith("gemm_f32") for s in _steps(plan)), (op, plan)
    # packed layouts and convolutions are outside the subset
    assert ga.explain_mlir(mm.linalg_op("mmt4d", [[2, 2, 4, 4], [2, 2, 4, 4]], [2, 2, 4, 4]))[0] == UNIMPL


def test_transpose_in_front_of_a_matmul_becomes_its_flag(ga):
    """x . transpose(w), as exporters write a Linear layer: one GEMM that reads w as it lies."""
    text = """func.func @f(%x: tensor<64x256xbf16>, %w: tensor<512x256xbf16>) -> tensor<64x512xbf16> {
      %et = tensor.empty() : tensor<256x512xbf16>
      %wt = linalg.transpose ins(%w : tensor<512x256xbf16>) outs(%et : tensor<256x512xbf16>) permutation = [1, 0]
      %c0 = arith.constant 0.0 : bf16
      %e = tensor.empty() : tensor<64x512xbf16>
      %z = linalg.fill ins(%c0 : bf16) outs(%e : tensor<64x512xbf16>) -> tensor<64x512xbf16>
      %y = linalg.matmul ins(%x, %wt : tensor<64x256xbf16>, tensor<256x512xbf16>) outs(%z : tensor<64x512xbf16>) -> tensor<64x512xbf16>
      return %y : tensor<64x512xbf16>
    }"""
    st, plan = ga.explain_mlir(text)
    assert st == OK and _steps(plan) == ["gemm_bf16: MatMul"], plan
    # a transpose that is not of the last two dims stays a copy
    other = text.replace("permutation = [1, 0]", "permutation = [0, 1]").replace("tensor<256x512xbf16>", "tensor<512x256xbf16>")
    st, plan = ga.explain_mlir(other)
    assert st != OK or "Transpose" in plan


REF_DIALECT = "/root/reference/test/mlir/test/gc/Dialect/OneDNNGraph"


@pytest.mark.skipif(not os.path.isdir(REF_DIALECT), reason="the reference tree is not on this machine")
def test_reference_onednn_graph_dialect_files(ga):
    """Every function of the reference's own front-end dialect tests parses and plans (one function per text)."""
    import re
    n = 0
    for name in ("onednn-graph-llama2.mlir", "onednn-graph-mlp.mlir", "onednn-graph-ops.mlir", "onednn-graph-to-linalg.mlir"):
        text = open(os.path.join(REF_DIALECT, name)).read()
        text = "\n".join(ln for ln in text.splitlines() if not ln.lstrip().startswith("//"))
        for fn in re.split(r"(?=func\.func)", text):
            if not fn.startswith("func.func") or "onednn_graph." not in fn:
                continue  # the @main drivers of the runnable tests call the function above them
            st, plan = ga.explain_mlir(fn)
            assert st == OK, (name, fn[:80], plan)
            n += 1
    assert n >= 20
    st, plan = ga.explain_mlir(open(os.path.join(REF_DIALECT, "onednn-graph-mlp.mlir")).read())
    assert _steps(plan) == ["gemm_bf16: MatMul+bias+act", "gemm_bf16: MatMul+bias+act"]


def test_onednn_graph_dialect_ops(ga):
    t = "tensor<64x128xbf16>"
    text = """func.func @f(%x: tensor<64x128xbf16>, %w: tensor<256x128xbf16>, %b: tensor<256xbf16>) -> tensor<64x1xf32> {
      %0 = onednn_graph.matmul %x, %w, %b {transpose_b = true}
           : (tensor<64x128xbf16>, tensor<256x128xbf16>, tensor<256xbf16>) -> tensor<64x256xbf16>
      %1 = onednn_graph.sigmoid %0 : (tensor<64x256xbf16>) -> tensor<64x256xbf16>
      %2 = onednn_graph.type_cast %1 : (tensor<64x256xbf16>) -> tensor<64x256xf32>
      %3 = onednn_graph.pow %2 {beta = 2.0 : f32} : (tensor<64x256xf32>) -> tensor<64x256xf32>
      %4 = onednn_graph.reduce_mean %3 {axes = array<i64: -1>, keep_dims = true} : (tensor<64x256xf32>) -> tensor<64x1xf32>
      return %4 : tensor<64x1xf32>
    }"""
    st, plan = ga.explain_mlir(text)
    assert st == OK, plan
    assert _steps(plan) == ["gemm_bf16: MatMul+bias+act", "reduce: ReduceMean of TypeCast+Pow"]
    assert ga.explain_mlir(text.replace("onednn_graph.sigmoid", "onednn_graph.softplus"))[0] == UNIMPL
    assert ga.explain_mlir(text.replace("{beta = 2.0 : f32} ", ""))[0] == INVALID_GRAPH


def test_residual_absorption_rules(ga):
    """A full-shape add behind a bf16 matmul goes into its epilogue and ends the chain; f32 matmuls, column
    broadcasts and results with a second reader keep the add as a kernel of its own."""
    def module(dt, res_shape="64x128", tail=""):
        t, a, w, r = "tensor<64x128x%s>" % dt, "tensor<64x32x%s>" % dt, "tensor<32x128x%s>" % dt, "tensor<%sx%s>" % (res_shape, dt)
        body = ("  %z = arith.constant 0.0 : " + dt + "\n  %e = tensor.empty() : " + t + "\n"
                "  %f = linalg.fill ins(%z : " + dt + ") outs(%e : " + t + ") -> " + t + "\n"
                "  %m = linalg.matmul ins(%a, %w : " + a + ", " + w + ") outs(%f : " + t + ") -> " + t + "\n")
        if res_shape == "64x128":
            body += "  %o = linalg.add ins(%m, %x : " + t + ", " + t + ") outs(%e : " + t + ") -> " + t + "\n"
        else:
            body += ("  %xb = linalg.broadcast ins(%x : " + r + ") outs(%e : " + t + ") dimensions = [1]\n"
                     "  %o = linalg.add ins(%m, %xb : " + t + ", " + t + ") outs(%e : " + t + ") -> " + t + "\n")
        body += tail.replace("T", t)
        last = "%q" if tail else "%o"
        return ("func.func @f(%a: " + a + ", %w: " + w + ", %x: " + r + ") -> " + t + " {\n" + body +
                "  return " + last + " : " + t + "\n}")

    st, plan = ga.explain_mlir(module("bf16"))
    assert st == OK and _steps(plan) == ["gemm_bf16: MatMul+residual"], plan
    st, plan = ga.explain_mlir(module("f32"))
    assert st == OK and _steps(plan) == ["gemm_f32: MatMul", "fused: Add"], plan
    st, plan = ga.explain_mlir(module("bf16", res_shape="64"))
    assert st == OK and _steps(plan)[0] == "gemm_bf16: MatMul" and len(_steps(plan)) == 2, plan
    # an activation behind the residual sum is not the epilogue's order (activation first): it stays outside
    st, plan = ga.explain_mlir(module("bf16", tail="  %q = linalg.max ins(%o, %f : T, T) outs(%e : T) -> T\n"))
    assert st == OK and _steps(plan)[0] == "gemm_bf16: MatMul+residual" and len(_steps(plan)) == 2, plan
    # the matmul's result is read again: it has to exist, so the add is a kernel of its own
    st, plan = ga.explain_mlir(module("bf16", tail="  %q = linalg.mul ins(%o, %m : T, T) outs(%e : T) -> T\n"))
    assert st == OK and _steps(plan)[0] == "gemm_bf16: MatMul" and len(_steps(plan)) == 2, plan


@pytest.mark.parametrize("shape,axis", [((5, 7, 3), 2), ((5, 7, 3), 0), ((9, 130), 1), ((2, 3, 5, 8), 1), ((640, 256), 1)])
def test_generated_kernels_compile_for_gfx950(ga, shape, axis):
    """The HIP source written for a module's fused groups -- element-at-a-time and four-at-a-time forms, strided
    rows, f16 storage, a row sum with ops before and after it and a second pass over the row -- is accepted by the
    run-time compiler for gfx950 (no GPU involved), and carries one kernel per fused group of the plan."""
    def t(s, dt="f16"):
        return "tensor<" + "".join("%dx" % d for d in s) + dt + ">"
    kept = [d for i, d in enumerate(shape) if i != axis]
    full, row, rowdims = t(shape), t(kept), str(axis)
    text = ("func.func @f(%x: " + full + ", %y: " + full + ") -> (" + full + ", " + row + ", " + full + ") {\n"
            "  %e = tensor.empty() : " + full + "\n  %er = tensor.empty() : " + row + "\n"
            "  %two = arith.constant dense<2.000000e+00> : " + full + "\n"
            "  %a = linalg.mul ins(%x, %two : " + full + ", " + full + ") outs(%e : " + full + ") -> " + full + "\n"
            "  %b = linalg.add ins(%a, %y : " + full + ", " + full + ") outs(%e : " + full + ") -> " + full + "\n"
            "  %c = linalg.exp ins(%b : " + full + ") outs(%e : " + full + ") -> " + full + "\n"
            "  %c0 = arith.constant 0.0 : f16\n"
            "  %z = linalg.fill ins(%c0 : f16) outs(%er : " + row + ") -> " + row + "\n"
            "  %s = linalg.reduce { arith.addf } ins(%c : " + full + ") outs(%z : " + row + ") dimensions = [" + rowdims + "]\n"
            "  %one = arith.constant dense<1.000000e+00> : " + row + "\n"
            "  %s1 = linalg.add ins(%s, %one : " + row + ", " + row + ") outs(%er : " + row + ") -> " + row + "\n"
            "  %sb = linalg.broadcast ins(%s1 : " + row + ") outs(%e : " + full + ") dimensions = [" + rowdims + "]\n"
            "  %n = linalg.div ins(%c, %sb : " + full + ", " + full + ") outs(%e : " + full + ") -> " + full + "\n"
            "  return %c, %s1, %n : " + full + ", " + row + ", " + full + "\n}")
    st, plan = ga.explain_mlir(text)
    assert st == OK, plan
    groups = [s for s in _steps(plan) if s.startswith("fused:") or s.startswith("reduce:")]
    st, src = ga.generated_source_mlir(text, "gfx950")
    assert st == OK, src
    assert src.count('extern "C" __global__') == len(groups) >= 2, (plan, src)


def test_generated_source_of_the_decoder_block(ga, mm):
    st, src = ga.generated_source_mlir(mm.decoder_mlp_block(32, 256, 512), "gfx950")
    assert st == OK, src
    assert src.count('extern "C" __global__') == 3  # two normalisations, the gate
    assert "__shfl_xor" in src and "gcmi::fused_op(" in src
    st, msg = ga.generated_source_mlir("func.func @f(", "gfx950")
    assert st != OK


def test_ops_whose_operands_are_all_broadcasts(ga):
    """linalg.broadcast is folded into its readers' strides only where each reader keeps an operand arrangement that
    still broadcasts to its result: add(row, row) over [8,64] would be a [64] result, so that broadcast stays a copy."""
    t = "tensor<8x64xf32>"
    text = ("func.func @f(%x: T, %r: tensor<64xf32>, %c: tensor<8xf32>) -> (T, T) {\n"
            "  %e = tensor.empty() : T\n"
            "  %rb = linalg.broadcast ins(%r : tensor<64xf32>) outs(%e : T) dimensions = [0]\n"
            "  %cb = linalg.broadcast ins(%c : tensor<8xf32>) outs(%e : T) dimensions = [1]\n"
            "  %v1 = linalg.sub ins(%x, %cb : T, T) outs(%e : T) -> T\n"
            "  %v2 = linalg.add ins(%rb, %rb : T, T) outs(%e : T) -> T\n"
            "  %v3 = linalg.mul ins(%v1, %v2 : T, T) outs(%e : T) -> T\n"
            "  %v4 = linalg.max ins(%cb, %x : T, T) outs(%e : T) -> T\n"
            "  return %v3, %v4 : T, T\n}").replace("T", t)
    st, plan = ga.explain_mlir(text)
    assert st == OK, plan
    assert _steps(plan) == ["eltwise: BroadcastTo (stride-0 copy)", "fused: Subtract+Add+Multiply", "fused: Maximum"], plan


def test_layer_normalisation_plan(ga, mm):
    """Two reductions: the mean is read by the variance group and by the scaling, so it is a kernel of its own; the
    variance group and the scaling (which alone reads the reciprocal deviation) share a launch."""
    st, plan = ga.explain_mlir(mm.layernorm(512, 1024))
    assert st == OK, plan
    assert _steps(plan) == ["reduce: Divide of ReduceSum",
                            "reduce: Subtract+Multiply+Multiply+Add after Divide+Add+Rsqrt of ReduceSum of Subtract+Square"], plan
    st, src = ga.generated_source_mlir(mm.layernorm(512, 1024, "bf16"), "gfx950")
    assert st == OK and src.count('extern "C" __global__') == 2, src
