"""CPU: host side of the oneDNN-Graph backend API -- JSON schema, error classes,
op verification and the fusion plan -- through the C ABI
(dnnl_graph_compiler_explain runs parse -> verify -> fuse -> plan without a GPU).
Cases follow test/dnnl/TestJsonParser.cpp and the error mapping of
src/dnnl/dnnl_graph_compiler.cpp:190-207 / src/dnnl/JsonParser.cpp."""
import ctypes as C
import importlib
import json
import os

import pytest

from conftest import ROOT

OK, UNIMPL, RUNTIME, INVALID_GRAPH = 0, 3, 5, 7


@pytest.fixture(scope="module")
def ga(gc):
    return importlib.import_module("graph_compiler_amd.graph_api")


def _res(name):
    return open(os.path.join(ROOT, "tests", "golden", name)).read()


def test_version_struct(ga):
    v = ga.api().dnnl_graph_compiler_get_version().contents
    assert (v.api_version.major, v.api_version.minor, v.api_version.patch) == (0, 1, 0)
    assert v.gc_version.hash == b"gfx950"
    assert ga.api().dnnl_graph_compiler_get_version().contents.gc_version.major == v.gc_version.major  # static storage


def test_create_destroy_without_gpu(ga):
    for threads in (None, 4):
        c = ga.Compiler(threads)
        assert c.h
        c.close()


@pytest.mark.parametrize("name", ["add", "add_relu", "div", "matmul", "mpl", "mul", "pow", "reduce_mean", "reduce_sum",
                                  "relu", "sigmoid", "sub", "typecast"])
def test_every_reference_fixture_parses_and_plans(ga, name):
    st, plan = ga.explain(_res(name + ".json"))
    assert st == OK, plan
    assert plan.strip()


def _steps(plan):
    """The launch lines of a plan (the last line reports the arena size)."""
    return [ln for ln in plan.splitlines() if not ln.startswith(("arena:", "  tile:"))]


def test_fusion_plan_of_reference_mlp(ga):
    """mpl.json (test/dnnl/resources): MatMul+bias -> ReLU -> MatMul -> Add -> ReLU
    becomes two GEMM launches with everything else in the epilogues."""
    st, plan = ga.explain(_res("mpl.json"))
    assert st == OK
    assert _steps(plan) == ["gemm_bf16: MatMul+bias+act", "gemm_bf16: MatMul+bias+act"]


def test_fusion_plans_of_benchmark_partitions(ga):
    assert _steps(ga.explain(ga.matmul_bias_relu_json(128, 512, 256))[1]) == ["gemm_f32: MatMul+bias+act"]
    assert _steps(ga.explain(_res("matmul.json"))[1]) == ["gemm_f32: MatMul+bias"]  # transpose_a folds into strides
    j, _ = ga.int8_mlp_json(256, 256, 512, 0.02, 128, [0.01] * 512)
    lines = _steps(ga.explain(j)[1])
    assert lines[0].startswith("colsum") and lines[1].startswith("gemm_int8: Dequantize x2 + MatMul+bias+act+cast") and len(lines) == 2
    assert _steps(ga.explain(ga.mlp_chain_json(256, 256, 512))[1]) == ["gemm_bf16: MatMul+act", "gemm_bf16: MatMul+bias"]
    assert ga.explain(ga.mha_json(2, 2, 128, 128, 128))[1].startswith("attention:")
    assert ga.explain(ga.mha_json(2, 2, 128, 128, 128, with_mask=False, scale_op="Divide"))[1].startswith("attention:")
    assert ga.explain(ga.mha_json(1, 2, 64, 64, 64))[1].startswith("attention:")
    # head_dim 32 has no fused kernel: falls back to per-op kernels, still a valid plan
    unfused = ga.explain(ga.mha_json(1, 2, 64, 64, 32))[1]
    assert "softmax: SoftMax" in unfused and "attention" not in unfused


def test_intermediate_that_is_an_output_is_not_fused_away(ga):
    g = json.loads(ga.matmul_bias_relu_json(64, 64, 64))
    g["output_ports"] = [3, 4]  # the pre-activation tensor is wanted too
    st, plan = ga.explain(json.dumps(g))
    assert st == OK and _steps(plan) == ["gemm_f32: MatMul+bias", "fused: ReLU"]


def _mutate(fn):
    g = json.loads(_res("add_relu.json"))
    fn(g)
    return json.dumps(g)


def test_error_classes(ga):
    ex = ga.explain
    # malformed / unknown key / missing pieces -> invalid_graph (std::invalid_argument)
    assert ex("{")[0] == INVALID_GRAPH
    assert ex(_mutate(lambda g: g.update(foo=1)))[0] == INVALID_GRAPH
    assert ex(_mutate(lambda g: g["graph"][0].update(bar=1)))[0] == INVALID_GRAPH
    assert ex(_mutate(lambda g: g["graph"][0]["inputs"][0].update(baz=1)))[0] == INVALID_GRAPH
    assert ex(_mutate(lambda g: g["graph"][0].pop("kind")))[0] == INVALID_GRAPH
    assert ex(_mutate(lambda g: g["graph"][0]["inputs"][0].pop("dtype")))[0] == INVALID_GRAPH
    assert ex(_mutate(lambda g: g.update(output_ports=[99])))[0] == INVALID_GRAPH           # Output value not found
    assert ex(_mutate(lambda g: g.update(input_ports=[0])))[0] == INVALID_GRAPH              # length mismatch
    assert ex(_mutate(lambda g: g.update(input_ports=[0, 77])))[0] == INVALID_GRAPH          # input not in input_ports
    assert ex(_mutate(lambda g: g["graph"][1]["inputs"][0].update(dtype="f32")))[0] == INVALID_GRAPH  # type mismatch
    assert ex(_mutate(lambda g: g["graph"][1]["outputs"][0].update(id=2)))[0] == INVALID_GRAPH  # duplicate output id
    # unsupported feature -> unimplemented (std::logic_error)
    assert ex(_mutate(lambda g: g.update(engine_kind="fpga")))[0] == UNIMPL
    assert ex(_mutate(lambda g: g.update(fpmath_mode="bf16")))[0] == UNIMPL
    assert ex(_mutate(lambda g: g["graph"][0].update(kind="Convolution")))[0] == UNIMPL
    assert ex(_mutate(lambda g: g["graph"][0]["inputs"][0].update(dtype="f128")))[0] == UNIMPL
    assert ex(_mutate(lambda g: g["graph"][0]["inputs"][0].update(layout_type="blocked")))[0] == UNIMPL
    assert ex(_mutate(lambda g: g["graph"][0].update(attrs={"x": {"type": "u64", "value": 1}})))[0] == UNIMPL
    assert ex(_mutate(lambda g: g["graph"][0].update(attrs={"auto_broadcast": {"type": "string", "value": "maybe"}})))[0] == INVALID_GRAPH
    # a graph that parses but does not verify -> runtime_error, like a failed JitModule::create
    assert ex(_mutate(lambda g: g["graph"][1]["outputs"][0].update(shape=[3, 3])))[0] == RUNTIME
    assert "gpu" and ex(_mutate(lambda g: g.update(engine_kind="gpu")))[0] == OK
    st, msg = ex(_mutate(lambda g: g["graph"][0].update(kind="Convolution")))
    assert "Unsupported operation" in msg


def test_parser_ids_strides_and_op_order(ga):
    """test/dnnl/TestJsonParser.cpp:71-225: add_relu.json declares a strided input;
    inputs are numbered in order of first use; outputs default to the last op's."""
    g = json.loads(_res("add_relu.json"))
    strided = [t for op in g["graph"] for t in op["inputs"] if t.get("layout_type") == "strided"]
    assert strided, "fixture lost its strided tensor"
    st, plan = ga.explain(_res("add_relu.json"))
    assert st == OK and plan.splitlines()[0] == "eltwise: copy"  # the strided input is gathered first
    g.pop("output_ports")
    assert ga.explain(json.dumps(g))[0] == OK  # output_ports absent -> last op's outputs


def test_matmul_shape_rules(ga):
    """lib/gc/Dialect/OneDNNGraph/OneDNNGraphOps.cpp:204-310"""
    def mm(a, b, o, **attrs):
        at = {k: {"type": "bool", "value": int(v)} for k, v in attrs.items()}
        return json.dumps({"graph": [{"kind": "MatMul", "attrs": at,
                                      "inputs": [{"id": 0, "dtype": "f32", "shape": a}, {"id": 1, "dtype": "f32", "shape": b}],
                                      "outputs": [{"id": 2, "dtype": "f32", "shape": o}]}]})
    ok = [([4, 8], [8, 3], [4, 3], {}), ([8, 4], [8, 3], [4, 3], {"transpose_a": 1}), ([4, 8], [3, 8], [4, 3], {"transpose_b": 1}),
          ([2, 5, 4, 8], [8, 3], [2, 5, 4, 3], {}), ([2, 1, 4, 8], [5, 8, 3], [2, 5, 4, 3], {}), ([8], [8], [1], {}),
          ([8], [2, 8, 3], [2, 3], {}), ([2, 4, 8], [8], [2, 4], {})]
    for a, b, o, at in ok:
        assert ga.explain(mm(a, b, o, **at))[0] == OK, (a, b, o)
    bad = [([4, 8], [7, 3], [4, 3], {}), ([4, 8], [8, 3], [4, 4], {}), ([2, 4, 8], [3, 8, 3], [2, 4, 3], {})]
    for a, b, o, at in bad:
        assert ga.explain(mm(a, b, o, **at))[0] == RUNTIME, (a, b, o)


def test_tensor_struct_layout_matches_the_reference_initialisers(ga):
    """{.id, .ndims, .dims, .data} (test/dnnl/TestApiOps.cpp:46-48) on LP64."""
    T = ga.Tensor
    assert (T.id.offset, T.ndims.offset, T.dims.offset, T.data.offset, C.sizeof(T)) == (0, 8, 16, 24, 32)
    assert C.sizeof(ga.Context) == 4


def test_arena_shares_memory_between_temporaries_with_disjoint_lifetimes(ga):
    """Four chained matmuls: t1 is dead once t2 exists, so t3 can take its place (the reference merges
    allocations by lifetime ticks, lib/gc/Transforms/MergeAllocTickBased.cpp).  The plan reports both sizes."""
    import json
    import re
    M = 4096  # 256 tiles each: these matmuls are not K-sliced and need no scratch
    ops = []
    for i in range(4):
        src = 0 if i == 0 else 10 + i - 1
        ops.append({"kind": "MatMul", "inputs": [ga._t(src, "bf16", [M, M]), ga._t(1 + i, "bf16", [M, M])],
                    "outputs": [ga._t(10 + i, "bf16", [M, M])]})
    st, plan = ga.explain(ga._graph(ops, [0, 1, 2, 3, 4], [13]))
    assert st == 0, plan
    m = re.search(r"arena: (\d+) bytes \((\d+) with one region per buffer\); staging for host buffers: (\d+) bytes", plan)
    assert m, plan
    shared, naive, staging = int(m.group(1)), int(m.group(2)), int(m.group(3))
    one = M * M * 2
    assert naive == 3 * one          # the 3 temporaries
    assert shared == 2 * one         # t3 reuses t1's region
    # the 5 inputs and the output are the caller's buffers: device copies exist only for host pointers, in a block
    # of their own that the first such execute allocates
    assert staging == 6 * one


def test_k_sliced_matmuls_get_scratch_of_their_own_in_the_arena(ga, gc):
    """A short A against a wide weight is K-sliced: its partial sums live in a slot of the executable's arena, alive
    for that step only (two such steps share the space), not in anything shared between executables."""
    import re
    M, K, N = 32, 4096, 4096
    ops = [{"kind": "MatMul", "inputs": [ga._t(0, "bf16", [M, K]), ga._t(1, "bf16", [K, N])],
            "outputs": [ga._t(10, "bf16", [M, N])]},
           {"kind": "MatMul", "inputs": [ga._t(10, "bf16", [M, N]), ga._t(2, "bf16", [N, K])],
            "outputs": [ga._t(11, "bf16", [M, K])]}]
    st, plan = ga.explain(ga._graph(ops, [0, 1, 2], [11]))
    assert st == 0, plan
    m = re.search(r"arena: (\d+) bytes \((\d+) with one region per buffer\); staging for host buffers: (\d+) bytes", plan)
    shared, naive, staging = int(m.group(1)), int(m.group(2)), int(m.group(3))
    ws = gc.lib().gcmi_gemm_bf16_workspace_bytes(M, N, K, 0)
    assert ws >= 2 * M * N * 4      # at least two slices of f32 partial sums
    hidden = M * N * 2
    assert naive == hidden + 2 * ws
    assert shared == hidden + ws    # the second step's scratch takes the place of the first's
    assert staging == 2 * M * K * 2 + 2 * K * N * 2   # A, both weights, the result


@pytest.mark.parametrize("M,N,K,kthreads", [(4096, 4096, 4096, 4), (1024, 4096, 4096, 8)])
def test_slices_named_by_a_matmul_config_get_their_workspace(ga, gc, M, N, K, kthreads):
    """Shapes the launcher would not slice by default: a MatmulConfig whose KThreads names slices must get the
    partial sums' slot planned (else the launch silently runs unsliced while the plan text says otherwise), and the
    plan text, the tile descriptor and the workspace query must tell the same story."""
    import ctypes as C
    import re
    nine = [1, 1, kthreads, 256, 256, 64, 128, 128, 32]
    assert gc.lib().gcmi_gemm_bf16_workspace_bytes(M, N, K, 0) == 0
    c, note = gc.tile_config(M, N, K, matmul_config=nine)
    assert (c.kernel, c.split_k, c.from_attrs, note) == (3, kthreads, 1, "")
    ws = gc.lib().gcmi_gemm_bf16_workspace_bytes_cfg(M, N, K, 0, (C.c_int64 * 9)(*nine))
    assert ws == kthreads * M * N * 4
    op = {"kind": "MatMul", "inputs": [ga._t(0, "bf16", [M, K]), ga._t(1, "bf16", [K, N])], "outputs": [ga._t(2, "bf16", [M, N])],
          "attrs": {k: {"type": "s64", "value": v} for k, v in zip(gc.MATMUL_CONFIG_NAMES, nine)}}
    st, plan = ga.explain(ga._graph([op], [0, 1], [2]))
    assert st == 0, plan
    assert re.search(r"split_k %d, \d+ workgroups, workspace %d B \[MatmulConfig attributes applied\]" % (kthreads, ws), plan), plan
    arena = int(re.search(r"arena: (\d+) bytes", plan).group(1))
    assert arena >= ws


def test_a_constant_attention_mask_is_classified_once(ga):
    """The tile classes of a mask that is a constant of the partition are a once-only step with a slot of its own
    (kept for the executable's lifetime); a variable mask is classified by every call into the step's scratch."""
    st, plan = ga.explain(ga.mha_json(2, 4, 512, 512, 128, True, "Multiply", mask_constant=True))
    assert st == 0 and "attention mask: mask tile classes, once: the mask is constant" in plan and "attention:" in plan, plan
    st, plan2 = ga.explain(ga.mha_json(2, 4, 512, 512, 128, True, "Multiply"))
    assert st == 0 and "once" not in plan2 and "attention:" in plan2, plan2
    st, plan3 = ga.explain(ga.mha_json(1, 1, 16, 16, 128, True, "Multiply", mask_constant=True))   # too small for classes
    assert st == 0 and "once" not in plan3, plan3
