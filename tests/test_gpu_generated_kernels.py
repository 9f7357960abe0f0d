"""GPU: the kernels generated for fused point-wise groups against the library's generic kernels for the same groups,
on seeded random programs -- random chains of the named unary and binary linalg ops over full-shape, row-broadcast
and column-broadcast operands, storage types f32 / bf16 / f16, shapes inside and outside the four-elements-per-thread
mode, optionally with a sum over the last or the first axis and a normalisation behind it.  The bar between the two
is bit equality (NaNs and infinities included: results are compared as integers), since both run the same expressions
in the same order.  Both share the planner, so the programs are also evaluated op by op with torch (f32 arithmetic,
every result rounded to the storage type) and compared within a tolerance, NaNs and infinities in the same places."""
import importlib
import re

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

UNARY = ["abs", "ceil", "floor", "negf", "exp", "tanh", "square", "erf", "sqrt", "rsqrt", "log", "reciprocal", "round"]
BINARY = ["add", "sub", "mul", "div", "max", "min"]
SHAPES = [(5, 7, 3), (8, 64), (33, 130), (4, 6, 10, 12), (300,), (2, 1028), (64, 2048), (3, 4100), (600, 8)]


@pytest.fixture(scope="module")
def ga(gc, dev):
    return importlib.import_module("graph_compiler_amd.graph_api")


def _t(shape, dt):
    return "tensor<" + "".join("%dx" % d for d in shape) + dt + ">"


def random_module(rng, shape, dt):
    """-> (text, argument shapes, result shapes).  Arguments: x, y (full shape), r (last dim), c (all but the last dim)."""
    full = _t(shape, dt)
    args = [("%x", shape), ("%y", shape)]
    lines = ["%e = tensor.empty() : " + full]
    values = ["%x", "%y"]
    if len(shape) > 1:
        args += [("%r", shape[-1:]), ("%c", shape[:-1])]
        lines.append("%rb = linalg.broadcast ins(%r : " + _t(shape[-1:], dt) + ") outs(%e : " + full + ") dimensions = [" +
                     ", ".join(str(i) for i in range(len(shape) - 1)) + "]")
        lines.append("%cb = linalg.broadcast ins(%c : " + _t(shape[:-1], dt) + ") outs(%e : " + full + ") dimensions = [" +
                     str(len(shape) - 1) + "]")
        values += ["%rb", "%cb"]
    n = 0

    def emit(op, operands, ty, outs):
        nonlocal n
        n += 1
        name = "%v" + str(n)
        lines.append(name + " = linalg." + op + " ins(" + ", ".join(operands) + " : " + ", ".join([ty] * len(operands)) + ") outs(" +
                     outs + " : " + ty + ") -> " + ty)
        return name

    for _ in range(int(rng.integers(1, 8))):
        if rng.random() < 0.45:
            values.append(emit(UNARY[int(rng.integers(len(UNARY)))], [values[int(rng.integers(len(values)))]], full, "%e"))
        else:
            a, b = values[int(rng.integers(len(values)))], values[int(rng.integers(len(values)))]
            values.append(emit(BINARY[int(rng.integers(len(BINARY)))], [a, b], full, "%e"))
    results, res_types = [values[-1]], [full]
    kind = rng.random()
    if len(shape) > 1 and kind < 0.7:
        # a sum over one axis and an op on the row values; then (sometimes) a normalisation by it, or a second sum
        # over values centred by the first -- the shape of a layer normalisation: a row statistic with two readers
        axis = len(shape) - 1 if kind < 0.5 else 0
        kept = [d for i, d in enumerate(shape) if i != axis]
        row = _t(kept, dt)
        lines.append("%er = tensor.empty() : " + row)
        lines.append("%c0 = arith.constant 0.0 : " + dt)
        lines.append("%z = linalg.fill ins(%c0 : " + dt + ") outs(%er : " + row + ") -> " + row)
        lines.append("%one = arith.constant dense<1.000000e+00> : " + row)

        def rowsum(v):
            nonlocal n
            n += 1
            name = "%s" + str(n)
            lines.append(name + " = linalg.reduce { arith.addf } ins(" + v + " : " + full + ") outs(%z : " + row + ") dimensions = [" +
                         str(axis) + "]")
            return name

        def spread(v):
            nonlocal n
            n += 1
            name = "%b" + str(n)
            lines.append(name + " = linalg.broadcast ins(" + v + " : " + row + ") outs(%e : " + full + ") dimensions = [" + str(axis) + "]")
            return name

        s1 = emit("add", [rowsum(values[-1]), "%one"], row, "%er")
        results, res_types = [s1], [row]
        form = rng.random()
        if form < 0.45:
            nrm = emit("div", [values[-1], spread(s1)], full, "%e")
            if rng.random() < 0.5:
                nrm = emit("mul", [nrm, "%rb"], full, "%e")
            results, res_types = [nrm], [full]
            if rng.random() < 0.5:
                results, res_types = [s1, nrm], [row, full]
        elif form < 0.85:
            centred = emit("sub", [values[-1], spread(s1)], full, "%e")
            spreadsq = emit(["square", "abs"][int(rng.integers(2))], [centred], full, "%e")
            s2 = emit("add", [rowsum(spreadsq), "%one"], row, "%er")
            if rng.random() < 0.5:
                s2 = emit("sqrt", [s2], row, "%er")
            out = emit("div", [centred, spread(s2)], full, "%e")
            if rng.random() < 0.5:
                out = emit("add", [emit("mul", [out, "%rb"], full, "%e"), "%rb"], full, "%e")
            results, res_types = [out], [full]
            pick = rng.random()
            if pick < 0.25:
                results, res_types = [s2, out], [row, full]
            elif pick < 0.4:
                results, res_types = [s1, out], [row, full]
    sig = ", ".join(a + ": " + _t(s, dt) for a, s in args)
    ret = ", ".join(results) + " : " + ", ".join(res_types)
    text = ("func.func @f(" + sig + ") -> (" + ", ".join(res_types) + ") {\n  " + "\n  ".join(lines) + "\n  return " + ret + "\n}")
    shapes_of = {full: list(shape)}
    if len(shape) > 1:
        shapes_of[_t([d for i, d in enumerate(shape) if i != len(shape) - 1], dt)] = list(shape[:-1])
        shapes_of[_t(list(shape[1:]), dt)] = list(shape[1:])
    return text, [s for _, s in args], [shapes_of[t] for t in res_types]


T_UNARY = {"abs": torch.abs, "ceil": torch.ceil, "floor": torch.floor, "negf": torch.neg, "exp": torch.exp, "tanh": torch.tanh,
           "square": lambda x: x * x, "erf": torch.erf, "sqrt": torch.sqrt, "rsqrt": torch.rsqrt, "log": torch.log,
           "reciprocal": torch.reciprocal,
           "round": lambda x: torch.where(x >= 0, torch.floor(x + 0.5), torch.ceil(x - 0.5))}  # halves away from zero
T_BINARY = {"add": torch.add, "sub": torch.sub, "mul": torch.mul, "div": torch.div,
            "max": lambda a, b: torch.where(torch.isnan(a) | torch.isnan(b), a + b, torch.maximum(a, b)),
            "min": lambda a, b: torch.where(torch.isnan(a) | torch.isnan(b), a + b, torch.minimum(a, b))}


def torch_reference(text, ins, td, shape):
    """The module of random_module(), line by line: f32 arithmetic, every op's result rounded to the storage type."""
    env = dict(zip(["%x", "%y", "%r", "%c"], [t.float() for t in ins]))
    env["%one"] = torch.ones((), device=ins[0].device)

    def rnd(v):
        return v.to(td).float()

    for line in text.splitlines():
        line = line.strip()
        m = re.match(r"(%\w+) = linalg\.(\w+)(?: \{ arith\.addf \})? ins\(([^:]+) :", line)
        if m and m.group(2) == "reduce":
            env[m.group(1)] = rnd(env[m.group(3).strip()].sum(int(re.search(r"dimensions = \[(\d+)\]", line).group(1))))
        elif m and m.group(2) == "broadcast":
            v = env[m.group(3).strip()]
            for d in sorted(int(d) for d in re.search(r"dimensions = \[([^\]]*)\]", line).group(1).split(",")):
                v = v.unsqueeze(d)
            env[m.group(1)] = v.expand(*shape)
        elif m and m.group(2) in T_UNARY:
            env[m.group(1)] = rnd(T_UNARY[m.group(2)](env[m.group(3).strip()]))
        elif m and m.group(2) in T_BINARY:
            a, b = [t.strip() for t in m.group(3).split(",")]
            env[m.group(1)] = rnd(T_BINARY[m.group(2)](env[a], env[b]))
        elif line.startswith("return"):
            return [env[n.strip()] for n in line[len("return"):].split(":")[0].split(",")]
    raise AssertionError("no return in the module")


def _run(ga, text, ins, outs):
    comp = ga.Compiler()
    try:
        st, exe = comp.compile_mlir(text)
        assert st == 0, "compile_mlir -> %d: %s\n%s" % (st, ga.api().dnnl_graph_compiler_last_error().decode(), text)
        try:
            assert exe.execute(ins, outs) == 0, ga.api().dnnl_graph_compiler_last_error().decode()
            torch.cuda.synchronize()
        finally:
            exe.close()
    finally:
        comp.close()


@pytest.mark.parametrize("seed", range(72))
def test_random_groups_generated_equals_library(ga, dev, monkeypatch, seed):
    rng = np.random.default_rng(1000 + seed)
    shape = SHAPES[seed % len(SHAPES)]
    dt = ["f32", "bf16", "f16"][(seed // len(SHAPES) + seed) % 3]
    td = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}[dt]
    text, arg_shapes, res_shapes = random_module(rng, shape, dt)
    torch.manual_seed(seed)
    ins = [((torch.rand(s, device=dev) - 0.4) * 3).to(td) for s in arg_shapes]
    runs = []
    for mode in ("generated", "library"):
        if mode == "library":
            monkeypatch.setenv("GCMI_NO_GENERATED_KERNELS", "1")
        else:
            monkeypatch.setenv("GCMI_GENERATED_KERNELS_REQUIRED", "1")
        before = ga.generated_kernel_launches()
        outs = [torch.full(s, 7.0, device=dev, dtype=td) for s in res_shapes]
        _run(ga, text, list(enumerate(ins)), [(len(ins) + j, o) for j, o in enumerate(outs)])
        assert (ga.generated_kernel_launches() > before) == (mode == "generated"), text
        runs.append(outs)
    bits = torch.int32 if dt == "f32" else torch.int16
    for a, b in zip(*runs):
        same = torch.equal(a.view(bits), b.view(bits))
        assert same, "%s\nfirst difference at %s" % (text, (a.view(bits) != b.view(bits)).nonzero()[:4].tolist())
    # against torch: one rounding of slack per op of the chain, libm-grade device functions
    tol = {"f32": 2e-4, "bf16": 3e-2, "f16": 4e-3}[dt]
    for got, ref in zip(runs[0], torch_reference(text, ins, td, list(shape))):
        got, ref = got.double(), ref.double().expand_as(got)
        assert torch.equal(torch.isnan(got), torch.isnan(ref)), text
        fin = torch.isfinite(ref) & torch.isfinite(got)
        rest = ~fin & ~torch.isnan(ref)
        assert torch.equal(got[rest], ref[rest]), text  # infinities, with their signs
        if fin.any():
            scale = torch.maximum(ref[fin].abs(), ref[fin].pow(2).mean().sqrt().clamp(max=1e300)).clamp(min=1e-30)
            err = ((got[fin] - ref[fin]).abs() / scale).max().item()
            assert err <= tol, "%s\nerror %g" % (text, err)
