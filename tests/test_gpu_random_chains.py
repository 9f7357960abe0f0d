"""GPU: seeded random matmul chains through compile_mlir against an op-by-op torch evaluation (f32 arithmetic, every
op's result rounded to the storage type): a matmul with its weight stored either way, then in random order and
presence a bias, an activation, a view to [1,M,N] and a residual add, a few point-wise ops with a second operand,
and sometimes a second matmul.  This is the planner's matching pass under test -- what goes into a GEMM epilogue, in
which order, and what stays a kernel of its own must not change the values."""
import importlib
import re

import numpy as np
import pytest
import torch

from conftest import assert_close

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ga(gc, dev):
    return importlib.import_module("graph_compiler_amd.graph_api")


def _t(shape, dt):
    return "tensor<" + "".join("%dx" % d for d in shape) + dt + ">"


def random_chain(rng, dt):
    M = int(rng.choice([32, 100, 256]))
    K = int(rng.choice([64, 256]))
    N = int(rng.choice([128, 200, 512]))
    nt = bool(rng.integers(2))
    args = [("%a", [M, K]), ("%w", [N, K] if nt else [K, N]), ("%b", [N]), ("%x", [1, M, N]), ("%y", [M, N])]
    mt, t3 = _t([M, N], dt), _t([1, M, N], dt)
    lines = ["%z = arith.constant 0.0 : " + dt, "%e = tensor.empty() : " + mt, "%e3 = tensor.empty() : " + t3,
             "%f = linalg.fill ins(%z : " + dt + ") outs(%e : " + mt + ") -> " + mt,
             "%bb = linalg.broadcast ins(%b : " + _t([N], dt) + ") outs(%e : " + mt + ") dimensions = [0]"]
    n = 0

    def emit(text):
        nonlocal n
        n += 1
        lines.append("%v" + str(n) + " = " + text)
        return "%v" + str(n)

    def binary(op, p, q, ty=mt, outs="%e"):
        return emit("linalg." + op + " ins(" + p + ", " + q + " : " + ty + ", " + ty + ") outs(" + outs + " : " + ty + ") -> " + ty)

    cur = emit("linalg." + ("matmul_transpose_b" if nt else "matmul") + " ins(%a, %w : " + _t([M, K], dt) + ", " +
               _t(args[1][1], dt) + ") outs(%f : " + mt + ") -> " + mt)
    steps = ["bias", "act", "residual", "pointwise"]
    rng.shuffle(steps)
    for s in steps:
        if rng.random() < 0.35:
            continue
        if s == "bias":
            cur = binary("add", cur, "%bb") if rng.random() < 0.5 else binary("add", "%bb", cur)
        elif s == "act":
            cur = binary("max", cur, "%f") if rng.random() < 0.6 else emit(
                "linalg.tanh ins(" + cur + " : " + mt + ") outs(%e : " + mt + ") -> " + mt)
        elif s == "residual":
            if rng.random() < 0.5:
                v = emit("tensor.expand_shape " + cur + " [[0, 1], [2]] output_shape [1, " + str(M) + ", " + str(N) + "] : " + mt +
                         " into " + t3)
                v = binary("add", "%x", v, t3, "%e3")
                cur = emit("tensor.collapse_shape " + v + " [[0, 1], [2]] : " + t3 + " into " + mt)
            else:
                cur = binary("add", cur, "%y")
        else:
            for _ in range(int(rng.integers(1, 4))):
                op = ["mul", "sub", "add", "max"][int(rng.integers(4))]
                cur = binary(op, cur, "%y") if rng.random() < 0.7 else binary(op, cur, cur)
    res_shape = [M, N]
    if rng.random() < 0.4:
        N2 = int(rng.choice([64, 256]))
        args.append(("%w2", [N, N2]))
        o2 = _t([M, N2], dt)
        lines.append("%e2 = tensor.empty() : " + o2)
        lines.append("%f2 = linalg.fill ins(%z : " + dt + ") outs(%e2 : " + o2 + ") -> " + o2)
        cur = emit("linalg.matmul ins(" + cur + ", %w2 : " + mt + ", " + _t([N, N2], dt) + ") outs(%f2 : " + o2 + ") -> " + o2)
        res_shape = [M, N2]
    sig = ", ".join(a + ": " + _t(s, dt) for a, s in args)
    rt = _t(res_shape, dt)
    text = "func.func @f(" + sig + ") -> " + rt + " {\n  " + "\n  ".join(lines) + "\n  return " + cur + " : " + rt + "\n}"
    return text, [s for _, s in args], res_shape, [a for a, _ in args]


def torch_reference(text, env, td):
    def rnd(v):
        return v.to(td).float()

    binary = {"add": torch.add, "sub": torch.sub, "mul": torch.mul,
              "max": lambda p, q: torch.where(torch.isnan(p) | torch.isnan(q), p + q, torch.maximum(p, q))}
    for line in text.splitlines():
        line = line.strip()
        m = re.match(r"(%\w+) = linalg\.(\w+) ins\(([^:]+) :", line)
        v = re.match(r"(%\w+) = tensor\.(expand|collapse)_shape (%\w+)", line)
        if m and m.group(2) == "fill":
            env[m.group(1)] = torch.zeros((), device=env["%a"].device)
        elif m and m.group(2) == "broadcast":
            env[m.group(1)] = env[m.group(3).strip()]  # a row vector: torch broadcasts it the same way
        elif m and m.group(2) in ("matmul", "matmul_transpose_b"):
            p, q = [env[t.strip()] for t in m.group(3).split(",")]
            env[m.group(1)] = rnd(p @ (q.t() if m.group(2).endswith("_b") else q))
        elif m and m.group(2) == "tanh":
            env[m.group(1)] = rnd(torch.tanh(env[m.group(3).strip()]))
        elif m and m.group(2) in binary:
            p, q = [env[t.strip()] for t in m.group(3).split(",")]
            env[m.group(1)] = rnd(binary[m.group(2)](p, q))
        elif v:
            src = env[v.group(3)]
            env[v.group(1)] = src.unsqueeze(0) if v.group(2) == "expand" else src.squeeze(0)
        elif line.startswith("return"):
            return env[line.split()[1]]
    raise AssertionError("no return in the module")


@pytest.mark.parametrize("mode", ["generated", "library"])
@pytest.mark.parametrize("seed", range(40))
def test_random_matmul_chains_against_torch(ga, dev, monkeypatch, seed, mode):
    monkeypatch.setenv("GCMI_NO_GENERATED_KERNELS" if mode == "library" else "GCMI_GENERATED_KERNELS_REQUIRED", "1")
    rng = np.random.default_rng(5000 + seed)
    dt = "bf16" if seed % 3 else "f32"
    td = torch.bfloat16 if dt == "bf16" else torch.float32
    text, arg_shapes, res_shape, names = random_chain(rng, dt)
    torch.manual_seed(seed)
    ins = [(torch.randn(s, device=dev) * (0.3 if len(s) == 2 and i in (1, 5) else 1.0)).to(td) for i, s in enumerate(arg_shapes)]
    out = torch.full(res_shape, 7.0, device=dev, dtype=td)
    comp = ga.Compiler()
    try:
        st, exe = comp.compile_mlir(text)
        assert st == 0, "compile_mlir -> %d: %s\n%s" % (st, ga.api().dnnl_graph_compiler_last_error().decode(), text)
        try:
            assert exe.execute(list(enumerate(ins)), [(len(ins), out)]) == 0, ga.api().dnnl_graph_compiler_last_error().decode()
            torch.cuda.synchronize()
        finally:
            exe.close()
    finally:
        comp.close()
    ref = torch_reference(text, {n: t.float() for n, t in zip(names, ins)}, td)
    st, plan = ga.explain_mlir(text)
    # bf16: one rounding per op of the chain on either side, and the MFMA's summation order against torch's
    assert_close(ref.double().cpu().numpy(), out.double().cpu().numpy(), 3e-2 if dt == "bf16" else 2e-4,
                 "chain\n" + text + "\n" + plan)
