"""Builders for modules in MLIR's textual form, in the shapes the reference's benchgc feeds to its
compiler: the MLP pattern (test/benchgc/src/benchgc/pattern/mlp.py) and a decoder MLP block with
RMSNorm and a gated feed-forward (the structure of test/benchgc/cases/llama2.mlir).  The text goes to
dnnl_graph_compiler_compile_mlir; argument i of the function has tensor id i, result j has id
(number of arguments) + j."""


class _Fn:
    """Collects SSA lines; every helper returns the name of the value it defines."""

    def __init__(self):
        self.lines = []
        self.n = 0

    def new(self):
        self.n += 1
        return "%%v%d" % self.n

    def emit(self, text):
        name = self.new()
        self.lines.append("    %s = %s" % (name, text))
        return name


def ttype(shape, dtype):
    return "tensor<%s%s>" % ("".join("%dx" % d for d in shape), dtype)


def _empty(f, shape, dtype):
    return f.emit("tensor.empty() : %s" % ttype(shape, dtype))


def _zeros(f, shape, dtype):
    c = f.emit("arith.constant 0.000000e+00 : %s" % dtype)
    e = _empty(f, shape, dtype)
    t = ttype(shape, dtype)
    return f.emit("linalg.fill ins(%s : %s) outs(%s : %s) -> %s" % (c, dtype, e, t, t))


def _splat(f, value, shape, dtype):
    return f.emit("arith.constant dense<%e> : %s" % (value, ttype(shape, dtype)))


def _named(f, op, ins, in_types, out_shape, dtype, tail=""):
    e = _empty(f, out_shape, dtype)
    t = ttype(out_shape, dtype)
    return f.emit("linalg.%s ins(%s : %s) outs(%s : %s)%s -> %s" % (op, ", ".join(ins), ", ".join(in_types), e, t, tail, t))


def _binary(f, op, a, b, shape, dtype):
    t = ttype(shape, dtype)
    return _named(f, op, [a, b], [t, t], shape, dtype)


def _matmul(f, op, a, a_shape, b, b_shape, out_shape, dtype):
    z = _zeros(f, out_shape, dtype)
    t = ttype(out_shape, dtype)
    return f.emit("linalg.%s ins(%s, %s : %s, %s) outs(%s : %s) -> %s" % (
        op, a, b, ttype(a_shape, dtype), ttype(b_shape, dtype), z, t, t))


def _broadcast(f, src, src_shape, out_shape, dims, dtype):
    e = _empty(f, out_shape, dtype)
    return f.emit("linalg.broadcast ins(%s : %s) outs(%s : %s) dimensions = [%s]" % (
        src, ttype(src_shape, dtype), e, ttype(out_shape, dtype), ", ".join(str(d) for d in dims)))


def _module(args, results, f, ret):
    sig = ", ".join("%%arg%d: %s" % (i, t) for i, t in enumerate(args))
    res = results[0] if len(results) == 1 else "(" + ", ".join(results) + ")"
    head = "  func.func @entry(%s) -> %s attributes {llvm.emit_c_interface} {" % (sig, res)
    tail = "    return %s : %s\n  }\n}" % (", ".join(ret), ", ".join(results))
    return "module {\n" + head + "\n" + "\n".join(f.lines) + "\n" + tail + "\n"


def mlp(batch, hidden, has_bias=None, act="noop", dtype="f32"):
    """benchgc's MLP pattern: arguments are the source [batch, hidden[0]], then one weight
    [hidden[i], hidden[i+1]] per layer, then the biases of the layers that have one."""
    layers = len(hidden) - 1
    has_bias = list(has_bias) if has_bias is not None else [False] * layers
    assert len(has_bias) == layers and act in ("noop", "relu", "sigmoid")
    args = [ttype([batch, hidden[0]], dtype)]
    args += [ttype([hidden[i], hidden[i + 1]], dtype) for i in range(layers)]
    args += [ttype([hidden[i + 1]], dtype) for i in range(layers) if has_bias[i]]
    f = _Fn()
    data, bias_idx = "%arg0", layers + 1
    for i in range(layers):
        shape = [batch, hidden[i + 1]]
        data = _matmul(f, "matmul", data, [batch, hidden[i]], "%%arg%d" % (i + 1), [hidden[i], hidden[i + 1]], shape, dtype)
        if has_bias[i]:
            bc = _broadcast(f, "%%arg%d" % bias_idx, [hidden[i + 1]], shape, [0], dtype)
            bias_idx += 1
            data = _binary(f, "add", data, bc, shape, dtype)
        if act == "relu":
            data = _binary(f, "max", data, _splat(f, 0.0, shape, dtype), shape, dtype)
        elif act == "sigmoid":
            t = ttype(shape, dtype)
            one = _splat(f, 1.0, shape, dtype)
            neg = _named(f, "negf", [data], [t], shape, dtype)
            ex = _named(f, "exp", [neg], [t], shape, dtype)
            data = _binary(f, "div", one, _binary(f, "add", one, ex, shape, dtype), shape, dtype)
    return _module(args, [ttype([batch, hidden[-1]], dtype)], f, [data])


def _rmsnorm(f, x, tokens, hidden, eps_arg, gamma_arg):
    """x: [1, tokens, hidden] bf16 -> gamma * bf16(x_f32 * (mean(x_f32^2) + eps)^-0.5)"""
    full, row = [1, tokens, hidden], [1, tokens]
    xf = _named(f, "copy", [x], [ttype(full, "bf16")], full, "f32")
    sq = f.emit("linalg.powf ins(%s, %s : %s, %s) outs(%s : %s) -> %s" % (
        xf, _splat(f, 2.0, full, "f32"), ttype(full, "f32"), ttype(full, "f32"), _empty(f, full, "f32"),
        ttype(full, "f32"), ttype(full, "f32")))
    z = _zeros(f, row, "f32")
    red = f.emit("linalg.reduce ins(%s : %s) outs(%s : %s) dimensions = [2]\n"
                 "      (%%in: f32, %%init: f32) {\n        %%s = arith.addf %%in, %%init : f32\n"
                 "        linalg.yield %%s : f32\n      }" % (sq, ttype(full, "f32"), z, ttype(row, "f32")))
    mean = _binary(f, "div", red, _splat(f, float(hidden), row, "f32"), row, "f32")
    col = [1, tokens, 1]
    mean3 = f.emit("tensor.expand_shape %s [[0], [1, 2]] output_shape [1, %d, 1] : %s into %s" % (
        mean, tokens, ttype(row, "f32"), ttype(col, "f32")))
    eps = _broadcast(f, eps_arg, [1], col, [0, 1], "f32")
    var = _binary(f, "add", mean3, eps, col, "f32")
    rs = f.emit("linalg.powf ins(%s, %s : %s, %s) outs(%s : %s) -> %s" % (
        var, _splat(f, -0.5, col, "f32"), ttype(col, "f32"), ttype(col, "f32"), _empty(f, col, "f32"),
        ttype(col, "f32"), ttype(col, "f32")))
    rs2 = f.emit("tensor.collapse_shape %s [[0], [1, 2]] : %s into %s" % (rs, ttype(col, "f32"), ttype(row, "f32")))
    rsb = _broadcast(f, rs2, row, full, [2], "f32")
    normed = _binary(f, "mul", xf, rsb, full, "f32")
    nb = _named(f, "copy", [normed], [ttype(full, "f32")], full, "bf16")
    g = _broadcast(f, gamma_arg, [hidden], full, [0, 1], "bf16")
    return _binary(f, "mul", g, nb, full, "bf16")


def rmsnorm(tokens, hidden):
    """The RMSNorm of test/benchgc/cases/llama2.mlir alone: (x [1,tokens,hidden] bf16, eps [1] f32, gamma [hidden]
    bf16) -> [1,tokens,hidden] bf16.  Tensor ids: arguments 0..2, the result 3."""
    f = _Fn()
    n = _rmsnorm(f, "%arg0", tokens, hidden, "%arg1", "%arg2")
    return _module([ttype([1, tokens, hidden], "bf16"), ttype([1], "f32"), ttype([hidden], "bf16")],
                   [ttype([1, tokens, hidden], "bf16")], f, [n])


def layernorm(rows, hidden, dtype="f32", eps=1e-5):
    """Layer normalisation over the last axis spelled with named linalg ops, two reductions: mean, then the variance
    of the centred values; (x [rows,hidden], gamma [hidden], beta [hidden]) -> [rows,hidden].  Ids 0..2, result 3."""
    full, col, vec = ttype([rows, hidden], dtype), ttype([rows], dtype), ttype([hidden], dtype)
    f = _Fn()
    e, er = _empty(f, [rows, hidden], dtype), _empty(f, [rows], dtype)
    z = _zeros(f, [rows], dtype)

    def op(name, ins, ty, outs):
        return f.emit("linalg.%s ins(%s : %s) outs(%s : %s) -> %s" % (name, ", ".join(ins), ", ".join([ty] * len(ins)), outs, ty, ty))

    def rowsum(v):
        return f.emit("linalg.reduce { arith.addf } ins(%s : %s) outs(%s : %s) dimensions = [1]" % (v, full, z, col))

    def along_row(v):
        return f.emit("linalg.broadcast ins(%s : %s) outs(%s : %s) dimensions = [1]" % (v, col, e, full))

    def along_col(v):
        return f.emit("linalg.broadcast ins(%s : %s) outs(%s : %s) dimensions = [0]" % (v, vec, e, full))

    n = _splat(f, float(hidden), [rows], dtype)
    mean = op("div", [rowsum("%arg0"), n], col, er)
    d = op("sub", ["%arg0", along_row(mean)], full, e)
    var = op("div", [rowsum(op("square", [d], full, e)), n], col, er)
    r = op("rsqrt", [op("add", [var, _splat(f, eps, [rows], dtype)], col, er)], col, er)
    y = op("mul", [op("mul", [d, along_row(r)], full, e), along_col("%arg1")], full, e)
    y = op("add", [y, along_col("%arg2")], full, e)
    return _module([full, vec, vec], [full], f, [y])


def decoder_mlp_block(tokens=32, hidden=4096, ffn=11008):
    """The second half of a llama-2 decoder layer, as test/benchgc/cases/llama2.mlir spells it:

        h   = residual + attn_out @ Wo^T
        n   = rmsnorm(h; eps, gamma1)
        out = h + (silu(n @ Wg^T) * (n @ Wu^T)) @ Wd^T
        return out, rmsnorm(out; eps2, gamma2)

    bf16 tensors, f32 inside the norms, weights stored [out_features, in_features].
    Arguments: 0 attn_out [1,T,H], 1 Wo [H,H], 2 residual [1,T,H], 3 eps [1] f32, 4 gamma1 [H],
    5 Wg [F,H], 6 Wu [F,H], 7 Wd [H,F], 8 eps2 [1] f32, 9 gamma2 [H].  Results: 10 out, 11 its norm."""
    T, H, F = tokens, hidden, ffn
    bt = "bf16"
    args = [ttype([1, T, H], bt), ttype([H, H], bt), ttype([1, T, H], bt), ttype([1], "f32"), ttype([H], bt),
            ttype([F, H], bt), ttype([F, H], bt), ttype([H, F], bt), ttype([1], "f32"), ttype([H], bt)]
    f = _Fn()

    def flat(v, n):
        return f.emit("tensor.collapse_shape %s [[0, 1], [2]] : %s into %s" % (v, ttype([1, T, n], bt), ttype([T, n], bt)))

    def unflat(v, n):
        return f.emit("tensor.expand_shape %s [[0, 1], [2]] output_shape [1, %d, %d] : %s into %s" % (
            v, T, n, ttype([T, n], bt), ttype([1, T, n], bt)))

    o = unflat(_matmul(f, "matmul_transpose_b", flat("%arg0", H), [T, H], "%arg1", [H, H], [T, H], bt), H)
    h = _binary(f, "add", "%arg2", o, [1, T, H], bt)
    n1 = _rmsnorm(f, h, T, H, "%arg3", "%arg4")
    gate = unflat(_matmul(f, "matmul_transpose_b", flat(n1, H), [T, H], "%arg5", [F, H], [T, F], bt), F)
    wide = [1, T, F]
    tw = ttype(wide, bt)
    one = _splat(f, 1.0, wide, bt)
    neg = _named(f, "negf", [gate], [tw], wide, bt)
    ex = _named(f, "exp", [neg], [tw], wide, bt)
    sig = _binary(f, "div", one, _binary(f, "add", one, ex, wide, bt), wide, bt)
    silu = _binary(f, "mul", sig, gate, wide, bt)
    up = unflat(_matmul(f, "matmul_transpose_b", flat(n1, H), [T, H], "%arg6", [F, H], [T, F], bt), F)
    act = _binary(f, "mul", silu, up, wide, bt)
    down = unflat(_matmul(f, "matmul_transpose_b", flat(act, F), [T, F], "%arg7", [H, F], [T, H], bt), H)
    out = _binary(f, "add", h, down, [1, T, H], bt)
    n2 = _rmsnorm(f, out, T, H, "%arg8", "%arg9")
    return _module(args, [ttype([1, T, H], bt)] * 2, f, [out, n2])


def generic_matmul(M, K, N, dtype="f32", transpose_b=False):
    """A matmul spelled as linalg.generic with indexing maps (test/benchgc/cases/generic.mlir)."""
    b_shape = [N, K] if transpose_b else [K, N]
    maps = ("#map = affine_map<(d0, d1, d2) -> (d0, d2)>\n"
            "#map1 = affine_map<(d0, d1, d2) -> (%s)>\n"
            "#map2 = affine_map<(d0, d1, d2) -> (d0, d1)>\n" % ("d1, d2" if transpose_b else "d2, d1"))
    f = _Fn()
    z = _zeros(f, [M, N], dtype)
    ta, tb, to = ttype([M, K], dtype), ttype(b_shape, dtype), ttype([M, N], dtype)
    r = f.emit('linalg.generic {indexing_maps = [#map, #map1, #map2], iterator_types = ["parallel", "parallel", "reduction"]} '
               "ins(%%arg0, %%arg1 : %s, %s) outs(%s : %s) {\n"
               "    ^bb0(%%in: %s, %%in_0: %s, %%out: %s):\n"
               "      %%p = arith.mulf %%in, %%in_0 : %s\n      %%s = arith.addf %%out, %%p : %s\n"
               "      linalg.yield %%s : %s\n    } -> %s" % (ta, tb, z, to, dtype, dtype, dtype, dtype, dtype, dtype, to))
    return maps + _module([ta, tb], [to], f, [r])


def attention(batch, seq, head_dim, scale, dtype="bf16"):
    """softmax(scale * Q K^T) V over [batch, seq, head_dim] operands, with named batch ops."""
    B, S, D = batch, seq, head_dim
    f = _Fn()
    qk = _matmul(f, "batch_matmul_transpose_b", "%arg0", [B, S, D], "%arg1", [B, S, D], [B, S, S], dtype)
    sc = _binary(f, "mul", qk, _splat(f, scale, [B, S, S], dtype), [B, S, S], dtype)
    e = _empty(f, [B, S, S], dtype)
    t = ttype([B, S, S], dtype)
    p = f.emit("linalg.softmax dimension(2) ins(%s : %s) outs(%s : %s) -> %s" % (sc, t, e, t, t))
    o = _matmul(f, "batch_matmul", p, [B, S, S], "%arg2", [B, S, D], [B, S, D], dtype)
    return _module([ttype([B, S, D], dtype)] * 3, [ttype([B, S, D], dtype)], f, [o])


def linalg_op(op, in_shapes, out_shape, dtype="f32"):
    """One named linalg op over the function's arguments, outs zero-filled: what benchgc's linalg driver builds
    (test/benchgc/src/benchgc/linalg/{eltwise,binary,matmul}.py)."""
    f = _Fn()
    z = _zeros(f, out_shape, dtype)
    ins = ["%%arg%d" % i for i in range(len(in_shapes))]
    types = [ttype(s, dtype) for s in in_shapes]
    to = ttype(out_shape, dtype)
    r = f.emit("linalg.%s ins(%s : %s) outs(%s : %s) -> %s" % (op, ", ".join(ins), ", ".join(types), z, to, to))
    return _module(types, [to], f, [r])
