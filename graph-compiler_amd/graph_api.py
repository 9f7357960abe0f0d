"""ctypes binding of the oneDNN-Graph compiler-backend C API (include/dnnl_graph_compiler.h)
and builders for the JSON partitions of the benchmark configurations.

The binding a maintainer of the reference would use is the C header itself;
this module exists so that the tests read like the reference's own API tests
(test/dnnl/TestApiBasic.cpp, test/dnnl/TestApiOps.cpp)."""
import ctypes as C
import json

import numpy as np

from . import lib, EXPORTS

EXPORTS["dnnl_graph_compiler.h"] = [
    "dnnl_graph_compiler_get_version", "dnnl_graph_compiler_create", "dnnl_graph_compiler_destroy",
    "dnnl_graph_compiler_compile", "dnnl_graph_compiler_destroy_executable", "dnnl_graph_compiler_execute",
    "dnnl_graph_compiler_execute_async", "dnnl_graph_compiler_explain", "dnnl_graph_compiler_last_error",
    "dnnl_graph_compiler_compile_mlir", "dnnl_graph_compiler_explain_mlir", "dnnl_graph_compiler_generated_source_mlir",
    "dnnl_graph_compiler_generated_kernel_launches"]

SUCCESS, OUT_OF_MEMORY, INVALID_ARGUMENTS, UNIMPLEMENTED, RUNTIME_ERROR, INVALID_GRAPH = 0, 1, 2, 3, 5, 7


class Version(C.Structure):
    class V(C.Structure):
        _fields_ = [("major", C.c_uint8), ("minor", C.c_uint8), ("patch", C.c_uint8), ("hash", C.c_char_p)]
    _fields_ = [("api_version", V), ("gc_version", V)]


class Context(C.Structure):
    _fields_ = [("num_threads", C.c_uint32)]


class Tensor(C.Structure):
    _fields_ = [("id", C.c_size_t), ("ndims", C.c_uint8), ("dims", C.POINTER(C.c_int64)), ("data", C.c_void_p)]


_bound = False


def api():
    global _bound
    L = lib()
    if not _bound:
        L.dnnl_graph_compiler_get_version.restype = C.POINTER(Version)
        L.dnnl_graph_compiler_create.restype = C.c_int
        L.dnnl_graph_compiler_create.argtypes = [C.POINTER(Context), C.POINTER(C.c_void_p)]
        L.dnnl_graph_compiler_destroy.restype = None
        L.dnnl_graph_compiler_destroy.argtypes = [C.c_void_p]
        L.dnnl_graph_compiler_compile.restype = C.c_int
        L.dnnl_graph_compiler_compile.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_void_p)]
        L.dnnl_graph_compiler_destroy_executable.restype = None
        L.dnnl_graph_compiler_destroy_executable.argtypes = [C.c_void_p]
        L.dnnl_graph_compiler_execute.restype = C.c_int
        L.dnnl_graph_compiler_execute.argtypes = [C.c_void_p, C.POINTER(Tensor), C.POINTER(Tensor)]
        L.dnnl_graph_compiler_execute_async.restype = C.c_int
        L.dnnl_graph_compiler_execute_async.argtypes = [C.c_void_p, C.POINTER(Tensor), C.POINTER(Tensor), C.c_void_p]
        L.dnnl_graph_compiler_explain.restype = C.c_int
        L.dnnl_graph_compiler_explain.argtypes = [C.c_char_p, C.c_char_p, C.c_size_t]
        L.dnnl_graph_compiler_last_error.restype = C.c_char_p
        L.dnnl_graph_compiler_compile_mlir.restype = C.c_int
        L.dnnl_graph_compiler_compile_mlir.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_void_p)]
        L.dnnl_graph_compiler_explain_mlir.restype = C.c_int
        L.dnnl_graph_compiler_explain_mlir.argtypes = [C.c_char_p, C.c_char_p, C.c_size_t]
        L.dnnl_graph_compiler_generated_source_mlir.restype = C.c_int
        L.dnnl_graph_compiler_generated_source_mlir.argtypes = [C.c_char_p, C.c_char_p, C.c_char_p, C.c_size_t]
        L.dnnl_graph_compiler_generated_kernel_launches.restype = C.c_long
        L.dnnl_graph_compiler_generated_kernel_launches.argtypes = []
        _bound = True
    return L


def explain(graph_json):
    """(status, plan text or error text) from the host-side stages; needs no GPU."""
    buf = C.create_string_buffer(1 << 16)
    st = api().dnnl_graph_compiler_explain(graph_json.encode(), buf, len(buf))
    return st, (buf.value.decode() if st == 0 else api().dnnl_graph_compiler_last_error().decode())


def explain_mlir(module_text):
    """explain() for a module in MLIR's textual form."""
    buf = C.create_string_buffer(1 << 16)
    st = api().dnnl_graph_compiler_explain_mlir(module_text.encode(), buf, len(buf))
    return st, (buf.value.decode() if st == 0 else api().dnnl_graph_compiler_last_error().decode())


def generated_source_mlir(module_text, check_arch=None):
    """HIP source of the kernels that compile_mlir generates for the fused groups of a module; with check_arch
    ("gfx950") the source is also compiled (no GPU needed) and a failure is reported with the compiler's log."""
    buf = C.create_string_buffer(1 << 20)
    st = api().dnnl_graph_compiler_generated_source_mlir(module_text.encode(), check_arch.encode() if check_arch else None,
                                                         buf, len(buf))
    return st, (buf.value.decode() if st == 0 else api().dnnl_graph_compiler_last_error().decode())


def generated_kernel_launches():
    return api().dnnl_graph_compiler_generated_kernel_launches()


def _tensor(tid, arr):
    """arr: numpy array (host) or torch tensor (host or device)."""
    if isinstance(arr, np.ndarray):
        shape, ptr = arr.shape, arr.ctypes.data
    else:
        shape, ptr = tuple(arr.shape), arr.data_ptr()
    dims = (C.c_int64 * max(len(shape), 1))(*shape)
    return Tensor(tid, len(shape), dims, ptr), dims


class Compiler:
    def __init__(self, num_threads=None):
        self.h = C.c_void_p()
        ctx = None if num_threads is None else C.byref(Context(num_threads))
        st = api().dnnl_graph_compiler_create(ctx, C.byref(self.h))
        if st:
            raise RuntimeError("dnnl_graph_compiler_create -> %d" % st)

    def compile(self, graph_json):
        exe = C.c_void_p()
        st = api().dnnl_graph_compiler_compile(self.h, graph_json.encode(), C.byref(exe))
        return st, (Executable(exe) if st == 0 else None)

    def compile_mlir(self, module_text):
        """Function argument i has tensor id i, result j has id (number of arguments) + j."""
        exe = C.c_void_p()
        st = api().dnnl_graph_compiler_compile_mlir(self.h, module_text.encode(), C.byref(exe))
        return st, (Executable(exe) if st == 0 else None)

    def close(self):
        if self.h:
            api().dnnl_graph_compiler_destroy(self.h)
            self.h = None


class Executable:
    def __init__(self, h):
        self.h = h

    def execute(self, inputs, outputs):
        """inputs / outputs: lists of (id, array).  Returns the status."""
        keep = []

        def pack(items):
            arr = (Tensor * max(len(items), 1))()
            for i, (tid, a) in enumerate(items):
                t, dims = _tensor(tid, a)
                keep.append(dims)
                arr[i] = t
            return arr

        return api().dnnl_graph_compiler_execute(self.h, pack(inputs), pack(outputs))

    def bind(self, inputs, outputs, stream=None):
        """The tensor arrays for execute(), built once: bind(...)() is then the C call alone, which is what a C or
        C++ caller pays (building the ctypes structures for a dozen tensors costs more than a small module runs).
        With `stream` (a hipStream_t as an integer, e.g. torch.cuda.current_stream().cuda_stream) the call is
        execute_async on that stream: launches only, device tensors only."""
        keep = []

        def pack(items):
            arr = (Tensor * max(len(items), 1))()
            for i, (tid, a) in enumerate(items):
                t, dims = _tensor(tid, a)
                keep.append((dims, a))
                arr[i] = t
            return arr

        ins, outs, h = pack(inputs), pack(outputs), self.h
        if stream is None:
            fn = api().dnnl_graph_compiler_execute

            def call(_keep=keep):
                return fn(h, ins, outs)
        else:
            fn_async, sp = api().dnnl_graph_compiler_execute_async, C.c_void_p(stream)

            def call(_keep=keep):
                return fn_async(h, ins, outs, sp)
        return call

    def close(self):
        if self.h:
            api().dnnl_graph_compiler_destroy_executable(self.h)
            self.h = None


def run(graph_json, inputs, outputs):
    """create -> compile -> execute -> destroy, as test/dnnl/TestApiOps.cpp:27-38.  Returns (compile_st, execute_st)."""
    gc = Compiler()
    try:
        st, exe = gc.compile(graph_json)
        if st:
            return st, None
        try:
            return 0, exe.execute(inputs, outputs)
        finally:
            exe.close()
    finally:
        gc.close()


# --------------------------------------------------------------------------- JSON builders
def _t(tid, dtype, shape, **kw):
    d = {"id": tid, "dtype": dtype, "shape": list(shape)}
    d.update(kw)
    return d


def _graph(ops, inputs=None, outputs=None, engine="cpu"):
    g = {"version": "3.5.0", "engine_kind": engine, "fpmath_mode": "any"}
    if inputs is not None:
        g["input_ports"] = list(inputs)
    if outputs is not None:
        g["output_ports"] = list(outputs)
    g["graph"] = ops
    return json.dumps(g)


def matmul_bias_relu_json(M, K, N, dtype="f32"):
    """MatMul(+bias) -> ReLU: ids 0 A, 1 B, 2 bias -> 4."""
    return _graph([
        {"kind": "MatMul", "inputs": [_t(0, dtype, [M, K]), _t(1, dtype, [K, N]), _t(2, dtype, [N])],
         "outputs": [_t(3, dtype, [M, N])]},
        {"kind": "ReLU", "inputs": [_t(3, dtype, [M, N])], "outputs": [_t(4, dtype, [M, N])]}], [0, 1, 2], [4])


def gemm_json(M, K, N, dtype="bf16"):
    return _graph([{"kind": "MatMul", "inputs": [_t(0, dtype, [M, K]), _t(1, dtype, [K, N])],
                    "outputs": [_t(2, dtype, [M, N])]}], [0, 1], [2])


def int8_mlp_json(M, K, N, scale_a, zp_a, scales_w, out_dtype="bf16", act="GELU", weights_nk=False, weights_constant=True):
    """Dequantize(u8 A) , Dequantize(s8 W, per channel) -> MatMul(+bias f32) -> GELU -> Typecast.
    ids: 0 A u8, 1 W s8, 2 bias f32 -> 7 (or 6 when out_dtype is f32).  weights_nk: W is stored [N,K] and the MatMul
    has transpose_b (the layout of torch.nn.Linear)."""
    wshape = [N, K] if weights_nk else [K, N]
    wprop = {"property_type": "constant"} if weights_constant else {}
    ops = [
        {"kind": "Dequantize", "attrs": {"qtype": {"type": "string", "value": "per_tensor"},
                                         "scales": {"type": "f32[]", "value": [float(scale_a)]},
                                         "zps": {"type": "s64[]", "value": [int(zp_a)]}},
         "inputs": [_t(0, "u8", [M, K])], "outputs": [_t(3, "f32", [M, K])]},
        {"kind": "Dequantize", "attrs": {"qtype": {"type": "string", "value": "per_channel"},
                                         "axis": {"type": "s64", "value": 0 if weights_nk else 1},
                                         "scales": {"type": "f32[]", "value": [float(s) for s in scales_w]},
                                         "zps": {"type": "s64[]", "value": [0] * len(scales_w)}},
         "inputs": [_t(1, "s8", wshape, **wprop)], "outputs": [_t(4, "f32", wshape)]},
        dict({"kind": "MatMul", "inputs": [_t(3, "f32", [M, K]), _t(4, "f32", wshape), _t(2, "f32", [N])],
              "outputs": [_t(5, "f32", [M, N])]},
             **({"attrs": {"transpose_b": {"type": "bool", "value": 1}}} if weights_nk else {}))]
    last = 5
    if act:
        ops.append({"kind": act, "inputs": [_t(5, "f32", [M, N])], "outputs": [_t(6, "f32", [M, N])]})
        last = 6
    if out_dtype == "bf16":
        ops.append({"kind": "Typecast", "inputs": [_t(last, "f32", [M, N])], "outputs": [_t(last + 1, "bf16", [M, N])]})
        last += 1
    return _graph(ops, [0, 1, 2], [last]), last


def mlp_chain_json(M, K, H):
    """x W1 -> ReLU -> W2 + bias (bf16).  ids: 0 x, 1 W1, 4 W2, 5 bias -> 6."""
    return _graph([
        {"kind": "MatMul", "inputs": [_t(0, "bf16", [M, K]), _t(1, "bf16", [K, H])], "outputs": [_t(2, "bf16", [M, H])]},
        {"kind": "ReLU", "inputs": [_t(2, "bf16", [M, H])], "outputs": [_t(3, "bf16", [M, H])]},
        {"kind": "MatMul", "inputs": [_t(3, "bf16", [M, H]), _t(4, "bf16", [H, K]), _t(5, "bf16", [K])],
         "outputs": [_t(6, "bf16", [M, K])]}], [0, 1, 4, 5], [6])


def mha_json(B, H, Sq, Sk, D, with_mask=True, scale_op="Multiply", mask_constant=False):
    """MatMul(Q,K^T) -> Multiply(scale) -> Add(mask) -> SoftMax -> MatMul(P,V).
    ids: 0 Q, 1 K, 2 scale f32[1], 3 mask f32[Sq,Sk], 4 V -> 9.  mask_constant: the mask is a constant of the
    partition (property_type "constant"): its contents are taken from the first execute."""
    s = [B, H, Sq, Sk]
    ops = [{"kind": "MatMul", "attrs": {"transpose_b": {"type": "bool", "value": 1}},
            "inputs": [_t(0, "bf16", [B, H, Sq, D]), _t(1, "bf16", [B, H, Sk, D])], "outputs": [_t(5, "f32", s)]},
           {"kind": scale_op, "inputs": [_t(5, "f32", s), _t(2, "f32", [1])], "outputs": [_t(6, "f32", s)]}]
    cur = 6
    ins = [0, 1, 2]
    if with_mask:
        mk = {"property_type": "constant"} if mask_constant else {}
        ops.append({"kind": "Add", "inputs": [_t(6, "f32", s), _t(3, "f32", [Sq, Sk], **mk)], "outputs": [_t(7, "f32", s)]})
        cur = 7
        ins.append(3)
    ops.append({"kind": "SoftMax", "attrs": {"axis": {"type": "s64", "value": -1}},
                "inputs": [_t(cur, "f32", s)], "outputs": [_t(8, "bf16", s)]})
    ops.append({"kind": "MatMul", "inputs": [_t(8, "bf16", s), _t(4, "bf16", [B, H, Sk, D])],
                "outputs": [_t(9, "bf16", [B, H, Sq, D])]})
    ins.append(4)
    return _graph(ops, ins, [9])
