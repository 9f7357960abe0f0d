"""numpy/ctypes face of the CPU oracle (oracle/gc_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg, always as the checker or the timed CPU baseline,
never by the shipped library.

The composite functions below restate, op by op and rounding point by rounding
point, what the reference's CPU pipeline computes for the partitions on the hot
path (citations are relative to the reference tree):

* f32 / bf16 MatMul(+bias)(+ReLU) : lib/gc/Transforms/OneDNNGraphToLinalg.cpp:
  421-499 (matmul, zero fill, bias broadcast + add), :355-358 (ReLU), deep-tile
  nest lib/gc/Transforms/DeepTileContractionOp.cpp:506-540, bf16 rounding after
  every bf16 op lib/gc/Transforms/Pipeline.cpp:79-95.
* int8 layer : legacy/core/src/ops/matmul_core.cpp:529-571 (compensation),
  legacy/core/src/compiler/ir/graph/quantization/quantize_op.cpp:259-277
  (dequantize), legacy/core/src/ops/gelu.cpp:72-133 (GELU).
* MHA : composition batch_matmul_transpose_b -> scale -> +mask -> softmax ->
  batch_matmul (test/benchgc/src/benchgc/linalg/matmul.py:29-32,65-68,
  test/benchgc/src/benchgc/linalg/softmax.py:28-32).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libgc_oracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libbrgemm_naive_ref.so")

BF16, F32, S8, U8 = 2, 3, 5, 6  # dnnl_data_type_t values


def build(force=False):
    """Compile the oracle (and oracle/_ref when the reference tree is there)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "all"])


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = C.CDLL(_LIB_PATH)
    i64, u64, f32, vp, ci = C.c_int64, C.c_uint64, C.c_float, C.c_void_p, C.c_int
    lib.gco_f32_to_bf16.restype = C.c_uint16
    lib.gco_f32_to_bf16.argtypes = [f32]
    lib.gco_bf16_to_f32.restype = f32
    lib.gco_bf16_to_f32.argtypes = [C.c_uint16]
    lib.gco_f32_to_bf16_array.argtypes = [vp, vp, i64]
    lib.gco_bf16_to_f32_array.argtypes = [vp, vp, i64]
    lib.gco_round_bf16_inplace.argtypes = [vp, i64]
    lib.gco_brgemm.restype = ci
    lib.gco_brgemm.argtypes = [i64] * 8 + [f32, i64, i64, vp, u64, vp, u64, vp, u64, ci]
    lib.gco_vnni_pack.restype = ci
    lib.gco_vnni_pack.argtypes = [vp, i64, i64, i64, ci, i64, i64, vp]
    lib.gco_validate_config.restype = ci
    lib.gco_validate_config.argtypes = [vp, i64, i64, i64, i64]
    lib.gco_default_config.argtypes = [i64, i64, i64, i64, vp]
    lib.gco_deep_tile_extents.argtypes = [vp, i64, i64, i64, vp]
    lib.gco_deep_tile_matmul.restype = ci
    lib.gco_deep_tile_matmul.argtypes = [vp, i64, i64, i64, i64, i64, vp, i64, vp, i64, vp, i64]
    lib.gco_bias_add.argtypes = [vp, vp, i64, i64, i64]
    lib.gco_relu.argtypes = [vp, i64]
    lib.gco_sigmoid.argtypes = [vp, i64]
    lib.gco_gelu_erf.argtypes = [vp, i64]
    lib.gco_gelu_tanh.argtypes = [vp, i64]
    lib.gco_colsum_s8.argtypes = [vp, i64, i64, i64, vp]
    lib.gco_dequant_comp.argtypes = [vp, i64, i64, i64, C.c_int32, vp, vp, vp, i64]
    lib.gco_softmax_rows.argtypes = [vp, i64, i64, i64]
    lib.gco_mha_bf16.restype = ci
    lib.gco_mha_bf16.argtypes = [vp, vp, vp, vp, f32, i64, i64, i64, i64, vp]
    lib.gco_compare_p2p.restype = i64
    lib.gco_compare_p2p.argtypes = [vp, vp, i64, f32, vp]
    lib.gco_compare_norm.restype = ci
    lib.gco_compare_norm.argtypes = [vp, vp, i64, f32, vp]
    lib.gco_compare_norm_rows.restype = i64
    lib.gco_compare_norm_rows.argtypes = [vp, vp, i64, i64, f32, vp]
    lib.gco_mha_f64.restype = ci
    lib.gco_mha_f64.argtypes = [vp, vp, vp, vp, C.c_double, i64, i64, i64, i64, ci, vp]
    lib.gco_num_threads.restype = ci
    return lib


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = _load()
    return _lib


def ref_lib():
    """The reference's own BrgemmNaive.cpp compiled into oracle/_ref, or None."""
    if not os.path.exists(_REF_PATH):
        return None
    r = C.CDLL(_REF_PATH)
    i64, u64, vp = C.c_int64, C.c_uint64, C.c_void_p
    r.dnnl_brgemm_dispatch.restype = i64
    r.dnnl_brgemm_dispatch.argtypes = [i64] * 8 + [C.c_float, i64, i64]
    r.dnnl_brgemm_execute.restype = None
    r.dnnl_brgemm_execute.argtypes = [i64, vp, u64, vp, u64, vp, u64, C.c_int]
    return r


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


# --------------------------------------------------------------------------- bf16
def f32_to_bf16(x):
    """RNE f32 -> bf16 bit patterns (uint16), NaN -> 0x7FC0."""
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().gco_f32_to_bf16_array(_p(x), _p(out), x.size)
    return out


def bf16_to_f32(h):
    h = _c(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().gco_bf16_to_f32_array(_p(h), _p(out), h.size)
    return out


def round_bf16(x):
    x = _c(x, np.float32).copy()
    lib().gco_round_bf16_inplace(_p(x), x.size)
    return x


# --------------------------------------------------------------------------- brgemm
def brgemm(M, N, K, LDA, LDB, LDC, stride_a, stride_b, beta, dtA, dtB, A, A_off, B, B_off, Cbuf, C_off, num):
    """In-place on Cbuf (numpy f32 / i32, flat).  Mirrors dnnl_brgemm_dispatch+execute."""
    rc = lib().gco_brgemm(M, N, K, LDA, LDB, LDC, stride_a, stride_b, float(beta), dtA, dtB,
                          _p(A), A_off, _p(B), B_off, _p(Cbuf), C_off, num)
    if rc:
        raise ValueError("unsupported dtype pair")
    return Cbuf


def vnni_pack(W, kb, nb):
    """W: 2-D array of 1- or 2-byte elements -> flat VNNI_MM2D blocked buffer."""
    W = np.ascontiguousarray(W)
    K, N = W.shape
    es = W.dtype.itemsize
    KO, NO = -(-K // kb), -(-N // nb)
    out = np.zeros(NO * KO * kb * nb, W.dtype)
    rc = lib().gco_vnni_pack(_p(W), K, N, N, es, kb, nb, _p(out))
    if rc:
        raise ValueError("bad vnni block")
    return out


def validate_config(cfg, M, N, K, num_threads=0):
    c = np.asarray(cfg, np.int64)
    return bool(lib().gco_validate_config(_p(c), M, N, K, num_threads))


def default_config(M, N, K, num_threads=1):
    c = np.zeros(9, np.int64)
    lib().gco_default_config(M, N, K, num_threads, _p(c))
    return c


def deep_tile_extents(cfg, M, N, K):
    c = np.asarray(cfg, np.int64)
    o = np.zeros(3, np.int64)
    lib().gco_deep_tile_extents(_p(c), M, N, K, _p(o))
    return tuple(int(v) for v in o)


_NP_OF = {F32: np.float32, BF16: np.uint16, S8: np.int8, U8: np.uint8}


def deep_tile_matmul(A, B, dtA, dtB, cfg=None, num_threads=None):
    """A [M,K], B [K,N] plain row-major (bf16 as uint16 patterns).
    Returns the accumulator-typed [M,N] result (f32 or s32)."""
    A = _c(A, _NP_OF[dtA])
    B = _c(B, _NP_OF[dtB])
    M, K = A.shape
    K2, N = B.shape
    assert K == K2
    if cfg is None:
        nt = num_threads or lib().gco_num_threads()
        # all threads on M when it splits evenly into 32-row blocks, else 1
        cfg = default_config(M, N, K, 1)
        mt = nt
        while mt > 1 and (M // cfg[6]) % mt:
            mt -= 1
        cfg[0] = mt
    cfg = np.asarray(cfg, np.int64)
    out = np.zeros((M, N), np.float32 if dtA in (F32, BF16) else np.int32)
    rc = lib().gco_deep_tile_matmul(_p(cfg), M, N, K, dtA, dtB, _p(A), K, _p(B), N, _p(out), N)
    if rc:
        raise ValueError("deep_tile_matmul failed rc=%d cfg=%s" % (rc, cfg.tolist()))
    return out


# --------------------------------------------------------------------------- post-ops
def bias_add(x, bias):
    x = _c(x, np.float32).copy()
    b = _c(bias, np.float32)
    M, N = x.shape
    lib().gco_bias_add(_p(x), _p(b), M, N, N)
    return x


def relu(x):
    x = _c(x, np.float32).copy()
    lib().gco_relu(_p(x), x.size)
    return x


def sigmoid(x):
    x = _c(x, np.float32).copy()
    lib().gco_sigmoid(_p(x), x.size)
    return x


def gelu(x, kind="erf"):
    x = _c(x, np.float32).copy()
    (lib().gco_gelu_erf if kind == "erf" else lib().gco_gelu_tanh)(_p(x), x.size)
    return x


def colsum_s8(W):
    W = _c(W, np.int8)
    K, N = W.shape
    out = np.zeros(N, np.int32)
    lib().gco_colsum_s8(_p(W), K, N, N, _p(out))
    return out


def dequant_comp(acc, zpA, colsum, scale):
    acc = _c(acc, np.int32)
    M, N = acc.shape
    cs = _c(colsum, np.int32)
    sc = _c(scale, np.float32)
    out = np.empty((M, N), np.float32)
    lib().gco_dequant_comp(_p(acc), M, N, N, int(zpA), _p(cs), _p(sc), _p(out), N)
    return out


def softmax_rows(x):
    x = _c(x, np.float32).copy()
    rows = int(np.prod(x.shape[:-1]))
    cols = x.shape[-1]
    lib().gco_softmax_rows(_p(x), rows, cols, cols)
    return x


# --------------------------------------------------------------------------- composites
def matmul_f32(A, B, bias=None, act=None, transpose_a=False, transpose_b=False, cfg=None):
    """f32 MatMul [+bias] [+ReLU/Sigmoid/GELU]; transposes are materialised
    first, as linalg.matmul_transpose_a/b index the same data."""
    A = np.asarray(A, np.float32)
    B = np.asarray(B, np.float32)
    if transpose_a:
        A = A.T
    if transpose_b:
        B = B.T
    y = deep_tile_matmul(A, B, F32, F32, cfg)
    if bias is not None:
        y = bias_add(y, bias)
    return _act(y, act)


def _act(y, act):
    if act in (None, "none"):
        return y
    if act == "relu":
        return relu(y)
    if act == "sigmoid":
        return sigmoid(y)
    if act == "gelu_erf":
        return gelu(y, "erf")
    if act == "gelu_tanh":
        return gelu(y, "tanh")
    raise ValueError(act)


def matmul_bf16(A16, B16, bias16=None, act=None, cfg=None):
    """bf16 MatMul [+bias] [+act] with the reference's rounding points:
    f32 accumulation over all of K, one rounding to bf16; then every bf16
    elementwise op = widen, f32 op, round (Pipeline.cpp:79-95).
    Inputs and result are uint16 bf16 patterns."""
    acc = deep_tile_matmul(A16, B16, BF16, BF16, cfg)
    y = round_bf16(acc)
    if bias16 is not None:
        y = round_bf16(bias_add(y, bf16_to_f32(bias16)))
    if act not in (None, "none"):
        y = round_bf16(_act(y, act))
    return f32_to_bf16(y)


def matmul_u8s8_acc(A8, W8, cfg=None):
    """Raw s32 accumulators of u8 x s8."""
    return deep_tile_matmul(A8, W8, U8, S8, cfg)


def int8_layer(A8, W8, scale, bias=None, zpA=128, act="gelu_erf", out_bf16=True, cfg=None):
    """u8 activations (zero point zpA) x s8 weights -> s32 -> compensation ->
    * scale[n] -> + bias[n] (f32) -> act (f32) -> bf16.  Returns (acc_s32, out)."""
    acc = matmul_u8s8_acc(A8, W8, cfg)
    x = dequant_comp(acc, zpA, colsum_s8(W8), scale)
    if bias is not None:
        x = bias_add(x, bias)
    x = _act(x, act)
    return acc, (f32_to_bf16(x) if out_bf16 else x)


def mlp_chain_bf16(x16, W1, W2, bias2):
    """h = relu(x W1) ; y = h W2 + bias2, all bf16 tensors."""
    h = matmul_bf16(x16, W1, None, "relu")
    return h, matmul_bf16(h, W2, bias2, None)


def mha_bf16(Q16, K16, V16, mask, scale):
    """Q,K,V: uint16 [B,H,S,D]; mask f32 [Sq,Sk] or None.  Returns uint16 [B,H,Sq,D]."""
    Q16 = _c(Q16, np.uint16)
    K16 = _c(K16, np.uint16)
    V16 = _c(V16, np.uint16)
    Bn, H, Sq, D = Q16.shape
    Sk = K16.shape[2]
    out = np.empty((Bn, H, Sq, D), np.uint16)
    m = None if mask is None else _c(mask, np.float32)
    rc = lib().gco_mha_bf16(_p(Q16), _p(K16), _p(V16), None if m is None else _p(m), float(scale),
                            Bn * H, Sq, Sk, D, _p(out))
    if rc:
        raise MemoryError
    return out


# --------------------------------------------------------------------------- compare
def compare_p2p(ref, res, thr):
    """benchgc point-to-point rule.  Returns (n_bad, max_d)."""
    ref = _c(ref, np.float32).ravel()
    res = _c(res, np.float32).ravel()
    md = C.c_float(0)
    bad = lib().gco_compare_p2p(_p(ref), _p(res), ref.size, float(thr), C.byref(md))
    return int(bad), float(md.value)


def compare_norm(ref, res, thr):
    """benchgc norm rule (test/benchgc/src/benchgc/arg/compare.py:41-57).  Returns (passed, l2)."""
    ref = _c(ref, np.float32).ravel()
    res = _c(res, np.float32).ravel()
    assert ref.size == res.size
    v = C.c_float(0)
    ok = lib().gco_compare_norm(_p(ref), _p(res), ref.size, float(thr), C.byref(v))
    return bool(ok), float(v.value)


def compare_norm_rows(ref, res, thr):
    """The norm rule per row of the last dim.  Returns (n_failing_rows, l2 per row)."""
    ref = _c(ref, np.float32)
    res = _c(res, np.float32)
    assert ref.shape == res.shape
    cols = ref.shape[-1]
    rows = ref.size // cols
    l2 = np.empty(rows, np.float32)
    bad = lib().gco_compare_norm_rows(_p(ref), _p(res), rows, cols, float(thr), _p(l2))
    return int(bad), l2


def mha_f64(Q16, K16, V16, mask, scale, round_p):
    """The attention composition in float64 (error attribution).  round_p: round the softmax weights to bf16 where the
    reference graph does.  Q,K,V: uint16 [B,H,S,D]; returns float64 [B,H,Sq,D], not rounded."""
    Q16 = _c(Q16, np.uint16)
    K16 = _c(K16, np.uint16)
    V16 = _c(V16, np.uint16)
    Bn, H, Sq, D = Q16.shape
    Sk = K16.shape[2]
    out = np.empty((Bn, H, Sq, D), np.float64)
    m = None if mask is None else _c(mask, np.float32)
    rc = lib().gco_mha_f64(_p(Q16), _p(K16), _p(V16), None if m is None else _p(m), float(scale),
                           Bn * H, Sq, Sk, D, 1 if round_p else 0, _p(out))
    if rc:
        raise MemoryError
    return out


def num_threads():
    return lib().gco_num_threads()
