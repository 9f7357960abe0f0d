"""ctypes face of libgraph_compiler_amd.so for tests and the benchmark.

The product is the shared library (C ABI declared in include/*.h).  This module
only loads it, declares the prototypes and offers thin helpers that pass torch
device tensors (torch is used for device memory and streams, nothing else).
There is no CPU fallback: a missing library or kernel is an error.

The directory name contains a hyphen, so load it by path, e.g.
    importlib.util.spec_from_file_location("graph_compiler_amd", ".../graph-compiler_amd/__init__.py")
"""
import ctypes as C
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libgraph_compiler_amd.so")

BF16, F32, S32, S8, U8, F16 = 2, 3, 4, 5, 6, 1
ACT = {None: 0, "none": 0, "relu": 1, "gelu_erf": 2, "gelu_tanh": 3, "sigmoid": 4}

# every symbol the public headers declare (checked by the CPU test-suite)
EXPORTS = {
    "gc_hip_kernels.h": ["gcmi_init", "gcmi_last_error", "gcmi_gemm_bf16", "gcmi_gemm_bf16_nt", "gcmi_gemm_bf16_batched", "gcmi_gemm_bf16_residual", "gcmi_gemm_f32_batched",
                         "gcmi_gemm_bf16_ws", "gcmi_gemm_bf16_workspace_bytes", "gcmi_gemm_bf16_workspace_bytes_cfg", "gcmi_mha_fwd_bf16_ws", "gcmi_mha_fwd_workspace_bytes", "gcmi_mha_classify_mask",
                         "gcmi_gemm_bf16_noalloc", "gcmi_noalloc_scratch_bytes", "gcmi_gemm_int8_cfg", "gcmi_gemm_tile_config_query",
                         "gcmi_gemm_int8", "gcmi_colsum_s8",
                         "gcmi_gemm_f32", "gcmi_mha_fwd_bf16", "gcmi_mha_fwd_bf16_opt"],
    "gc_brgemm.h": ["dnnl_brgemm_dispatch", "dnnl_brgemm_tileconfig", "dnnl_brgemm_tilerelease",
                    "dnnl_brgemm_execute"],
}


def build(jobs=8):
    """Compile the library in-tree with hipcc for gfx950 (always recompiles)."""
    subprocess.check_call(["make", "-C", os.path.join(_HERE, "csrc"), "-B", "-j%d" % jobs, "all"])


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("libgraph_compiler_amd.so is not built (%s); run __graft_entry__.build() -- "
                           "there is no CPU fallback" % LIB_PATH)
    L = C.CDLL(LIB_PATH)
    i64, u64, vp, ci, f32 = C.c_int64, C.c_uint64, C.c_void_p, C.c_int, C.c_float
    L.gcmi_init.restype = ci
    L.gcmi_init.argtypes = [ci]
    L.gcmi_last_error.restype = C.c_char_p
    L.gcmi_gemm_bf16.restype = ci
    L.gcmi_gemm_bf16.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, vp, ci, ci, ci, vp]
    L.gcmi_gemm_bf16_nt.restype = ci
    L.gcmi_gemm_bf16_batched.restype = ci
    L.gcmi_gemm_bf16_batched.argtypes = [vp, vp, vp] + [i64] * 10 + [ci, vp, ci, ci, ci, vp]
    L.gcmi_gemm_bf16_residual.restype = ci
    L.gcmi_gemm_bf16_residual.argtypes = [vp, vp, vp] + [i64] * 10 + [ci, vp, ci, ci, vp, i64, ci, ci, vp]
    L.gcmi_gemm_bf16_workspace_bytes.restype = C.c_size_t
    L.gcmi_gemm_bf16_workspace_bytes.argtypes = [i64, i64, i64, ci]
    L.gcmi_gemm_bf16_workspace_bytes_cfg.restype = C.c_size_t
    L.gcmi_gemm_bf16_workspace_bytes_cfg.argtypes = [i64, i64, i64, ci, C.POINTER(C.c_int64)]
    L.gcmi_gemm_bf16_ws.restype = ci
    L.gcmi_gemm_bf16_ws.argtypes = [vp, vp, vp] + [i64] * 10 + [ci, vp, ci, ci, vp, i64, ci, ci, vp, C.c_size_t, vp, vp]
    L.gcmi_gemm_int8_cfg.restype = ci
    L.gcmi_gemm_int8_cfg.argtypes = [vp, ci, vp, vp, i64, i64, i64, i64, i64, i64, vp, C.c_int32, vp, vp, ci, ci, vp, vp]
    L.gcmi_gemm_tile_config_query.restype = ci
    L.gcmi_gemm_tile_config_query.argtypes = [ci, i64, i64, i64, ci, ci, vp, vp, C.c_char_p, C.c_size_t]
    L.gcmi_mha_fwd_workspace_bytes.restype = C.c_size_t
    L.gcmi_mha_fwd_workspace_bytes.argtypes = [i64, i64, i64, ci]
    L.gcmi_mha_fwd_bf16_ws.restype = ci
    L.gcmi_mha_fwd_bf16_ws.argtypes = [vp, vp, vp, vp, i64, vp, i64, i64, i64, i64, f32, ci, vp, C.c_size_t, vp]
    L.gcmi_mha_classify_mask.restype = ci
    L.gcmi_mha_classify_mask.argtypes = [vp, i64, i64, i64, i64, vp, C.c_size_t, vp]
    L.gcmi_gemm_bf16_noalloc.restype = ci
    L.gcmi_gemm_bf16_noalloc.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, ci, vp, ci, ci, ci, vp]
    L.gcmi_noalloc_scratch_bytes.restype = C.c_size_t
    L.gcmi_noalloc_scratch_bytes.argtypes = []
    L.gcmi_gemm_f32_batched.restype = ci
    L.gcmi_gemm_f32_batched.argtypes = [vp, vp, vp] + [i64] * 10 + [ci, ci, vp, ci, vp]
    L.gcmi_gemm_bf16_nt.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, vp, ci, ci, ci, vp]
    L.gcmi_gemm_int8.restype = ci
    L.gcmi_gemm_int8.argtypes = [vp, ci, vp, vp, i64, i64, i64, i64, i64, i64, vp, C.c_int32, vp, vp, ci, ci, vp]
    L.gcmi_colsum_s8.restype = ci
    L.gcmi_colsum_s8.argtypes = [vp, i64, i64, i64, vp, vp]
    L.gcmi_gemm_f32.restype = ci
    L.gcmi_gemm_f32.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, ci, ci, vp, ci, vp]
    L.gcmi_mha_fwd_bf16.restype = ci
    L.gcmi_mha_fwd_bf16.argtypes = [vp, vp, vp, vp, i64, vp, i64, i64, i64, i64, f32, vp]
    L.gcmi_mha_fwd_bf16_opt.restype = ci
    L.gcmi_mha_fwd_bf16_opt.argtypes = [vp, vp, vp, vp, i64, vp, i64, i64, i64, i64, f32, ci, vp]
    L.dnnl_brgemm_dispatch.restype = i64
    L.dnnl_brgemm_dispatch.argtypes = [i64] * 8 + [f32, i64, i64]
    L.dnnl_brgemm_tileconfig.restype = None
    L.dnnl_brgemm_tileconfig.argtypes = [i64]
    L.dnnl_brgemm_tilerelease.restype = None
    L.dnnl_brgemm_tilerelease.argtypes = []
    L.dnnl_brgemm_execute.restype = None
    L.dnnl_brgemm_execute.argtypes = [i64, vp, u64, vp, u64, vp, u64, ci]
    _lib = L
    return L


class TileConfig(C.Structure):
    """gcmi_gemm_tile_config of include/gc_hip_kernels.h"""
    _fields_ = [(n, C.c_int32) for n in ("kernel", "bm", "bn", "kbytes", "stages", "waves_m", "waves_n", "wave_m", "wave_n",
                                         "mfma_m", "mfma_n", "mfma_k", "split_k", "group_m", "workgroups", "from_attrs")]


MATMUL_CONFIG_NAMES = ("MThreads", "NThreads", "KThreads", "MBlock", "NBlock", "KBlock", "innermostMBlock",
                       "innermostNBlock", "innermostKBlock")


def tile_config(M, N, K, a_dtype=BF16, trans_b=False, out_dtype=BF16, matmul_config=None):
    """What the launcher chooses for this GEMM (no GPU needed).  matmul_config: the nine MatmulConfig integers in
    MATMUL_CONFIG_NAMES order, or None.  Returns (TileConfig, note)."""
    c = TileConfig()
    note = C.create_string_buffer(200)
    arr = None if matmul_config is None else (C.c_int64 * 9)(*matmul_config)
    check(lib().gcmi_gemm_tile_config_query(a_dtype, M, N, K, int(trans_b), out_dtype, arr, C.byref(c), note, 200),
          "gcmi_gemm_tile_config_query")
    return c, note.value.decode()


class GcError(RuntimeError):
    pass


def check(rc, what=""):
    if rc != 0:
        raise GcError("%s failed with status %d: %s" % (what, rc, lib().gcmi_last_error().decode()))


def _stream():
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def gemm_bf16(A, B, bias=None, act=None, out_dtype=BF16, out=None):
    """A [M,K], B [K,N] torch.bfloat16 cuda tensors (row strides may exceed the row)."""
    import torch
    M, K = A.shape
    K2, N = B.shape
    assert K == K2 and (A.stride(1) == 1 or K == 1) and (B.stride(1) == 1 or N == 1)
    if out is None:
        out = torch.empty((M, N), device=A.device, dtype=torch.bfloat16 if out_dtype == BF16 else torch.float32)
    bdt = BF16
    if bias is not None:
        bdt = BF16 if bias.dtype == torch.bfloat16 else F32
    check(lib().gcmi_gemm_bf16(_ptr(A), _ptr(B), _ptr(out), M, N, K, A.stride(0) if M > 1 else K,
                               B.stride(0) if K > 1 else N, out.stride(0) if M > 1 else N, _ptr(bias), bdt,
                               ACT[act], out_dtype, _stream()), "gcmi_gemm_bf16")
    return out


def gemm_bf16_nt(A, Bt, bias=None, act=None, out_dtype=BF16, out=None):
    """A [M,K], Bt [N,K] (the weight as torch.nn.Linear stores it): A @ Bt.T without a transposed copy."""
    import torch
    M, K = A.shape
    N, K2 = Bt.shape
    assert K == K2 and (A.stride(1) == 1 or K == 1) and (Bt.stride(1) == 1 or K == 1)
    if out is None:
        out = torch.empty((M, N), device=A.device, dtype=torch.bfloat16 if out_dtype == BF16 else torch.float32)
    bdt = BF16
    if bias is not None:
        bdt = BF16 if bias.dtype == torch.bfloat16 else F32
    check(lib().gcmi_gemm_bf16_nt(_ptr(A), _ptr(Bt), _ptr(out), M, N, K, A.stride(0) if M > 1 else K,
                                  Bt.stride(0) if N > 1 else K, out.stride(0) if M > 1 else N, _ptr(bias), bdt,
                                  ACT[act], out_dtype, _stream()), "gcmi_gemm_bf16_nt")
    return out


def gemm_bf16_residual(A, B, residual, trans_b=False, bias=None, act=None, out_dtype=BF16, out=None):
    """act(A @ B + bias) + residual in one launch; B is [K,N], or [N,K] with trans_b.  residual: [M,N] bf16 or f32."""
    import torch
    M, K = A.shape
    N = B.shape[0] if trans_b else B.shape[1]
    assert B.shape[1 if trans_b else 0] == K and (A.stride(1) == 1 or K == 1) and (B.stride(1) == 1 or B.shape[1] == 1)
    assert tuple(residual.shape) == (M, N) and (residual.stride(1) == 1 or N == 1)
    if out is None:
        out = torch.empty((M, N), device=A.device, dtype=torch.bfloat16 if out_dtype == BF16 else torch.float32)
    bdt = BF16
    if bias is not None:
        bdt = BF16 if bias.dtype == torch.bfloat16 else F32
    rdt = BF16 if residual.dtype == torch.bfloat16 else F32
    check(lib().gcmi_gemm_bf16_residual(_ptr(A), _ptr(B), _ptr(out), 1, M, N, K, A.stride(0) if M > 1 else K,
                                        B.stride(0) if B.shape[0] > 1 else B.shape[1], out.stride(0) if M > 1 else N,
                                        0, 0, 0, int(trans_b), _ptr(bias), bdt, ACT[act],
                                        _ptr(residual), residual.stride(0) if M > 1 else N, rdt, out_dtype, _stream()),
          "gcmi_gemm_bf16_residual")
    return out


def gemm_batched(A, B, trans_b=False, bias=None, act=None, out=None):
    """A [batch, M, K]; B [batch, K, N] ([batch, N, K] with trans_b) or 2-D (shared by all batches); bf16 or f32."""
    import torch
    nb, M, K = A.shape
    Bm = B if B.dim() == 3 else B.unsqueeze(0)
    N = Bm.shape[1] if trans_b else Bm.shape[2]
    assert A.is_contiguous() and B.is_contiguous() and (Bm.shape[2] if trans_b else Bm.shape[1]) == K
    if out is None:
        out = torch.empty((nb, M, N), device=A.device, dtype=A.dtype)
    sb = 0 if B.dim() == 2 else Bm.shape[1] * Bm.shape[2]
    if A.dtype == torch.float32:
        check(lib().gcmi_gemm_f32_batched(_ptr(A), _ptr(B), _ptr(out), nb, M, N, K, K, Bm.shape[2], N, M * K, sb, M * N,
                                          0, int(trans_b), _ptr(bias), ACT[act], _stream()), "gcmi_gemm_f32_batched")
    else:
        bdt = BF16 if bias is None or bias.dtype == torch.bfloat16 else F32
        check(lib().gcmi_gemm_bf16_batched(_ptr(A), _ptr(B), _ptr(out), nb, M, N, K, K, Bm.shape[2], N, M * K, sb, M * N,
                                           int(trans_b), _ptr(bias), bdt, ACT[act], BF16, _stream()),
              "gcmi_gemm_bf16_batched")
    return out


def colsum_s8(W):
    import torch
    K, N = W.shape
    out = torch.empty((N,), device=W.device, dtype=torch.int32)
    check(lib().gcmi_colsum_s8(_ptr(W), K, N, W.stride(0) if K > 1 else N, _ptr(out), _stream()), "gcmi_colsum_s8")
    return out


def gemm_int8(A, W, colsum=None, zp_a=0, scale=None, bias=None, act=None, out_dtype=S32, out=None, matmul_config=None):
    """A [M,K] uint8 or int8, W [K,N] int8 cuda tensors.  matmul_config: the nine MatmulConfig integers, or None."""
    import torch
    M, K = A.shape
    K2, N = W.shape
    assert K == K2 and A.stride(1) == 1 and W.stride(1) == 1
    adt = U8 if A.dtype == torch.uint8 else S8
    odt = {S32: torch.int32, F32: torch.float32, BF16: torch.bfloat16}[out_dtype]
    if out is None:
        out = torch.empty((M, N), device=A.device, dtype=odt)
    if matmul_config is not None:
        arr = (C.c_int64 * 9)(*matmul_config)
        check(lib().gcmi_gemm_int8_cfg(_ptr(A), adt, _ptr(W), _ptr(out), M, N, K, A.stride(0) if M > 1 else K,
                                       W.stride(0) if K > 1 else N, out.stride(0) if M > 1 else N, _ptr(colsum), int(zp_a),
                                       _ptr(scale), _ptr(bias), ACT[act], out_dtype, arr, _stream()), "gcmi_gemm_int8_cfg")
        return out
    check(lib().gcmi_gemm_int8(_ptr(A), adt, _ptr(W), _ptr(out), M, N, K, A.stride(0) if M > 1 else K,
                               W.stride(0) if K > 1 else N, out.stride(0) if M > 1 else N, _ptr(colsum), int(zp_a),
                               _ptr(scale), _ptr(bias), ACT[act], out_dtype, _stream()), "gcmi_gemm_int8")
    return out


def gemm_f32(A, B, bias=None, act=None, trans_a=False, trans_b=False, out=None):
    """Stored A is [K,M] when trans_a else [M,K]; stored B is [N,K] when trans_b else [K,N]."""
    import torch
    if trans_a:
        K, M = A.shape
    else:
        M, K = A.shape
    if trans_b:
        N, K2 = B.shape
    else:
        K2, N = B.shape
    assert K == K2 and (A.stride(1) == 1 or K == 1) and (B.stride(1) == 1 or N == 1)
    if out is None:
        out = torch.empty((M, N), device=A.device, dtype=torch.float32)
    check(lib().gcmi_gemm_f32(_ptr(A), _ptr(B), _ptr(out), M, N, K, A.stride(0), B.stride(0), out.stride(0),
                              int(trans_a), int(trans_b), _ptr(bias), ACT[act], _stream()), "gcmi_gemm_f32")
    return out


def mha_fwd_bf16(Q, K, V, mask=None, scale=None, out=None, skip_masked=True):
    """Q [B,H,Sq,D], K,V [B,H,Sk,D] contiguous bf16; mask f32 [Sq,Sk] or None."""
    import torch
    Bn, H, Sq, D = Q.shape
    Sk = K.shape[2]
    assert Q.is_contiguous() and K.is_contiguous() and V.is_contiguous()
    if scale is None:
        scale = 1.0 / (D ** 0.5)
    if out is None:
        out = torch.empty_like(Q)
    mld = 0 if mask is None else mask.stride(0)
    check(lib().gcmi_mha_fwd_bf16_opt(_ptr(Q), _ptr(K), _ptr(V), _ptr(mask), mld, _ptr(out), Bn * H, Sq, Sk, D,
                                      float(scale), int(bool(skip_masked)), _stream()), "gcmi_mha_fwd_bf16")
    return out


def mha_mask_classes(mask, Sq, Sk, D):
    """The tile classes of a mask that stays the same between calls: one classification pass into a workspace the
    caller keeps (None: this shape uses no classes).  Pass it to mha_fwd_bf16_classified."""
    import torch
    n = lib().gcmi_mha_fwd_workspace_bytes(Sq, Sk, D, 1)
    if n == 0:
        return None
    ws = torch.empty(n, dtype=torch.uint8, device=mask.device)
    check(lib().gcmi_mha_classify_mask(_ptr(mask), mask.stride(0), Sq, Sk, D, _ptr(ws), n, _stream()), "gcmi_mha_classify_mask")
    return ws


def mha_fwd_bf16_classified(Q, K, V, mask, classes, scale=None, out=None, skip_masked=True):
    """mha_fwd_bf16 for a mask whose classes were prepared by mha_mask_classes (no classification pass per call)."""
    import torch
    Bn, H, Sq, D = Q.shape
    Sk = K.shape[2]
    assert Q.is_contiguous() and K.is_contiguous() and V.is_contiguous()
    if scale is None:
        scale = 1.0 / (D ** 0.5)
    if out is None:
        out = torch.empty_like(Q)
    flags = (1 if skip_masked else 0) | (2 if classes is not None else 0)
    check(lib().gcmi_mha_fwd_bf16_ws(_ptr(Q), _ptr(K), _ptr(V), _ptr(mask), mask.stride(0), _ptr(out), Bn * H, Sq, Sk, D,
                                     float(scale), flags, _ptr(classes), 0 if classes is None else classes.numel(), _stream()),
          "gcmi_mha_fwd_bf16_ws")
    return out
