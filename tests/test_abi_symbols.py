"""CPU: the C-ABI library loads and exports every symbol include/*.h declares."""
import ctypes
import os
import re

from conftest import ROOT


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b((?:gcmi|dnnl_brgemm|dnnl_graph_compiler|mlir)\w*)\s*\(", text)
    return sorted(set(names))


def test_library_exports_every_declared_symbol(gc):
    assert os.path.exists(gc.LIB_PATH), "library not built: run __graft_entry__.build()"
    lib = ctypes.CDLL(gc.LIB_PATH)
    headers = [h for h in os.listdir(os.path.join(ROOT, "include")) if h.endswith(".h")]
    gc_c = os.path.join(ROOT, "include", "gc-c")
    if os.path.isdir(gc_c):
        headers += [os.path.join("gc-c", h) for h in os.listdir(gc_c) if h.endswith(".h")]
    assert headers
    total = 0
    for h in headers:
        for name in _declared(h):
            assert hasattr(lib, name), "%s declares %s but the library does not export it" % (h, name)
            total += 1
    assert total >= 11


def test_python_prototypes_cover_headers(gc):
    for header, names in gc.EXPORTS.items():
        declared = _declared(header)
        for n in names:
            assert n in declared, (header, n)


def test_validation_errors_need_no_gpu(gc):
    """Argument checks run before any HIP call."""
    L = gc.lib()
    assert L.gcmi_gemm_bf16(None, None, None, 4, 4, 4, 4, 4, 4, None, 2, 0, 2, None) == 2
    assert b"null" in L.gcmi_last_error()
    assert L.gcmi_gemm_bf16(None, None, None, -1, 4, 4, 4, 4, 4, None, 2, 0, 2, None) == 2
    assert L.gcmi_gemm_bf16(None, None, None, 0, 4, 4, 4, 4, 4, None, 2, 0, 2, None) == 0  # empty: nothing to do
    assert L.gcmi_mha_fwd_bf16(None, None, None, None, 0, None, 1, 8, 8, 96, 1.0, None) == 3  # head_dim 96 not built
    assert L.gcmi_gemm_int8(None, 3, None, None, 4, 4, 4, 4, 4, 4, None, 0, None, None, 0, 4, None) == 2
    assert L.dnnl_brgemm_dispatch(4, 4, 4, 4, 4, 4, 16, 16, 0.0, 3, 2) == -1  # f32 x bf16 is not a pair
    h = L.dnnl_brgemm_dispatch(4, 4, 4, 4, 4, 4, 16, 16, 0.0, 3, 3)
    h2 = L.dnnl_brgemm_dispatch(4, 4, 4, 4, 4, 4, 16, 16, 1.0, 2, 2)
    assert h >= 0 and h2 == h + 1  # dense, increasing handles
