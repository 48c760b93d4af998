"""The C-ABI library loads and exports exactly what include/dxhip.h declares (no GPU, no compute)."""
import ctypes as C
import os
import re

from deepx_amd import lib as dx

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared():
    text = open(os.path.join(ROOT, "include", "dxhip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"DXH_API\s+(?:const\s+)?\w+\s*\*?\s*(dxh_\w+)\s*\(", text))


def test_header_matches_python_signatures():
    d = declared()
    assert d, "no declarations parsed"
    assert d == set(dx.SIGNATURES), (d ^ set(dx.SIGNATURES))


def test_library_exports_every_declared_symbol():
    L = dx.load()  # raises if the library is not built or a symbol is missing
    for name in declared():
        assert hasattr(L, name), name
    assert L.dxh_version() >= 100
    assert L.dxh_error_string(-1).decode().startswith("dtype")
    assert L.dxh_error_string(0).decode() == "ok"


def test_argument_errors_need_no_gpu():
    L = dx.load()
    # validation happens before any HIP call
    assert L.dxh_add(dx.F32, None, None, None, -5, None) == -2
    assert L.dxh_add(dx.F32, None, None, None, 0, None) == 0
    assert L.dxh_add(0x4000, C.c_void_p(16), C.c_void_p(16), C.c_void_p(16), 4, None) == -1
    assert L.dxh_tan(dx.BF16, C.c_void_p(16), C.c_void_p(16), 4, None) == -1
    assert L.dxh_transpose(dx.F32, C.c_void_p(16), dx.i32arr([2, 3]), 2, dx.i32arr([1, 1]), C.c_void_p(16), None) == -2
    assert L.dxh_broadcastTo(dx.F32, C.c_void_p(16), dx.i32arr([2, 3]), 2, dx.i32arr([5, 3]), 2, C.c_void_p(16), None) == -3
    n = C.c_size_t(7)
    assert L.dxh_reduce_workspace_bytes(dx.F32, dx.i32arr([8192, 8192]), 2, dx.i32arr([1]), 1, C.byref(n)) == 0 and n.value == 0
    assert L.dxh_reduce_workspace_bytes(dx.F32, dx.i32arr([8192, 8192]), 2, dx.i32arr([0]), 1, C.byref(n)) == 0 and n.value > 0
    assert L.dxh_reduce_workspace_bytes(dx.F32, dx.i32arr([8192, 8192]), 2, dx.i32arr([2]), 1, C.byref(n)) == -2
    assert L.dxh_matmul(dx.BOOL, None, None, None, 1, 2, 2, 2, None) == -1
