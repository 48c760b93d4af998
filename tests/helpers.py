"""Shared test plumbing: the CPU oracle (ctypes), numpy<->device transfers, ulp distance.

The oracle is the checker only; nothing here is imported by the product.
"""
import ctypes as C
import os
import subprocess

import numpy as np

from deepx_amd import lib as dx

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_SO = os.path.join(ORACLE_DIR, "liboracle.so")

F64, F32, F16, BF16 = dx.F64, dx.F32, dx.F16, dx.BF16
I64, I32, I16, I8, BOOL = dx.I64, dx.I32, dx.I16, dx.I8, dx.BOOL

# storage numpy dtype per deepx dtype (16-bit floats travel as raw uint16 bit patterns)
NP = {F64: np.float64, F32: np.float32, F16: np.uint16, BF16: np.uint16,
      I64: np.int64, I32: np.int32, I16: np.int16, I8: np.int8, BOOL: np.uint8}
ALL_NUMERIC = [F64, F32, F16, BF16, I64, I32, I16, I8]
FLOATS = [F64, F32, F16, BF16]
INTS = [I64, I32, I16, I8]

_orc = None


def oracle():
    global _orc
    if _orc is None:
        if not os.path.exists(ORACLE_SO):
            subprocess.check_call(["make", "-C", ORACLE_DIR, "liboracle.so"])
        L = C.CDLL(ORACLE_SO)
        # the oracle mirrors the dxh_* signatures minus stream/workspace
        for name, (argtypes, restype) in dx.SIGNATURES.items():
            oname = "orc_" + name[4:]
            if not hasattr(L, oname):
                continue
            at = list(argtypes)
            if name in ("dxh_sum", "dxh_prod", "dxh_reducemax", "dxh_reducemin"):
                at = at[:7]
            elif name == "dxh_matmul":
                at = at[:8]  # no workspace, no stream
            else:
                at = at[:-1]  # drop the stream
            fn = getattr(L, oname)
            fn.argtypes = at
            fn.restype = restype
        L.orc_reduced_shape.argtypes = [C.POINTER(C.c_int32), C.c_int, C.POINTER(C.c_int32), C.c_int, C.c_int,
                                        C.POINTER(C.c_int32)]
        L.orc_faithful_reduce_f32.argtypes = [C.c_int, C.c_void_p, C.POINTER(C.c_int32), C.c_int,
                                              C.POINTER(C.c_int32), C.c_int, C.c_int, C.c_void_p]
        for name in ("transpose", "concat", "broadcastTo", "indexselect"):  # same arguments as the plain functions
            getattr(L, "orc_faithful_" + name).argtypes = getattr(L, "orc_" + name).argtypes
        L.orc_f32_to_bf16.argtypes = [C.c_float]; L.orc_f32_to_bf16.restype = C.c_uint16
        L.orc_f32_to_f16.argtypes = [C.c_float]; L.orc_f32_to_f16.restype = C.c_uint16
        L.orc_bf16_to_f32.argtypes = [C.c_uint16]; L.orc_bf16_to_f32.restype = C.c_float
        L.orc_f16_to_f32.argtypes = [C.c_uint16]; L.orc_f16_to_f32.restype = C.c_float
        _orc = L
    return _orc


def hp(a):
    """host pointer of a numpy array"""
    return a.ctypes.data_as(C.c_void_p)


# ---- 16-bit float helpers (numpy float16 and a bit-twiddled bf16 are independent of the
# oracle's own conversion code, so they can pin it) --------------------------------------
def f32_to_bf16_bits(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    nan = (u & 0x7fffffff) > 0x7f800000
    r = ((u + 0x7fff + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_f16_bits(x):
    return np.ascontiguousarray(x, dtype=np.float32).astype(np.float16).view(np.uint16)


def f16_bits_to_f32(b):
    return np.ascontiguousarray(b, dtype=np.uint16).view(np.float16).astype(np.float32)


def to_storage(x, dtype):
    """float/int numpy values -> storage array for `dtype`"""
    if dtype == BF16:
        return f32_to_bf16_bits(np.asarray(x, dtype=np.float32))
    if dtype == F16:
        return f32_to_f16_bits(np.asarray(x, dtype=np.float32))
    return np.ascontiguousarray(x, dtype=NP[dtype])


def to_float(a, dtype):
    """storage array -> float64 values (for tolerance checks)"""
    if dtype == BF16:
        return bf16_bits_to_f32(a).astype(np.float64)
    if dtype == F16:
        return f16_bits_to_f32(a).astype(np.float64)
    return a.astype(np.float64)


def rand(rng, dtype, n, lo=-1.0, hi=1.0):
    """seeded test data in storage form"""
    if dtype in FLOATS:
        return to_storage(rng.uniform(lo, hi, size=n), dtype)
    info = np.iinfo(NP[dtype])
    lo_i = max(info.min, -(2 ** 20)) if lo == -1.0 else int(lo)
    hi_i = min(info.max, 2 ** 20) if hi == 1.0 else int(hi)
    return rng.integers(lo_i, hi_i, size=n, endpoint=True).astype(NP[dtype])


def ulp_diff(a, b, dtype):
    """max distance in units of last place between two storage arrays of a float dtype"""
    if dtype == F64:
        ia, ib = a.view(np.int64).astype(np.int64), b.view(np.int64).astype(np.int64)
        sign = np.int64(-2 ** 63)
    elif dtype == F32:
        ia, ib = a.view(np.int32).astype(np.int64), b.view(np.int32).astype(np.int64)
        sign = np.int64(-2 ** 31)
    else:
        ia, ib = a.view(np.int16).astype(np.int64), b.view(np.int16).astype(np.int64)
        sign = np.int64(-2 ** 15)
    # map sign-magnitude to a monotonic integer line
    ia = np.where(ia < 0, sign - ia, ia)
    ib = np.where(ib < 0, sign - ib, ib)
    both_nan = np.isnan(to_float(a, dtype)) & np.isnan(to_float(b, dtype))
    d = np.abs(ia - ib)
    d[both_nan] = 0
    return int(d.max()) if d.size else 0


# ---- device side: torch owns HBM buffers, libdxhip gets raw pointers ---------------------
class Dev:
    """A device buffer holding the bytes of a numpy array."""

    def __init__(self, arr=None, nbytes=None):
        import torch
        if arr is not None:
            arr = np.ascontiguousarray(arr)
            self.np_dtype, self.shape = arr.dtype, arr.shape
            host = torch.from_numpy(arr.view(np.uint8).reshape(-1).copy())
            self.t = host.cuda()
        else:
            self.np_dtype, self.shape = np.uint8, (nbytes,)
            self.t = torch.empty(max(1, nbytes), dtype=torch.uint8, device="cuda")
        self.ptr = C.c_void_p(self.t.data_ptr())

    @staticmethod
    def empty(shape, np_dtype):
        n = int(np.prod(shape)) if len(np.shape(shape)) else int(shape)
        d = Dev(nbytes=n * np.dtype(np_dtype).itemsize)
        d.np_dtype, d.shape = np.dtype(np_dtype), tuple(np.atleast_1d(shape))
        return d

    def get(self):
        import torch
        torch.cuda.synchronize()
        nbytes = int(np.prod(self.shape)) * np.dtype(self.np_dtype).itemsize
        return self.t[:nbytes].cpu().numpy().view(self.np_dtype).reshape(self.shape).copy()


_mm_ws = {}


def matmul(dxh, dtype, a, b, c, batch, m, k, n, stream=None):
    """dxh_matmul with the workspace its own query asks for (one grow-only device buffer per
    stream, as a caller of the C ABI would keep).  Returns the entry point's return code."""
    need = C.c_size_t(0)
    rc = dxh.dxh_matmul_workspace_bytes(dtype, a, b, c, batch, m, k, n, C.byref(need))
    if rc != 0:
        return rc
    ws_ptr, ws_bytes = None, 0
    if need.value:
        key = stream.value if isinstance(stream, C.c_void_p) else stream
        ws = _mm_ws.get(key)
        if ws is None or ws.shape[0] < need.value:
            import torch
            torch.cuda.synchronize()  # work that still uses the old buffer
            ws = _mm_ws[key] = Dev.empty(max(need.value, 1 << 22), np.uint8)
        ws_ptr, ws_bytes = ws.ptr, ws.shape[0]
    return dxh.dxh_matmul(dtype, a, b, c, batch, m, k, n, ws_ptr, ws_bytes, stream)
