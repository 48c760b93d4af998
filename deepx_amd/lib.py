"""ctypes binding of libdxhip.so, the C ABI declared in include/dxhip.h.

This is the harness-side view of the library (tests, bench, smoke).  The product's host
side is the C++ executor in deepx_amd/executor, which links the same entry points.
There is no CPU fallback: `load()` raises if the library has not been built.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libdxhip.so")

# Precision bit values, executor/deepxcore/src/deepx/dtype.hpp:120-146
F64, F32, F16, BF16 = 1 << 0, 1 << 1, 1 << 2, 1 << 3
I64, I32, I16, I8, BOOL = 1 << 8, 1 << 9, 1 << 10, 1 << 11, 1 << 13

DTYPE_NAMES = {
    F64: "float64", F32: "float32", F16: "float16", BF16: "bfloat16",
    I64: "int64", I32: "int32", I16: "int16", I8: "int8", BOOL: "bool",
}
DTYPE_SIZE = {F64: 8, F32: 4, F16: 2, BF16: 2, I64: 8, I32: 4, I16: 2, I8: 1, BOOL: 1}


class Scalar(C.Structure):
    """dxh_scalar: floating dtypes read .f, integer dtypes read .i."""
    _fields_ = [("f", C.c_double), ("i", C.c_int64)]


class ChainOp(C.Structure):
    """dxh_chain_op: one op of a dxh_chain run."""
    _fields_ = [("code", C.c_int32), ("lhs", C.c_int32), ("rhs", C.c_int32), ("scalar", Scalar), ("out", C.c_void_p)]


class ChainTensor(C.Structure):
    """dxh_chain_tensor: one input of a dxh_chain_rows run."""
    _fields_ = [("data", C.c_void_p), ("dtype", C.c_int32), ("extent", C.c_int32)]


class ChainRowsOp(C.Structure):
    """dxh_chain_rows_op: one op of a dxh_chain_rows run."""
    _fields_ = [("code", C.c_int32), ("lhs", C.c_int32), ("rhs", C.c_int32), ("scalar", Scalar), ("out", C.c_void_p),
                ("dtype", C.c_int32), ("extent", C.c_int32)]


# enum dxh_chain_code, in the header's order (the last three: dxh_chain_rows only)
CHAIN_CODES = ["add", "sub", "mul", "div", "max", "min", "addscalar", "subscalar", "rsubscalar", "mulscalar",
               "divscalar", "rdivscalar", "maxscalar", "minscalar", "sqrt", "exp", "log", "square", "copy", "rowsum", "rowmax", "rowmin"]
CHAIN_RESULT = 16
CHAIN_FULL, CHAIN_ROW, CHAIN_COLUMN = 0, 1, 2  # enum dxh_chain_extent


def scalar(v):
    """Both views of one scalar, as the executor fills them from T(std::stof(text))."""
    f = float(v)
    try:
        i = int(v)
    except (OverflowError, ValueError):
        i = 0
    return Scalar(f, i)


class PoolStats(C.Structure):
    """dxh_pool_stats_t of include/dxhip.h"""
    _fields_ = [(n, C.c_uint64) for n in ("hits", "misses", "kept", "released", "kept_bytes", "kept_blocks", "live_bytes", "live_blocks")]


_p, _i, _i64, _sz, _f = C.c_void_p, C.c_int, C.c_int64, C.c_size_t, C.c_float
_pi32 = C.POINTER(C.c_int32)
_pp = C.POINTER(C.c_void_p)

_BIN = [_i, _p, _p, _p, _i64, _p]
_SCL = [_i, _p, Scalar, _p, _i64, _p]
_RSCL = [_i, Scalar, _p, _p, _i64, _p]
_UN = [_i, _p, _p, _i64, _p]
_RED = [_i, _p, _pi32, _i, _pi32, _i, _p, _p, _sz, _p]

ABI_VERSION = 200  # DXH_ABI_VERSION of include/dxhip.h, the layout SIGNATURES below describes

SIGNATURES = {
    "dxh_version": ([], _i),
    "dxh_error_string": ([_i], C.c_char_p),
    "dxh_tune": ([_i, _i64], _i),
    "dxh_device_count": ([C.POINTER(_i)], _i),
    "dxh_set_device": ([_i], _i),
    "dxh_device_name": ([C.c_char_p, _sz], _i),
    "dxh_malloc": ([_pp, _sz], _i),
    "dxh_free": ([_p], _i),
    "dxh_pool_alloc": ([_pp, _sz], _i),
    "dxh_pool_free": ([_p], _i),
    "dxh_pool_trim": ([_sz, C.POINTER(_sz)], _i),
    "dxh_pool_limit": ([_sz], _i),
    "dxh_pool_stats": ([C.POINTER(PoolStats)], _i),
    "dxh_memcpy_h2d": ([_p, _p, _sz, _p], _i),
    "dxh_memcpy_d2h": ([_p, _p, _sz, _p], _i),
    "dxh_memcpy_d2d": ([_p, _p, _sz, _p], _i),
    "dxh_stream_create": ([_pp], _i),
    "dxh_stream_destroy": ([_p], _i),
    "dxh_stream_sync": ([_p], _i),
    "dxh_device_sync": ([], _i),
    "dxh_event_create": ([_pp], _i),
    "dxh_event_destroy": ([_p], _i),
    "dxh_event_record": ([_p, _p], _i),
    "dxh_event_sync": ([_p], _i),
    "dxh_stream_wait_event": ([_p, _p], _i),
    "dxh_event_elapsed_ms": ([_p, _p, C.POINTER(_f)], _i),
    "dxh_ipc_export": ([_p, _p], _i),
    "dxh_ipc_open": ([_p, C.POINTER(_p)], _i),
    "dxh_ipc_close": ([_p], _i),
    "dxh_graph_begin_capture": ([_p], _i),
    "dxh_graph_end_capture": ([_p, C.POINTER(_p)], _i),
    "dxh_graph_launch": ([_p, _p], _i),
    "dxh_graph_destroy": ([_p], _i),
    "dxh_graph_counter_stats": ([C.POINTER(_i64), C.POINTER(_i64)], _i),
    "dxh_add": (_BIN, _i), "dxh_sub": (_BIN, _i), "dxh_mul": (_BIN, _i), "dxh_div": (_BIN, _i),
    "dxh_max": (_BIN, _i), "dxh_min": (_BIN, _i), "dxh_pow": (_BIN, _i),
    "dxh_addscalar": (_SCL, _i), "dxh_subscalar": (_SCL, _i), "dxh_rsubscalar": (_RSCL, _i),
    "dxh_mulscalar": (_SCL, _i), "dxh_divscalar": (_SCL, _i), "dxh_rdivscalar": (_RSCL, _i),
    "dxh_maxscalar": (_SCL, _i), "dxh_minscalar": (_SCL, _i),
    "dxh_powscalar": (_SCL, _i), "dxh_rpowscalar": (_RSCL, _i),
    "dxh_sqrt": (_UN, _i), "dxh_exp": (_UN, _i), "dxh_log": (_UN, _i),
    "dxh_sin": (_UN, _i), "dxh_cos": (_UN, _i), "dxh_tan": (_UN, _i), "dxh_invert": (_UN, _i),
    "dxh_chain": ([_i, _pp, _i, C.POINTER(ChainOp), _i, _i64, _p], _i),
    "dxh_chain_rows": ([C.POINTER(ChainTensor), _i, C.POINTER(ChainRowsOp), _i, _i64, _i64, _p], _i),
    "dxh_chain_rows_can_sum": ([_i64, _i64], _i),
    "dxh_chain_rows_check": ([C.POINTER(ChainTensor), _i, C.POINTER(ChainRowsOp), _i, _i64, _i64], _i),
    "dxh_chain_stats": ([C.POINTER(_i64), C.POINTER(_i64)], _i),
    "dxh_todtype": ([_i, _p, _i, _p, _i64, _p], _i),
    "dxh_equal": ([_i, _p, _p, _f, _p, _i64, _p], _i),
    "dxh_notequal": ([_i, _p, _p, _f, _p, _i64, _p], _i),
    "dxh_equalscalar": ([_i, _p, Scalar, _f, _p, _i64, _p], _i),
    "dxh_notequalscalar": ([_i, _p, Scalar, _f, _p, _i64, _p], _i),
    "dxh_less": (_BIN, _i), "dxh_greater": (_BIN, _i),
    "dxh_lessscalar": (_SCL, _i), "dxh_greaterscalar": (_SCL, _i),
    "dxh_switch": ([_i, _pp, _i, _i, _p, _p, _i64, _p], _i),
    "dxh_reduce_workspace_bytes": ([_i, _pi32, _i, _pi32, _i, C.POINTER(_sz)], _i),
    "dxh_sum": (_RED, _i), "dxh_prod": (_RED, _i),
    "dxh_reducemax": (_RED, _i), "dxh_reducemin": (_RED, _i),
    "dxh_sum_noalloc": ([_i, _p, _pi32, _i, _pi32, _i, _p, _p], _i),
    "dxh_transpose": ([_i, _p, _pi32, _i, _pi32, _p, _p], _i),
    "dxh_concat": ([_i, _pp, _i, _pi32, _pi32, _i, _i, _p, _p], _i),
    "dxh_broadcastTo": ([_i, _p, _pi32, _i, _pi32, _i, _p, _p], _i),
    "dxh_indexselect": ([_i, _p, _pi32, _i, _i, _p, _pi32, _i, _i, _p, _p], _i),
    "dxh_repeat": ([_i, _p, _pi32, _i, _pi32, _p, _p], _i),
    "dxh_constant": ([_i, _p, _i64, Scalar, _p], _i),
    "dxh_arange": ([_i, _p, _i64, Scalar, Scalar, _p], _i),
    "dxh_uniform": ([_i, _p, _i64, Scalar, Scalar, C.c_uint32, _p], _i),
    "dxh_normal": ([_i, _p, _i64, Scalar, Scalar, C.c_uint32, _p], _i),
    "dxh_dropout": ([_i, _p, _i64, _f, C.c_uint32, _p], _i),
    "dxh_matmul_workspace_bytes": ([_i, _p, _p, _p, _i64, _i64, _i64, _i64, C.POINTER(_sz)], _i),
    "dxh_matmul": ([_i, _p, _p, _p, _i64, _i64, _i64, _i64, _p, _sz, _p], _i),
    "dxh_matmul_shared_a_workspace_bytes": ([_i, _p, _pp, _pp, _i, _i64, _i64, _i64, C.POINTER(_sz)], _i),
    "dxh_matmul_shared_a": ([_i, _p, _pp, _pp, _i, _i64, _i64, _i64, _p, _sz, _p], _i),
}

_lib = None


class DxhError(RuntimeError):
    pass


def load(path=None):
    """Load libdxhip.so and declare every entry point.  Raises if it is not built."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or LIB_PATH
    if not os.path.exists(p):
        raise DxhError(
            f"{p} is missing: build it with `make -C deepx_amd/csrc` "
            "(or __graft_entry__.build()); there is no CPU fallback")
    lib = C.CDLL(p)
    for name, (argtypes, restype) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.argtypes = argtypes
        fn.restype = restype
    got = lib.dxh_version()
    if got != ABI_VERSION:
        raise DxhError(f"{p} was built for ABI {got}, these bindings are written for {ABI_VERSION} (DXH_ABI_VERSION in include/dxhip.h): rebuild it")
    if path is None:
        _lib = lib
    return lib


def check(code, what=""):
    if code != 0:
        msg = load().dxh_error_string(code).decode()
        raise DxhError(f"{what}: dxh error {code}: {msg}")


def i32arr(values):
    values = list(values)
    return (C.c_int32 * max(1, len(values)))(*values)


def ptrarr(ptrs):
    ptrs = list(ptrs)
    return (C.c_void_p * len(ptrs))(*ptrs)
