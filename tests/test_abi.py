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
    # the header's macro, the bindings' constant and the built library agree
    macro = int(re.search(r"#define\s+DXH_ABI_VERSION\s+(\d+)", open(os.path.join(ROOT, "include", "dxhip.h")).read()).group(1))
    assert L.dxh_version() == macro == dx.ABI_VERSION
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
    assert L.dxh_matmul(dx.BOOL, None, None, None, 1, 2, 2, 2, None, 0, None) == -1
    # the matmul workspace query is host arithmetic: 0 for the BASELINE shapes' first GEMM, partial tiles
    # for a product cut along K, padded copies for rows that are not 16-byte pieces; it needs no GPU
    P = lambda v: C.c_void_p(v)
    assert L.dxh_matmul_workspace_bytes(dx.BF16, P(256), P(512), P(1024), 1, 2048, 896, 4864, C.byref(n)) == 0 and n.value == 0
    assert L.dxh_matmul_workspace_bytes(dx.F32, P(256), P(512), P(1024), 1, 16, 4096, 256, C.byref(n)) == 0 and n.value >= 2 * 16 * 256 * 4
    assert L.dxh_matmul_workspace_bytes(dx.BF16, P(256), P(512), P(1024), 1, 333, 777, 555, C.byref(n)) == 0 and n.value >= 832 * 560 * 2
    assert L.dxh_matmul_workspace_bytes(dx.I32, P(256), P(512), P(1024), 1, 64, 64, 64, C.byref(n)) == 0 and n.value == 0
    assert L.dxh_matmul_workspace_bytes(dx.BOOL, P(256), P(512), P(1024), 1, 64, 64, 64, C.byref(n)) == -1
    assert L.dxh_matmul(dx.F32, P(256), P(512), P(1024), 1, 16, 4096, 256, P(100), 1 << 20, None) == -4  # workspace not 256-byte aligned
    # the sum that allocates nothing refuses what its fixed scratch array cannot hold, before any HIP call
    assert L.dxh_sum_noalloc(dx.F32, C.c_void_p(256), dx.i32arr([4096, 4096, 16]), 3, dx.i32arr([0, 2]), 2, C.c_void_p(512), None) == -6
    assert L.dxh_sum_noalloc(dx.F32, C.c_void_p(256), dx.i32arr([64, 64]), 2, dx.i32arr([2]), 1, C.c_void_p(512), None) == -2
    assert L.dxh_sum_noalloc(dx.BOOL, C.c_void_p(256), dx.i32arr([64, 64]), 2, dx.i32arr([1]), 1, C.c_void_p(512), None) == -1
    assert L.dxh_error_string(-6).decode().startswith("input needs more scratch")
    # dxh_chain: operand references, op codes, counts, alignment and dtype are checked on the host
    ins = (C.c_void_p * 2)(16, 32)
    op = lambda code, lhs, rhs, out: dx.ChainOp(code, lhs, rhs, dx.scalar(1.0), out)
    one = (dx.ChainOp * 1)(op(0, 0, 1, 48))
    assert L.dxh_chain(dx.F32, ins, 2, one, 1, 0, None) == 0            # nothing to do
    assert L.dxh_chain(dx.F32, ins, 2, one, 0, 8, None) == -2           # no ops
    assert L.dxh_chain(dx.F32, ins, 2, one, 9, 8, None) == -2           # too many ops
    assert L.dxh_chain(dx.I32, ins, 2, one, 1, 8, None) == -1           # float dtypes only
    assert L.dxh_chain(dx.F32, ins, 2, one, 1, 7, None) == -5           # not a whole number of vectors
    assert L.dxh_chain(dx.F32, ins, 2, (dx.ChainOp * 1)(op(0, 0, 2, 48)), 1, 8, None) == -2    # input 2 does not exist
    assert L.dxh_chain(dx.F32, ins, 2, (dx.ChainOp * 1)(op(0, 0, dx.CHAIN_RESULT, 48)), 1, 8, None) == -2  # its own result
    assert L.dxh_chain(dx.F32, ins, 2, (dx.ChainOp * 1)(op(17, 0, 1, 48)), 1, 8, None) == -2   # unknown op code
    assert L.dxh_chain(dx.F32, ins, 2, (dx.ChainOp * 1)(op(0, 0, 1, 50)), 1, 8, None) == -5    # output off a 16-byte boundary
    assert L.dxh_chain(dx.F32, ins, 2, (dx.ChainOp * 1)(op(0, 0, 1, None)), 1, 8, None) == -2  # the last op must store
    assert len(dx.CHAIN_CODES) == 22 and dx.CHAIN_CODES[16] == "log" and dx.CHAIN_CODES[18] == "copy" and dx.CHAIN_CODES[21] == "rowmin"
    # dxh_chain_rows: the same checks, and those on extents: a [rows, cols] op takes any operand, an op on
    # vectors only vectors of its kind; a vector input may not be an output of the run
    T, R = dx.ChainTensor, dx.ChainRowsOp
    FULL, ROW, COL = dx.CHAIN_FULL, dx.CHAIN_ROW, dx.CHAIN_COLUMN
    tin = (T * 3)(T(64, dx.F32, FULL), T(128, dx.BF16, ROW), T(256, dx.F32, COL))
    rop = lambda code, lhs, rhs, out, dtype=dx.F32, extent=FULL: R(code, lhs, rhs, dx.scalar(1.0), out, dtype, extent)
    run = lambda *ops, n_in=3, rows=8, cols=16: L.dxh_chain_rows(tin, n_in, (R * len(ops))(*ops), len(ops), rows, cols, None)
    assert run(rop(2, 0, 1, 512), rows=0) == 0                               # nothing to do
    assert run(rop(2, 0, 1, 512), cols=18) == -5                             # cols not a multiple of 4
    assert run(rop(2, 0, 1, 512, dx.F64)) == -1                              # no fp64 in this form
    assert L.dxh_chain_rows((T * 1)(T(64, dx.I32, FULL)), 1, (R * 1)(rop(18, 0, 0, 512)), 1, 8, 16, None) == -1
    assert run(rop(22, 0, 0, 512)) == -2                                     # unknown op code
    assert run(rop(2, 0, 3, 512)) == -2                                      # input 3 does not exist
    assert run(rop(2, 0, 1, 512, extent=3)) == -2                            # unknown extent
    assert run(rop(2, 0, 1, None)) == -2                                     # the last op must store
    assert run(rop(2, 0, 1, 520)) == -5                                      # fp32 output off a 16-byte boundary
    assert run(rop(18, 1, 0, 516, dx.BF16, ROW)) == -5                       # bf16 row off an 8-byte boundary
    assert run(rop(18, 2, 0, 516, dx.F32, COL), rop(2, 0, dx.CHAIN_RESULT, 512), rows=0) == 0  # a column needs its element size only
    assert run(rop(9, 0, 0, 512, dx.F32, ROW)) == -2                         # an op on row vectors cannot read a [rows, cols] tensor
    assert run(rop(9, 2, 0, 512, dx.F32, ROW)) == -2                         # ... nor a column vector
    assert run(rop(18, 1, 0, 1024, dx.F32, ROW), rop(0, dx.CHAIN_RESULT, 2, 512, dx.F32, COL)) == -2  # a row result into a column op
    assert run(rop(9, 2, 0, 256, dx.F32, COL), rop(2, 0, dx.CHAIN_RESULT, 512)) == -2  # overwrites the column vector it reads
    # the row sum: an fp32 [rows, cols] operand into an fp32 column, over views whose rows one lane group folds
    assert run(rop(19, 0, 0, 512, dx.F32, FULL)) == -2                       # its result is a column
    assert run(rop(19, 2, 0, 512, dx.F32, COL)) == -2                        # its operand is not
    assert run(rop(19, 0, 0, 512, dx.BF16, COL)) == -1                       # fp32 only
    assert L.dxh_chain_rows((T * 1)(T(64, dx.BF16, FULL)), 1, (R * 1)(rop(19, 0, 0, 512, dx.F32, COL)), 1, 8, 16, None) == -1
    assert L.dxh_chain_rows_can_sum(2048, 896) == 1 and L.dxh_chain_rows_can_sum(8, 16) == 1
    assert L.dxh_chain_rows_can_sum(8, 18) == 0 and L.dxh_chain_rows_can_sum(0, 16) == 0
    assert L.dxh_chain_rows_can_sum(64, 1 << 20) == 0                        # a row that long is cut or takes the whole workgroup
    assert run(rop(19, 0, 0, 512, dx.F32, COL), rows=64, cols=1 << 20) == -3
    assert run(*([rop(2, 0, 0, 512)] * 17)) == -2                            # too many ops
    # dxh_chain_rows_check: the checks of a call without its launch.  A softmax (row max, sub, exp, row sum, exp,
    # div) is one of the runs with a compiled kernel, which takes 16-bit rows and rows of up to eight 16-byte
    # vectors per lane; other runs with a row reduction need fp32 and rows short enough for the interpreter.
    RES = dx.CHAIN_RESULT
    def softmax(dt, rows, cols):
        tin1 = (T * 1)(T(4096, dt, FULL))
        ops = [rop(20, 0, 0, 8192, dt, COL), rop(18, RES, 0, None, dt, FULL), rop(1, 0, RES + 1, None, dt, FULL), rop(15, RES + 2, 0, None, dt, FULL),
               rop(19, RES + 3, 0, 8192, dt, COL), rop(15, RES + 2, 0, None, dt, FULL), rop(18, RES + 4, 0, None, dt, FULL), rop(3, RES + 5, RES + 6, 4096, dt, FULL)]
        return L.dxh_chain_rows_check(tin1, 1, (R * len(ops))(*ops), len(ops), rows, cols)
    assert softmax(dx.F32, 2048, 2048) == 0 and softmax(dx.BF16, 2048, 4096) == 0 and softmax(dx.F16, 7, 8) == 0
    assert softmax(dx.F32, 64, 1 << 20) == -3 and softmax(dx.BF16, 64, 8192) == -1 and softmax(dx.BF16, 64, 12) == -1
    assert L.dxh_tune(12, 0) == 0
    try:
        assert softmax(dx.F32, 2048, 896) == 0 and softmax(dx.F32, 2048, 2048) == -3 and softmax(dx.BF16, 2048, 896) == -1
    finally:
        assert L.dxh_tune(12, 1) == 0
    a, b = C.c_int64(-1), C.c_int64(-1)
    assert L.dxh_chain_stats(C.byref(a), C.byref(b)) == 0 and a.value >= 0 and b.value >= 0 and L.dxh_chain_stats(None, None) == -2


def test_tuning_knobs_validate_their_values():
    """dxh_tune is host state only: every knob of the header accepts its documented range and
    rejects values outside it (and unknown knobs) with DXH_ERR_ARG."""
    L = dx.load()
    text = open(os.path.join(ROOT, "include", "dxhip.h")).read()
    knobs = {name: int(val) for name, val in re.findall(r"(DXH_TUNE_\w+)\s*=\s*(\d+)", text)}
    assert sorted(knobs.values()) == list(range(len(knobs))), knobs  # dense numbering, no duplicates
    good = {"DXH_TUNE_NT_STORE_BYTES": [0, 1 << 20], "DXH_TUNE_REDUCE_TARGET_BLOCKS": [256, 1024], "DXH_TUNE_REDUCE_COL_MIN_ROWS": [1, 16],
            "DXH_TUNE_REDUCE_COL_MAX_LANES": [4, 32, 128, 256], "DXH_TUNE_MATMUL_TILE": [1, 6, 15, 0], "DXH_TUNE_REDUCE_ROW_LOADS": [1, 4],
            "DXH_TUNE_MATMUL_SPLITK": [1, 7, 1024, 0], "DXH_TUNE_NT_LOAD": [1, 2, 0], "DXH_TUNE_SKINNY_PER_CU": [2, 4, 1],
            "DXH_TUNE_SKINNY_MIN_ROWS": [8, 512, 256], "DXH_TUNE_SKINNY_HALF": [1, 0], "DXH_TUNE_REDUCE_FUSED_FINISH": [0, 1],
            "DXH_TUNE_CHAIN_STATIC": [0, 1]}
    bad = {"DXH_TUNE_REDUCE_TARGET_BLOCKS": [0], "DXH_TUNE_REDUCE_COL_MIN_ROWS": [0], "DXH_TUNE_REDUCE_COL_MAX_LANES": [3, 512],
           "DXH_TUNE_MATMUL_TILE": [-1, 16], "DXH_TUNE_REDUCE_ROW_LOADS": [0, 65], "DXH_TUNE_MATMUL_SPLITK": [-1, 1025], "DXH_TUNE_NT_LOAD": [-1, 3], "DXH_TUNE_SKINNY_PER_CU": [0, 65],
           "DXH_TUNE_SKINNY_MIN_ROWS": [7], "DXH_TUNE_SKINNY_HALF": [-1, 2], "DXH_TUNE_REDUCE_FUSED_FINISH": [-1, 2], "DXH_TUNE_CHAIN_STATIC": [-1, 2]}
    assert set(good) == set(knobs), set(good) ^ set(knobs)
    defaults = {"DXH_TUNE_NT_STORE_BYTES": 0, "DXH_TUNE_REDUCE_TARGET_BLOCKS": 1024, "DXH_TUNE_REDUCE_COL_MIN_ROWS": 16,
                "DXH_TUNE_REDUCE_COL_MAX_LANES": 128, "DXH_TUNE_MATMUL_TILE": 0, "DXH_TUNE_REDUCE_ROW_LOADS": 4,
                "DXH_TUNE_MATMUL_SPLITK": 0, "DXH_TUNE_NT_LOAD": 0, "DXH_TUNE_SKINNY_PER_CU": 1, "DXH_TUNE_SKINNY_MIN_ROWS": 256,
                "DXH_TUNE_SKINNY_HALF": 0, "DXH_TUNE_REDUCE_FUSED_FINISH": 1, "DXH_TUNE_CHAIN_STATIC": 1}
    try:
        for name, values in good.items():
            for v in values:
                assert L.dxh_tune(knobs[name], v) == 0, (name, v)
        for name, values in bad.items():
            for v in values:
                assert L.dxh_tune(knobs[name], v) == -2, (name, v)
        assert L.dxh_tune(len(knobs), 0) == -2
        assert L.dxh_tune(-1, 0) == -2
    finally:
        for name, v in defaults.items():
            assert L.dxh_tune(knobs[name], v) == 0


def test_chain_codes_follow_the_header():
    """The op codes of dxh_chain are positional: the binding's list must be the header's enum, in order."""
    text = open(os.path.join(ROOT, "include", "dxhip.h")).read()
    body = text[text.index("enum dxh_chain_code {"):]
    body = re.sub(r"/\*.*?\*/", "", body[:body.index("};")], flags=re.S)
    names = re.findall(r"DXH_CHAIN_(\w+)", body)
    assert [n.lower() for n in names] == dx.CHAIN_CODES
    assert int(re.search(r"#define DXH_CHAIN_RESULT (\d+)", text).group(1)) == dx.CHAIN_RESULT
