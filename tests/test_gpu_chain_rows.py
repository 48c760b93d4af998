"""GPU parity: dxh_chain_rows (a run of elementwise ops over a [rows, cols] view whose tensors may
differ in dtype and may be row or column vectors) against the separate entry points, the CPU
oracle and a numpy model.

Bars: bit-identical to what todtype / powscalar / broadcastTo / mul ... store when called one
after another; each op of such a run bit-exact against the oracle fed with the device's own
operands (casts, squares, copies and products are correctly rounded on both sides); random runs
of exactly rounded ops bit-exact against numpy float32 arithmetic with one rounding to the op's
dtype (NaN payloads aside).
"""
import ctypes as C

import numpy as np
import pytest

from deepx_amd import lib as dx
from tests import helpers as H
from tests.helpers import Dev, hp

pytestmark = pytest.mark.gpu

FULL, ROW, COL = dx.CHAIN_FULL, dx.CHAIN_ROW, dx.CHAIN_COLUMN
R = dx.CHAIN_RESULT
BINARY = ["add", "sub", "mul", "div", "max", "min"]
SCALAR = ["addscalar", "subscalar", "rsubscalar", "mulscalar", "divscalar", "rdivscalar", "maxscalar", "minscalar"]


def count(extent, rows, cols):
    return rows * cols if extent == FULL else cols if extent == ROW else rows


def run_rows(dxh, inputs, prog, rows, cols, outs=None):
    """inputs: (Dev, dtype, extent); prog: (name, lhs, rhs, scalar, dtype, extent).  Returns rc and the outputs."""
    if outs is None:
        outs = [Dev.empty(count(e, rows, cols), H.NP[dt]) for (_, _, _, _, dt, e) in prog]
    tin = (dx.ChainTensor * max(1, len(inputs)))(*[dx.ChainTensor(d.ptr, dt, e) for d, dt, e in inputs])
    ops = (dx.ChainRowsOp * len(prog))()
    for k, (name, lhs, rhs, s, dt, e) in enumerate(prog):
        ops[k] = dx.ChainRowsOp(dx.CHAIN_CODES.index(name), lhs, rhs, dx.scalar(s), outs[k].ptr if outs[k] is not None else None, dt, e)
    return dxh.dxh_chain_rows(tin, len(inputs), ops, len(prog), rows, cols, None), outs


def shape_of(extent, rows, cols):
    return [rows, cols] if extent == FULL else [1, cols] if extent == ROW else [rows, 1]


def run_separately(dxh, orc, inputs, prog, rows, cols):
    """The lines a front end would send, one entry point each, on the device; every result also
    against the oracle applied to the device's operands of that op."""
    outs = []
    for k, (name, lhs, rhs, s, dt, e) in enumerate(prog):
        src = lambda r: inputs[r] if r < R else (outs[r - R], prog[r - R][4], prog[r - R][5])
        a, adt, ae = src(lhs)
        n = count(e, rows, cols)
        out = Dev.empty(n, H.NP[dt])
        want = np.empty(n, dtype=H.NP[dt])
        ah = a.get()
        if name == "copy" and ae != e:
            assert adt == dt and e == FULL
            ish, osh = shape_of(ae, rows, cols), [rows, cols]
            dx.check(dxh.dxh_broadcastTo(dt, a.ptr, dx.i32arr(ish), 2, dx.i32arr(osh), 2, out.ptr, None), "broadcastTo")
            assert orc.orc_broadcastTo(dt, hp(ah), dx.i32arr(ish), 2, dx.i32arr(osh), 2, hp(want)) == 0
        elif name == "copy":
            dx.check(dxh.dxh_todtype(adt, a.ptr, dt, out.ptr, n, None), "todtype")
            assert orc.orc_todtype(adt, hp(ah), dt, hp(want), n) == 0
        elif name == "square":
            assert adt == dt == dx.F32 and ae == e
            dx.check(dxh.dxh_powscalar(dt, a.ptr, dx.scalar(2.0), out.ptr, n, None), "powscalar")
            assert orc.orc_powscalar(dt, hp(ah), dx.scalar(2.0), hp(want), n) == 0
            # the device squares with one multiplication (correctly rounded); the oracle's powf is within an ulp of that,
            # and has its bits whenever the square needs no rounding (operands that came from a 16-bit type)
            assert np.array_equal(out.get(), (ah.astype(np.float64) ** 2).astype(np.float32)), ("square", rows, cols)
            assert H.ulp_diff(out.get(), want, dt) <= 1, ("square", rows, cols)
            want = None
        elif name in BINARY:
            b, bdt, be = src(rhs)
            assert adt == bdt == dt and ae == be == e
            dx.check(getattr(dxh, "dxh_" + name)(dt, a.ptr, b.ptr, out.ptr, n, None), name)
            assert getattr(orc, "orc_" + name)(dt, hp(ah), hp(b.get()), hp(want), n) == 0
        elif name in ("rsubscalar", "rdivscalar"):
            assert adt == dt and ae == e
            dx.check(getattr(dxh, "dxh_" + name)(dt, dx.scalar(s), a.ptr, out.ptr, n, None), name)
            assert getattr(orc, "orc_" + name)(dt, dx.scalar(s), hp(ah), hp(want), n) == 0
        elif name in SCALAR:
            assert adt == dt and ae == e
            dx.check(getattr(dxh, "dxh_" + name)(dt, a.ptr, dx.scalar(s), out.ptr, n, None), name)
            assert getattr(orc, "orc_" + name)(dt, hp(ah), dx.scalar(s), hp(want), n) == 0
        elif name == "rowsum":
            assert adt == dt and ae == FULL and e == COL
            dx.check(dxh.dxh_sum(dt, a.ptr, dx.i32arr([rows, cols]), 2, dx.i32arr([1]), 1, out.ptr, None, 0, None), "sum")
            want = None  # the order of a float sum is the kernel's own: checked against float64 below
            ref = H.to_float(ah, dt).astype(np.float64).reshape(rows, cols)
            rel = 1e-6 if dt == dx.F32 else 2.0 ** -8 if dt == dx.BF16 else 2.0 ** -11  # fp32 accumulation, one rounding to a 16-bit result
            assert np.all(np.abs(H.to_float(out.get(), dt).astype(np.float64) - ref.sum(1)) <= rel * np.abs(ref).sum(1) + 1e-30), ("sum", rows, cols)
        elif name in ("rowmax", "rowmin"):
            assert adt == dt and ae == FULL and e == COL
            fn = "reducemax" if name == "rowmax" else "reducemin"
            dx.check(getattr(dxh, "dxh_" + fn)(dt, a.ptr, dx.i32arr([rows, cols]), 2, dx.i32arr([1]), 1, out.ptr, None, 0, None), fn)
            assert getattr(orc, "orc_" + fn)(dt, hp(ah), dx.i32arr([rows, cols]), 2, dx.i32arr([1]), 1, hp(want)) == 0
        elif name in ("exp", "log"):
            assert adt == dt and ae == e
            dx.check(getattr(dxh, "dxh_" + name)(dt, a.ptr, out.ptr, n, None), name)
            assert getattr(orc, "orc_" + name)(dt, hp(ah), hp(want), n) == 0
            g64, w64 = H.to_float(out.get(), dt).astype(np.float64), H.to_float(want, dt).astype(np.float64)
            ulp = 2.0 ** -23 if dt == dx.F32 else 2.0 ** -7 if dt == dx.BF16 else 2.0 ** -10
            fin = np.isfinite(w64)
            assert np.array_equal(fin, np.isfinite(g64)) and np.all(np.abs(g64[fin] - w64[fin]) <= (4 if dt == dx.F32 else 1) * ulp * np.abs(w64[fin]) + 1e-45), (name, rows, cols)
            want = None  # within 4 ulp of libm (1 ulp of a 16-bit result), not its bits
        else:
            assert adt == dt and ae == e and name == "sqrt"
            dx.check(dxh.dxh_sqrt(dt, a.ptr, out.ptr, n, None), name)
            assert orc.orc_sqrt(dt, hp(ah), hp(want), n) == 0
        got = out.get()
        assert want is None or np.array_equal(got.view(np.uint8), want.view(np.uint8)), ("oracle", k, name, rows, cols)
        outs.append(out)
    return outs


def same_bits(a, b):
    return np.array_equal(a.get().view(np.uint8), b.get().view(np.uint8))


@pytest.mark.parametrize("half", [dx.BF16, dx.F16])
def test_rmsnorm_lines_as_runs(dxh, orc, half):
    """The elementwise lines of an RMSNorm either side of its row sum (t5layernorm.py:17-22 as the
    front end emits it): cast and square before the sum; after it the reciprocal root spread over
    the columns, the product, the weight cast, spread over the rows and multiplied, and the cast of
    the result.  Every tensor a line writes, bit for bit what the separate entry points store, and
    each of those against the oracle."""
    rng = np.random.default_rng(1200 + half)
    for rows, cols in [(2048, 896), (5, 12), (2, 4), (257, 1000), (64, 4096), (2100, 500), (4099, 260)]:
        x = Dev(H.rand(rng, half, rows * cols, -2.0, 2.0))
        w = Dev(H.rand(rng, half, cols, 0.5, 1.5))
        var = Dev(H.rand(rng, dx.F32, rows, 0.05, 3.0))  # stands for 1/sqrt(mean + eps) of each row
        before = [("copy", 0, 0, 0, dx.F32, FULL), ("square", R + 0, 0, 2.0, dx.F32, FULL)]
        ins = [(x, half, FULL)]
        want = run_separately(dxh, orc, ins, before, rows, cols)
        rc, got = run_rows(dxh, ins, before, rows, cols)
        dx.check(rc, "chain_rows")
        for k in range(len(before)):
            assert same_bits(got[k], want[k]), ("before", rows, cols, k)
        xf = got[0]
        after = [("copy", 0, 0, 0, dx.F32, FULL),        # broadcastTo(var) -> rs
                 ("mul", 1, R + 0, 0, dx.F32, FULL),      # xf * rs -> xn
                 ("copy", 2, 0, 0, dx.F32, ROW),          # todtype(w) -> wf1
                 ("copy", R + 2, 0, 0, dx.F32, FULL),     # broadcastTo(wf1) -> wf
                 ("mul", R + 3, R + 1, 0, dx.F32, FULL),  # wf * xn -> xn
                 ("copy", R + 4, 0, 0, half, FULL)]       # todtype(xn) -> h
        ins = [(var, dx.F32, COL), (xf, dx.F32, FULL), (w, half, ROW)]
        want = run_separately(dxh, orc, ins, after, rows, cols)
        rc, got = run_rows(dxh, ins, after, rows, cols)
        dx.check(rc, "chain_rows")
        for k in range(len(after)):
            assert same_bits(got[k], want[k]), ("after", rows, cols, k)
        # the same with the first product not stored (the second overwrites xn in the IR)
        outs = [Dev.empty(count(e, rows, cols), H.NP[dt]) for (_, _, _, _, dt, e) in after]
        outs[1] = None
        rc, got2 = run_rows(dxh, ins, after, rows, cols, outs=outs)
        dx.check(rc, "chain_rows")
        for k in (0, 2, 3, 4, 5):
            assert same_bits(got2[k], want[k]), ("after, xn stored once", rows, cols, k)


@pytest.mark.parametrize("half", [dx.BF16, dx.F16])
def test_whole_rmsnorm_as_one_run(dxh, orc, half):
    """All thirteen elementwise and reduce lines of the RMSNorm in one launch: the row sum sits in
    the middle of the run (its operand produced by the run, its result a column vector that the
    scalar lines then work on), with the lanes laid out as dxh_sum's own kernel has them, so every
    tensor — the sums included — has the bits of the thirteen separate launches.  Shapes: rows of
    one to four vector groups per lane, row counts that leave the last workgroup ragged, the
    config-5 size; and shapes whose rows dxh_sum would not give to one lane group are refused."""
    rng = np.random.default_rng(1300 + half)
    for rows, cols in [(2048, 896), (5, 12), (2, 4), (257, 1000), (64, 1024), (1000, 256), (33, 64), (7, 520), (2100, 500), (4099, 260), (1029, 1024)]:
        assert dxh.dxh_chain_rows_can_sum(rows, cols) == 1, (rows, cols)
        x = Dev(H.rand(rng, half, rows * cols, -2.0, 2.0))
        w = Dev(H.rand(rng, half, cols, 0.5, 1.5))
        prog = [("copy", 0, 0, 0, dx.F32, FULL),             # todtype(x) -> xf
                ("square", R + 0, 0, 2.0, dx.F32, FULL),      # powscalar(xf, 2) -> sq
                ("rowsum", R + 1, 0, 0, dx.F32, COL),         # sum(sq, [-1], keepdims) -> var
                ("divscalar", R + 2, 0, float(cols), dx.F32, COL),
                ("addscalar", R + 3, 0, 1e-6, dx.F32, COL),
                ("sqrt", R + 4, 0, 0, dx.F32, COL),
                ("rdivscalar", R + 5, 0, 1.0, dx.F32, COL),
                ("copy", R + 6, 0, 0, dx.F32, FULL),          # broadcastTo(var) -> rs
                ("mul", R + 0, R + 7, 0, dx.F32, FULL),       # xf * rs -> xn
                ("copy", 1, 0, 0, dx.F32, ROW),               # todtype(w) -> wf1
                ("copy", R + 9, 0, 0, dx.F32, FULL),          # broadcastTo(wf1) -> wf
                ("mul", R + 10, R + 8, 0, dx.F32, FULL),      # wf * xn -> xn
                ("copy", R + 11, 0, 0, half, FULL)]           # todtype(xn) -> h
        ins = [(x, half, FULL), (w, half, ROW)]
        want = run_separately(dxh, orc, ins, prog, rows, cols)
        rc, got = run_rows(dxh, ins, prog, rows, cols)
        dx.check(rc, "chain_rows")
        for k in range(len(prog)):
            assert same_bits(got[k], want[k]), (rows, cols, k, prog[k][0])
        # as the IR has it: var and xn written several times, stored once
        outs = [Dev.empty(count(e, rows, cols), H.NP[dt]) for (_, _, _, _, dt, e) in prog]
        for k in (2, 3, 4, 5, 8):
            outs[k] = None
        rc, got2 = run_rows(dxh, ins, prog, rows, cols, outs=outs)
        dx.check(rc, "chain_rows")
        for k in (0, 1, 6, 7, 9, 10, 11, 12):
            assert same_bits(got2[k], want[k]), ("stored once", rows, cols, k)
    # rows too long for one lane group: refused, the caller runs the lines one by one
    for rows, cols in [(4, 8192), (2, 1 << 16)]:
        assert dxh.dxh_chain_rows_can_sum(rows, cols) == 0
        x = Dev(H.rand(rng, dx.F32, rows * cols))
        rc, _ = run_rows(dxh, [(x, dx.F32, FULL)], [("rowsum", 0, 0, 0, dx.F32, COL)], rows, cols)
        assert rc == -3


def model(inputs_host, prog, rows, cols):
    """numpy float32 arithmetic on operands spread to [rows, cols], one rounding to the op's dtype."""
    def spread(values, extent):
        v = np.asarray(values, dtype=np.float32)
        return v.reshape(rows, cols) if extent == FULL else np.broadcast_to(v.reshape(1, cols), (rows, cols)) if extent == ROW \
            else np.broadcast_to(v.reshape(rows, 1), (rows, cols))
    results = []
    with np.errstate(all="ignore"):
        for name, lhs, rhs, s, dt, e in prog:
            src = lambda r: inputs_host[r] if r < R else results[r - R]
            a, b = src(lhs), src(rhs)
            sc = np.float32(H.to_float(H.to_storage(np.array([s]), dt), dt)[0])
            if name == "add": y = a + b
            elif name == "sub": y = a - b
            elif name == "mul": y = a * b
            elif name == "div": y = a / b
            elif name == "max": y = np.where(a < b, b, a)
            elif name == "min": y = np.where(b < a, b, a)
            elif name == "addscalar": y = a + sc
            elif name == "subscalar": y = a - sc
            elif name == "rsubscalar": y = sc - a
            elif name == "mulscalar": y = a * sc
            elif name == "divscalar": y = a / sc
            elif name == "rdivscalar": y = sc / a
            elif name == "maxscalar": y = np.where(a < sc, sc, a)
            elif name == "minscalar": y = np.where(sc < a, sc, a)
            elif name == "sqrt": y = np.sqrt(a)
            elif name == "square": y = a * a
            else: y = a
            y = np.asarray(y, dtype=np.float32)
            results.append(H.to_float(H.to_storage(y.reshape(-1), dt), dt).astype(np.float32).reshape(rows, cols))
    return results


def test_random_mixed_runs_match_the_model(dxh):
    """Random runs of 1..8 ops over up to 8 inputs of mixed dtype (f32, bf16, f16) and extent; ops of
    full extent draw operands of any extent (a vector counts for every row or column), ops on vectors
    only vectors of their kind.  Shapes from one group of four columns to several workgroups, row
    counts that leave the last workgroup ragged."""
    rng = np.random.default_rng(4242)
    dtypes = [dx.F32, dx.BF16, dx.F16]
    names = BINARY + SCALAR + ["sqrt", "square", "copy"]
    for trial in range(40):
        rows, cols = [(1, 4), (3, 8), (7, 36), (64, 256), (33, 1000), (300, 132), (2051, 516)][trial % 7]
        n_in = int(rng.integers(1, 9))
        inputs, host = [], []
        for j in range(n_in):
            dt = dtypes[int(rng.integers(0, 3))]
            e = FULL if rows == 1 or j == 0 else int(rng.integers(0, 3))
            data = H.rand(rng, dt, count(e, rows, cols), 0.25, 2.0)
            inputs.append((Dev(data), dt, e))
            v = H.to_float(data, dt).astype(np.float32)
            host.append(np.broadcast_to(v.reshape(shape_of(e, rows, cols)), (rows, cols)))
        prog, extents = [], []
        for k in range(int(rng.integers(1, 9))):
            e = FULL if rows == 1 else int(rng.choice([FULL, FULL, ROW, COL]))
            fits = [j for j in range(n_in) if e == FULL or inputs[j][2] == e] + [R + j for j in range(k) if e == FULL or extents[j] == e]
            if not fits:
                e = FULL
                fits = list(range(n_in)) + [R + j for j in range(k)]
            pick = lambda: int(fits[int(rng.integers(0, len(fits)))])
            prog.append((str(rng.choice(names)), pick(), pick(), float(rng.choice([0.5, 1.0, 2.0, -1.0, 3.1])), dtypes[int(rng.integers(0, 3))], e))
            extents.append(e)
        rc, got = run_rows(dxh, inputs, prog, rows, cols)
        dx.check(rc, "chain_rows")
        want = model(host, prog, rows, cols)
        for k, (name, _, _, _, dt, e) in enumerate(prog):
            g = H.to_float(got[k].get(), dt).astype(np.float32)
            w = want[k][0, :] if e == ROW else want[k][:, 0] if e == COL else want[k].reshape(-1)
            assert np.array_equal(g, w, equal_nan=True), (trial, rows, cols, k, prog)


def test_long_run_with_many_live_results(dxh):
    """Sixteen ops over eight inputs in which every result is read again three ops later, so that
    nine results are alive beside the inputs: more LDS per workgroup than a launch gets unasked
    (17 slots of 4 KiB), which makes the entry point raise the kernel's limit first.  Against the
    numpy model, and twice in a row (the second launch finds the limit raised)."""
    rng = np.random.default_rng(31)
    rows, cols = 96, 200
    inputs, host = [], []
    for j in range(8):
        dt = [dx.F32, dx.BF16, dx.F16][j % 3]
        data = H.rand(rng, dt, rows * cols, 0.5, 1.5)
        inputs.append((Dev(data), dt, FULL))
        host.append(H.to_float(data, dt).astype(np.float32).reshape(rows, cols))
    prog = []
    for k in range(16):
        name = ["add", "mul", "max", "sub"][k % 4]
        lhs = k % 8 if k < 3 else R + (k - 3)   # a result from three ops back: not the one in registers
        prog.append((name, lhs, (k + 3) % 8, 0.0, [dx.F32, dx.F32, dx.BF16][k % 3], FULL))
    want = model(host, prog, rows, cols)
    for attempt in range(2):
        rc, got = run_rows(dxh, inputs, prog, rows, cols)
        dx.check(rc, "chain_rows")
        for k, (_, _, _, _, dt, _) in enumerate(prog):
            g = H.to_float(got[k].get(), dt).astype(np.float32)
            assert np.array_equal(g, want[k].reshape(-1), equal_nan=True), (attempt, k)


def test_in_place_and_refusals(dxh):
    """A [rows, cols] output may be one of the inputs (a lane reads its own elements before it writes
    them); a vector input may not (DXH_ERR_ARG), nor may an op on vectors read a [rows, cols] tensor."""
    rng = np.random.default_rng(5)
    rows, cols = 48, 64
    a, v = H.rand(rng, dx.F32, rows * cols), H.rand(rng, dx.F32, rows)
    A, Vc = Dev(a), Dev(v)
    prog = [("mul", 0, 1, 0, dx.F32, FULL), ("add", R + 0, 0, 0, dx.F32, FULL)]  # a *= v (per row); c = a_new + a_old
    out2 = Dev.empty(rows * cols, np.float32)
    rc, _ = run_rows(dxh, [(A, dx.F32, FULL), (Vc, dx.F32, COL)], prog, rows, cols, outs=[A, out2])
    dx.check(rc, "chain_rows")
    prod = (a.reshape(rows, cols) * v.reshape(rows, 1)).astype(np.float32)
    assert np.array_equal(A.get().reshape(rows, cols), prod) and np.array_equal(out2.get().reshape(rows, cols), prod + a.reshape(rows, cols))
    rc, _ = run_rows(dxh, [(A, dx.F32, FULL), (Vc, dx.F32, COL)], [("sqrt", 1, 0, 0, dx.F32, COL), ("mul", 0, R + 0, 0, dx.F32, FULL)], rows, cols, outs=[Vc, out2])
    assert rc == -2
    rc, _ = run_rows(dxh, [(A, dx.F32, FULL), (Vc, dx.F32, COL)], [("sqrt", 0, 0, 0, dx.F32, COL)], rows, cols)
    assert rc == -2
