"""GPU parity: dxh_chain (a run of elementwise ops in one launch) against the CPU oracle and
against the separate entry points.

Bars: every output of a run is compared op by op with the oracle applied to the operands the
device used for that op (so errors do not compound): bit-exact for add / sub / mul / div / max /
min, their scalar forms and sqrt (correctly rounded on both sides), <= 4 ulp for exp and log
(glibc on the host, ROCm's device libm here; 16-bit floats compute in fp32 and round once, which
leaves at most 1 ulp of the storage type).  And bit-identical to what add / mulscalar / exp ...
store when called one after another.
"""
import ctypes as C

import numpy as np
import pytest

from deepx_amd import lib as dx
from tests import helpers as H
from tests.helpers import Dev, hp

pytestmark = pytest.mark.gpu

BINARY = ["add", "sub", "mul", "div", "max", "min"]
SCALAR = ["addscalar", "subscalar", "rsubscalar", "mulscalar", "divscalar", "rdivscalar", "maxscalar", "minscalar"]
UNARY = ["sqrt", "exp", "log"]
VEC = {dx.F64: 2, dx.F32: 4, dx.F16: 8, dx.BF16: 8}


def run_separately(dxh, dtype, inputs, prog, n):
    """prog: list of (name, lhs, rhs, scalar); refs < 16 are inputs, 16 + j results.  Returns device outputs."""
    outs = []
    for name, lhs, rhs, s in prog:
        src = lambda r: inputs[r] if r < dx.CHAIN_RESULT else outs[r - dx.CHAIN_RESULT]
        out = Dev.empty(n, H.NP[dtype])
        fn = getattr(dxh, "dxh_" + name)
        if name in BINARY:
            dx.check(fn(dtype, src(lhs).ptr, src(rhs).ptr, out.ptr, n, None), name)
        elif name in ("rsubscalar", "rdivscalar"):
            dx.check(fn(dtype, dx.scalar(s), src(lhs).ptr, out.ptr, n, None), name)
        elif name in SCALAR:
            dx.check(fn(dtype, src(lhs).ptr, dx.scalar(s), out.ptr, n, None), name)
        else:
            dx.check(fn(dtype, src(lhs).ptr, out.ptr, n, None), name)
        outs.append(out)
    return outs


def run_chain(dxh, dtype, inputs, prog, n, outs=None):
    outs = outs or [Dev.empty(n, H.NP[dtype]) for _ in prog]
    ops = (dx.ChainOp * len(prog))()
    for k, (name, lhs, rhs, s) in enumerate(prog):
        ops[k] = dx.ChainOp(dx.CHAIN_CODES.index(name), lhs, rhs, dx.scalar(s), outs[k].ptr if outs[k] is not None else None)
    ptrs = (C.c_void_p * max(1, len(inputs)))(*[d.ptr for d in inputs])
    return dxh.dxh_chain(dtype, ptrs, len(inputs), ops, len(prog), n, None), outs


def check_against_oracle(orc, dtype, inputs, prog, outs, n, what):
    """Op k of the run on the oracle, fed with the device's own operands of that op."""
    host_in = [d.get() for d in inputs]
    host_out = [o.get() for o in outs]
    for k, (name, lhs, rhs, s) in enumerate(prog):
        src = lambda r: host_in[r] if r < dx.CHAIN_RESULT else host_out[r - dx.CHAIN_RESULT]
        want = np.empty(n, dtype=H.NP[dtype])
        fn = getattr(orc, "orc_" + name)
        if name in BINARY:
            rc = fn(dtype, hp(src(lhs)), hp(src(rhs)), hp(want), n)
        elif name in ("rsubscalar", "rdivscalar"):
            rc = fn(dtype, dx.scalar(s), hp(src(lhs)), hp(want), n)
        elif name in SCALAR:
            rc = fn(dtype, hp(src(lhs)), dx.scalar(s), hp(want), n)
        else:
            rc = fn(dtype, hp(src(lhs)), hp(want), n)
        assert rc == 0, (name, rc)
        if name in ("exp", "log"):
            ulps = H.ulp_diff(host_out[k], want, dtype)
            assert ulps <= (4 if dtype in (dx.F32, dx.F64) else 1), (what, dtype, k, name, ulps)
        else:
            same = (host_out[k].view(np.uint8) == want.view(np.uint8)).all() or \
                np.array_equal(host_out[k], want, equal_nan=dtype in (dx.F32, dx.F64))
            if not same and dtype in (dx.F16, dx.BF16):  # NaN payloads aside, the bits must agree
                f, w = H.to_float(host_out[k], dtype), H.to_float(want, dtype)
                same = np.array_equal(np.isnan(f), np.isnan(w)) and np.array_equal(host_out[k][~np.isnan(w)], want[~np.isnan(w)])
            assert same, (what, dtype, k, name)


def same_bits(a, b):
    return np.array_equal(a.get().view(np.uint8), b.get().view(np.uint8))


def same_bits_nans_aside(a, b, dtype):
    """the same bits wherever the result is a number, and NaN in the same places: which NaN an op returns (sign, payload) is
    the compiler's choice per kernel — sqrt of a negative float16 comes back as 0x7e00 from one kernel and 0xfe00 from another"""
    x, y = a.get(), b.get()
    if np.array_equal(x.view(np.uint8), y.view(np.uint8)):
        return True
    fx, fy = H.to_float(x, dtype), H.to_float(y, dtype)
    nan = np.isnan(fx)
    return bool(nan.any()) and np.array_equal(nan, np.isnan(fy)) and np.array_equal(x[~nan], y[~nan])


@pytest.mark.parametrize("dtype", [dx.F32, dx.BF16, dx.F16, dx.F64])
def test_config1_chain_in_one_launch(dxh, orc, dtype):
    """The 8-op elementwise chain of BASELINE config 1 (abs composed from mulscalar and max) and
    the SiLU gate of config 5, each as one run; every intermediate tensor against the oracle and
    bit-identical to the separate kernels."""
    rng = np.random.default_rng(40 + dtype)
    n = 1 << 18
    A, B = Dev(H.rand(rng, dtype, n)), Dev(H.rand(rng, dtype, n))
    R = dx.CHAIN_RESULT
    c1 = [("add", 0, 1, 0), ("mul", R + 0, 1, 0), ("addscalar", R + 1, 0, 0.5), ("exp", R + 2, 0, 0),
          ("mulscalar", 1, 0, -1), ("max", 1, R + 4, 0), ("addscalar", R + 5, 0, 1), ("div", R + 3, R + 6, 0)]
    silu = [("mulscalar", 0, 0, -1), ("exp", R + 0, 0, 0), ("addscalar", R + 1, 0, 1), ("rdivscalar", R + 2, 0, 1),
            ("mul", 0, R + 3, 0), ("mul", R + 4, 1, 0)]
    for prog in (c1, silu):
        want = run_separately(dxh, dtype, [A, B], prog, n)
        rc, got = run_chain(dxh, dtype, [A, B], prog, n)
        dx.check(rc, "chain")
        check_against_oracle(orc, dtype, [A, B], prog, got, n, "config chain")
        for k, (g, w) in enumerate(zip(got, want)):
            assert same_bits(g, w), (dtype, prog[k][0], k)


@pytest.mark.parametrize("dtype", [dx.F32, dx.BF16, dx.F16, dx.F64])
def test_random_runs_match_separate_calls(dxh, orc, dtype):
    """Random runs of 1..8 ops over up to 8 inputs, every op code, operands drawn from inputs and
    earlier results; sizes from one vector to several workgroups."""
    rng = np.random.default_rng(700 + dtype)
    v = VEC[dtype]
    for trial in range(12):
        n = int(rng.choice([v, 3 * v, 256 * v, 256 * v * 5 + 7 * v, 1 << 17]))
        n_in = int(rng.integers(1, 9))
        inputs = [Dev(H.rand(rng, dtype, n, 0.25, 2.0)) for _ in range(n_in)]
        prog = []
        for k in range(int(rng.integers(1, 9))):
            name = str(rng.choice(BINARY + SCALAR + UNARY))
            ref = lambda: int(rng.integers(0, n_in)) if (k == 0 or rng.random() < 0.5) else dx.CHAIN_RESULT + int(rng.integers(0, k))
            prog.append((name, ref(), ref(), float(rng.choice([0.5, 1.0, 2.0, -1.0, 3.1]))))
        want = run_separately(dxh, dtype, inputs, prog, n)
        rc, got = run_chain(dxh, dtype, inputs, prog, n)
        dx.check(rc, "chain")
        check_against_oracle(orc, dtype, inputs, prog, got, n, ("random run", trial, n))
        for k, (g, w) in enumerate(zip(got, want)):
            assert same_bits_nans_aside(g, w, dtype), (dtype, trial, n, prog, k)


def test_in_place_and_argument_checks(dxh):
    """An output may be one of the inputs (inputs are read before anything is written); bad
    operand references, op codes, counts, alignment and dtypes are refused without a launch."""
    rng = np.random.default_rng(9)
    n = 4096
    a, b = H.rand(rng, dx.F32, n), H.rand(rng, dx.F32, n)
    A, B = Dev(a), Dev(b)
    R = dx.CHAIN_RESULT
    prog = [("add", 0, 1, 0), ("mul", R + 0, 0, 0)]  # a += b; c = a_new * a_old
    out2 = Dev.empty(n, np.float32)
    rc, _ = run_chain(dxh, dx.F32, [A, B], prog, n, outs=[A, out2])
    dx.check(rc, "chain")
    assert np.array_equal(A.get(), a + b) and np.array_equal(out2.get(), (a + b) * a)
    # results that are not stored (out = NULL) still feed later ops; the last op must store
    keep = Dev.empty(n, np.float32)
    silu = [("mulscalar", 0, 0, -1), ("exp", R + 0, 0, 0), ("addscalar", R + 1, 0, 1), ("rdivscalar", R + 2, 0, 1), ("mul", 0, R + 3, 0)]
    want = run_separately(dxh, dx.F32, [B], silu, n)[-1]
    rc, _ = run_chain(dxh, dx.F32, [B], silu, n, outs=[None, None, None, None, keep])
    dx.check(rc, "chain")
    assert np.array_equal(keep.get().view(np.uint32), want.get().view(np.uint32))
    rc, _ = run_chain(dxh, dx.F32, [B], silu[:2], n, outs=[keep, None])
    assert rc == -2
    o = Dev.empty(n, np.float32)
    bad = [([("add", 0, 5, 0)], dx.F32, n, -2),             # input that is not there
           ([("add", 0, R + 0, 0)], dx.F32, n, -2),         # its own result
           ([("exp", 0, 0, 0)] * 9, dx.F32, n, -2),         # too many ops
           ([("add", 0, 1, 0)], dx.I32, n, -1),             # integer dtype
           ([("add", 0, 1, 0)], dx.F32, n - 1, -5)]         # not a whole number of vectors
    for prog, dtype, cnt, want in bad:
        rc, _ = run_chain(dxh, dtype, [A, B], prog, cnt, outs=[o] * len(prog))
        assert rc == want, (prog, rc)
    ops = (dx.ChainOp * 1)(dx.ChainOp(99, 0, 0, dx.scalar(0), o.ptr))
    ptrs = (C.c_void_p * 2)(A.ptr, B.ptr)
    assert dxh.dxh_chain(dx.F32, ptrs, 2, ops, 1, n, None) == -2
    assert dxh.dxh_chain(dx.F32, ptrs, 2, ops, 0, n, None) == -2
