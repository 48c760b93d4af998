"""GPU parity: the runs that libdxhip holds compiled kernels for (the front's RMSNorm, softmax and
SiLU gate as the batch path spells them) against the same runs through the interpreting kernel and
against the separate entry points, each of which is held to the CPU oracle.

Bar: every tensor a run stores is bit-identical three ways (compiled, interpreted where the
interpreter takes the run, separate launches); the separate launches are checked against the oracle
op by op inside run_separately (exact ops bit for bit, exp within 4 ulp, float sums against float64).
"""
import ctypes as C

import numpy as np
import pytest

from deepx_amd import lib as dx
from tests import helpers as H
from tests.helpers import Dev
from tests.test_gpu_chain_rows import COL, FULL, R, ROW, count, run_rows, run_separately, same_bits

pytestmark = pytest.mark.gpu

KNOB_STATIC = 12  # DXH_TUNE_CHAIN_STATIC


def stats(dxh):
    a, b = C.c_int64(), C.c_int64()
    dx.check(dxh.dxh_chain_stats(C.byref(a), C.byref(b)))
    return a.value, b.value


def rmsnorm_prog(half, cols, eps=1e-6):
    return [("copy", 0, 0, 0, dx.F32, FULL), ("square", R + 0, 0, 2.0, dx.F32, FULL), ("rowsum", R + 1, 0, 0, dx.F32, COL),
            ("divscalar", R + 2, 0, float(cols), dx.F32, COL), ("addscalar", R + 3, 0, eps, dx.F32, COL), ("sqrt", R + 4, 0, 0, dx.F32, COL),
            ("rdivscalar", R + 5, 0, 1.0, dx.F32, COL), ("copy", R + 6, 0, 0, dx.F32, FULL), ("mul", R + 0, R + 7, 0, dx.F32, FULL),
            ("copy", 1, 0, 0, dx.F32, ROW), ("copy", R + 9, 0, 0, dx.F32, FULL), ("mul", R + 10, R + 8, 0, dx.F32, FULL),
            ("copy", R + 11, 0, 0, half, FULL)]


def softmax_prog(dt, short=False):
    head = [("rowmax", 0, 0, 0, dt, COL), ("copy", R + 0, 0, 0, dt, FULL), ("sub", 0, R + 1, 0, dt, FULL), ("exp", R + 2, 0, 0, dt, FULL),
            ("rowsum", R + 3, 0, 0, dt, COL)]
    if short:
        return head + [("copy", R + 4, 0, 0, dt, FULL), ("div", R + 3, R + 5, 0, dt, FULL)]
    return head + [("exp", R + 2, 0, 0, dt, FULL), ("copy", R + 4, 0, 0, dt, FULL), ("div", R + 5, R + 6, 0, dt, FULL)]


def three_ways(dxh, orc, ins, prog, rows, cols, label, interpreter_takes_it=True, skip_outs=()):
    """compiled == interpreted == separate launches, for every op of `prog` that stores"""
    want = run_separately(dxh, orc, ins, prog, rows, cols)
    outs = lambda: [None if k in skip_outs else Dev.empty(count(e, rows, cols), H.NP[dt]) for k, (_, _, _, _, dt, e) in enumerate(prog)]
    c0, i0 = stats(dxh)
    rc, got = run_rows(dxh, ins, prog, rows, cols, outs=outs())
    dx.check(rc, label)
    c1, i1 = stats(dxh)
    assert (c1 - c0, i1 - i0) == (1, 0), (label, rows, cols, "the run did not take its compiled kernel")
    for k in range(len(prog)):
        if k not in skip_outs:
            assert same_bits(got[k], want[k]), (label, "compiled vs separate", rows, cols, k, prog[k][0])
    dx.check(dxh.dxh_tune(KNOB_STATIC, 0))
    try:
        rc, got2 = run_rows(dxh, ins, prog, rows, cols, outs=outs())
        c2, i2 = stats(dxh)
        if interpreter_takes_it:
            dx.check(rc, label + " interpreted")
            assert (c2 - c1, i2 - i1) == (0, 1)
            for k in range(len(prog)):
                if k not in skip_outs:
                    assert same_bits(got2[k], want[k]), (label, "interpreted vs separate", rows, cols, k)
        else:
            assert rc in (-1, -3), (label, rc)  # 16-bit row reductions / rows too long for its lane layout
    finally:
        dx.check(dxh.dxh_tune(KNOB_STATIC, 1))


@pytest.mark.parametrize("half", [dx.BF16, dx.F16, dx.F32])
def test_rmsnorm_compiled(dxh, orc, half):
    """The thirteen lines of the front's RMSNorm (t5layernorm.py:17-22) as one compiled launch: rows of 1 to 8
    vectors per lane, rows that end inside a lane's vectors, fewer rows than a workgroup holds, lane groups
    narrower than a wave."""
    rng = np.random.default_rng(700 + half)
    for rows, cols in [(2048, 896), (5, 12), (2, 4), (257, 1000), (33, 2048), (2100, 500), (4099, 260), (1, 64), (300, 1028)]:
        x = Dev(H.rand(rng, half, rows * cols, -2.0, 2.0))
        w = Dev(H.rand(rng, half, cols, 0.5, 1.5))
        prog = rmsnorm_prog(half, cols)
        ins = [(x, half, FULL), (w, half, ROW)]
        takes = bool(dxh.dxh_chain_rows_can_sum(rows, cols))
        three_ways(dxh, orc, ins, prog, rows, cols, "rmsnorm", interpreter_takes_it=takes)
        # as the executor launches it: tensors that a later line of the run overwrites are not stored
        three_ways(dxh, orc, ins, prog, rows, cols, "rmsnorm", interpreter_takes_it=takes, skip_outs=(2, 3, 4, 5, 8))


@pytest.mark.parametrize("dt", [dx.F32, dx.BF16, dx.F16])
@pytest.mark.parametrize("short", [False, True])
def test_softmax_compiled(dxh, orc, dt, short):
    """The front's softmax over the last axis (normalization.py:4-17: reducemax, sub, exp, sum, exp, div with
    the two broadcasts between) as one compiled launch, fp32 and 16-bit, attention-shaped and ragged views."""
    rng = np.random.default_rng(900 + dt + short)
    shapes = [(2048, 2048), (2048, 896), (7, 8), (300, 1000), (1, 16), (515, 264), (64, 4096 if dt != dx.F32 else 1536)]
    for rows, cols in shapes:
        span = 6.0 if dt == dx.F32 else 3.0  # a 16-bit difference t - max carries an absolute error that exp turns into a relative one
        t = H.rand(rng, dt, rows * cols, -span, span).reshape(rows, cols)
        if rows > 2:  # ties and signed zeros in the maximum, a row of one repeated value
            t[1, :] = t[1, 0]
            t[2, :3] = H.to_storage(np.array([0.0, -0.0, 0.0]), dt)
            t[2, 3:] = H.to_storage(np.full(cols - 3, -1.0), dt)
        ins = [(Dev(t.reshape(-1)), dt, FULL)]
        prog = softmax_prog(dt, short)
        takes = dt == dx.F32 and bool(dxh.dxh_chain_rows_can_sum(rows, cols))
        three_ways(dxh, orc, ins, prog, rows, cols, "softmax", interpreter_takes_it=takes)
        # the result against the textbook formula in float64 (every row sums to one)
        rc, got = run_rows(dxh, ins, prog, rows, cols)
        y = H.to_float(got[-1].get(), dt).reshape(rows, cols)
        x64 = H.to_float(t.reshape(-1), dt).reshape(rows, cols)
        e = np.exp(x64 - x64.max(1, keepdims=True))
        ref = e / e.sum(1, keepdims=True)
        tol = 1e-5 if dt == dx.F32 else 2.0 ** -4 if dt == dx.BF16 else 2.0 ** -7
        floor = 1e-7 if dt == dx.F16 else 1e-30  # results under 6e-5 are subnormal in float16
        assert np.all(np.abs(y - ref) <= tol * ref + floor), (rows, cols, float(np.max(np.abs(y - ref) / (ref + floor))))


@pytest.mark.parametrize("dt", [dx.F32, dx.BF16, dx.F16])
def test_scaled_softmax_compiled(dxh, orc, dt):
    """Attention weights as the front computes them (attention.py:15,24): the scores times the scaling factor, then the
    softmax's eight lines on the product — nine lines, one compiled launch, every stored tensor with the bits of nine
    separate launches, and the result against the formula in float64."""
    rng = np.random.default_rng(950 + dt)
    scale = 64 ** -0.5
    for rows, cols in [(14 * 256, 2048), (2048, 896), (7, 8), (300, 1000), (1, 16), (515, 264)]:
        span = 40.0 if dt == dx.F32 else 20.0
        t = H.rand(rng, dt, rows * cols, -span, span)
        ins = [(Dev(t), dt, FULL)]
        shifted = [(name, l + 1 if l >= R else R + 0, r + 1 if r >= R else r, s, d, e) for name, l, r, s, d, e in softmax_prog(dt)]
        prog = [("mulscalar", 0, 0, scale, dt, FULL)] + shifted
        takes = dt == dx.F32 and bool(dxh.dxh_chain_rows_can_sum(rows, cols))
        three_ways(dxh, orc, ins, prog, rows, cols, "scaled softmax", interpreter_takes_it=takes)
        rc, got = run_rows(dxh, ins, prog, rows, cols)
        y = H.to_float(got[-1].get(), dt).reshape(rows, cols)
        a64 = H.to_float(got[0].get(), dt).reshape(rows, cols).astype(np.float64)  # the stored product, as the softmax sees it
        x64 = H.to_float(t, dt).reshape(rows, cols).astype(np.float64)
        assert np.all(np.abs(a64 - x64 * scale) <= np.abs(x64 * scale) * (2.0 ** -23 if dt == dx.F32 else 2.0 ** -8 if dt == dx.BF16 else 2.0 ** -11) + (2.0 ** -24 if dt == dx.F16 else 1e-30))  # float16 products under 6e-5 are subnormal
        e = np.exp(a64 - a64.max(1, keepdims=True))
        ref = e / e.sum(1, keepdims=True)
        tol = 1e-5 if dt == dx.F32 else 2.0 ** -4 if dt == dx.BF16 else 2.0 ** -7
        floor = 1e-7 if dt == dx.F16 else 1e-30
        assert np.all(np.abs(y - ref) <= tol * ref + floor), (rows, cols, float(np.max(np.abs(y - ref) / (ref + floor))))


def test_softmax_nan_and_infinities_follow_the_separate_kernels(dxh, orc):
    """reducemax is (a < b) ? b : a in the kernel's own order: where a NaN sits in a row decides whether it
    wins.  The compiled run must agree with the separate launch on every such row."""
    rows, cols = 64, 1024
    rng = np.random.default_rng(77)
    t = rng.uniform(-3, 3, (rows, cols)).astype(np.float32)
    for r in range(rows):
        t[r, (r * 37) % cols] = np.nan if r % 3 == 0 else np.inf if r % 3 == 1 else -np.inf
    ins = [(Dev(t.reshape(-1)), dx.F32, FULL)]
    prog = softmax_prog(dx.F32)[:3]
    want = run_rows_separately_bits(dxh, ins, prog, rows, cols)
    rc, got = run_rows(dxh, ins, softmax_prog(dx.F32), rows, cols)
    dx.check(rc)
    for k in range(3):
        assert same_bits(got[k], want[k]), k


def run_rows_separately_bits(dxh, ins, prog, rows, cols):
    """reducemax, broadcastTo, sub through their own entry points (no oracle: NaN rows)"""
    t = ins[0][0]
    m, mb, d = Dev.empty(rows, np.float32), Dev.empty(rows * cols, np.float32), Dev.empty(rows * cols, np.float32)
    dx.check(dxh.dxh_reducemax(dx.F32, t.ptr, dx.i32arr([rows, cols]), 2, dx.i32arr([1]), 1, m.ptr, None, 0, None))
    dx.check(dxh.dxh_broadcastTo(dx.F32, m.ptr, dx.i32arr([rows, 1]), 2, dx.i32arr([rows, cols]), 2, mb.ptr, None))
    dx.check(dxh.dxh_sub(dx.F32, t.ptr, mb.ptr, d.ptr, rows * cols, None))
    return [m, mb, d]


@pytest.mark.parametrize("dt", [dx.F32, dx.BF16, dx.F16])
def test_silu_gate_compiled(dxh, orc, dt):
    """The six lines of the front's SiLU gate (activite.py:11-18, gatedmlp.py:20-26) through dxh_chain: the compiled
    kernel, the interpreting one and the separate launches store the same bits."""
    rng = np.random.default_rng(60 + dt)
    for n in (2048 * 4864, 4096, 8 * 1031):
        g, u = Dev(H.rand(rng, dt, n, -8.0, 8.0)), Dev(H.rand(rng, dt, n, -2.0, 2.0))
        prog = [("mulscalar", 0, 0, -1.0), ("exp", R + 0, 0, 0), ("addscalar", R + 1, 0, 1.0), ("rdivscalar", R + 2, 0, 1.0), ("mul", 0, R + 3, 0), ("mul", R + 4, 1, 0)]

        def run(store_all):
            outs = [Dev.empty(n, H.NP[dt]) if (store_all or k == len(prog) - 1) else None for k in range(len(prog))]
            ops = (dx.ChainOp * len(prog))(*[dx.ChainOp(dx.CHAIN_CODES.index(nm), l, r, dx.scalar(s), outs[k].ptr if outs[k] is not None else None)
                                             for k, (nm, l, r, s) in enumerate(prog)])
            dx.check(dxh.dxh_chain(dt, (C.c_void_p * 2)(g.ptr, u.ptr), 2, ops, len(prog), n, None), "chain")
            return outs

        c0, i0 = stats(dxh)
        comp = run(True)
        last = run(False)
        assert stats(dxh) == (c0 + 2, i0)
        dx.check(dxh.dxh_tune(KNOB_STATIC, 0))
        try:
            interp = run(True)
            assert stats(dxh) == (c0 + 2, i0 + 1)
        finally:
            dx.check(dxh.dxh_tune(KNOB_STATIC, 1))
        # separate launches
        sep = []
        cur = Dev.empty(n, H.NP[dt]); dx.check(dxh.dxh_mulscalar(dt, g.ptr, dx.scalar(-1.0), cur.ptr, n, None)); sep.append(cur)
        cur = Dev.empty(n, H.NP[dt]); dx.check(dxh.dxh_exp(dt, sep[0].ptr, cur.ptr, n, None)); sep.append(cur)
        cur = Dev.empty(n, H.NP[dt]); dx.check(dxh.dxh_addscalar(dt, sep[1].ptr, dx.scalar(1.0), cur.ptr, n, None)); sep.append(cur)
        cur = Dev.empty(n, H.NP[dt]); dx.check(dxh.dxh_rdivscalar(dt, dx.scalar(1.0), sep[2].ptr, cur.ptr, n, None)); sep.append(cur)
        cur = Dev.empty(n, H.NP[dt]); dx.check(dxh.dxh_mul(dt, g.ptr, sep[3].ptr, cur.ptr, n, None)); sep.append(cur)
        cur = Dev.empty(n, H.NP[dt]); dx.check(dxh.dxh_mul(dt, sep[4].ptr, u.ptr, cur.ptr, n, None)); sep.append(cur)
        for k in range(len(prog)):
            assert same_bits(comp[k], sep[k]) and same_bits(interp[k], sep[k]), (n, k)
        assert same_bits(last[-1], sep[-1])
        # and the value: silu(g) * u in float64, a handful of roundings to the dtype away
        g64, u64 = H.to_float(g.get(), dt), H.to_float(u.get(), dt)
        ref = g64 / (1.0 + np.exp(-g64)) * u64
        tol = 1e-5 if dt == dx.F32 else 2.0 ** -5 if dt == dx.BF16 else 2.0 ** -8
        assert np.all(np.abs(H.to_float(comp[-1].get(), dt) - ref) <= tol * np.abs(ref) + 1e-6)


@pytest.mark.parametrize("dt", [dx.F32, dx.BF16, dx.F16])
@pytest.mark.parametrize("gated", [True, False, "sigmoid"])
def test_swish_as_the_front_spells_it(dxh, orc, dt, gated):
    """swish(x, beta) of the front is x * sigmoid(x * beta) with sigmoid(t) = 1 / (exp(t * -1) + 1) (activite.py:10-16):
    one more mulscalar in front of the sequence above, seven lines with the gate's `* up`.  Compiled, interpreted
    and as separate launches: the same bits in every tensor."""
    rng = np.random.default_rng(70 + dt)
    for n, beta in ((2048 * 896, 1.0), (8 * 1031, 1.702)):
        x, u = Dev(H.rand(rng, dt, n, -6.0, 6.0)), Dev(H.rand(rng, dt, n, -2.0, 2.0))  # exp(6 * 1.702) still fits float16
        prog = [("mulscalar", 0, 0, beta), ("mulscalar", R + 0, 0, -1.0), ("exp", R + 1, 0, 0), ("addscalar", R + 2, 0, 1.0),
                ("rdivscalar", R + 3, 0, 1.0), ("mul", 0, R + 4, 0)] + ([("mul", R + 5, 1, 0)] if gated is True else [])
        if gated == "sigmoid":  # sigmoid on its own (activite.py:10-12): 1 / (exp(t * -1) + 1), four lines
            prog = [("mulscalar", 0, 0, -1.0), ("exp", R + 0, 0, 0), ("addscalar", R + 1, 0, 1.0), ("rdivscalar", R + 2, 0, 1.0)]
        ins = [x, u] if gated is True else [x]

        def run():
            outs = [Dev.empty(n, H.NP[dt]) for _ in prog]
            ops = (dx.ChainOp * len(prog))(*[dx.ChainOp(dx.CHAIN_CODES.index(nm), l, r, dx.scalar(s), outs[k].ptr) for k, (nm, l, r, s) in enumerate(prog)])
            dx.check(dxh.dxh_chain(dt, (C.c_void_p * len(ins))(*[t.ptr for t in ins]), len(ins), ops, len(prog), n, None), "chain")
            return outs

        c0, i0 = stats(dxh)
        comp = run()
        assert stats(dxh) == (c0 + 1, i0)
        dx.check(dxh.dxh_tune(KNOB_STATIC, 0))
        try:
            interp = run()
            assert stats(dxh) == (c0 + 1, i0 + 1)
        finally:
            dx.check(dxh.dxh_tune(KNOB_STATIC, 1))
        sep = []
        for k, (nm, l, r, sc) in enumerate(prog):
            a = ins[l] if l < R else sep[l - R]
            out = Dev.empty(n, H.NP[dt])
            if nm == "mul":
                b = ins[r] if r < R else sep[r - R]
                dx.check(dxh.dxh_mul(dt, a.ptr, b.ptr, out.ptr, n, None))
            elif nm == "exp":
                dx.check(dxh.dxh_exp(dt, a.ptr, out.ptr, n, None))
            elif nm == "rdivscalar":
                dx.check(dxh.dxh_rdivscalar(dt, dx.scalar(sc), a.ptr, out.ptr, n, None))
            else:
                dx.check(getattr(dxh, "dxh_" + nm)(dt, a.ptr, dx.scalar(sc), out.ptr, n, None))
            sep.append(out)
        for k in range(len(prog)):
            assert same_bits(comp[k], sep[k]) and same_bits(interp[k], sep[k]), (n, k)
        x64 = H.to_float(x.get(), dt)
        ref = x64 / (1.0 + np.exp(-x64 * H.to_float(H.to_storage(np.array([beta]), dt), dt)[0]))
        if gated == "sigmoid":
            ref, beta = 1.0 / (1.0 + np.exp(-x64)), 1.0
        elif gated:
            ref = ref * H.to_float(u.get(), dt)
        # the rounding of x * beta to the dtype is a relative error of the exponent: exp turns it into |x beta| times as much
        tol = 1e-5 if dt == dx.F32 else 2.0 ** -5 if dt == dx.BF16 else 2.0 ** -8
        assert np.all(np.abs(H.to_float(comp[-1].get(), dt) - ref) <= tol * (1.0 + np.abs(x64 * beta)) * np.abs(ref) + 1e-6)


def test_attention_sized_softmax_compiled_equals_separate(dxh):
    """[14 * 2048, 2048] fp32 scores (one head group of the BASELINE attention shape): the compiled softmax against
    the separate launches, compared on the device."""
    import torch
    rows, cols = 14 * 2048, 2048
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    t = torch.randn(rows, cols, generator=g, device="cuda") * 3
    p = lambda x: C.c_void_p(x.data_ptr())
    names = ["m", "mb", "d", "e", "s", "e2", "sb", "y"]
    sep = {n: torch.empty((rows, 1) if n in ("m", "s") else (rows, cols), device="cuda") for n in names}
    sh, ax, col_sh = dx.i32arr([rows, cols]), dx.i32arr([1]), dx.i32arr([rows, 1])
    n = rows * cols
    dx.check(dxh.dxh_reducemax(dx.F32, p(t), sh, 2, ax, 1, p(sep["m"]), None, 0, None))
    dx.check(dxh.dxh_broadcastTo(dx.F32, p(sep["m"]), col_sh, 2, sh, 2, p(sep["mb"]), None))
    dx.check(dxh.dxh_sub(dx.F32, p(t), p(sep["mb"]), p(sep["d"]), n, None))
    dx.check(dxh.dxh_exp(dx.F32, p(sep["d"]), p(sep["e"]), n, None))
    dx.check(dxh.dxh_sum(dx.F32, p(sep["e"]), sh, 2, ax, 1, p(sep["s"]), None, 0, None))
    dx.check(dxh.dxh_exp(dx.F32, p(sep["d"]), p(sep["e2"]), n, None))
    dx.check(dxh.dxh_broadcastTo(dx.F32, p(sep["s"]), col_sh, 2, sh, 2, p(sep["sb"]), None))
    dx.check(dxh.dxh_div(dx.F32, p(sep["e2"]), p(sep["sb"]), p(sep["y"]), n, None))
    got = {k: torch.empty_like(v) for k, v in sep.items()}
    prog = softmax_prog(dx.F32)
    tin = (dx.ChainTensor * 1)(dx.ChainTensor(t.data_ptr(), dx.F32, FULL))
    ops = (dx.ChainRowsOp * len(prog))(*[dx.ChainRowsOp(dx.CHAIN_CODES.index(nm), l, r, dx.scalar(s), got[names[k]].data_ptr(), dt, e)
                                         for k, (nm, l, r, s, dt, e) in enumerate(prog)])
    c0, i0 = stats(dxh)
    dx.check(dxh.dxh_chain_rows(tin, 1, ops, len(prog), rows, cols, None))
    assert stats(dxh) == (c0 + 1, i0)
    torch.cuda.synchronize()
    for k in names:
        assert torch.equal(got[k].view(torch.int32), sep[k].view(torch.int32)), k
    assert torch.allclose(got["y"].sum(1), torch.ones(rows, device="cuda"), atol=1e-5)
