"""GPU parity: libdxhip elementwise / compare / switch / todtype / init vs the CPU oracle.

Bars: bit-exact for integer, compare, select and cast ops and for fp add/sub/mul/div/sqrt/
max/min (IEEE correctly rounded on both sides); <= 4 ulp for transcendentals (the oracle is
glibc libm, the device is ROCm's device libm).
"""
import ctypes as C

import numpy as np
import pytest

from deepx_amd import lib as dx
from tests import helpers as H
from tests.helpers import Dev, hp

pytestmark = pytest.mark.gpu

# sizes: vector body + ragged tail, one below a vector, several grid-stride trips
SIZES = [1, 3, 17, 1000, 4096, 262144 + 5, (1 << 21) + 3]


def run_binary(dxh, orc, name, dtype, a, b):
    n = a.size
    da, db, dc = Dev(a), Dev(b), Dev.empty(n, a.dtype)
    dx.check(getattr(dxh, "dxh_" + name)(dtype, da.ptr, db.ptr, dc.ptr, n, None), name)
    want = np.empty_like(a)
    assert getattr(orc, "orc_" + name)(dtype, hp(a), hp(b), hp(want), n) == 0
    return dc.get(), want


@pytest.mark.parametrize("name", ["add", "sub", "mul", "div", "max", "min"])
@pytest.mark.parametrize("dtype", H.ALL_NUMERIC)
def test_binary_bit_exact(dxh, orc, name, dtype):
    rng = np.random.default_rng(1000 + dtype)
    for n in SIZES:
        a, b = H.rand(rng, dtype, n), H.rand(rng, dtype, n)
        if name == "div" and dtype in H.INTS:
            b[::7] = 0  # division by zero is defined (0) on both sides
        got, want = run_binary(dxh, orc, name, dtype, a, b)
        assert np.array_equal(got, want), f"{name} {dx.DTYPE_NAMES[dtype]} n={n}"


def test_int_wraparound(dxh, orc):
    for dtype in H.INTS:
        info = np.iinfo(H.NP[dtype])
        a = np.array([info.max, info.min, info.max, info.min, -1, 0, info.min], dtype=H.NP[dtype])
        b = np.array([1, -1, info.max, info.min, info.min, 0, -1], dtype=H.NP[dtype])
        for name in ["add", "sub", "mul", "div"]:
            got, want = run_binary(dxh, orc, name, dtype, a, b)
            assert np.array_equal(got, want), (name, dtype)


@pytest.mark.parametrize("dtype", [dx.F32, dx.F64])
def test_pow(dxh, orc, dtype):
    rng = np.random.default_rng(7)
    n = 100003
    a = H.to_storage(rng.uniform(0.1, 4.0, n), dtype)
    b = H.to_storage(rng.uniform(-3.0, 3.0, n), dtype)
    got, want = run_binary(dxh, orc, "pow", dtype, a, b)
    assert H.ulp_diff(got, want, dtype) <= 4


SCALAR_OPS = ["addscalar", "subscalar", "rsubscalar", "mulscalar", "divscalar", "rdivscalar", "maxscalar", "minscalar"]


def run_scalar(dxh, orc, name, dtype, a, s):
    n = a.size
    da, dc = Dev(a), Dev.empty(n, a.dtype)
    sc = dx.scalar(s)
    f, g = getattr(dxh, "dxh_" + name), getattr(orc, "orc_" + name)
    want = np.empty_like(a)
    if name.startswith("r"):
        dx.check(f(dtype, sc, da.ptr, dc.ptr, n, None), name)
        assert g(dtype, sc, hp(a), hp(want), n) == 0
    else:
        dx.check(f(dtype, da.ptr, sc, dc.ptr, n, None), name)
        assert g(dtype, hp(a), sc, hp(want), n) == 0
    return dc.get(), want


@pytest.mark.parametrize("name", SCALAR_OPS)
@pytest.mark.parametrize("dtype", H.ALL_NUMERIC)
def test_scalar_bit_exact(dxh, orc, name, dtype):
    rng = np.random.default_rng(2000 + dtype)
    for n in [5, 4099, 300001]:
        a = H.rand(rng, dtype, n)
        if name == "rdivscalar" and dtype in H.INTS:
            a[::5] = 0
        for s in ([0.5, -3.0] if dtype in H.FLOATS else [3, -7]):
            got, want = run_scalar(dxh, orc, name, dtype, a, s)
            assert np.array_equal(got, want), f"{name} {dx.DTYPE_NAMES[dtype]} n={n} s={s}"


@pytest.mark.parametrize("dtype", [dx.F32, dx.F64])
def test_powscalar(dxh, orc, dtype):
    rng = np.random.default_rng(8)
    a = H.to_storage(rng.uniform(0.1, 4.0, 65537), dtype)
    for name, s in [("powscalar", 2.0), ("powscalar", 0.5), ("rpowscalar", 2.0), ("rpowscalar", 1.5)]:
        got, want = run_scalar(dxh, orc, name, dtype, a, s)
        assert H.ulp_diff(got, want, dtype) <= 4, (name, s)
    # x**2 must equal x*x to 1 ulp (closed form)
    got, _ = run_scalar(dxh, orc, "powscalar", dtype, a, 2.0)
    assert H.ulp_diff(got, (a * a).astype(a.dtype), dtype) <= 1
    # the square has its own kernel: special values must come out as pow(x, 2) gives them
    sp = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, -3.0, 1e-30, -1e30, 1e30, np.finfo(a.dtype).tiny], dtype=a.dtype)
    got, want = run_scalar(dxh, orc, "powscalar", dtype, sp, 2.0)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok], want[ok]) and np.array_equal(np.signbit(got[ok]), np.signbit(want[ok])), (got, want)


def run_unary(dxh, orc, name, dtype, a):
    n = a.size
    da, dc = Dev(a), Dev.empty(n, a.dtype)
    dx.check(getattr(dxh, "dxh_" + name)(dtype, da.ptr, dc.ptr, n, None), name)
    want = np.empty_like(a)
    assert getattr(orc, "orc_" + name)(dtype, hp(a), hp(want), n) == 0
    return dc.get(), want


@pytest.mark.parametrize("dtype", H.FLOATS)
def test_sqrt_bit_exact(dxh, orc, dtype):
    rng = np.random.default_rng(9)
    a = H.to_storage(rng.uniform(0.0, 100.0, 100001), dtype)
    got, want = run_unary(dxh, orc, "sqrt", dtype, a)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("name,lo,hi", [("exp", -10.0, 10.0), ("log", 1e-3, 100.0), ("sin", -6.0, 6.0),
                                        ("cos", -6.0, 6.0), ("tan", -1.5, 1.5)])
@pytest.mark.parametrize("dtype", H.FLOATS)
def test_transcendental_4ulp(dxh, orc, name, lo, hi, dtype):
    if name == "tan" and dtype in (dx.F16, dx.BF16):
        a = H.to_storage(np.zeros(4), dtype)
        assert dxh.dxh_tan(dtype, Dev(a).ptr, Dev(a).ptr, 4, None) == -1  # DXH_ERR_DTYPE, as op-cuda
        return
    rng = np.random.default_rng(10)
    a = H.to_storage(rng.uniform(lo, hi, 200003), dtype)
    got, want = run_unary(dxh, orc, name, dtype, a)
    assert H.ulp_diff(got, want, dtype) <= 4, f"{name} {dx.DTYPE_NAMES[dtype]}"


@pytest.mark.parametrize("dtype", [dx.BF16, dx.F16])
def test_exp_every_16bit_input(dxh, orc, dtype):
    """exp of a 16-bit float runs on the hardware's exp2 instead of the fp32 expansion.  Every one of
    the 65,536 input patterns: within one unit in the last place of the oracle's expf rounded once,
    NaN where it has NaN, and the same zeros, infinities and denormal results."""
    a = np.arange(65536, dtype=np.uint32).astype(np.uint16).view(H.NP[dtype])
    got, want = run_unary(dxh, orc, "exp", dtype, a)
    gf, wf = H.to_float(got, dtype), H.to_float(want, dtype)
    assert np.array_equal(np.isnan(gf), np.isnan(wf))
    assert np.array_equal(np.isinf(gf), np.isinf(wf))
    assert np.array_equal(gf == 0.0, wf == 0.0)
    assert H.ulp_diff(got, want, dtype) <= 1
    differing = np.count_nonzero(got.view(np.uint16) != want.view(np.uint16)) - np.count_nonzero(np.isnan(gf))
    assert differing <= 65536 * 0.05, differing


def _same_nans_aside(got, want, dtype):
    gf, wf = H.to_float(got, dtype), H.to_float(want, dtype)
    nan = np.isnan(wf)
    return np.array_equal(np.isnan(gf), nan) and np.array_equal(got.view(np.uint16)[~nan], want.view(np.uint16)[~nan])


@pytest.mark.parametrize("dtype", [dx.BF16, dx.F16])
def test_every_16bit_input_through_the_unary_ops(dxh, orc, dtype):
    """All 65,536 patterns of a 16-bit float — zeros, denormals, infinities, NaNs, negatives — through sqrt (the oracle's
    bits, NaN for NaN) and through log, sin and cos (NaN and infinities where the oracle has them, finite results within
    one unit in the last place; in fact all but a handful of float16 logarithms have the oracle's bits)."""
    a = np.arange(65536, dtype=np.uint32).astype(np.uint16).view(H.NP[dtype])
    got, want = run_unary(dxh, orc, "sqrt", dtype, a)
    assert _same_nans_aside(got, want, dtype)
    for name in ("log", "sin", "cos"):
        got, want = run_unary(dxh, orc, name, dtype, a)
        gf, wf = H.to_float(got, dtype), H.to_float(want, dtype)
        assert np.array_equal(np.isnan(gf), np.isnan(wf)), name
        inf = np.isinf(wf)
        assert np.array_equal(np.isinf(gf), inf) and np.array_equal(gf[inf], wf[inf]), name
        fin = ~np.isnan(wf) & ~inf
        assert H.ulp_diff(got[fin], want[fin], dtype) <= 1, name
        assert np.count_nonzero(got.view(np.uint16)[fin] != want.view(np.uint16)[fin]) <= 16, name


@pytest.mark.parametrize("dtype", [dx.BF16, dx.F16])
def test_every_16bit_input_through_the_binary_ops(dxh, orc, dtype):
    """All 65,536 patterns as the left operand of add, sub, mul, div, max and min against 48 right operands (signed
    zeros, one, a half, the largest finite value, denormals, infinities, NaN, 32 random patterns): the oracle's bits
    everywhere a number comes out, NaN where it has NaN — 3.1 million pairs per op."""
    rng = np.random.default_rng(5)
    with np.errstate(over="ignore"):
        special = H.to_storage(np.array([0.0, -0.0, 1.0, -1.0, 2.0, 0.5, 3.0, 1e-3, 65504.0, 1e-7, np.inf, -np.inf, np.nan, 1e30, -1e30, 1e-30]), dtype)
    partners = np.concatenate([special, rng.integers(0, 65536, 32).astype(np.uint16).view(H.NP[dtype])])
    allx = np.arange(65536, dtype=np.uint32).astype(np.uint16).view(H.NP[dtype])
    a, b = np.repeat(allx, len(partners)), np.tile(partners, 65536)
    for name in ("add", "sub", "mul", "div", "max", "min"):
        got, want = run_binary(dxh, orc, name, dtype, a, b)
        assert _same_nans_aside(got, want, dtype), name


@pytest.mark.parametrize("dtype", [dx.F32, dx.F64])
def test_special_values_through_every_float_op(dxh, orc, dtype):
    """A grid of 131 values — signed zeros, denormals and their neighbours, the largest finite value, the thresholds of exp,
    numbers next to one, 1e±30, infinities, NaN, 64 random magnitudes over eighty decades — in all pairs through add, sub,
    mul, div, max and min (the oracle's bits, NaN for NaN) and one by one through sqrt (exact) and exp, log, sin, cos, tan
    (NaN and infinities where the oracle has them, 4 units in the last place elsewhere, arguments of 1e30 included)."""
    npd = H.NP[dtype]
    fi = np.finfo(npd)
    base = [0.0, 1.0, 2.0, 0.5, 3.0, 1.0 / 3.0, 10.0, 1e-3, 1e3, np.pi, np.e, fi.max, fi.max / 2, fi.tiny, fi.tiny * 2, fi.tiny / 2, fi.smallest_subnormal,
            fi.smallest_subnormal * 3, fi.eps, 1 + fi.eps, 1 - fi.eps / 2, 88.0, 89.0, 709.0, 710.0, 1e-20, 1e20, 1e-30, 1e30, 0.1, 0.7, 123456.789]
    rng = np.random.default_rng(3)
    with np.errstate(all="ignore"):
        grid = np.array(base + [-x for x in base] + [np.inf, -np.inf, np.nan], dtype=npd)
        grid = np.concatenate([grid, (rng.standard_normal(64) * 10.0 ** rng.integers(-40, 40, 64)).astype(npd)])

    def exact(got, want):
        nan = np.isnan(want)
        return np.array_equal(np.isnan(got), nan) and np.array_equal(got[~nan].view(np.uint8), want[~nan].view(np.uint8))

    a, b = np.repeat(grid, grid.size), np.tile(grid, grid.size)
    for name in ("add", "sub", "mul", "div", "max", "min"):
        got, want = run_binary(dxh, orc, name, dtype, a, b)
        assert exact(got, want), name
    got, want = run_unary(dxh, orc, "sqrt", dtype, grid)
    assert exact(got, want)
    for name in ("exp", "log", "sin", "cos", "tan"):
        got, want = run_unary(dxh, orc, name, dtype, grid)
        assert np.array_equal(np.isnan(got), np.isnan(want)), name
        inf = np.isinf(want)
        assert np.array_equal(np.isinf(got), inf) and np.array_equal(got[inf], want[inf]), name
        fin = ~np.isnan(want) & ~inf
        assert H.ulp_diff(got[fin], want[fin], dtype) <= 4, name


def test_exp_special_values(dxh, orc):
    a = np.array([0.0, -np.inf, np.inf, 1000.0, -1000.0], dtype=np.float32)
    got, _ = run_unary(dxh, orc, "exp", dx.F32, a)
    assert got[0] == 1.0 and got[1] == 0.0 and np.isinf(got[2]) and np.isinf(got[3]) and got[4] == 0.0
    got, _ = run_unary(dxh, orc, "log", dx.F32, np.array([1.0, 0.0], dtype=np.float32))
    assert got[0] == 0.0 and np.isneginf(got[1])


@pytest.mark.parametrize("dtype", H.INTS + [dx.BOOL])
def test_invert(dxh, orc, dtype):
    rng = np.random.default_rng(11)
    a = rng.integers(0, 2, 10007).astype(np.uint8) if dtype == dx.BOOL else H.rand(rng, dtype, 10007)
    got, want = run_unary(dxh, orc, "invert", dtype, a)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("src", H.ALL_NUMERIC)
@pytest.mark.parametrize("dst", H.ALL_NUMERIC)
def test_todtype(dxh, orc, src, dst):
    rng = np.random.default_rng(12)
    n = 70001
    a = H.rand(rng, src, n, -100.0, 100.0) if src in H.FLOATS else H.rand(rng, src, n)
    da, dc = Dev(a), Dev.empty(n, H.NP[dst])
    dx.check(dxh.dxh_todtype(src, da.ptr, dst, dc.ptr, n, None), "todtype")
    want = np.empty(n, dtype=H.NP[dst])
    assert orc.orc_todtype(src, hp(a), dst, hp(want), n) == 0
    assert np.array_equal(dc.get(), want), f"{dx.DTYPE_NAMES[src]}->{dx.DTYPE_NAMES[dst]}"


@pytest.mark.parametrize("half", [dx.BF16, dx.F16])
def test_todtype_every_16bit_input_and_every_rounding_tie(dxh, orc, half):
    """Casts between the float types on all 65,536 patterns of a 16-bit type (to float64, float32 and both 16-bit types:
    denormals, overflow to infinity, NaN for NaN), and from float32 into the 16-bit type on every halfway point between
    two neighbouring 16-bit values and on its two float32 neighbours — where round-to-nearest-even is decided."""
    allx = np.arange(65536, dtype=np.uint32).astype(np.uint16).view(H.NP[half])

    def cast(src, a, dst):
        da, dc = Dev(a), Dev.empty(a.size, H.NP[dst])
        dx.check(dxh.dxh_todtype(src, da.ptr, dst, dc.ptr, a.size, None), "todtype")
        want = np.empty(a.size, dtype=H.NP[dst])
        assert orc.orc_todtype(src, hp(a), dst, hp(want), a.size) == 0
        return dc.get(), want

    for dst in (dx.F64, dx.F32, dx.F16, dx.BF16):
        got, want = cast(half, allx, dst)
        if dst in (dx.F16, dx.BF16):
            assert _same_nans_aside(got, want, dst), dx.DTYPE_NAMES[dst]
        else:
            nan = np.isnan(want)
            assert np.array_equal(np.isnan(got), nan) and np.array_equal(got[~nan], want[~nan]), dx.DTYPE_NAMES[dst]
    vals = np.sort(np.unique(H.to_float(allx, half)[np.isfinite(H.to_float(allx, half))].astype(np.float64)))
    ties = ((vals[:-1] + vals[1:]) / 2).astype(np.float32)  # one bit more than the 16-bit type holds: exact in float32
    assert np.array_equal(ties.astype(np.float64), (vals[:-1] + vals[1:]) / 2)
    probes = np.concatenate([ties, np.nextafter(ties, np.float32(np.inf)), np.nextafter(ties, np.float32(-np.inf)),
                             np.array([np.inf, -np.inf, np.nan, 3.0e38, -3.0e38, 1e-45, -1e-45, 65520.0, 65519.996], dtype=np.float32)])
    got, want = cast(dx.F32, probes, half)
    assert _same_nans_aside(got, want, half)


CMP = ["equal", "notequal", "less", "greater"]


@pytest.mark.parametrize("name", CMP)
@pytest.mark.parametrize("dtype", H.ALL_NUMERIC)
def test_compare(dxh, orc, name, dtype):
    rng = np.random.default_rng(13 + dtype)
    for n in [7, 4099, 500001]:
        a = H.rand(rng, dtype, n, -4, 4) if dtype in H.INTS else H.rand(rng, dtype, n)
        b = a.copy()
        flip = rng.random(n) < 0.5
        b[flip] = H.rand(rng, dtype, int(flip.sum()), -4, 4) if dtype in H.INTS else H.rand(rng, dtype, int(flip.sum()))
        da, db, dm = Dev(a), Dev(b), Dev.empty(n, np.uint8)
        want = np.empty(n, dtype=np.uint8)
        for eps in ([0.0, 0.25] if name in ("equal", "notequal") else [None]):
            f, g = getattr(dxh, "dxh_" + name), getattr(orc, "orc_" + name)
            if eps is None:
                dx.check(f(dtype, da.ptr, db.ptr, dm.ptr, n, None), name)
                assert g(dtype, hp(a), hp(b), hp(want), n) == 0
            else:
                dx.check(f(dtype, da.ptr, db.ptr, eps, dm.ptr, n, None), name)
                assert g(dtype, hp(a), hp(b), eps, hp(want), n) == 0
            got = dm.get()
            assert np.array_equal(got, want), f"{name} {dx.DTYPE_NAMES[dtype]} n={n} eps={eps}"
            assert set(np.unique(got)) <= {0, 1}


@pytest.mark.parametrize("dtype", [dx.BF16, dx.F16])
def test_compare_every_16bit_input(dxh, orc, dtype):
    """All 65,536 patterns of a 16-bit float against 48 partners (signed zeros, infinities, NaN, denormals, neighbours of
    one, random patterns) through equal / notequal with and without an epsilon and through less / greater: the oracle's
    mask, byte for byte — NaN compares as the reference's `<=` and `<` make it compare."""
    rng = np.random.default_rng(6)
    with np.errstate(over="ignore"):
        special = H.to_storage(np.array([0.0, -0.0, 1.0, -1.0, 1.0078125, 0.9921875, 0.5, 65504.0, 1e-7, -1e-7, np.inf, -np.inf, np.nan, 1e30, -1e30, 0.25]), dtype)
    partners = np.concatenate([special, rng.integers(0, 65536, 32).astype(np.uint16).view(H.NP[dtype])])
    allx = np.arange(65536, dtype=np.uint32).astype(np.uint16).view(H.NP[dtype])
    a, b = np.repeat(allx, len(partners)), np.tile(partners, 65536)
    n = a.size
    da, db, dm = Dev(a), Dev(b), Dev.empty(n, np.uint8)
    want = np.empty(n, dtype=np.uint8)
    for name in CMP:
        for eps in ([0.0, 0.25, 1e-3] if name in ("equal", "notequal") else [None]):
            f, g = getattr(dxh, "dxh_" + name), getattr(orc, "orc_" + name)
            if eps is None:
                dx.check(f(dtype, da.ptr, db.ptr, dm.ptr, n, None), name)
                assert g(dtype, hp(a), hp(b), hp(want), n) == 0
            else:
                dx.check(f(dtype, da.ptr, db.ptr, eps, dm.ptr, n, None), name)
                assert g(dtype, hp(a), hp(b), eps, hp(want), n) == 0
            got = dm.get()
            assert np.array_equal(got, want), (name, eps, int(np.count_nonzero(got != want)))


@pytest.mark.parametrize("name", ["equalscalar", "notequalscalar", "lessscalar", "greaterscalar"])
@pytest.mark.parametrize("dtype", H.ALL_NUMERIC)
def test_compare_scalar(dxh, orc, name, dtype):
    rng = np.random.default_rng(14 + dtype)
    n = 30011
    a = H.rand(rng, dtype, n, -4, 4) if dtype in H.INTS else H.to_storage(rng.integers(-4, 4, n) * 0.25, dtype)
    s = dx.scalar(1 if dtype in H.INTS else 0.25)
    da, dm = Dev(a), Dev.empty(n, np.uint8)
    want = np.empty(n, dtype=np.uint8)
    f, g = getattr(dxh, "dxh_" + name), getattr(orc, "orc_" + name)
    if "equal" in name:
        for eps in [0.0, 0.3]:
            dx.check(f(dtype, da.ptr, s, eps, dm.ptr, n, None), name)
            assert g(dtype, hp(a), s, eps, hp(want), n) == 0
            assert np.array_equal(dm.get(), want)
    else:
        dx.check(f(dtype, da.ptr, s, dm.ptr, n, None), name)
        assert g(dtype, hp(a), s, hp(want), n) == 0
        assert np.array_equal(dm.get(), want)


@pytest.mark.parametrize("dtype", H.ALL_NUMERIC + [dx.BOOL])
def test_switch_bool_and_int(dxh, orc, dtype):
    rng = np.random.default_rng(15)
    for n in [9, 100003]:
        mk = (lambda: rng.integers(0, 2, n).astype(np.uint8)) if dtype == dx.BOOL else (lambda: H.rand(rng, dtype, n))
        ts = [mk() for _ in range(3)]
        devs = [Dev(t) for t in ts]
        out = Dev.empty(n, ts[0].dtype)
        want = np.empty_like(ts[0])
        # bool cases: where(c, t1, t0)
        cases = rng.integers(0, 2, n).astype(np.uint8)
        dcs = Dev(cases)
        dx.check(dxh.dxh_switch(dtype, dx.ptrarr([d.ptr.value for d in devs[:2]]), 2, dx.BOOL, dcs.ptr, out.ptr, n, None), "switch")
        assert orc.orc_switch(dtype, dx.ptrarr([t.ctypes.data for t in ts[:2]]), 2, dx.BOOL, hp(cases), hp(want), n) == 0
        got = out.get()
        assert np.array_equal(got, want)
        assert np.array_equal(got, np.where(cases != 0, ts[1], ts[0]))
        # int32 cases over three tensors
        cases = rng.integers(0, 3, n).astype(np.int32)
        dcs = Dev(cases)
        dx.check(dxh.dxh_switch(dtype, dx.ptrarr([d.ptr.value for d in devs]), 3, dx.I32, dcs.ptr, out.ptr, n, None), "switch")
        assert orc.orc_switch(dtype, dx.ptrarr([t.ctypes.data for t in ts]), 3, dx.I32, hp(cases), hp(want), n) == 0
        assert np.array_equal(out.get(), want)
    # bool cases need exactly two tensors
    assert dxh.dxh_switch(dtype, dx.ptrarr([d.ptr.value for d in devs]), 3, dx.BOOL, dcs.ptr, out.ptr, n, None) == -2


@pytest.mark.parametrize("dtype", H.ALL_NUMERIC)
def test_constant_arange(dxh, orc, dtype):
    n = 10007
    out = Dev.empty(n, H.NP[dtype])
    want = np.empty(n, dtype=H.NP[dtype])
    v = dx.scalar(1.5 if dtype in H.FLOATS else 7)
    dx.check(dxh.dxh_constant(dtype, out.ptr, n, v, None), "constant")
    assert orc.orc_constant(dtype, hp(want), n, v) == 0
    assert np.array_equal(out.get(), want)
    s0, s1 = dx.scalar(2), dx.scalar(0.5 if dtype in H.FLOATS else 3)
    nn = 200 if dtype in (dx.I8, dx.BF16) else 2000
    dx.check(dxh.dxh_arange(dtype, out.ptr, nn, s0, s1, None), "arange")
    assert orc.orc_arange(dtype, hp(want), nn, s0, s1) == 0
    assert np.array_equal(out.get()[:nn], want[:nn])


def test_misaligned_pointers_take_scalar_path(dxh, orc):
    """A tensor view that starts off a 16-byte boundary must still be correct."""
    rng = np.random.default_rng(16)
    n = 5003
    a, b = H.rand(rng, dx.F32, n + 1), H.rand(rng, dx.F32, n + 1)
    da, db, dc = Dev(a), Dev(b), Dev.empty(n + 1, np.float32)
    off = lambda d: C.c_void_p(d.ptr.value + 4)
    dx.check(dxh.dxh_add(dx.F32, off(da), off(db), off(dc), n, None), "add")
    assert np.array_equal(dc.get()[1:], a[1:] + b[1:])
    # off by one byte for a 4-byte dtype is rejected, not faulted
    assert dxh.dxh_add(dx.F32, C.c_void_p(da.ptr.value + 1), db.ptr, dc.ptr, n, None) == -5


@pytest.mark.parametrize("dtype", [dx.F64, dx.F32, dx.BF16, dx.I64, dx.I32, dx.I16, dx.I8])
def test_store_policy_leaves_the_bits_alone(dxh, orc, dtype):
    """Outputs of up to 32 MiB leave with write-through stores, larger ones with non-temporal stores
    (knob 0 moves the limit).  Every width of both kinds: 16-byte vectors, and the 8-, 4-, 2- and 1-byte
    stores of a tensor that starts off a 16-byte boundary; add, a scalar form and a cast against the
    oracle under either policy."""
    rng = np.random.default_rng(160 + dtype)
    n = 40007
    es = np.dtype(H.NP[dtype]).itemsize
    a, b = H.rand(rng, dtype, n + 16), H.rand(rng, dtype, n + 16)
    want = np.empty(n, dtype=a.dtype)
    for shift in (0, 1):  # elements off the allocation's start: 0 keeps 16-byte alignment, 1 loses it
        av, bv = a[shift:shift + n].copy(), b[shift:shift + n].copy()
        assert orc.orc_add(dtype, hp(av), hp(bv), hp(want), n) == 0
        for limit in (1 << 40, 0):  # everything written through / everything non-temporal
            dx.check(dxh.dxh_tune(0, limit))
            try:
                da, db, dc = Dev(a), Dev(b), Dev.empty(n + 16, a.dtype)
                at = lambda d: C.c_void_p(d.ptr.value + shift * es)
                dx.check(dxh.dxh_add(dtype, at(da), at(db), at(dc), n, None), "add")
                assert np.array_equal(dc.get()[shift:shift + n], want), (shift, limit)
                dst = dx.F32 if dtype != dx.F32 else dx.BF16
                dd = Dev.empty(n + 16, H.NP[dst])
                ds = np.dtype(H.NP[dst]).itemsize
                dx.check(dxh.dxh_todtype(dtype, at(da), dst, C.c_void_p(dd.ptr.value + shift * ds), n, None), "todtype")
                cast_want = np.empty(n, dtype=H.NP[dst])
                assert orc.orc_todtype(dtype, hp(av), dst, hp(cast_want), n) == 0
                assert np.array_equal(dd.get()[shift:shift + n], cast_want), (shift, limit)
            finally:
                dx.check(dxh.dxh_tune(0, 32 << 20))


def test_error_codes(dxh):
    a = Dev(np.zeros(16, dtype=np.float32))
    assert dxh.dxh_add(12345, a.ptr, a.ptr, a.ptr, 16, None) == -1
    assert dxh.dxh_add(dx.F32, None, a.ptr, a.ptr, 16, None) == -2
    assert dxh.dxh_add(dx.F32, a.ptr, a.ptr, a.ptr, -1, None) == -2
    assert dxh.dxh_add(dx.F32, None, None, None, 0, None) == 0  # empty tensor is a no-op
    assert dxh.dxh_pow(dx.I32, a.ptr, a.ptr, a.ptr, 16, None) == -1


def test_config1_chain_full_size(dxh, orc):
    """BASELINE config 1 at full size, each op checked on the oracle's own inputs."""
    n = 4096 * 4096
    rng = np.random.default_rng(1)
    A = rng.uniform(-1, 1, n).astype(np.float32)
    B = np.random.default_rng(2).uniform(-1, 1, n).astype(np.float32)
    half, one, neg = dx.scalar(0.5), dx.scalar(1.0), dx.scalar(-1.0)
    dA, dB = Dev(A), Dev(B)
    d = {k: Dev.empty(n, np.float32) for k in "CDEFGnad"}
    dx.check(dxh.dxh_add(dx.F32, dA.ptr, dB.ptr, d["C"].ptr, n, None))
    dx.check(dxh.dxh_mul(dx.F32, d["C"].ptr, dB.ptr, d["D"].ptr, n, None))
    dx.check(dxh.dxh_addscalar(dx.F32, d["D"].ptr, half, d["E"].ptr, n, None))
    dx.check(dxh.dxh_exp(dx.F32, d["E"].ptr, d["F"].ptr, n, None))
    dx.check(dxh.dxh_mulscalar(dx.F32, dB.ptr, neg, d["n"].ptr, n, None))
    dx.check(dxh.dxh_max(dx.F32, dB.ptr, d["n"].ptr, d["a"].ptr, n, None))
    dx.check(dxh.dxh_addscalar(dx.F32, d["a"].ptr, one, d["d"].ptr, n, None))
    dx.check(dxh.dxh_div(dx.F32, d["F"].ptr, d["d"].ptr, d["G"].ptr, n, None))
    Cc = A + B
    assert np.array_equal(d["C"].get(), Cc)
    Dd = Cc * B
    assert np.array_equal(d["D"].get(), Dd)
    Ee = Dd + np.float32(0.5)
    assert np.array_equal(d["E"].get(), Ee)
    Fw = np.empty_like(Ee)
    assert orc.orc_exp(dx.F32, hp(Ee), hp(Fw), n) == 0
    Fg = d["F"].get()
    assert H.ulp_diff(Fg, Fw, dx.F32) <= 4
    den = np.abs(B) + np.float32(1.0)
    assert np.array_equal(d["d"].get(), den)
    assert np.array_equal(d["G"].get(), Fg / den)  # div is exact on the device's own F


def test_nt_load_knob_gives_identical_results(dxh):
    """The non-temporal hint on loads is a cache policy, chosen per launch by op class and size:
    forcing it on (1) or off (2) through the tuning knob must not change a single bit of an
    elementwise, compare, cast or reduce result."""
    NT_LOAD_KNOB = 7  # DXH_TUNE_NT_LOAD
    rng = np.random.default_rng(4242)
    n = 300_001
    A = rng.standard_normal(n).astype(np.float32)
    B = rng.standard_normal(n).astype(np.float32)
    dA, dB = Dev(A), Dev(B)
    results = {}
    for knob in (0, 1, 2):
        dx.check(dxh.dxh_tune(NT_LOAD_KNOB, knob))
        try:
            dC, dS, dU, dM, dH = Dev.empty(n, np.float32), Dev.empty(n, np.float32), Dev.empty(n, np.float32), Dev.empty(n, np.uint8), Dev.empty(n, np.uint16)
            dx.check(dxh.dxh_add(dx.F32, dA.ptr, dB.ptr, dC.ptr, n, None))
            dx.check(dxh.dxh_mulscalar(dx.F32, dA.ptr, dx.scalar(1.5), dS.ptr, n, None))
            dx.check(dxh.dxh_exp(dx.F32, dA.ptr, dU.ptr, n, None))
            dx.check(dxh.dxh_less(dx.F32, dA.ptr, dB.ptr, dM.ptr, n, None))
            dx.check(dxh.dxh_todtype(dx.F32, dA.ptr, dx.BF16, dH.ptr, n, None))
            rows, cols = 300, 1000
            dR, dK = Dev.empty(rows, np.float32), Dev.empty(cols, np.float32)
            ws = Dev.empty(1 << 20, np.uint8)
            sh = dx.i32arr([rows, cols])
            dx.check(dxh.dxh_sum(dx.F32, dA.ptr, sh, 2, dx.i32arr([1]), 1, dR.ptr, ws.ptr, 1 << 20, None))
            dx.check(dxh.dxh_reducemax(dx.F32, dA.ptr, sh, 2, dx.i32arr([0]), 1, dK.ptr, ws.ptr, 1 << 20, None))
            results[knob] = [d.get().copy() for d in (dC, dS, dU, dM, dH, dR, dK)]
        finally:
            dx.check(dxh.dxh_tune(NT_LOAD_KNOB, 0))
    for knob in (1, 2):
        for got, want in zip(results[knob], results[0]):
            assert np.array_equal(got, want), knob
