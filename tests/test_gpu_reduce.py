"""GPU parity: reductions vs the CPU oracle.

Bars: reducemax/reducemin and every integer reduction bit-exact; fp32 sum/prod within
rel 1e-5*sqrt(N) of the oracle (N = reduced length; the reference's own summation order is
thread-schedule dependent); bf16/f16 within rel 1e-2.
"""
import ctypes as C

import numpy as np
import pytest

from deepx_amd import lib as dx
from tests import helpers as H
from tests.helpers import Dev, hp

pytestmark = pytest.mark.gpu

OPS = ["sum", "prod", "reducemax", "reducemin"]


def gpu_reduce(dxh, name, dtype, a, shape, dims):
    sh, dm = dx.i32arr(shape), dx.i32arr(dims)
    kept = [s for i, s in enumerate(shape) if i not in [d % len(shape) for d in dims]] if dims else []
    nout = int(np.prod(kept)) if kept else 1
    ws_bytes = C.c_size_t(0)
    dx.check(dxh.dxh_reduce_workspace_bytes(dtype, sh, len(shape), dm, len(dims), C.byref(ws_bytes)), "ws")
    ws = Dev.empty(max(1, ws_bytes.value), np.uint8)
    da, out = Dev(a), Dev.empty(nout, a.dtype)
    dx.check(getattr(dxh, "dxh_" + name)(dtype, da.ptr, sh, len(shape), dm, len(dims), out.ptr, ws.ptr, ws_bytes.value, None), name)
    return out.get(), nout


def cpu_reduce(orc, name, dtype, a, shape, dims, nout):
    want = np.empty(nout, dtype=a.dtype)
    assert getattr(orc, "orc_" + name)(dtype, hp(a), dx.i32arr(shape), len(shape), dx.i32arr(dims), len(dims), hp(want)) == 0
    return want


def check(name, dtype, got, want, nred):
    if dtype in H.INTS or name in ("reducemax", "reducemin"):
        assert np.array_equal(got, want)
        return
    g, w = H.to_float(got, dtype), H.to_float(want, dtype)
    tol = 1e-2 if dtype in (dx.F16, dx.BF16) else (1e-5 if dtype == dx.F32 else 1e-13) * np.sqrt(nred)
    scale = np.maximum(np.abs(w), 1e-30)
    if name == "sum":  # cancellation: measure against the magnitude that was summed
        scale = np.maximum(scale, 1.0)
    assert np.all(np.abs(g - w) <= tol * scale), f"max rel {np.max(np.abs(g - w) / scale)}"


SHAPES = [
    ((1000,), [0]),
    ((37, 129), [1]),
    ((37, 129), [0]),
    ((64, 256), [-1]),
    ((33, 64), [1]),          # sub-wave row groups
    ((5, 7, 11), [1]),
    ((5, 7, 11), [0, 2]),     # two reduced groups
    ((5, 7, 11), [0, 1, 2]),
    ((5, 7, 11), []),         # empty = all axes
    ((4, 3, 8, 16), [1, 3]),
    ((2, 3, 4, 5, 6), [0, 2, 4]),
    ((3, 1, 5), [1]),         # size-1 axis: copy
    ((300, 2), [0]),          # narrow strided
    ((8, 4096), [0]),         # split-R col stage
    ((2, 70000), [1]),        # split-R row stage
    ((1 << 20,), [0]),        # full reduce with two passes
]


@pytest.mark.parametrize("name", OPS)
@pytest.mark.parametrize("dtype", H.ALL_NUMERIC)
def test_reduce_shapes(dxh, orc, name, dtype):
    rng = np.random.default_rng(300 + dtype)
    for shape, dims in SHAPES:
        n = int(np.prod(shape))
        if name == "prod":
            a = H.to_storage(rng.uniform(0.98, 1.02, n), dtype) if dtype in H.FLOATS else rng.integers(-3, 4, n).astype(H.NP[dtype])
        else:
            a = H.rand(rng, dtype, n)
        if dtype in (dx.F16, dx.BF16) and name == "prod" and n > 100000:
            continue
        got, nout = gpu_reduce(dxh, name, dtype, a, shape, dims)
        want = cpu_reduce(orc, name, dtype, a, shape, dims, nout)
        check(name, dtype, got, want, n // nout)


def test_sum_closed_forms(dxh):
    # sum(arange(n)) = n(n-1)/2 exactly representable in f64; all-ones rows sum to the row length
    n = 1 << 16
    a = np.arange(n, dtype=np.float64)
    got, _ = gpu_reduce(dxh, "sum", dx.F64, a, (n,), [0])
    assert got[0] == n * (n - 1) / 2
    ones = np.ones((512, 8192), dtype=np.float32)
    got, _ = gpu_reduce(dxh, "sum", dx.F32, ones.reshape(-1), (512, 8192), [1])
    assert np.all(got == 8192.0)
    got, _ = gpu_reduce(dxh, "sum", dx.F32, ones.reshape(-1), (512, 8192), [0])
    assert np.all(got == 512.0)
    i = np.arange(100000, dtype=np.int64)
    got, _ = gpu_reduce(dxh, "sum", dx.I64, i, (100000,), [0])
    assert got[0] == 100000 * 99999 // 2


def test_dims_errors(dxh):
    a = Dev(np.zeros(16, dtype=np.float32))
    sh = dx.i32arr([4, 4])
    assert dxh.dxh_sum(dx.F32, a.ptr, sh, 2, dx.i32arr([2]), 1, a.ptr, None, 0, None) == -2
    assert dxh.dxh_sum(dx.F32, a.ptr, sh, 2, dx.i32arr([-3]), 1, a.ptr, None, 0, None) == -2
    assert dxh.dxh_sum(dx.BOOL, a.ptr, sh, 2, dx.i32arr([0]), 1, a.ptr, None, 0, None) == -1
    # a reduction that needs scratch refuses to run without it
    big = dx.i32arr([1 << 20])
    need = C.c_size_t(0)
    assert dxh.dxh_reduce_workspace_bytes(dx.F32, big, 1, dx.i32arr([0]), 1, C.byref(need)) == 0
    assert need.value > 0
    b = Dev(np.zeros(1 << 20, dtype=np.float32))
    assert dxh.dxh_sum(dx.F32, b.ptr, big, 1, dx.i32arr([0]), 1, a.ptr, None, 0, None) == -4


def test_config2_full_size(dxh, orc):
    """BASELINE config 2: fp32 [8192,8192] N(0,1): sum axis 1 / axis 0, reducemax/min axis 1; prod of
    [8192,64] U(0.9,1.1).  keepdims only reshapes the result, so both settings share one buffer."""
    rng = np.random.default_rng(3)
    X = rng.standard_normal((8192, 8192), dtype=np.float32)
    flat = X.reshape(-1)
    got, _ = gpu_reduce(dxh, "sum", dx.F32, flat, (8192, 8192), [1])
    ref = X.astype(np.float64).sum(axis=1)
    assert np.all(np.abs(got - ref) <= 1e-5 * np.sqrt(8192) * np.maximum(np.abs(ref), 1.0))
    got, _ = gpu_reduce(dxh, "sum", dx.F32, flat, (8192, 8192), [0])
    ref = X.astype(np.float64).sum(axis=0)
    assert np.all(np.abs(got - ref) <= 1e-5 * np.sqrt(8192) * np.maximum(np.abs(ref), 1.0))
    got, _ = gpu_reduce(dxh, "reducemax", dx.F32, flat, (8192, 8192), [1])
    assert np.array_equal(got, X.max(axis=1))
    got, _ = gpu_reduce(dxh, "reducemin", dx.F32, flat, (8192, 8192), [1])
    assert np.array_equal(got, X.min(axis=1))
    got, _ = gpu_reduce(dxh, "reducemax", dx.F32, flat, (8192, 8192), [0])
    assert np.array_equal(got, X.max(axis=0))
    P = np.random.default_rng(4).uniform(0.9, 1.1, (8192, 64)).astype(np.float32)
    got, nout = gpu_reduce(dxh, "prod", dx.F32, P.reshape(-1), (8192, 64), [1])
    want = cpu_reduce(orc, "prod", dx.F32, P.reshape(-1), (8192, 64), [1], nout)
    ref = P.astype(np.float64).prod(axis=1)
    assert np.all(np.abs(got - ref) <= 1e-5 * 8 * np.abs(ref))
    assert np.all(np.abs(want - ref) <= 1e-5 * 8 * np.abs(ref))


FUSED_KNOB = 11  # DXH_TUNE_REDUCE_FUSED_FINISH


def _reduce_on(dxh, name, dtype, da, shape, dims, out, ws, ws_bytes, stream):
    dx.check(getattr(dxh, "dxh_" + name)(dtype, da.ptr, dx.i32arr(shape), len(shape), dx.i32arr(dims), len(dims), out.ptr, ws.ptr, ws_bytes, stream), name)


@pytest.mark.parametrize("dtype", [dx.F32, dx.F64, dx.BF16, dx.I32, dx.I8])
def test_split_strided_axis_finishes_in_one_launch(dxh, orc, dtype):
    """A strided axis cut into slices: the last workgroup of a tile adds the slices inside the same
    launch (knob 11 = 1, default) or a second launch does (0).  Both against the oracle to the
    file's bars; integers and max / min bit-equal between the two; the one-launch path called
    three times in a row (its completion counters must be back at zero) gives the same bits."""
    rng = np.random.default_rng(500 + dtype)
    for shape, dims in [((4096, 512), [0]), ((3, 2048, 256), [1]), ((8, 4096), [0]), ((5000, 1000), [0]), ((2, 3000, 40), [1]), ((7, 1024, 64), [0, 1])]:
        a = H.rand(rng, dtype, int(np.prod(shape)), 0.5, 1.5) if dtype not in H.INTS else H.rand(rng, dtype, int(np.prod(shape)))
        for name in OPS:
            if name == "prod" and dtype not in H.INTS:
                a = H.rand(rng, dtype, int(np.prod(shape)), 0.999, 1.001)
            res = {}
            for knob in (1, 0):
                dx.check(dxh.dxh_tune(FUSED_KNOB, knob))
                try:
                    runs = [gpu_reduce(dxh, name, dtype, a, shape, dims) for _ in range(3 if knob else 1)]
                finally:
                    dx.check(dxh.dxh_tune(FUSED_KNOB, 1))
                got, nout = runs[0]
                for other, _ in runs[1:]:
                    assert np.array_equal(got.view(np.uint8), other.view(np.uint8)), (name, shape, dims)
                res[knob] = got
                nred = int(np.prod(shape)) // nout
                check(name, dtype, got, cpu_reduce(orc, name, dtype, a, shape, dims, nout), nred)
            if dtype in H.INTS or name in ("reducemax", "reducemin"):
                assert np.array_equal(res[0], res[1]), (name, shape, dims)


def test_one_launch_finish_on_two_streams_and_under_capture(dxh):
    """Two streams reduce different tensors at the same time (each owns its completion counters), and
    a reduction recorded under stream capture replays three times next to eager calls on the
    capture stream; every result equals the eager one-launch result on the default stream."""
    rng = np.random.default_rng(77)
    shape, dims = (4096, 2048), [0]
    sh, dm = dx.i32arr(shape), dx.i32arr(dims)
    n, nout = shape[0] * shape[1], shape[1]
    X = [rng.standard_normal(n).astype(np.float32) for _ in range(2)]
    want = [gpu_reduce(dxh, "sum", dx.F32, x, shape, dims)[0] for x in X]
    wsb = C.c_size_t(0)
    dx.check(dxh.dxh_reduce_workspace_bytes(dx.F32, sh, 2, dm, 1, C.byref(wsb)))
    assert wsb.value > 0  # the axis is cut
    streams = [C.c_void_p(), C.c_void_p()]
    for s in streams:
        dx.check(dxh.dxh_stream_create(C.byref(s)))
    dev = [Dev(x) for x in X]
    outs = [Dev.empty(nout, np.float32) for _ in range(2)]
    wss = [Dev.empty(wsb.value, np.uint8) for _ in range(2)]
    for _ in range(20):
        for i in range(2):
            _reduce_on(dxh, "sum", dx.F32, dev[i], shape, dims, outs[i], wss[i], wsb.value, streams[i])
    for i in range(2):
        dx.check(dxh.dxh_stream_sync(streams[i]))
        assert np.array_equal(outs[i].get(), want[i])
    # capture on stream 0, replay on stream 1 while stream 0 keeps reducing eagerly
    gout, gws = Dev.empty(nout, np.float32), Dev.empty(wsb.value, np.uint8)
    graph = C.c_void_p()
    dx.check(dxh.dxh_graph_begin_capture(streams[0]))
    rc = dxh.dxh_sum(dx.F32, dev[1].ptr, sh, 2, dm, 1, gout.ptr, gws.ptr, wsb.value, streams[0])
    dx.check(dxh.dxh_graph_end_capture(streams[0], C.byref(graph)))
    dx.check(rc, "sum under capture")
    for _ in range(3):
        dx.check(dxh.dxh_graph_launch(graph, streams[1]))
        for _ in range(5):
            _reduce_on(dxh, "sum", dx.F32, dev[0], shape, dims, outs[0], wss[0], wsb.value, streams[0])
        dx.check(dxh.dxh_stream_sync(streams[1]))
        dx.check(dxh.dxh_stream_sync(streams[0]))
        assert np.array_equal(gout.get(), want[1])
        assert np.array_equal(outs[0].get(), want[0])
    dx.check(dxh.dxh_graph_destroy(graph))
    for s in streams:
        dx.check(dxh.dxh_stream_destroy(s))


def test_one_launch_finish_many_launches(dxh):
    """The workgroup that stores a tile's last slice must see every other slice: 2000 launches of the
    one-launch finish over four shapes and max / min / integer sum (order-independent, so the
    two-launch path gives the same bits), compared after every launch; stops at the first mismatch."""
    rng = np.random.default_rng(4242)
    cases = [("reducemax", dx.F32, (4096, 512), [0]), ("reducemin", dx.F32, (3, 2048, 256), [1]),
             ("sum", dx.I32, (5000, 1000), [0]), ("reducemax", dx.BF16, (8192, 2048), [0])]
    prepared = []
    for name, dtype, shape, dims in cases:
        a = H.rand(rng, dtype, int(np.prod(shape)))
        dx.check(dxh.dxh_tune(FUSED_KNOB, 0))
        try:
            want, nout = gpu_reduce(dxh, name, dtype, a, shape, dims)
        finally:
            dx.check(dxh.dxh_tune(FUSED_KNOB, 1))
        sh, dm = dx.i32arr(shape), dx.i32arr(dims)
        wsb = C.c_size_t(0)
        dx.check(dxh.dxh_reduce_workspace_bytes(dtype, sh, len(shape), dm, len(dims), C.byref(wsb)))
        assert wsb.value > 0, "the axis must be cut for this test to mean anything"
        prepared.append((name, dtype, shape, dims, Dev(a), Dev.empty(nout, a.dtype), Dev.empty(wsb.value, np.uint8), wsb.value, want))
    for it in range(500):
        for name, dtype, shape, dims, da, out, ws, wsb, want in prepared:
            _reduce_on(dxh, name, dtype, da, shape, dims, out, ws, wsb, None)
            got = out.get()
            assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (it, name, shape)


def test_two_slice_exchange_finish_many_launches(dxh, orc):
    """A strided axis cut into exactly two slices with a 4-byte accumulator meets in one atomic
    exchange per output element (each 64-bit slot must be zero again when the launch ends).  1200
    launches over four cases, compared after every launch with the first launch's bits (a + b and
    a * b do not depend on which half arrives second); the first launch is held to the oracle, and
    for integers to the two-launch path bit for bit."""
    rng = np.random.default_rng(9191)
    cases = [("sum", dx.F32, (8192, 8192), [0]), ("prod", dx.F32, (2048, 16384), [0]),
             ("sum", dx.I32, (2048, 16384), [0]), ("reducemax", dx.I32, (2, 2048, 4096), [1])]
    prepared = []
    for name, dtype, shape, dims in cases:
        n = int(np.prod(shape))
        a = H.rand(rng, dtype, n, 0.999, 1.001) if name == "prod" else H.rand(rng, dtype, n)
        first, nout = gpu_reduce(dxh, name, dtype, a, shape, dims)
        check(name, dtype, first, cpu_reduce(orc, name, dtype, a, shape, dims, nout), n // nout)
        if dtype in H.INTS:
            dx.check(dxh.dxh_tune(FUSED_KNOB, 0))
            try:
                two, _ = gpu_reduce(dxh, name, dtype, a, shape, dims)
            finally:
                dx.check(dxh.dxh_tune(FUSED_KNOB, 1))
            assert np.array_equal(first, two), (name, shape)
        sh, dm = dx.i32arr(shape), dx.i32arr(dims)
        wsb = C.c_size_t(0)
        dx.check(dxh.dxh_reduce_workspace_bytes(dtype, sh, len(shape), dm, len(dims), C.byref(wsb)))
        prepared.append((name, dtype, shape, dims, Dev(a), Dev.empty(nout, a.dtype), Dev.empty(max(wsb.value, 16), np.uint8), wsb.value, first))
    for it in range(300):
        for name, dtype, shape, dims, da, out, ws, wsb, want in prepared:
            _reduce_on(dxh, name, dtype, da, shape, dims, out, ws, wsb, None)
            got = out.get()
            assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (it, name, shape)
