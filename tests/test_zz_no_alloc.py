"""GPU parity: dxh_sum_noalloc (partial results in a device array inside the library, no
allocation, no workspace argument) against dxh_sum with a caller workspace.

Bar: the two run the same kernels in the same launch shapes, so every output is bit-identical
(integer and float alike); dxh_sum itself is held to the oracle in test_gpu_reduce.py, and the
float64 check here repeats that bar (rel 1e-5*sqrt(N) for fp32, 1e-2 for bf16) on the new entry
point's own output.  Each case makes two calls in a row, the second on a smaller input, so the
second call runs over whatever the first left in the shared array.
"""
import ctypes as C

import numpy as np
import pytest

from deepx_amd import lib as dx
from tests import helpers as H
from tests.helpers import Dev

pytestmark = pytest.mark.gpu


def both(dxh, dtype, a, shape, dims):
    sh, dm = dx.i32arr(shape), dx.i32arr(dims)
    kept = [s for i, s in enumerate(shape) if i not in [d % len(shape) for d in dims]]
    nout = int(np.prod(kept)) if kept else 1
    wsb = C.c_size_t(0)
    dx.check(dxh.dxh_reduce_workspace_bytes(dtype, sh, len(shape), dm, len(dims), C.byref(wsb)), "ws")
    ws = Dev.empty(max(1, wsb.value), np.uint8)
    da = Dev(a)
    want, got = Dev.empty(nout, a.dtype), Dev.empty(nout, a.dtype)
    dx.check(dxh.dxh_sum(dtype, da.ptr, sh, len(shape), dm, len(dims), want.ptr, ws.ptr, wsb.value, None), "sum")
    dx.check(dxh.dxh_sum_noalloc(dtype, da.ptr, sh, len(shape), dm, len(dims), got.ptr, None), "sum_noalloc")
    return got.get(), want.get(), wsb.value


# (first call, smaller second call); every first shape needs partial results (a cut axis or two stages)
CASES = [
    (((8192, 8192), [0]), ((1024, 2048), [0])),          # BASELINE config 2, strided axis
    (((4, 262144), [1]), ((2, 70000), [1])),             # contiguous axis cut into chunks
    (((96, 64, 128), [0, 2]), ((5, 7, 11), [0, 2])),     # two stages, the first one's output in scratch
    (((1 << 22,), [0]), ((1 << 20,), [0])),              # everything reduced, two passes
]


@pytest.mark.parametrize("dtype", [dx.F32, dx.BF16, dx.F64, dx.I32])
@pytest.mark.parametrize("case", CASES)
def test_sum_noalloc_equals_sum_twice_in_a_row(dxh, dtype, case):
    rng = np.random.default_rng(900 + dtype)
    used = 0
    for shape, dims in case:
        n = int(np.prod(shape))
        if dtype == dx.F64 and n > (1 << 25):
            shape = (shape[0] // 4,) + tuple(shape[1:])
            n = int(np.prod(shape))
        a = H.rand(rng, dtype, n)
        got, want, wsb = both(dxh, dtype, a, shape, dims)
        used = max(used, wsb)
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (dtype, shape, dims)
        # the bar of the oracle comparison, on the new entry point's own output
        if dtype in H.INTS:  # exact: wrap-around arithmetic in the storage width
            ref = a.reshape(shape).astype(np.int64).sum(axis=tuple(dims)).astype(H.NP[dtype])
            assert np.array_equal(got.reshape(ref.shape), ref), (dtype, shape, dims)
        else:
            ref = H.to_float(a, dtype).reshape(shape).sum(axis=tuple(dims))
            nred = n // max(1, got.size)
            tol = 1e-2 if dtype == dx.BF16 else (1e-5 if dtype == dx.F32 else 1e-13) * np.sqrt(nred)
            g = H.to_float(got, dtype).reshape(ref.shape)
            assert np.all(np.abs(g - ref) <= tol * np.maximum(np.abs(ref), np.sqrt(nred))), (dtype, shape, dims)
    assert used > 0, "no case here used the scratch array"


def test_sum_noalloc_refuses_what_does_not_fit(dxh):
    """A reduction whose partial results exceed the array is refused before anything is launched."""
    shape, dims = (4096, 4096, 16), [0, 2]  # stage 1 leaves 16 Mi fp32 partials
    sh, dm = dx.i32arr(shape), dx.i32arr(dims)
    wsb = C.c_size_t(0)
    dx.check(dxh.dxh_reduce_workspace_bytes(dx.F32, sh, 3, dm, 2, C.byref(wsb)))
    assert wsb.value > (4 << 20)
    assert dxh.dxh_sum_noalloc(dx.F32, C.c_void_p(256), sh, 3, dm, 2, C.c_void_p(512), None) == -6
