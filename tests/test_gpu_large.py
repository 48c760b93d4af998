"""GPU: tensors with more than 2^31 elements (int8, so > 2 GiB each) through every kernel family.
Dimensions stay below 2^31 as the reference's int shapes require, but flat offsets do not: this is
where 32-bit index arithmetic would wrap.  Everything is integer work, checked bit for bit against
numpy on the whole tensor."""
import ctypes as C

import numpy as np
import pytest

from deepx_amd import lib as dx
from tests.helpers import Dev

pytestmark = pytest.mark.gpu

ROWS, COLS = 70001, 32768          # 2,293,792,768 elements
N = ROWS * COLS


@pytest.fixture(scope="module")
def big():
    """a[i] = (i * 7 + i // 251) mod 256 as int8: no short period along either axis"""
    a = np.empty(N, dtype=np.int8)
    step = 1 << 26
    for start in range(0, N, step):  # in chunks: the int64 index vector of the whole tensor would take 18 GB
        i = np.arange(start, min(N, start + step), dtype=np.int64)
        a[start:start + i.size] = ((i * 7 + i // 251) & 0xff).astype(np.uint8).view(np.int8)
    return a, Dev(a)


def test_elementwise_and_compare_past_2g(dxh, big):
    a, da = big
    dc = Dev.empty(N, np.int8)
    dx.check(dxh.dxh_addscalar(dx.I8, da.ptr, dx.scalar(3), dc.ptr, N, None))
    want = (a.view(np.uint8) + np.uint8(3)).view(np.int8)
    got = dc.get()
    assert np.array_equal(got, want)
    dx.check(dxh.dxh_mul(dx.I8, da.ptr, dc.ptr, dc.ptr, N, None))       # in place, wraps
    want = (a.view(np.uint8) * want.view(np.uint8)).view(np.int8)
    assert np.array_equal(dc.get(), want)
    dm = Dev.empty(N, np.uint8)
    dx.check(dxh.dxh_greater(dx.I8, da.ptr, dc.ptr, dm.ptr, N, None))
    assert np.array_equal(dm.get(), (a > want).astype(np.uint8))
    dx.check(dxh.dxh_constant(dx.I8, dc.ptr, N, dx.scalar(-5), None))
    tail = dc.get()
    assert tail[0] == -5 and tail[-1] == -5 and np.all(tail == -5)


def test_reductions_past_2g(dxh, big):
    a, da = big
    shape = dx.i32arr([ROWS, COLS])
    A = a.reshape(ROWS, COLS)
    for axis, nout in ((0, COLS), (1, ROWS)):
        dims = dx.i32arr([axis])
        need = C.c_size_t(0)
        dx.check(dxh.dxh_reduce_workspace_bytes(dx.I8, shape, 2, dims, 1, C.byref(need)))
        ws = Dev.empty(max(1, need.value), np.uint8)
        out = Dev.empty(nout, np.int8)
        dx.check(dxh.dxh_sum(dx.I8, da.ptr, shape, 2, dims, 1, out.ptr, ws.ptr, need.value, None))
        assert np.array_equal(out.get(), A.sum(axis=axis, dtype=np.int64).astype(np.int8)), axis  # int8 accumulation wraps
        dx.check(dxh.dxh_reducemax(dx.I8, da.ptr, shape, 2, dims, 1, out.ptr, ws.ptr, need.value, None))
        assert np.array_equal(out.get(), A.max(axis=axis)), axis


def test_changeshape_past_2g(dxh, big):
    a, da = big
    A = a.reshape(ROWS, COLS)
    shape = dx.i32arr([ROWS, COLS])
    out = Dev.empty(N, np.int8)
    dx.check(dxh.dxh_transpose(dx.I8, da.ptr, shape, 2, dx.i32arr([1, 0]), out.ptr, None))
    got = out.get().reshape(COLS, ROWS)
    assert np.array_equal(got, A.T)
    del got
    # gather rows from both ends of the table: row offsets beyond 2^31 bytes
    idx = np.array([ROWS - 1, 0, 65537, ROWS - 2, 40000, 69999], dtype=np.int64)
    di, dg = Dev(idx), Dev.empty(idx.size * COLS, np.int8)
    dx.check(dxh.dxh_indexselect(dx.I8, da.ptr, shape, 2, dx.I64, di.ptr, dx.i32arr([idx.size]), 1, 0, dg.ptr, None))
    assert np.array_equal(dg.get().reshape(idx.size, COLS), A[idx])
    # broadcast one row to the full height: the output alone passes 2^31 elements
    row = Dev(A[12345].copy())
    dx.check(dxh.dxh_broadcastTo(dx.I8, row.ptr, dx.i32arr([1, COLS]), 2, shape, 2, out.ptr, None))
    got = out.get().reshape(ROWS, COLS)
    assert np.array_equal(got[0], A[12345]) and np.array_equal(got[-1], A[12345]) and np.all(got == A[12345][None, :])
    del got
    # concat two halves along axis 0 back into the whole
    half = ROWS // 2
    top, bottom = Dev(A[:half].copy()), Dev(A[half:].copy())
    ins = dx.ptrarr([top.t.data_ptr(), bottom.t.data_ptr()])
    dx.check(dxh.dxh_concat(dx.I8, ins, 2, dx.i32arr([half, ROWS - half]), shape, 2, 0, out.ptr, None))
    assert np.array_equal(out.get().reshape(ROWS, COLS), A)
