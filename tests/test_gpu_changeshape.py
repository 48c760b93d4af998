"""GPU parity: transpose / concat / broadcastTo / indexselect / repeat, bit-exact vs the oracle
(and numpy) on raw element bits."""
import numpy as np
import pytest

from deepx_amd import lib as dx
from tests import helpers as H
from tests.helpers import Dev, hp

pytestmark = pytest.mark.gpu

RAW = {1: (dx.I8, np.uint8), 2: (dx.BF16, np.uint16), 4: (dx.F32, np.uint32), 8: (dx.I64, np.uint64)}


def rnd(rng, shape, es):
    return rng.integers(0, 256, size=int(np.prod(shape)) * es, dtype=np.uint8).view(RAW[es][1]).reshape(shape)


TRANSPOSES = [
    ((6, 10), [1, 0]),
    ((65, 130), [1, 0]),
    ((3, 5, 7), [2, 0, 1]),
    ((3, 5, 7), [0, 2, 1]),
    ((3, 5, 7), [1, 0, 2]),       # keeps the last axis
    ((2, 16, 3, 8), [0, 2, 1, 3]),  # attention permute
    ((2, 3, 4, 5), [3, 2, 1, 0]),
    ((4, 1, 6), [2, 1, 0]),
    ((7,), [0]),
    ((2, 3, 4), [0, 1, 2]),       # identity
    ((129, 3, 67), [2, 1, 0]),
]


@pytest.mark.parametrize("es", [1, 2, 4, 8])
def test_transpose(dxh, orc, es):
    rng = np.random.default_rng(40 + es)
    dtype = RAW[es][0]
    for shape, order in TRANSPOSES:
        a = rnd(rng, shape, es)
        da, out = Dev(a), Dev.empty(a.size, a.dtype)
        dx.check(dxh.dxh_transpose(dtype, da.ptr, dx.i32arr(shape), len(shape), dx.i32arr(order), out.ptr, None), "transpose")
        want = np.empty(a.size, dtype=a.dtype)
        assert orc.orc_transpose(dtype, hp(a), dx.i32arr(shape), len(shape), dx.i32arr(order), hp(want)) == 0
        got = out.get()
        assert np.array_equal(got, want), (shape, order)
        assert np.array_equal(got, np.transpose(a, order).reshape(-1))


# shapes whose extents are multiples of 16 elements in the two moving axes: the 16-byte tiled
# kernel for every element size (tiles of 16..256 elements per side), with ragged tile edges,
# batch axes before / between / after the moving axes, and short innermost runs (2..16 bytes)
# that are folded into the element
VEC_TRANSPOSES = [
    ((256, 512), [1, 0]),
    ((272, 48), [1, 0]),            # partial tiles on both sides
    ((3, 64, 96), [0, 2, 1]),
    ((32, 5, 48), [2, 1, 0]),
    ((16, 7, 32, 3), [2, 1, 0, 3]),   # batch axis between, innermost run of 3 elements stays
    ((48, 64, 4), [1, 0, 2]),       # innermost run of 4 elements: folded for 1/2/4-byte elements
    ((48, 64, 2), [1, 0, 2]),
    ((2, 48, 16, 8), [0, 2, 1, 3]),
    ((5, 16, 2, 32), [0, 3, 2, 1]),
    ((512, 16), [1, 0]),
    ((16, 1024), [1, 0]),
]


@pytest.mark.parametrize("es", [1, 2, 4, 8])
def test_transpose_vector_tiles(dxh, es):
    rng = np.random.default_rng(140 + es)
    dtype = RAW[es][0]
    for shape, order in VEC_TRANSPOSES:
        a = rnd(rng, shape, es)
        da, out = Dev(a), Dev.empty(a.size, a.dtype)
        dx.check(dxh.dxh_transpose(dtype, da.ptr, dx.i32arr(shape), len(shape), dx.i32arr(order), out.ptr, None), "transpose")
        assert np.array_equal(out.get(), np.transpose(a, order).reshape(-1)), (es, shape, order)


def test_transpose_unaligned_base_takes_the_elementwise_tiles(dxh):
    """Same shapes from a base address that is only element-aligned: the 16-byte kernel must not be
    chosen (it would fault or read the wrong bytes)."""
    rng = np.random.default_rng(150)
    for es in (1, 2, 4):
        dtype = RAW[es][0]
        for shape, order in [((256, 512), [1, 0]), ((48, 64, 4), [1, 0, 2])]:
            a = rnd(rng, shape, es)
            n = a.size
            buf_in, buf_out = Dev.empty(n + 16, a.dtype), Dev.empty(n + 16, a.dtype)
            import torch
            buf_in.t[es:es + n * es].copy_(torch.from_numpy(a.reshape(-1).view(np.uint8).copy()))
            pin, pout = buf_in.t.data_ptr() + es, buf_out.t.data_ptr() + es
            dx.check(dxh.dxh_transpose(dtype, pin, dx.i32arr(shape), len(shape), dx.i32arr(order), pout, None), "transpose")
            torch.cuda.synchronize()
            got = buf_out.t[es:es + n * es].cpu().numpy().view(a.dtype)
            assert np.array_equal(got, np.transpose(a, order).reshape(-1)), (es, shape, order)


def test_transpose_bad_order(dxh):
    a = Dev(np.zeros(24, dtype=np.float32))
    assert dxh.dxh_transpose(dx.F32, a.ptr, dx.i32arr([2, 3, 4]), 3, dx.i32arr([0, 0, 1]), a.ptr, None) == -2
    assert dxh.dxh_transpose(dx.F32, a.ptr, dx.i32arr([2, 3, 4]), 3, dx.i32arr([0, 1, 3]), a.ptr, None) == -2


def test_concat_reference_expectation_on_the_hip_path(dxh):
    """The expectation the reference's own concat test holds
    (executor/op-ompsimd/test/tensorfunc/8_tensor_concat.cpp:47-129: four constant-filled [2,3,4]
    tensors joined along each axis), through dxh_concat."""
    import json
    import os
    g = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "concat_kat.json")))
    arrs = [np.full(t["shape"], t["fill"], dtype=np.float32) for t in g["inputs"]]
    devs = [Dev(a) for a in arrs]
    for axis_s, exp in g["expected"].items():
        axis, shape = int(axis_s), exp["shape"]
        out = Dev.empty(int(np.prod(shape)), np.float32)
        dx.check(dxh.dxh_concat(dx.F32, dx.ptrarr([d.ptr.value for d in devs]), len(devs), dx.i32arr([a.shape[axis] for a in arrs]),
                                dx.i32arr(shape), 3, axis, out.ptr, None), "concat")
        got = out.get().reshape(shape)
        if axis == 0:
            for i, v in enumerate(exp["blocks"]):
                assert np.all(got[i] == v)
        elif axis == 1:
            for i in range(2):
                assert np.array_equal(got[i], np.repeat(np.array(exp["rows"], dtype=np.float32)[:, None], 4, axis=1))
        else:
            assert np.all(got == np.array(exp["row"], dtype=np.float32))


@pytest.mark.parametrize("es", [1, 2, 4, 8])
def test_concat(dxh, orc, es):
    rng = np.random.default_rng(50 + es)
    dtype = RAW[es][0]
    cases = [([(2, 3), (2, 5), (2, 1)], 1), ([(2, 3), (4, 3)], 0), ([(2, 3, 8), (2, 4, 8), (2, 1, 8)], 1),
             ([(3, 4, 5)] * 3, 2), ([(1, 7)] * 11, 0), ([(2, 0, 4), (2, 3, 4)], 1)]
    for shapes, axis in cases:
        arrs = [rnd(rng, s, es) for s in shapes]
        want_np = np.concatenate(arrs, axis=axis)
        devs = [Dev(a) for a in arrs]
        out = Dev.empty(want_np.size, want_np.dtype)
        axs = dx.i32arr([s[axis] for s in shapes])
        osh = dx.i32arr(want_np.shape)
        dx.check(dxh.dxh_concat(dtype, dx.ptrarr([d.ptr.value for d in devs]), len(arrs), axs, osh, want_np.ndim, axis, out.ptr, None), "concat")
        want = np.empty(want_np.size, dtype=want_np.dtype)
        assert orc.orc_concat(dtype, dx.ptrarr([a.ctypes.data for a in arrs]), len(arrs), axs, osh, want_np.ndim, axis, hp(want)) == 0
        got = out.get()
        assert np.array_equal(got, want), (shapes, axis)
        assert np.array_equal(got, want_np.reshape(-1))


@pytest.mark.parametrize("es", [1, 2, 4, 8])
def test_broadcast(dxh, orc, es):
    rng = np.random.default_rng(60 + es)
    dtype = RAW[es][0]
    cases = [((1, 8), (5, 8)), ((8,), (3, 5, 8)), ((5, 1), (5, 9)), ((3, 1, 4), (3, 6, 4)), ((1,), (4, 4)),
             ((2, 1, 3, 1), (2, 5, 3, 7)), ((4, 4), (4, 4)), ((1, 1, 6), (2, 3, 6)), ((7, 1), (2, 7, 33))]
    for ishape, oshape in cases:
        a = rnd(rng, ishape, es)
        want_np = np.broadcast_to(a, oshape)
        da, out = Dev(a), Dev.empty(want_np.size, a.dtype)
        dx.check(dxh.dxh_broadcastTo(dtype, da.ptr, dx.i32arr(ishape), len(ishape), dx.i32arr(oshape), len(oshape), out.ptr, None), "broadcastTo")
        want = np.empty(want_np.size, dtype=a.dtype)
        assert orc.orc_broadcastTo(dtype, hp(a), dx.i32arr(ishape), len(ishape), dx.i32arr(oshape), len(oshape), hp(want)) == 0
        got = out.get()
        assert np.array_equal(got, want), (ishape, oshape)
        assert np.array_equal(got, np.ascontiguousarray(want_np).reshape(-1))
    a = Dev(np.zeros(6, dtype=np.float32))
    assert dxh.dxh_broadcastTo(dx.F32, a.ptr, dx.i32arr([2, 3]), 2, dx.i32arr([4, 3]), 2, a.ptr, None) == -3


@pytest.mark.parametrize("es", [1, 2, 4, 8])
@pytest.mark.parametrize("idt", [dx.I32, dx.I64])
def test_indexselect(dxh, orc, es, idt):
    rng = np.random.default_rng(70 + es)
    dtype = RAW[es][0]
    cases = [((50, 8), (7,), 0), ((50, 9), (7,), 0), ((4, 10, 6), (3, 2), 1), ((4, 10, 6), (5,), -1), ((6, 5), (2, 3), 1)]
    for ishape, xshape, axis in cases:
        a = rnd(rng, ishape, es)
        ax = axis % len(ishape)
        idx = rng.integers(0, ishape[ax], size=xshape).astype(np.int32 if idt == dx.I32 else np.int64)
        want_np = np.take(a, idx, axis=ax)
        da, di, out = Dev(a), Dev(idx), Dev.empty(want_np.size, a.dtype)
        dx.check(dxh.dxh_indexselect(dtype, da.ptr, dx.i32arr(ishape), len(ishape), idt, di.ptr, dx.i32arr(xshape), len(xshape), axis, out.ptr, None), "indexselect")
        want = np.empty(want_np.size, dtype=a.dtype)
        assert orc.orc_indexselect(dtype, hp(a), dx.i32arr(ishape), len(ishape), idt, hp(idx), dx.i32arr(xshape), len(xshape), axis, hp(want)) == 0
        got = out.get()
        assert np.array_equal(got, want), (ishape, xshape, axis)
        assert np.array_equal(got, want_np.reshape(-1))


def test_indexselect_out_of_range_is_clamped(dxh):
    a = np.arange(40, dtype=np.float32).reshape(10, 4)
    idx = np.array([-5, 0, 9, 10, 1000], dtype=np.int64)
    da, di, out = Dev(a), Dev(idx), Dev.empty(20, np.float32)
    dx.check(dxh.dxh_indexselect(dx.F32, da.ptr, dx.i32arr([10, 4]), 2, dx.I64, di.ptr, dx.i32arr([5]), 1, 0, out.ptr, None))
    assert np.array_equal(out.get().reshape(5, 4), a[[0, 0, 9, 9, 9]])


@pytest.mark.parametrize("es", [1, 2, 4, 8])
def test_repeat(dxh, orc, es):
    rng = np.random.default_rng(80 + es)
    dtype = RAW[es][0]
    for shape, reps in [((3, 4), (2, 3)), ((2, 3, 4), (1, 2, 1)), ((5,), (4,)), ((64, 48), (3, 2)), ((16, 1, 32), (1, 5, 1)), ((4096,), (7,)),
                        ((2, 3, 2, 3, 2, 3, 2, 3), (2, 2, 2, 2, 2, 2, 2, 2)),   # 16 interleaved axes: more than the row kernels index
                        ((3, 2, 2, 2, 2, 2, 2), (1, 2, 1, 2, 1, 2, 3))]:
        a = rnd(rng, shape, es)
        want_np = a
        for ax, r in enumerate(reps):
            want_np = np.repeat(want_np, r, axis=ax)
        da, out = Dev(a), Dev.empty(want_np.size, a.dtype)
        dx.check(dxh.dxh_repeat(dtype, da.ptr, dx.i32arr(shape), len(shape), dx.i32arr(reps), out.ptr, None), "repeat")
        want = np.empty(want_np.size, dtype=a.dtype)
        assert orc.orc_repeat(dtype, hp(a), dx.i32arr(shape), len(shape), dx.i32arr(reps), hp(want)) == 0
        got = out.get()
        assert np.array_equal(got, want)
        assert np.array_equal(got, want_np.reshape(-1))


def test_config3_full_size(dxh):
    """BASELINE config 3 at full size: round-trip and numpy equality on bit patterns."""
    rng = np.random.default_rng(5)
    shape = (32, 2048, 14, 64)
    T = rng.integers(0, 65536, size=shape, dtype=np.uint16)
    dT, out, back = Dev(T), Dev.empty(T.size, np.uint16), Dev.empty(T.size, np.uint16)
    dx.check(dxh.dxh_transpose(dx.BF16, dT.ptr, dx.i32arr(shape), 4, dx.i32arr([0, 2, 1, 3]), out.ptr, None))
    assert np.array_equal(out.get().reshape(32, 14, 2048, 64), T.transpose(0, 2, 1, 3))
    # transposing back with the inverse permutation restores the input (involution)
    dx.check(dxh.dxh_transpose(dx.BF16, out.ptr, dx.i32arr([32, 14, 2048, 64]), 4, dx.i32arr([0, 2, 1, 3]), back.ptr, None))
    assert np.array_equal(back.get().reshape(shape), T)
    del dT, out, back
    cs = [np.random.default_rng(6 + i).integers(0, 65536, size=(16, 1024, 4096), dtype=np.uint16) for i in range(3)]
    devs = [Dev(c) for c in cs]
    out = Dev.empty(3 * cs[0].size, np.uint16)
    dx.check(dxh.dxh_concat(dx.F16, dx.ptrarr([d.ptr.value for d in devs]), 3, dx.i32arr([1024] * 3), dx.i32arr([16, 3072, 4096]), 3, 1, out.ptr, None))
    got = out.get().reshape(16, 3072, 4096)
    for i in range(3):
        assert np.array_equal(got[:, 1024 * i:1024 * (i + 1), :], cs[i])
    del devs, out
    r = np.random.default_rng(9).integers(0, 65536, size=(1, 4096), dtype=np.uint16)
    dr, out = Dev(r), Dev.empty(8192 * 4096, np.uint16)
    dx.check(dxh.dxh_broadcastTo(dx.BF16, dr.ptr, dx.i32arr([1, 4096]), 2, dx.i32arr([8192, 4096]), 2, out.ptr, None))
    assert np.array_equal(out.get().reshape(8192, 4096), np.broadcast_to(r, (8192, 4096)))


def test_config4_full_size(dxh, orc):
    """BASELINE config 4: int32 2^26 max/min/greater/where, and the bf16 embedding gather."""
    n = 1 << 26
    a = np.random.default_rng(10).integers(-2 ** 20, 2 ** 20, n, endpoint=True).astype(np.int32)
    b = np.random.default_rng(11).integers(-2 ** 20, 2 ** 20, n, endpoint=True).astype(np.int32)
    da, db, dc, dm = Dev(a), Dev(b), Dev.empty(n, np.int32), Dev.empty(n, np.uint8)
    dx.check(dxh.dxh_max(dx.I32, da.ptr, db.ptr, dc.ptr, n, None))
    assert np.array_equal(dc.get(), np.maximum(a, b))
    dx.check(dxh.dxh_min(dx.I32, da.ptr, db.ptr, dc.ptr, n, None))
    assert np.array_equal(dc.get(), np.minimum(a, b))
    dx.check(dxh.dxh_greater(dx.I32, da.ptr, db.ptr, dm.ptr, n, None))
    m = dm.get()
    assert np.array_equal(m, (a > b).astype(np.uint8))
    # where(m, a, b) == switch([b a], m)
    dx.check(dxh.dxh_switch(dx.I32, dx.ptrarr([db.ptr.value, da.ptr.value]), 2, dx.BOOL, dm.ptr, dc.ptr, n, None))
    w = dc.get()
    assert np.array_equal(w, np.where(a > b, a, b))
    assert np.array_equal(w, np.maximum(a, b))  # where(a>b,a,b) is max: a checksum of the whole chain
    del da, db, dc, dm
    E = H.f32_to_bf16_bits(np.random.default_rng(12).standard_normal((151936, 896), dtype=np.float32) * 0.02)
    idx = np.random.default_rng(13).integers(0, 151936, 4096).astype(np.int64)
    dE, di, out = Dev(E), Dev(idx), Dev.empty(4096 * 896, np.uint16)
    dx.check(dxh.dxh_indexselect(dx.BF16, dE.ptr, dx.i32arr([151936, 896]), 2, dx.I64, di.ptr, dx.i32arr([4096]), 1, 0, out.ptr, None))
    assert np.array_equal(out.get().reshape(4096, 896), E[idx])
