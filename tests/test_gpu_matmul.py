"""GPU parity: matmul vs the oracle (float64 accumulation) and the reference's known answer.

Bars: fp32/f64 within rel 1e-5*sqrt(K) (f64: 1e-13*sqrt(K)) of |A||B| row-column magnitude;
bf16/f16 (MFMA, fp32 accumulate, one rounding) within rel 1e-2; integers bit-exact.
"""
import numpy as np
import pytest

from deepx_amd import lib as dx
from tests import helpers as H
from tests.helpers import Dev, hp

pytestmark = pytest.mark.gpu


def run(dxh, orc, dtype, A, B, batch, m, k, n):
    dA, dB, dC = Dev(A), Dev(B), Dev.empty(batch * m * n, A.dtype)
    dx.check(H.matmul(dxh, dtype, dA.ptr, dB.ptr, dC.ptr, batch, m, k, n, None), "matmul")
    want = np.empty(batch * m * n, dtype=A.dtype)
    assert orc.orc_matmul(dtype, hp(A), hp(B), hp(want), batch, m, k, n) == 0
    return dC.get(), want


SHAPES = [(1, 1, 1, 1), (1, 3, 4, 5), (2, 3, 4, 5), (1, 64, 64, 64), (1, 128, 32, 128), (3, 130, 70, 150),
          (1, 257, 129, 65), (2, 31, 200, 17), (1, 256, 896, 384),
          (3, 320, 2048, 64)]  # attention weights x values: one tile across N, rows of A 4 KiB apart in 16-bit types


@pytest.mark.parametrize("dtype", [dx.F32, dx.F64, dx.BF16, dx.F16])
def test_matmul_float(dxh, orc, dtype):
    rng = np.random.default_rng(90 + dtype)
    for batch, m, k, n in SHAPES:
        A = H.to_storage(rng.standard_normal(batch * m * k), dtype)
        B = H.to_storage(rng.standard_normal(batch * k * n), dtype)
        got, want = run(dxh, orc, dtype, A, B, batch, m, k, n)
        g, w = H.to_float(got, dtype), H.to_float(want, dtype)
        Af = np.abs(H.to_float(A, dtype)).reshape(batch, m, k)
        Bf = np.abs(H.to_float(B, dtype)).reshape(batch, k, n)
        mag = np.matmul(Af, Bf).reshape(-1)  # sum_k |a||b|: the scale rounding errors grow with
        rel = {dx.F32: 1e-5 * np.sqrt(k), dx.F64: 1e-13 * np.sqrt(k), dx.BF16: 1e-2, dx.F16: 1e-2}[dtype]
        assert np.all(np.abs(g - w) <= rel * np.maximum(mag, 1e-30)), (dtype, batch, m, k, n, np.max(np.abs(g - w) / np.maximum(mag, 1e-30)))


@pytest.mark.parametrize("dtype", H.INTS)
def test_matmul_int_exact(dxh, orc, dtype):
    rng = np.random.default_rng(95 + dtype)
    for batch, m, k, n in SHAPES[:7]:
        A = rng.integers(-5, 6, batch * m * k).astype(H.NP[dtype])
        B = rng.integers(-5, 6, batch * k * n).astype(H.NP[dtype])
        got, want = run(dxh, orc, dtype, A, B, batch, m, k, n)
        assert np.array_equal(got, want)


def test_matmul_reference_known_answer(dxh):
    """arange(24).reshape(2,3,4) @ arange(40).reshape(2,4,5), the expectation held in
    executor/op-ompsimd/test/tensorfunc/4_tensor_matmul.cpp:18-36."""
    A = np.arange(24, dtype=np.float32)
    B = np.arange(40, dtype=np.float32)
    dA, dB, dC = Dev(A), Dev(B), Dev.empty(30, np.float32)
    dx.check(H.matmul(dxh, dx.F32, dA.ptr, dB.ptr, dC.ptr, 2, 3, 4, 5, None))
    want = np.array([[[70, 76, 82, 88, 94], [190, 212, 234, 256, 278], [310, 348, 386, 424, 462]],
                     [[1510, 1564, 1618, 1672, 1726], [1950, 2020, 2090, 2160, 2230], [2390, 2476, 2562, 2648, 2734]]],
                    dtype=np.float32)
    assert np.array_equal(dC.get().reshape(2, 3, 5), want)


@pytest.mark.parametrize("dtype", [dx.BF16, dx.F16])
def test_config5_gemm_shapes_half(dxh, orc, dtype):
    """BASELINE config 5 GEMM shapes, bf16 (and f16) in / fp32 accumulate / 16-bit out: every element of
    every output tile against float64 numpy (the launches these shapes take, one round of 160x256
    tiles and 128x128 tiles whose K is cut in two, are checked whole, not on a sample); bar rel 1e-2 of
    sum_k |a||b|."""
    rng = np.random.default_rng(14)
    for (m, k, n), seed in [((2048, 896, 4864), 15), ((2048, 4864, 896), 17)]:
        A = H.to_storage(rng.standard_normal(m * k).astype(np.float32), dtype)
        B = H.to_storage(np.random.default_rng(seed).standard_normal(k * n).astype(np.float32) * 0.02, dtype)
        dA, dB, dC = Dev(A), Dev(B), Dev.empty(m * n, np.uint16)
        dx.check(H.matmul(dxh, dtype, dA.ptr, dB.ptr, dC.ptr, 1, m, k, n, None))
        got = H.to_float(dC.get(), dtype).reshape(m, n).astype(np.float64)
        Af = H.to_float(A, dtype).reshape(m, k).astype(np.float64)
        Bf = H.to_float(B, dtype).reshape(k, n).astype(np.float64)
        ref = Af @ Bf
        mag = np.abs(Af) @ np.abs(Bf)
        bad = np.abs(got - ref) > 1e-2 * mag
        assert not bad.any(), (m, k, n, int(bad.sum()), np.argwhere(bad)[:4].tolist())
        # and tighter in the mean: one rounding to 8 (11) significant bits of a sum accumulated in fp32
        assert np.mean(np.abs(got - ref) / np.maximum(np.abs(ref), 1e-30) * (np.abs(ref) > 1e-3 * mag)) < (2.0 ** -9 if dtype == dx.BF16 else 2.0 ** -12)


TILE_KNOB = 4  # DXH_TUNE_MATMUL_TILE


@pytest.mark.parametrize("tile", [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15])
@pytest.mark.parametrize("dtype", [dx.BF16, dx.F16])
def test_matmul_tile_configs(dxh, dtype, tile):
    """Every workgroup tile of the MFMA kernel (forced through the tuning knob) on aligned shapes
    with ragged tile edges, more than one batch and M, N below one tile; float64 numpy is the
    reference, bar rel 1e-2 of sum_k |a||b| as above.  K = 72, 8, 1000, 56 end in a partial K step
    (zero-filled in the kernel; tiles 7 to 15, whose operands go straight into LDS in whole K steps,
    hand those to their register-staged twins); K = 32 and 64 are shorter than the LDS pipeline of
    those tiles, K = 192 and 448 wrap around its stages.  Tiles 11 and 12 (160 and 128 rows, four
    waves side by side) meet M below, at and above a tile, with a last tile of 1 to 159 rows."""
    rng = np.random.default_rng(300 + tile + dtype)
    dx.check(dxh.dxh_tune(TILE_KNOB, tile))
    try:
        for batch, m, k, n in [(2, 300, 128, 264), (1, 520, 192, 520), (3, 70, 64, 8), (1, 257, 64, 1032), (1, 1, 64, 16),
                               (1, 1024, 448, 768), (1, 300, 72, 264), (2, 130, 8, 16), (1, 257, 1000, 520), (1, 64, 56, 64),
                               (1, 300, 32, 264), (2, 511, 96, 776)]:
            A = H.to_storage(rng.standard_normal(batch * m * k), dtype)
            B = H.to_storage(rng.standard_normal(batch * k * n), dtype)
            dA, dB, dC = Dev(A), Dev(B), Dev.empty(batch * m * n, A.dtype)
            dx.check(H.matmul(dxh, dtype, dA.ptr, dB.ptr, dC.ptr, batch, m, k, n, None), "matmul")
            got = H.to_float(dC.get(), dtype).astype(np.float64).reshape(batch, m, n)
            Af = H.to_float(A, dtype).astype(np.float64).reshape(batch, m, k)
            Bf = H.to_float(B, dtype).astype(np.float64).reshape(batch, k, n)
            ref, mag = np.matmul(Af, Bf), np.matmul(np.abs(Af), np.abs(Bf))
            assert np.all(np.abs(got - ref) <= 1e-2 * np.maximum(mag, 1e-30)), (tile, dtype, batch, m, k, n)
    finally:
        dx.check(dxh.dxh_tune(TILE_KNOB, 0))


def test_matmul_tiles_exact_on_small_integers(dxh):
    """Small integer operands are exact in bf16 and their dot products exact in fp32, whatever the
    summation order: every tile must return the exact product rounded once (RNE) to bf16.  A wrong
    fragment, k-permutation or edge clamp changes an integer and fails bit-exactly."""
    rng = np.random.default_rng(77)
    # the second K ends in a partial K step; the third is one tile wide with rows of A 4 KiB apart: its tiles start at K steps of their own
    for m, k, n in [(384, 256, 520), (200, 200, 136), (704, 2048, 64)]:
        lim = 4 if k <= 256 else 1  # |sum| <= 16*256 = 4096 or 2048: exact in fp32
        Ai, Bi = rng.integers(-lim, lim + 1, (m, k)), rng.integers(-lim, lim + 1, (k, n))
        A = H.to_storage(Ai.astype(np.float64).reshape(-1), dx.BF16)
        B = H.to_storage(Bi.astype(np.float64).reshape(-1), dx.BF16)
        want = (Ai @ Bi).astype(np.float64)
        dA, dB, dC = Dev(A), Dev(B), Dev.empty(m * n, np.uint16)
        for tile in (0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15):
            dx.check(dxh.dxh_tune(TILE_KNOB, tile))
            try:
                dx.check(H.matmul(dxh, dx.BF16, dA.ptr, dB.ptr, dC.ptr, 1, m, k, n, None))
                got = H.to_float(dC.get(), dx.BF16).astype(np.float64).reshape(m, n)
            finally:
                dx.check(dxh.dxh_tune(TILE_KNOB, 0))
            # one RNE rounding of the exact integer to bf16
            assert np.array_equal(got, H.to_float(H.to_storage(want.reshape(-1), dx.BF16), dx.BF16).astype(np.float64).reshape(m, n)), (tile, k)


@pytest.mark.parametrize("tile", [1, 2, 3, 4])
def test_matmul_f32_tile_configs(dxh, tile):
    """Every tile of the fp32 matrix-pipe kernel, on 16-byte-friendly shapes (vector path) and on
    odd K / N / unaligned bases (element-wise path), ragged edges, batches and a K that is not a
    multiple of the K step.  Bar: rel 1e-5*sqrt(K) of sum_k |a||b| against float64 numpy."""
    rng = np.random.default_rng(500 + tile)
    dx.check(dxh.dxh_tune(TILE_KNOB, tile))
    try:
        for batch, m, k, n in [(2, 300, 128, 264), (1, 130, 100, 68), (3, 70, 33, 9), (1, 257, 64, 1030), (1, 1, 4, 4),
                               (1, 520, 1000, 260), (2, 65, 7, 129)]:
            A = rng.standard_normal(batch * m * k).astype(np.float32)
            B = rng.standard_normal(batch * k * n).astype(np.float32)
            dA, dB, dC = Dev(A), Dev(B), Dev.empty(batch * m * n, np.float32)
            dx.check(H.matmul(dxh, dx.F32, dA.ptr, dB.ptr, dC.ptr, batch, m, k, n, None), "matmul")
            got = dC.get().astype(np.float64).reshape(batch, m, n)
            Af, Bf = A.astype(np.float64).reshape(batch, m, k), B.astype(np.float64).reshape(batch, k, n)
            ref, mag = np.matmul(Af, Bf), np.matmul(np.abs(Af), np.abs(Bf))
            assert np.all(np.abs(got - ref) <= 1e-5 * np.sqrt(k) * np.maximum(mag, 1e-30)), (tile, batch, m, k, n)
        # exact on small integers whatever the summation order
        m, k, n = 200, 96, 132
        Ai, Bi = rng.integers(-8, 9, (m, k)), rng.integers(-8, 9, (k, n))
        dA, dB, dC = Dev(Ai.astype(np.float32).reshape(-1)), Dev(Bi.astype(np.float32).reshape(-1)), Dev.empty(m * n, np.float32)
        dx.check(H.matmul(dxh, dx.F32, dA.ptr, dB.ptr, dC.ptr, 1, m, k, n, None))
        assert np.array_equal(dC.get().reshape(m, n), (Ai @ Bi).astype(np.float32))
    finally:
        dx.check(dxh.dxh_tune(TILE_KNOB, 0))


@pytest.mark.parametrize("tile", [1, 2, 3])
def test_matmul_f64_tile_configs(dxh, tile):
    """Every tile of the fp64 matrix-pipe kernel: vector path (even K, N), element-wise path (odd
    K / N), ragged edges, batches, K not a multiple of the K step.  Bar: rel 1e-13*sqrt(K) of
    sum_k |a||b| against numpy's float64 product (a different summation order), and exact on
    small integers."""
    rng = np.random.default_rng(600 + tile)
    dx.check(dxh.dxh_tune(TILE_KNOB, tile))
    try:
        for batch, m, k, n in [(2, 300, 128, 264), (1, 130, 100, 68), (3, 70, 33, 9), (1, 257, 64, 1030), (1, 1, 2, 2),
                               (1, 520, 1000, 260), (2, 65, 7, 129)]:
            A = rng.standard_normal(batch * m * k)
            B = rng.standard_normal(batch * k * n)
            dA, dB, dC = Dev(A), Dev(B), Dev.empty(batch * m * n, np.float64)
            dx.check(H.matmul(dxh, dx.F64, dA.ptr, dB.ptr, dC.ptr, batch, m, k, n, None), "matmul")
            got = dC.get().reshape(batch, m, n)
            Af, Bf = A.reshape(batch, m, k), B.reshape(batch, k, n)
            ref, mag = np.matmul(Af, Bf), np.matmul(np.abs(Af), np.abs(Bf))
            assert np.all(np.abs(got - ref) <= 1e-13 * np.sqrt(k) * np.maximum(mag, 1e-300)), (tile, batch, m, k, n)
        m, k, n = 200, 96, 132
        Ai, Bi = rng.integers(-1000, 1001, (m, k)), rng.integers(-1000, 1001, (k, n))
        dA, dB, dC = Dev(Ai.astype(np.float64).reshape(-1)), Dev(Bi.astype(np.float64).reshape(-1)), Dev.empty(m * n, np.float64)
        dx.check(H.matmul(dxh, dx.F64, dA.ptr, dB.ptr, dC.ptr, 1, m, k, n, None))
        assert np.array_equal(dC.get().reshape(m, n), (Ai @ Bi).astype(np.float64))
    finally:
        dx.check(dxh.dxh_tune(TILE_KNOB, 0))


SPLITK_KNOB = 6  # DXH_TUNE_MATMUL_SPLITK


def _ref_product(A, B, dtype, batch, m, k, n):
    Af = H.to_float(A, dtype).astype(np.float64).reshape(batch, m, k)
    Bf = H.to_float(B, dtype).astype(np.float64).reshape(batch, k, n)
    return np.matmul(Af, Bf), np.matmul(np.abs(Af), np.abs(Bf))


@pytest.mark.parametrize("dtype", [dx.BF16, dx.F16, dx.F32, dx.F64])
@pytest.mark.parametrize("splits", [2, 3, 7])
def test_matmul_split_k_forced(dxh, dtype, splits):
    """A product cut into K slices (forced through the tuning knob) against float64 numpy, on
    batches, ragged tiles, a K that ends in a partial K step and a K shorter than `splits` K steps;
    same bars as the unsplit kernels.  Small-integer operands must come out exact, and a second
    run bit-identical (the slices are added in a fixed order)."""
    rng = np.random.default_rng(700 + dtype + splits)
    rel = {dx.F32: 1e-5, dx.F64: 1e-13, dx.BF16: 1e-2, dx.F16: 1e-2}[dtype]
    dx.check(dxh.dxh_tune(SPLITK_KNOB, splits))
    try:
        for batch, m, k, n in [(1, 64, 1024, 64), (2, 70, 520, 72), (1, 16, 4096, 136), (3, 1, 200, 8), (1, 130, 64, 64), (1, 33, 1000, 264)]:
            A = H.to_storage(rng.standard_normal(batch * m * k), dtype)
            B = H.to_storage(rng.standard_normal(batch * k * n), dtype)
            dA, dB, dC = Dev(A), Dev(B), Dev.empty(batch * m * n, A.dtype)
            dx.check(H.matmul(dxh, dtype, dA.ptr, dB.ptr, dC.ptr, batch, m, k, n, None), "matmul")
            first = dC.get()
            got = H.to_float(first, dtype).astype(np.float64).reshape(batch, m, n)
            ref, mag = _ref_product(A, B, dtype, batch, m, k, n)
            scale = np.sqrt(k) if dtype in (dx.F32, dx.F64) else 1.0
            assert np.all(np.abs(got - ref) <= rel * scale * np.maximum(mag, 1e-300)), (dtype, splits, batch, m, k, n)
            dC2 = Dev.empty(batch * m * n, A.dtype)
            dx.check(H.matmul(dxh, dtype, dA.ptr, dB.ptr, dC2.ptr, batch, m, k, n, None), "matmul")
            assert np.array_equal(first, dC2.get()), "split-K result varies between runs"
        m, k, n = 96, 456, 72
        Ai, Bi = rng.integers(-4, 5, (m, k)), rng.integers(-4, 5, (k, n))
        A = H.to_storage(Ai.astype(np.float64).reshape(-1), dtype)
        B = H.to_storage(Bi.astype(np.float64).reshape(-1), dtype)
        dA, dB, dC = Dev(A), Dev(B), Dev.empty(m * n, A.dtype)
        dx.check(H.matmul(dxh, dtype, dA.ptr, dB.ptr, dC.ptr, 1, m, k, n, None))
        want = H.to_float(H.to_storage((Ai @ Bi).astype(np.float64).reshape(-1), dtype), dtype)  # one rounding of the exact integer
        assert np.array_equal(H.to_float(dC.get(), dtype), want)
    finally:
        dx.check(dxh.dxh_tune(SPLITK_KNOB, 0))


@pytest.mark.parametrize("dtype", [dx.BF16, dx.F32, dx.F64])
def test_matmul_skinny_shapes_auto_split(dxh, dtype):
    """Shapes that the launcher cuts along K by itself (few output tiles, long K), and the same
    shapes with the knob at 1 (never cut): both within the bar of float64 numpy."""
    rng = np.random.default_rng(800 + dtype)
    rel = {dx.F32: 1e-5, dx.F64: 1e-13, dx.BF16: 1e-2}[dtype]
    for knob in (0, 1):
        dx.check(dxh.dxh_tune(SPLITK_KNOB, knob))
        try:
            for batch, m, k, n in [(1, 1, 4096, 512), (1, 16, 2048, 1024), (1, 64, 20000, 64), (2, 300, 1024, 8)]:
                A = H.to_storage(rng.standard_normal(batch * m * k), dtype)
                B = H.to_storage(rng.standard_normal(batch * k * n), dtype)
                dA, dB, dC = Dev(A), Dev(B), Dev.empty(batch * m * n, A.dtype)
                dx.check(H.matmul(dxh, dtype, dA.ptr, dB.ptr, dC.ptr, batch, m, k, n, None), "matmul")
                got = H.to_float(dC.get(), dtype).astype(np.float64).reshape(batch, m, n)
                ref, mag = _ref_product(A, B, dtype, batch, m, k, n)
                scale = np.sqrt(k) if dtype in (dx.F32, dx.F64) else 1.0
                assert np.all(np.abs(got - ref) <= rel * scale * np.maximum(mag, 1e-300)), (dtype, knob, batch, m, k, n)
        finally:
            dx.check(dxh.dxh_tune(SPLITK_KNOB, 0))


@pytest.mark.parametrize("dtype,m,k,n", [(dx.F32, 16, 4096, 256), (dx.BF16, 64, 8192, 64), (dx.BF16, 333, 777, 555),
                                         (dx.F32, 4, 4096, 1024), (dx.F64, 130, 515, 67), (dx.BF16, 1000, 4160, 904), (dx.F16, 2048, 4864, 896), (dx.BF16, 1000, 4160, 2824)])
def test_matmul_under_capture_equals_eager(dxh, dtype, m, k, n):
    """Products that are cut along K or run on padded copies keep their partial results in the
    caller's workspace, so the same kernels run under stream capture: a recorded matmul replays
    the bits of the eager call (and neither allocates).  The last two shapes take 128x128 tiles whose
    two halves of K meet inside the launch (a ragged M and N, K steps that do not halve evenly; the
    second config-5 shape; the last one 128x256 tiles of that kind)."""
    import ctypes as C
    rng = np.random.default_rng(900 + m)
    A = H.to_storage(rng.standard_normal(m * k), dtype)
    B = H.to_storage(rng.standard_normal(k * n), dtype)
    dA, dB, dC, dG = Dev(A), Dev(B), Dev.empty(m * n, A.dtype), Dev.empty(m * n, A.dtype)
    need = C.c_size_t(0)
    dx.check(dxh.dxh_matmul_workspace_bytes(dtype, dA.ptr, dB.ptr, dC.ptr, 1, m, k, n, C.byref(need)))
    assert need.value > 0, "shape chosen to need scratch"
    ws = Dev.empty(need.value, np.uint8)
    assert dxh.dxh_matmul(dtype, dA.ptr, dB.ptr, dC.ptr, 1, m, k, n, None, 0, None) == -4
    assert dxh.dxh_matmul(dtype, dA.ptr, dB.ptr, dC.ptr, 1, m, k, n, ws.ptr, need.value - 1, None) == -4
    dx.check(dxh.dxh_matmul(dtype, dA.ptr, dB.ptr, dC.ptr, 1, m, k, n, ws.ptr, need.value, None))
    want = dC.get()
    ref = H.to_float(A, dtype).reshape(m, k) @ H.to_float(B, dtype).reshape(k, n)
    bound = np.abs(H.to_float(A, dtype).reshape(m, k)) @ np.abs(H.to_float(B, dtype).reshape(k, n))
    tol = 1e-2 if dtype == dx.BF16 else 2e-3 if dtype == dx.F16 else (1e-5 if dtype == dx.F32 else 1e-13) * np.sqrt(k)
    assert np.all(np.abs(H.to_float(want, dtype).reshape(m, n) - ref) <= tol * bound + 1e-30)
    st = C.c_void_p()
    dx.check(dxh.dxh_stream_create(C.byref(st)))
    graph = C.c_void_p()
    dx.check(dxh.dxh_graph_begin_capture(st))
    rc = dxh.dxh_matmul(dtype, dA.ptr, dB.ptr, dG.ptr, 1, m, k, n, ws.ptr, need.value, st)
    dx.check(dxh.dxh_graph_end_capture(st, C.byref(graph)))
    dx.check(rc, "matmul under capture")
    for _ in range(3):
        dx.check(dxh.dxh_graph_launch(graph, st))
        dx.check(dxh.dxh_stream_sync(st))
        assert np.array_equal(dG.get().view(np.uint8), want.view(np.uint8))
        dx.check(dxh.dxh_matmul(dtype, dA.ptr, dB.ptr, dC.ptr, 1, m, k, n, ws.ptr, need.value, None))  # eager work between replays
        dx.check(dxh.dxh_device_sync())
    dx.check(dxh.dxh_graph_destroy(graph))
    dx.check(dxh.dxh_stream_destroy(st))


def test_k_cut_inside_the_launch_many_launches(dxh):
    """The two halves of a K cut meet through device memory and a counter that strided-axis
    reductions of the same stream use as well: 400 launches, a fused-finish reduction between any
    two, every product bit-identical to the first (which half arrives last varies from launch to
    launch; their sum may not) and within the float64 bar, every reduction identical to the first."""
    import ctypes as C
    rng = np.random.default_rng(77)
    m, k, n = 1000, 4160, 904
    A = H.to_storage(rng.standard_normal(m * k), dx.BF16)
    B = H.to_storage(rng.standard_normal(k * n), dx.BF16)
    dA, dB, dC = Dev(A), Dev(B), Dev.empty(m * n, np.uint16)
    need = C.c_size_t(0)
    dx.check(dxh.dxh_matmul_workspace_bytes(dx.BF16, dA.ptr, dB.ptr, dC.ptr, 1, m, k, n, C.byref(need)))
    assert need.value == 8 * 8 * 2 * 128 * 128 * 4, "64 tiles of 128x128, two fp32 partial tiles each"
    ws = Dev.empty(need.value, np.uint8)
    R, Cc = 4096, 2048
    X = Dev(rng.standard_normal(R * Cc).astype(np.float32))
    col = Dev.empty(Cc, np.float32)
    rneed = C.c_size_t(0)
    dx.check(dxh.dxh_reduce_workspace_bytes(dx.F32, dx.i32arr([R, Cc]), 2, dx.i32arr([0]), 1, C.byref(rneed)))
    rws = Dev.empty(max(rneed.value, 1), np.uint8)
    first = first_col = None
    for it in range(400):
        dx.check(dxh.dxh_matmul(dx.BF16, dA.ptr, dB.ptr, dC.ptr, 1, m, k, n, ws.ptr, need.value, None))
        dx.check(dxh.dxh_sum(dx.F32, X.ptr, dx.i32arr([R, Cc]), 2, dx.i32arr([0]), 1, col.ptr, rws.ptr, rneed.value, None))
        if it % 40 == 0 or it == 399:
            got, gcol = dC.get(), col.get()
            if first is None:
                first, first_col = got, gcol
                Af, Bf = H.to_float(A, dx.BF16).reshape(m, k), H.to_float(B, dx.BF16).reshape(k, n)
                assert np.all(np.abs(H.to_float(got, dx.BF16).reshape(m, n) - Af @ Bf) <= 1e-2 * (np.abs(Af) @ np.abs(Bf)))
            assert np.array_equal(got, first) and np.array_equal(gcol, first_col), it


@pytest.mark.parametrize("dtype", [dx.BF16, dx.F16])
@pytest.mark.parametrize("tile", [0, 1])
def test_matmul_half_rows_not_16_byte_aligned(dxh, dtype, tile):
    """Odd K / N and bases that are only 2-byte aligned: with the tile knob at 0 the product runs on
    zero-padded copies of the operands, with the knob set it stays on the element-wise fallback
    kernel; both against float64 numpy (rel 1e-2 of sum_k |a||b|) and exact on small integers."""
    rng = np.random.default_rng(1000 + dtype + tile)
    dx.check(dxh.dxh_tune(TILE_KNOB, tile))
    try:
        for batch, m, k, n, off in [(1, 333, 777, 555, 0), (2, 130, 71, 150, 0), (1, 257, 129, 65, 0), (3, 31, 200, 17, 0),
                                    (1, 64, 72, 61, 0), (1, 200, 63, 64, 0), (1, 128, 64, 128, 1), (2, 65, 96, 72, 3)]:
            A = H.to_storage(rng.standard_normal(batch * m * k), dtype)
            B = H.to_storage(rng.standard_normal(batch * k * n), dtype)
            # `off` elements of slack in front: the operands then start 2 * off bytes past a 256-byte boundary
            dA, dB, dC = Dev(np.concatenate([np.zeros(off, A.dtype), A])), Dev(np.concatenate([np.zeros(off, B.dtype), B])), Dev.empty(batch * m * n + off, A.dtype)
            dx.check(H.matmul(dxh, dtype, dA.ptr.value + 2 * off, dB.ptr.value + 2 * off, dC.ptr.value + 2 * off, batch, m, k, n, None), "matmul")
            got = H.to_float(dC.get()[off:], dtype).astype(np.float64).reshape(batch, m, n)
            ref, mag = _ref_product(A, B, dtype, batch, m, k, n)
            assert np.all(np.abs(got - ref) <= 1e-2 * np.maximum(mag, 1e-30)), (dtype, tile, batch, m, k, n, off)
        m, k, n = 131, 203, 77
        Ai, Bi = rng.integers(-4, 5, (m, k)), rng.integers(-4, 5, (k, n))
        A = H.to_storage(Ai.astype(np.float64).reshape(-1), dtype)
        B = H.to_storage(Bi.astype(np.float64).reshape(-1), dtype)
        dA, dB, dC = Dev(A), Dev(B), Dev.empty(m * n, A.dtype)
        dx.check(H.matmul(dxh, dtype, dA.ptr, dB.ptr, dC.ptr, 1, m, k, n, None))
        want = H.to_float(H.to_storage((Ai @ Bi).astype(np.float64).reshape(-1), dtype), dtype)
        assert np.array_equal(H.to_float(dC.get(), dtype), want)
    finally:
        dx.check(dxh.dxh_tune(TILE_KNOB, 0))


def test_matmul_int8_matrix_pipe_wraps_like_the_reference(dxh):
    """int8 products large enough for the matrix-pipe kernel (int32 accumulate, low 8 bits
    stored), full-range operands: the result must equal the exact integer product reduced modulo
    2^8, which is what accumulating in int8 (the reference's arithmetic) gives.  Aligned and
    ragged shapes, batches, a K long enough for the int32 accumulators to wrap as well."""
    rng = np.random.default_rng(1234)
    for batch, m, k, n in [(1, 512, 256, 512), (2, 300, 200, 520), (1, 1000, 77, 333), (8, 128, 64, 128), (1, 129, 1000, 1040),
                           (1, 256, 140000, 512)]:
        A = rng.integers(-128, 128, (batch, m, k), dtype=np.int8)
        B = rng.integers(-128, 128, (batch, k, n), dtype=np.int8)
        dA, dB, dC = Dev(A.reshape(-1)), Dev(B.reshape(-1)), Dev.empty(batch * m * n, np.int8)
        dx.check(H.matmul(dxh, dx.I8, dA.ptr, dB.ptr, dC.ptr, batch, m, k, n, None), "matmul")
        # float64 BLAS matmul is exact here: |sum| <= 140000 * 2^14 < 2^53
        want = np.matmul(A.astype(np.float64), B.astype(np.float64)).astype(np.int64).astype(np.int8)
        assert np.array_equal(dC.get().reshape(batch, m, n), want), (batch, m, k, n)


@pytest.mark.parametrize("dtype", [dx.BF16, dx.F16, dx.F32, dx.F64])
def test_matmul_few_rows(dxh, dtype):
    """At most 8 rows of A with K >= 256 take the streaming kernel (vector ALU, K in slices, fp32 /
    fp64 sums; by default for fp32 and fp64 only, here forced for the 16-bit types too): every row-count template, batches, odd K, a K of several slices and sub-chunks, N
    down to one vector; float64 numpy is the reference (same bars as the matrix-pipe kernels),
    small-integer operands must be exact and a second run bit-identical."""
    rng = np.random.default_rng(1100 + dtype)
    rel = {dx.F32: 1e-5, dx.F64: 1e-13, dx.BF16: 1e-2, dx.F16: 1e-2}[dtype]
    dx.check(dxh.dxh_tune(10, 1))  # DXH_TUNE_SKINNY_HALF: by default the kernel serves fp32 / fp64 only
    try:
        _few_rows_cases(dxh, dtype, rng, rel)
    finally:
        dx.check(dxh.dxh_tune(10, 0))


def _few_rows_cases(dxh, dtype, rng, rel):
    for batch, m, k, n in [(1, 1, 4096, 512), (2, 3, 1000, 264), (1, 8, 300, 8), (1, 5, 257, 1040), (1, 4, 70000, 64), (3, 2, 256, 4096),
                           (1, 7, 2048, 4864), (1, 1, 896, 151936 // 8)]:
        A = H.to_storage(rng.standard_normal(batch * m * k), dtype)
        B = H.to_storage(rng.standard_normal(batch * k * n), dtype)
        dA, dB, dC, dC2 = Dev(A), Dev(B), Dev.empty(batch * m * n, A.dtype), Dev.empty(batch * m * n, A.dtype)
        dx.check(H.matmul(dxh, dtype, dA.ptr, dB.ptr, dC.ptr, batch, m, k, n, None), "matmul")
        dx.check(H.matmul(dxh, dtype, dA.ptr, dB.ptr, dC2.ptr, batch, m, k, n, None), "matmul")
        first = dC.get()
        assert np.array_equal(first, dC2.get()), "result varies between runs"
        got = H.to_float(first, dtype).astype(np.float64).reshape(batch, m, n)
        ref, mag = _ref_product(A, B, dtype, batch, m, k, n)
        scale = np.sqrt(k) if dtype in (dx.F32, dx.F64) else 1.0
        assert np.all(np.abs(got - ref) <= rel * scale * np.maximum(mag, 1e-300)), (dtype, batch, m, k, n)
    m, k, n = 6, 1500, 136
    Ai, Bi = rng.integers(-4, 5, (m, k)), rng.integers(-4, 5, (k, n))
    A = H.to_storage(Ai.astype(np.float64).reshape(-1), dtype)
    B = H.to_storage(Bi.astype(np.float64).reshape(-1), dtype)
    dA, dB, dC = Dev(A), Dev(B), Dev.empty(m * n, A.dtype)
    dx.check(H.matmul(dxh, dtype, dA.ptr, dB.ptr, dC.ptr, 1, m, k, n, None))
    want = H.to_float(H.to_storage((Ai @ Bi).astype(np.float64).reshape(-1), dtype), dtype)
    assert np.array_equal(H.to_float(dC.get(), dtype), want)


@pytest.mark.parametrize("dtype", [dx.F32, dx.F64, dx.BF16, dx.F16])
def test_matmul_few_rows_any_n(dxh, dtype):
    """At most 8 rows and an N that is not a multiple of the 16-byte vector (rows of B then start
    on any element boundary), bases off a 16-byte boundary, N below one workgroup's width and a K
    of several slices: float64 numpy reference, exact on small integers, runs bit-identical, and
    nothing written past the end of C."""
    rng = np.random.default_rng(1200 + dtype)
    rel = {dx.F32: 1e-5, dx.F64: 1e-13, dx.BF16: 1e-2, dx.F16: 1e-2}[dtype]
    npd = H.NP[dtype]
    for batch, m, k, n, off in [(1, 1, 768, 50257, 0), (2, 3, 1000, 263, 0), (1, 8, 300, 9, 0), (1, 5, 257, 1041, 1), (1, 4, 70000, 67, 0),
                                (3, 2, 256, 4097, 3), (1, 7, 2048, 4863, 0), (1, 1, 4096, 5, 1), (1, 13, 1024, 1001, 0), (2, 16, 512, 127, 1)]:
        A = H.to_storage(rng.standard_normal(batch * m * k), dtype)
        B = H.to_storage(rng.standard_normal(batch * k * n), dtype)
        guard = 64
        dA = Dev(np.concatenate([np.zeros(off, npd), A]))
        dB = Dev(np.concatenate([np.zeros(off, npd), B]))
        outs = []
        seven = H.to_storage(np.full(1, 7.0), dtype)[0]
        for _ in range(2):
            dC = Dev(np.full(off + batch * m * n + guard, seven, npd))
            es = np.dtype(npd).itemsize
            dx.check(H.matmul(dxh, dtype, dA.ptr.value + es * off, dB.ptr.value + es * off, dC.ptr.value + es * off, batch, m, k, n, None), "matmul")
            outs.append(dC.get())
        assert np.array_equal(outs[0], outs[1]), "result varies between runs"
        assert np.all(outs[0][:off] == seven) and np.all(outs[0][off + batch * m * n:] == seven), "wrote outside C"
        got = H.to_float(outs[0][off:off + batch * m * n], dtype).astype(np.float64).reshape(batch, m, n)
        ref, mag = _ref_product(A, B, dtype, batch, m, k, n)
        scale = np.sqrt(k) if dtype in (dx.F32, dx.F64) else 1.0
        assert np.all(np.abs(got - ref) <= rel * scale * np.maximum(mag, 1e-300)), (dtype, batch, m, k, n, off)
    m, k, n = 6, 1500, 137
    Ai, Bi = rng.integers(-4, 5, (m, k)), rng.integers(-4, 5, (k, n))
    A = H.to_storage(Ai.astype(np.float64).reshape(-1), dtype)
    B = H.to_storage(Bi.astype(np.float64).reshape(-1), dtype)
    dA, dB, dC = Dev(A), Dev(B), Dev.empty(m * n, npd)
    dx.check(H.matmul(dxh, dtype, dA.ptr, dB.ptr, dC.ptr, 1, m, k, n, None))
    want = H.to_float(H.to_storage((Ai @ Bi).astype(np.float64).reshape(-1), dtype), dtype)
    assert np.array_equal(H.to_float(dC.get(), dtype), want)


@pytest.mark.parametrize("dtype", [dx.BF16, dx.F16])
def test_products_that_share_their_left_operand(dxh, dtype):
    """dxh_matmul_shared_a: C_j = A B_j for 2, 3, 4 and 5 pairs is, pair by pair, bit for bit what dxh_matmul
    stores — as one launch where the shape takes a large tile uncut (the gate / up projections of config 5,
    2048x896x4864; square and ragged shapes), as separate products otherwise (a K cut in two, rows that are not
    16-byte pieces, few tiles).  The first shape is also held to float64."""
    import ctypes as C
    rng = np.random.default_rng(500 + dtype)
    for (m, k, n), counts in [((2048, 896, 4864), (2, 3)), ((300, 128, 520), (2, 4, 5)), ((2048, 4864, 896), (2,)), ((333, 777, 555), (2,)),
                              ((64, 64, 64), (3,)), ((1024, 448, 768), (2,)), ((4096, 1024, 1024), (4,))]:
        A = H.to_storage(rng.standard_normal(m * k), dtype)
        dA = Dev(A)
        for count in counts:
            Bs = [H.to_storage(rng.standard_normal(k * n) * 0.05, dtype) for _ in range(count)]
            dBs = [Dev(b) for b in Bs]
            want = []
            for j in range(count):
                dC = Dev.empty(m * n, A.dtype)
                dx.check(H.matmul(dxh, dtype, dA.ptr, dBs[j].ptr, dC.ptr, 1, m, k, n, None), "matmul")
                want.append(dC.get())
            dCs = [Dev(np.full(m * n, 0x7fc1, dtype=A.dtype)) for _ in range(count)]
            bs, cs = dx.ptrarr([b.ptr.value for b in dBs]), dx.ptrarr([c.ptr.value for c in dCs])
            need = C.c_size_t(0)
            dx.check(dxh.dxh_matmul_shared_a_workspace_bytes(dtype, dA.ptr, bs, cs, count, m, k, n, C.byref(need)), "workspace")
            ws = Dev.empty(max(1, need.value), np.uint8)
            dx.check(dxh.dxh_matmul_shared_a(dtype, dA.ptr, bs, cs, count, m, k, n, ws.ptr if need.value else None, need.value, None), "shared")
            for j in range(count):
                assert np.array_equal(dCs[j].get(), want[j]), (m, k, n, count, j)
            if (m, k, n) == (2048, 896, 4864) and count == 2:
                Af = H.to_float(A, dtype).reshape(m, k)
                for j in range(count):
                    Bf = H.to_float(Bs[j], dtype).reshape(k, n)
                    assert np.all(np.abs(H.to_float(dCs[j].get(), dtype).reshape(m, n) - Af @ Bf) <= 1e-2 * (np.abs(Af) @ np.abs(Bf)))
    # argument errors: two products into one result, a missing result, no pairs
    p = Dev.empty(64 * 64, np.uint16)
    same = dx.ptrarr([p.ptr.value, p.ptr.value])
    assert dxh.dxh_matmul_shared_a(dtype, p.ptr, same, same, 2, 64, 64, 64, None, 0, None) == -2
    assert dxh.dxh_matmul_shared_a(dtype, p.ptr, same, dx.ptrarr([p.ptr.value, 0]), 2, 64, 64, 64, None, 0, None) == -2
    assert dxh.dxh_matmul_shared_a(dtype, p.ptr, same, same, 0, 64, 64, 64, None, 0, None) == -2
