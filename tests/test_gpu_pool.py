"""GPU: freed device blocks handed out again (dxh_pool_*), through the C ABI and under the executor's `newtensor` /
`deltensor`.  The pool never waits for the device, so the cases that matter are blocks that come back while launches
on them are still queued: whoever gets the block next must see its own data only.  Also here: where a tensor's bytes
come from and go to outside the device (large `.data` files through the page cache)."""
import ctypes as C
import os

import numpy as np
import pytest

from deepx_amd import lib as dx
from tests import helpers as H
from tests.executor_client import InProc
from tests.test_gpu_batch import Host, T, V

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _torch_owns_the_hip_runtime(dxh):
    yield


def pool_stats(L):
    s = dx.PoolStats()
    assert L.dxh_pool_stats(C.byref(s)) == 0
    return {n: int(getattr(s, n)) for n, _ in dx.PoolStats._fields_}


def pool_alloc(L, nbytes):
    p = C.c_void_p()
    assert L.dxh_pool_alloc(C.byref(p), nbytes) == 0 and p.value
    return p.value


def test_a_freed_block_is_the_next_one_of_its_class(dxh):
    L = dxh
    MB = 1 << 20
    assert L.dxh_pool_trim(0, None) == 0
    s0 = pool_stats(L)
    assert s0["kept_blocks"] == 0
    p, q = pool_alloc(L, 20 * MB), pool_alloc(L, 20 * MB)
    assert p != q
    pattern = np.arange(5 * MB, dtype=np.uint32)
    assert L.dxh_memcpy_h2d(p, pattern.ctypes.data, pattern.nbytes, None) == 0
    assert L.dxh_pool_free(p) == 0
    r = pool_alloc(L, 20 * MB - 100)  # same class: the block just freed, with what it held (the pool clears nothing)
    assert r == p
    back = np.empty_like(pattern)
    assert L.dxh_memcpy_d2h(back.ctypes.data, r, back.nbytes, None) == 0
    assert np.array_equal(back, pattern)
    other = pool_alloc(L, 3 * MB)  # another class: never one of these blocks
    assert other not in (p, q)
    s1 = pool_stats(L)
    assert s1["hits"] - s0["hits"] == 1 and s1["misses"] - s0["misses"] == 3
    assert s1["live_blocks"] - s0["live_blocks"] == 3 and s1["live_bytes"] - s0["live_bytes"] == 43 * MB
    # a pointer the pool did not hand out, or has back already, is refused and left alone
    raw = C.c_void_p()
    assert L.dxh_malloc(C.byref(raw), 4096) == 0
    assert L.dxh_pool_free(raw) == -2
    assert L.dxh_free(raw) == 0
    assert L.dxh_pool_free(q) == 0 and L.dxh_pool_free(q) == -2
    assert L.dxh_pool_free(r) == 0 and L.dxh_pool_free(other) == 0 and L.dxh_pool_free(None) == 0
    s2 = pool_stats(L)
    assert s2["kept_blocks"] == 3 and s2["kept_bytes"] == 43 * MB and s2["live_blocks"] == s0["live_blocks"]
    released = C.c_size_t()
    assert L.dxh_pool_trim(24 * MB, C.byref(released)) == 0  # largest first: one 20 MiB block and the small one stay
    assert released.value == 20 * MB and pool_stats(L)["kept_bytes"] == 23 * MB
    assert L.dxh_pool_trim(0, C.byref(released)) == 0 and released.value == 23 * MB
    assert pool_stats(L)["kept_blocks"] == 0
    # zero bytes still get a pointer of their own
    z1, z2 = pool_alloc(L, 0), pool_alloc(L, 0)
    assert z1 != z2
    assert L.dxh_pool_free(z1) == 0 and L.dxh_pool_free(z2) == 0


def test_the_limit_on_kept_bytes(dxh):
    L = dxh
    MB = 1 << 20
    assert L.dxh_pool_trim(0, None) == 0
    try:
        assert L.dxh_pool_limit(8 * MB) == 0
        a, b, c = pool_alloc(L, 6 * MB), pool_alloc(L, 4 * MB), pool_alloc(L, 16 * MB)
        before = pool_stats(L)
        assert L.dxh_pool_free(c) == 0  # alone over the limit: straight back to the driver
        assert pool_stats(L)["kept_blocks"] == 0 and pool_stats(L)["released"] == before["released"] + 1
        assert L.dxh_pool_free(a) == 0 and pool_stats(L)["kept_bytes"] == 6 * MB
        assert L.dxh_pool_free(b) == 0  # 10 MiB would be kept: the larger block goes
        assert pool_stats(L)["kept_bytes"] == 4 * MB and pool_stats(L)["kept_blocks"] == 1
    finally:
        assert L.dxh_pool_limit(64 << 30) == 0
    assert L.dxh_pool_trim(0, None) == 0


@pytest.mark.parametrize("mode", ["in_order", "streams", "held"])
def test_newtensor_on_a_block_still_in_use_is_zero(dxh, tmp_path, mode):
    """`deltensor` right behind launches that write the tensor, then `newtensor` of the same size: the new tensor gets the
    block that those launches are still writing (the pool says so), and must read as zeros afterwards, and a result
    computed into it must be that result — in order, with independent lines on side streams, and with runs held back."""
    L = dxh
    shape = [4096, 8192]  # 128 MiB: each launch on it runs for tens of microseconds, several are queued at the free
    rng = np.random.default_rng(197)
    src = rng.uniform(-1, 1, shape).astype(np.float32)
    ex = InProc()
    ex.set_streams(3 if mode == "streams" else 1)
    ex.set_defer(mode == "held")
    h = Host(ex, tmp_path)
    p = f"pool_{mode}_"
    h.put(p + "src", src)
    h.put(p + "src2", -src)
    assert L.dxh_pool_trim(0, None) == 0
    for it in range(4):
        hits = pool_stats(L)["hits"]
        lines = [f"newtensor({V(shape)})->({T(p + 'x')})", f"newtensor({V(shape)})->({T(p + 'w')})"]
        lines += [f"addscalar({T(p + 'src')}, var<float32>:{it + 1})->({T(p + 'x')})",
                  f"mulscalar({T(p + 'src2')}, var<float32>:3)->({T(p + 'w')})",
                  f"mul({T(p + 'x')}, {T(p + 'w')})->({T(p + 'x')})",
                  f"add({T(p + 'src')}, {T(p + 'src2')})->({T(p + 'w')})",
                  f"exp({T(p + 'x')})->({T(p + 'x')})",
                  f"deltensor()->({T(p + 'x')})", f"deltensor()->({T(p + 'w')})",
                  f"newtensor({V(shape)})->({T(p + 'y')})", f"newtensor({V(shape)})->({T(p + 'y2')})"]
        for line in lines:
            h.run(line)
        if it:  # the first pass fills the pool
            assert pool_stats(L)["hits"] - hits == 4, "the blocks were not handed out again"
        y, y2 = h.get(p + "y"), h.get(p + "y2")
        assert not y.any() and not y2.any(), f"pass {it}: a new tensor is not zero"
        h.run(f"addscalar({T(p + 'src')}, var<float32>:5)->({T(p + 'y')})")
        h.run(f"deltensor()->({T(p + 'y2')})")
        assert np.array_equal(h.get(p + "y"), src + np.float32(5))
        h.run(f"deltensor()->({T(p + 'y')})")
    if mode == "streams":
        assert ex.side_launches() > 0
    if mode == "held":
        assert ex.defer_stats()["held_lines"] > 0


def test_tensors_from_the_driver_when_the_pool_is_off(dxh, tmp_path):
    L = dxh
    ex = InProc()
    h = Host(ex, tmp_path)
    try:
        ex.set_pool(False)
        before = pool_stats(L)
        h.run(f"newtensor({V([512, 512])})->({T('pool_off_a')})")
        h.run(f"addscalar({T('pool_off_a')}, var<float32>:2)->({T('pool_off_a')})")
        assert np.array_equal(h.get("pool_off_a"), np.full([512, 512], 2, np.float32))
        ex.set_pool(True)
        h.run(f"newtensor({V([512, 512])})->({T('pool_off_b')})")  # pooled, beside one that is not
        h.run(f"deltensor()->({T('pool_off_a')})")
        h.run(f"deltensor()->({T('pool_off_b')})")
        after = pool_stats(L)
        assert after["hits"] + after["misses"] - before["hits"] - before["misses"] == 1
        assert after["kept"] - before["kept"] == 1 and after["live_blocks"] == before["live_blocks"]
    finally:
        ex.set_pool(True)


def dirty_blocks(h, L, prefix, shape, count, dt="float32"):
    """leaves `count` blocks of this shape's class in the pool, full of sevens"""
    for i in range(count):
        h.run(f"newtensor({V(shape)})->({T(prefix + f'dirt{i}', dt)})")
        h.run(f"constant(var<float32>:7)->({T(prefix + f'dirt{i}', dt)})")
    for i in range(count):
        h.run(f"deltensor()->({T(prefix + f'dirt{i}', dt)})")


@pytest.mark.parametrize("mode", ["lines", "batch", "batch_unfused", "graph", "streams", "held", "fill_at_once"])
def test_a_new_tensor_reads_as_zeros_whoever_touches_it_first(dxh, tmp_path, mode):
    """`newtensor` owes its zero fill to the first launch that names the tensor.  On blocks full of sevens: a tensor that is
    read before anything wrote it reads as zeros (as an operand, in place, inside a fused run, by two lines that may sit on
    two streams, by a replayed graph whose tensors were deleted and made again at the same addresses); a tensor that an op
    overwrites holds that op's result; and a tensor whose op failed reads as zeros afterwards."""
    L = dxh
    shape = [1024, 2048]
    rng = np.random.default_rng(199)
    src = rng.uniform(-1, 1, shape).astype(np.float32)
    ex = InProc()
    ex.set_streams(3 if mode == "streams" else 1)
    ex.set_defer(mode == "held")
    ex.set_graphs(mode == "graph")
    ex.set_fusion(mode != "batch_unfused")
    ex.set_zero_later(mode != "fill_at_once")
    h = Host(ex, tmp_path)
    p = f"lz_{mode}_"
    n = lambda name: T(p + name)
    h.put(p + "src", src)
    h.run(f"newtensor({V([3, 5])})->({n('small')})")
    fresh = ["y", "y2", "y3", "z", "z2", "w", "t1", "t2", "r", "never"]
    block = [f"add({n('y')}, {n('src')})->({n('z')})",            # y read first: zeros
             f"mul({n('y')}, {n('src')})->({n('z2')})",           # and by a second line that depends on nothing the first one writes
             f"addscalar({n('y2')}, var<float32>:2)->({n('y2')})",  # in place
             f"mulscalar({n('y3')}, var<float32>:3)->({n('t1')})",  # a run that starts by reading a fresh tensor
             f"add({n('t1')}, {n('src')})->({n('t2')})",
             f"exp({n('t2')})->({n('w')})",
             f"sum({n('src')}, {V([1])}, var<bool>:false)->({n('r')})"]
    block = [f"{l} // author=miaobyte id={i + 1}" for i, l in enumerate(block)]
    for it in range(4):  # with graphs: eager, recorded, replayed, replayed — the tensors deleted and made again in between
        dirty_blocks(h, L, p, shape, len(fresh))
        hits = pool_stats(L)["hits"]
        for name in fresh:
            h.run(f"newtensor({V(shape if name != 'r' else [shape[0]])})->({n(name)})")
        assert pool_stats(L)["hits"] - hits >= len(fresh) - 1, "the new tensors did not get used blocks"
        if mode in ("lines", "streams", "held", "fill_at_once"):
            replies = [ex.execute(l) for l in block]
        else:
            replies = ex.execute_batch(block)
        assert all(r.split(" ")[1].startswith("ok") for r in replies), replies
        bad = ex.execute(f"add({n('src')}, {n('small')})->({n('never')}) // id=77")  # fails: shapes differ
        assert bad.startswith("77 error"), bad
        ex.flush()
        assert np.array_equal(h.get(p + "z"), src), it
        assert not h.get(p + "z2").any() and not h.get(p + "y").any(), it
        assert np.array_equal(h.get(p + "y2"), np.full(shape, 2, np.float32)), it
        assert not h.get(p + "t1").any() and np.array_equal(h.get(p + "t2"), src), it
        assert np.allclose(h.get(p + "w"), np.exp(src), rtol=1e-6), it
        assert np.allclose(h.get(p + "r"), src.astype(np.float64).sum(1), rtol=1e-5, atol=1e-4), it
        assert not h.get(p + "never").any(), "a tensor whose op failed does not read as zeros"
        if mode == "graph":
            # the same batch again with one tensor deleted and made again on its own block, now full of sevens: every
            # pointer the recorded graph holds is still right, so it is replayed, and must still read that tensor as zeros
            replays = ex.stats()["replays"]
            h.run(f"constant(var<float32>:7)->({n('y')})")
            y_hits = pool_stats(L)["hits"]
            h.run(f"deltensor()->({n('y')})")
            h.run(f"newtensor({V(shape)})->({n('y')})")
            assert pool_stats(L)["hits"] == y_hits + 1
            replies = ex.execute_batch(block)
            assert all(r.split(" ")[1].startswith("ok") for r in replies), replies
            if it:  # the pass before recorded it
                assert ex.stats()["replays"] == replays + 1, ex.stats()
            assert np.array_equal(h.get(p + "z"), src) and not h.get(p + "z2").any() and not h.get(p + "y").any(), it
        for name in fresh:
            h.run(f"deltensor()->({n(name)})")
    if mode == "graph":
        assert ex.stats()["replays"] >= 1, ex.stats()
    if mode == "streams":
        assert ex.side_launches() > 0
    if mode in ("batch", "held"):
        assert ex.fusion_stats()["runs"] >= 4


def test_random_programs_with_allocations_in_every_mode(dxh, tmp_path):
    """Random programs in which tensors come and go between the compute lines — `newtensor` under fresh names and under
    names that exist, `deltensor`, lines that read a tensor nobody has written yet, lines that fail on one — on pool
    blocks full of sevens.  Reference: storage from the driver, zero fill at allocation, one line at a time, no fusion.
    Against it, with pooled storage and the fill owed: line by line, as one datagram with fused runs, with runs held back,
    on side streams (one datagram and line by line), and as a datagram sent three times with graphs on.  Same replies,
    same bits in every tensor that is left."""
    L = dxh
    rng = np.random.default_rng(20261)
    code = {"float32": dx.F32, "bfloat16": dx.BF16}
    modes = ("reference", "lines", "batch", "held", "streams", "streams_lines", "graph")
    fused = held = side = hits = 0
    for trial in range(40):
        rows, cols = [(16, 64), (64, 896), (33, 260), (128, 32), (5, 1000)][trial % 5]
        shapes = {"F": [rows, cols], "C": [rows, 1]}
        inputs = [(f"rp{trial}_in{i}_{dt[:2]}", "F", dt) for i in range(2) for dt in code]
        data = {name: (rng.uniform(-1, 1, shapes[k]).astype(np.float32) if dt == "float32"
                       else H.to_storage(rng.uniform(-1, 1, int(np.prod(shapes[k]))), dx.BF16).reshape(shapes[k])) for name, k, dt in inputs}
        live = list(inputs)  # (name, kind, dtype), as the program goes
        lines, fresh_no = [], 0
        def some(k=None, dt=None):
            fits = [t for t in live if (k is None or t[1] == k) and (dt is None or t[2] == dt)]
            return fits[int(rng.integers(0, len(fits)))] if fits else None
        for _ in range(int(rng.integers(24, 40))):
            kind = str(rng.choice(["new", "new", "new", "del", "renew", "bin", "bin", "scalar", "scalar", "exp", "sum", "broadcast", "cast", "bad"]))
            dt = str(rng.choice(list(code)))
            if kind == "new":
                k = str(rng.choice(["F", "F", "C"]))
                name = f"rp{trial}_t{fresh_no}_{dt[:2]}"
                fresh_no += 1
                lines.append(f"newtensor({V(shapes[k])})->({T(name, dt)})")
                live.append((name, k, dt))
            elif kind == "del":
                t = some()
                if t and t not in inputs:
                    lines.append(f"deltensor()->({T(t[0], t[2])})")
                    live.remove(t)
            elif kind == "renew":  # a name that exists: the tensor stays as it is
                t = some()
                lines.append(f"newtensor({V(shapes[t[1]])})->({T(t[0], t[2])})")
            elif kind == "bin":
                k = str(rng.choice(["F", "F", "C"]))
                a, b, c = some(k, dt), some(k, dt), some(k, dt)
                if a and b and c:
                    lines.append(f"{rng.choice(['add', 'mul', 'sub', 'max'])}({T(a[0], dt)}, {T(b[0], dt)})->({T(c[0], dt)})")
            elif kind == "scalar":
                a = some(None, dt)
                c = some(a[1], dt) if a else None
                if a and c:
                    lines.append(f"{rng.choice(['addscalar', 'mulscalar', 'maxscalar'])}({T(a[0], dt)}, var<float32>:{float(rng.choice([0.5, 2.0, -1.25]))})->({T(c[0], dt)})")
            elif kind == "exp":
                a = some(None, dt)
                c = some(a[1], dt) if a else None
                if a and c:
                    lines.append(f"exp({T(a[0], dt)})->({T(c[0], dt)})")
            elif kind == "sum":
                a, c = some("F", dt), some("C", dt)
                if a and c:
                    lines.append(f"sum({T(a[0], dt)}, {V([-1])}, var<bool>:true)->({T(c[0], dt)})")
            elif kind == "broadcast":
                a, c = some("C", dt), some("F", dt)
                if a and c:
                    lines.append(f"broadcastTo({T(a[0], dt)}, {V(shapes['F'])})->({T(c[0], dt)})")
            elif kind == "cast":
                a = some()
                d2 = str(rng.choice(list(code)))
                c = some(a[1], d2)
                if a and c:
                    lines.append(f"todtype({T(a[0], a[2])})->({T(c[0], d2)})")
            else:  # fails: a column where a full tensor is needed
                a, b, c = some("F", dt), some("C", dt), some("F", dt)
                if a and b and c:
                    lines.append(f"add({T(a[0], dt)}, {T(b[0], dt)})->({T(c[0], dt)})")
        text = [f"{line} // author=miaobyte id={700 + i}" for i, line in enumerate(lines)]
        results, replies = {}, {}
        for mode in modes:
            ex = InProc()
            ex.set_pool(mode != "reference")
            ex.set_zero_later(mode != "reference")
            ex.set_fusion(mode in ("batch", "held", "streams", "graph"))
            ex.set_defer(mode == "held")
            ex.set_streams(3 if mode.startswith("streams") else 1)
            ex.set_graphs(mode == "graph")
            try:
                h = Host(ex, tmp_path)
                if mode != "reference":
                    for k in shapes:
                        for dt in code:
                            dirty_blocks(h, L, f"rp{trial}_{mode}_{k}_", shapes[k], 6, dt)
                for name, k, dt in inputs:
                    h.put(name, data[name], dt)
                before = pool_stats(L)["hits"]
                if mode in ("batch", "streams"):
                    replies[mode] = ex.execute_batch(text)
                elif mode == "graph":
                    # a program with allocations is never recorded; what must hold is that asking for graphs changes nothing
                    replies[mode] = ex.execute_batch(text)
                else:
                    replies[mode] = [ex.execute(t) for t in text]
                ex.flush()
                hits += pool_stats(L)["hits"] - before
                fused += ex.fusion_stats()["lines"] if mode == "batch" else 0
                held += ex.defer_stats()["held_lines"] if mode == "held" else 0
                side += ex.side_launches() if mode.startswith("streams") else 0
                results[mode] = {name: h.get(name) for name, _, _ in live}
                for name, _, dt in live:
                    if (name, _, dt) not in inputs:
                        h.run(f"deltensor()->({T(name, dt)})")
            finally:
                ex.set_pool(True)
            ex.close()
        want = [r.split("//")[0] for r in replies["reference"]]
        for mode in modes[1:]:
            assert [r.split("//")[0] for r in replies[mode]] == want, (trial, mode, lines)
            for name, _, dt in live:
                a, b = results["reference"][name], results[mode][name]
                same = np.array_equal(a.view(np.uint8), b.view(np.uint8))
                if not same:
                    same = np.array_equal(H.to_float(a.reshape(-1), code[dt]), H.to_float(b.reshape(-1), code[dt]), equal_nan=True)
                assert same, (trial, mode, name, lines)
    assert hits > 500, "the pooled modes did not get their blocks from the pool"
    assert fused > 100 and held > 100 and side > 100, (fused, held, side)


def test_a_failed_runtime_call_is_reported_once(dxh):
    """A call of the C ABI that fails (here: freeing a pointer the driver never gave out) returns its code to its caller
    and leaves nothing behind for the next launch to find: the launchers ask the runtime for its last error after every
    launch, and would otherwise report the old failure as their own."""
    L = dxh
    host = np.zeros(16, np.float32)
    rc = L.dxh_free(host.ctypes.data)
    assert rc > 0, "freeing host memory must fail"
    x = np.arange(1024, dtype=np.float32)
    a, out = H.Dev(x), H.Dev.empty(1024, np.float32)
    assert L.dxh_add(dx.F32, a.ptr, a.ptr, out.ptr, 1024, None) == 0
    assert np.array_equal(out.get(), x + x)
    # a product that needs no workspace, right after an allocation the driver must refuse
    p = C.c_void_p()
    assert L.dxh_malloc(C.byref(p), 1 << 60) > 0 and not p.value
    assert L.dxh_pool_alloc(C.byref(p), 1 << 60) > 0 and not p.value
    assert L.dxh_mulscalar(dx.F32, a.ptr, dx.scalar(2.0), out.ptr, 1024, None) == 0
    assert np.array_equal(out.get(), x * 2)


def test_kept_blocks_give_way_when_the_driver_is_out_of_memory(dxh):
    """With a third of the free device memory kept in the pool, an allocation of seven tenths of it cannot be served
    beside them: the pool gives its blocks back and the allocation succeeds, through dxh_pool_alloc and through
    dxh_malloc alike.  (Nothing is touched: the blocks are address space and page tables only.)"""
    import torch
    L = dxh
    assert L.dxh_pool_trim(0, None) == 0
    free_b, total_b = torch.cuda.mem_get_info()
    small, large = int(free_b * 0.35), int(free_b * 0.7)
    assert small < total_b // 2, "the kept block must fit under the pool's limit (half the device)"
    try:
        assert L.dxh_pool_limit(total_b // 2) == 0
        for via_pool in (True, False):
            kept = pool_alloc(L, small)
            assert L.dxh_pool_free(kept) == 0
            before = pool_stats(L)
            assert before["kept_blocks"] == 1 and before["kept_bytes"] >= small
            p = C.c_void_p()
            rc = L.dxh_pool_alloc(C.byref(p), large) if via_pool else L.dxh_malloc(C.byref(p), large)
            assert rc == 0 and p.value, f"allocation failed with the pool in the way ({rc})"
            after = pool_stats(L)
            assert after["kept_blocks"] == 0 and after["released"] == before["released"] + 1
            assert (L.dxh_pool_free(p) if via_pool else L.dxh_free(p)) == 0
            assert L.dxh_pool_trim(0, None) == 0
        # and with nothing to give back the driver's own answer comes through, once
        p = C.c_void_p()
        assert L.dxh_pool_alloc(C.byref(p), total_b * 2) > 0 and not p.value
    finally:
        assert L.dxh_pool_limit(64 << 30) == 0
        assert L.dxh_pool_trim(0, None) == 0


def test_large_tensor_files_go_through_the_page_cache_unchanged(dxh, tmp_path):
    """`load` of a large `.data` file copies from the file's pages and `save` of a large tensor copies into them, without
    a buffer in between: the bytes on the device are the bytes of the file and the other way round, a file of the
    wrong size and a missing one are refused with the messages of the buffered path, and small tensors (which keep that
    path) sit beside them."""
    from tests.executor_client import read_tensor, write_tensor
    ex = InProc()
    rng = np.random.default_rng(211)
    try:
        for shape, dt, npd in (([4096, 3000], "float32", np.float32), ([5000, 1000], "bfloat16", np.uint16), ([300, 7], "float32", np.float32), ([6000, 4096], "int16", np.int16)):
            a = rng.integers(-30000, 30000, size=shape).astype(npd) if npd != np.float32 else rng.standard_normal(shape).astype(np.float32)
            name = f"pc_{shape[0]}"
            p = str(tmp_path / name)
            write_tensor(p, a, dt)
            assert ex.execute(f"load(var<string>:{p})->() // id=1").startswith("1 ok")
            q = str(tmp_path / (name + "_back"))
            assert ex.execute(f"save(tensor<{dt}>:{name}, var<string>:{q})->() // id=2").startswith("2 ok")
            with open(q + ".data", "rb") as f:
                assert f.read() == a.tobytes(), shape
            assert np.array_equal(read_tensor(q)[0].reshape(shape), a)
            # the same tensor overwritten on the device, saved over the old file (which is emptied first)
            assert ex.execute(f"constant(var<float32>:3)->(tensor<{dt}>:{name}) // id=3").startswith("3 ok")
            assert ex.execute(f"save(tensor<{dt}>:{name}, var<string>:{q})->() // id=4").startswith("4 ok")
            assert os.path.getsize(q + ".data") == a.nbytes
        # a large file of the wrong size, then a missing one
        big = str(tmp_path / "pc_4096")
        with open(big + ".data", "ab") as f:
            f.write(b"\0" * 8)
        r = ex.execute(f"loadtensordata(var<string>:{big})->(tensor<float32>:pc_4096) // id=5")
        assert r.startswith("5 error") and "file size mismatch" in r, r
        os.remove(big + ".data")
        r = ex.execute(f"loadtensordata(var<string>:{big})->(tensor<float32>:pc_4096) // id=6")
        assert r.startswith("6 error") and "Failed to open file" in r, r
        r = ex.execute(f"save(tensor<float32>:pc_4096, var<string>:{tmp_path}/no/such/dir/x)->() // id=7")
        assert r.startswith("7 error") and "Failed to open file for writing" in r, r
    finally:
        ex.close()
