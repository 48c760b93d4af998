"""GPU: several deepxIR lines per datagram — run as one batch (one wait for the device) and, with
DEEPX_GRAPH=1, recorded into a HIP graph on the second arrival and replayed afterwards.  Every
replay is checked bit for bit against the same lines executed one by one, with eager work and
synchronisations between the replays."""
import ctypes as C

import numpy as np
import pytest

from deepx_amd import lib as dx
from tests import helpers as H
from tests.executor_client import InProc, UdpExecutor, read_tensor, write_tensor

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _torch_owns_the_hip_runtime(dxh):
    """The in-process executor pulls in the HIP runtime; torch must have loaded its own copy first
    (the session fixture imports torch), or a later torch import in this process finds no GPU."""
    yield


def T(name, dt="float32"):
    return f"tensor<{dt}>:{name}"


def V(values):
    return "vector<int32>:[" + " ".join(str(v) for v in values) + "]"


class Host:
    """tensor upload/download through the executor's own load/save ops"""

    def __init__(self, ex, tmp_path):
        self.ex, self.tmp, self.n = ex, tmp_path, 0

    def run(self, line):
        self.n += 1
        r = self.ex.execute(f"{line} // id={self.n}")
        assert r.startswith(f"{self.n} ok//"), r

    def put(self, name, arr, dtype_name="float32"):
        p = str(self.tmp / name)
        write_tensor(p, arr, dtype_name)
        self.run(f"load(var<string>:{p})->()")

    def get(self, name):
        p = str(self.tmp / (name + "_out"))
        self.run(f"save({T(name, 'any')}, var<string>:{p})->()")
        return read_tensor(p)[0]


CHAIN = ["add({A}, {B})->({C})", "mul({C}, {B})->({D})", "addscalar({D}, var<float32>:0.5)->({E})", "exp({E})->({F})",
         "mulscalar({B}, var<float32>:-1)->({nB})", "max({B}, {nB})->({absB})", "addscalar({absB}, var<float32>:1)->({den})",
         "div({F}, {den})->({G})"]
NAMES = ["A", "B", "C", "D", "E", "F", "nB", "absB", "den", "G"]


def chain_lines(prefix, first_id):
    names = {n: T(prefix + n) for n in NAMES}
    return [line.format(**names) + f" // author=miaobyte id={first_id + i}" for i, line in enumerate(CHAIN)]


def make_chain(h, prefix, shape, rng):
    for n in NAMES[2:]:
        h.run(f"newtensor({V(shape)})->({T(prefix + n)})")
    h.put(prefix + "A", rng.uniform(-1, 1, shape).astype(np.float32))
    h.put(prefix + "B", rng.uniform(-1, 1, shape).astype(np.float32))


def test_batch_equals_line_by_line(tmp_path):
    ex = InProc()
    h = Host(ex, tmp_path)
    rng = np.random.default_rng(41)
    make_chain(h, "s_", [257, 129], rng)
    for line in chain_lines("s_", 1000):
        assert ex.execute(line).split(" ")[1].startswith("ok")
    want = {n: h.get("s_" + n) for n in NAMES[2:]}
    for n in NAMES[2:]:
        h.run(f"constant(var<float32>:0)->({T('s_' + n)})")
    rs = ex.execute_batch(chain_lines("s_", 2000))
    assert [r.split(" ")[0] for r in rs] == [str(2000 + i) for i in range(8)] and all(r.split(" ")[1].startswith("ok") for r in rs)
    for n in NAMES[2:]:
        assert np.array_equal(h.get("s_" + n).view(np.uint32), want[n].view(np.uint32)), n
    assert ex.stats()["captures"] == 0  # graphs are off unless asked for
    assert ex.fusion_stats() == {"runs": 0, "lines": 0, "matmul_groups": 0, "matmul_lines": 0}  # 257 * 129 floats are not a whole number of 16-byte vectors


def test_graph_replays_track_new_inputs(tmp_path):
    ex = InProc()
    ex.set_graphs(True)
    h = Host(ex, tmp_path)
    rng = np.random.default_rng(42)
    shape = [300, 200]
    make_chain(h, "g_", shape, rng)
    # a reduction (workspace), a transpose and a matmul ride along in the same datagram
    h.run(f"newtensor({V([200])})->({T('g_colsum')})")
    h.run(f"newtensor({V([200, 300])})->({T('g_Gt')})")
    h.run(f"newtensor({V([300, 300])})->({T('g_GGt')})")
    extra = [f"sum({T('g_G')}, {V([0])}, var<bool>:false)->({T('g_colsum')}) // author=miaobyte id=3008",
             f"transpose({T('g_G')}, {V([1, 0])})->({T('g_Gt')}) // author=miaobyte id=3009",
             f"matmul({T('g_G')}, {T('g_Gt')})->({T('g_GGt')}) // author=cublas id=3010"]
    lines = chain_lines("g_", 3000) + extra
    outs = NAMES[2:] + ["colsum", "Gt", "GGt"]
    for round_no in range(5):
        a = rng.uniform(-1, 1, shape).astype(np.float32)
        b = rng.uniform(-1, 1, shape).astype(np.float32)
        h.put("g_A", a)   # load replaces an existing tensor by a fresh allocation: a recorded graph must notice
        h.put("g_B", b)   # new addresses and record again, or replay if the allocator handed the old ones back
        for line in lines:  # line by line: the expectation
            assert ex.execute(line).split(" ")[1].startswith("ok")
        want = {n: h.get("g_" + n) for n in outs}
        for n in outs:
            h.run(f"constant(var<float32>:0)->({T('g_' + n)})")
        rs = ex.execute_batch(lines)
        assert all(r.split(" ")[1].startswith("ok") for r in rs), rs
        for n in outs:
            got = h.get("g_" + n)
            assert np.array_equal(got.view(np.uint32), want[n].view(np.uint32)), (round_no, n)
    st = ex.stats()
    assert st["rejects"] == 0 and st["captures"] >= 1 and st["captures"] + st["replays"] == 4, st


def test_graph_replay_with_stable_addresses(tmp_path):
    """Inputs refreshed in place (copytensor into the same allocation): the recorded graph is
    replayed, not re-recorded, and every replay sees the new data."""
    ex = InProc()
    ex.set_graphs(True)
    h = Host(ex, tmp_path)
    rng = np.random.default_rng(43)
    shape = [64, 96]
    make_chain(h, "r_", shape, rng)
    lines = chain_lines("r_", 4000)
    for round_no in range(6):
        h.put("r_stageA", rng.uniform(-1, 1, shape).astype(np.float32))
        h.put("r_stageB", rng.uniform(-1, 1, shape).astype(np.float32))
        h.run(f"copytensor({T('r_stageA')})->({T('r_A')})")
        h.run(f"copytensor({T('r_stageB')})->({T('r_B')})")
        for line in lines:
            assert ex.execute(line).split(" ")[1].startswith("ok")
        want = h.get("r_G")
        h.run(f"constant(var<float32>:0)->({T('r_G')})")
        assert all(r.split(" ")[1].startswith("ok") for r in ex.execute_batch(lines))
        assert np.array_equal(h.get("r_G").view(np.uint32), want.view(np.uint32)), round_no
    st = ex.stats()
    assert st == {"batches": 6, "captures": 1, "replays": 4, "rejects": 0}, st


def test_batches_that_must_not_be_recorded(tmp_path):
    ex = InProc()
    ex.set_graphs(True)
    h = Host(ex, tmp_path)
    h.put("n_A", np.arange(12, dtype=np.float32).reshape(3, 4))
    h.run(f"newtensor({V([3, 4])})->({T('n_C')})")
    h.run("argset(var<float32>:2)->(var<float32>:two)")
    named = [f"mulscalar({T('n_A')}, var<float32>:two)->({T('n_C')}) // id=5001", f"addscalar({T('n_C')}, var<float32>:1)->({T('n_C')}) // id=5002"]
    for _ in range(3):
        assert all(r.split(" ")[1].startswith("ok") for r in ex.execute_batch(named))
    assert np.array_equal(h.get("n_C"), np.arange(12, dtype=np.float32).reshape(3, 4) * 2 + 1)
    h.run("argset(var<float32>:3)->(var<float32>:two)")  # the named scalar changes: a recorded graph would have frozen it
    assert all(r.split(" ")[1].startswith("ok") for r in ex.execute_batch(named))
    assert np.array_equal(h.get("n_C"), np.arange(12, dtype=np.float32).reshape(3, 4) * 3 + 1)
    lifecycle = [f"newtensor({V([2, 2])})->({T('n_tmp')}) // id=5003", f"constant(var<float32>:7)->({T('n_tmp')}) // id=5004",
                 f"deltensor()->({T('n_tmp')}) // id=5005"]
    for _ in range(3):
        assert all(r.split(" ")[1].startswith("ok") for r in ex.execute_batch(lifecycle))
    failing = [f"add({T('n_A')}, {T('n_missing')})->({T('n_C')}) // id=5006", f"addscalar({T('n_A')}, var<float32>:1)->({T('n_C')}) // id=5007"]
    for _ in range(3):
        rs = ex.execute_batch(failing)
        assert rs[0].endswith("tensor not found: n_missing") and rs[1].split(" ")[1].startswith("ok")
    assert ex.stats()["captures"] == 0 and ex.stats()["replays"] == 0


def test_graphs_over_udp(tmp_path):
    srv = UdpExecutor(env={"DEEPX_GRAPH": "1"})
    try:
        rng = np.random.default_rng(44)
        a, b = rng.uniform(-1, 1, (50, 70)).astype(np.float32), rng.uniform(-1, 1, (50, 70)).astype(np.float32)
        for name, arr in (("u_A", a), ("u_B", b)):
            p = str(tmp_path / name)
            write_tensor(p, arr, "float32")
            srv.must("load", [f"var<string>:{p}"], [], author="")
        for n in NAMES[2:]:
            srv.must("newtensor", [V([50, 70])], [T("u_" + n)], author="")
        datagram = "\n".join(chain_lines("u_", 6000))
        for _ in range(4):
            srv.must("constant", ["var<float32>:0"], [T("u_G")])
            rs = srv.raw(datagram, 8)
            assert [r.id for r in rs] == [str(6000 + i) for i in range(8)] and all(r.ok for r in rs)
            p = str(tmp_path / "u_G_out")
            srv.must("save", [T("u_G", "any"), f"var<string>:{p}"], [], author="")
            f = np.exp((a + b) * b + np.float32(0.5))
            want = f / (np.maximum(b, -b) + np.float32(1))
            got = read_tensor(p)[0]
            assert np.allclose(got, want, rtol=1e-6, atol=0)
    finally:
        srv.close()
    assert srv.proc.returncode == 0


def test_side_streams_over_udp(tmp_path):
    """The server started with DEEPX_STREAMS=3 and DEEPX_FUSE=0: the eight lines of the chain as one datagram, whose
    independent lines leave the default stream, give the values of in-order execution every time."""
    srv = UdpExecutor(env={"DEEPX_STREAMS": "3", "DEEPX_FUSE": "0"})
    try:
        rng = np.random.default_rng(45)
        a, b = rng.uniform(-1, 1, (512, 640)).astype(np.float32), rng.uniform(-1, 1, (512, 640)).astype(np.float32)
        for name, arr in (("v_A", a), ("v_B", b)):
            p = str(tmp_path / name)
            write_tensor(p, arr, "float32")
            srv.must("load", [f"var<string>:{p}"], [], author="")
        for n in NAMES[2:]:
            srv.must("newtensor", [V([512, 640])], [T("v_" + n)], author="")
        datagram = "\n".join(chain_lines("v_", 7000))
        f = np.exp((a + b) * b + np.float32(0.5))
        want = f / (np.maximum(b, -b) + np.float32(1))
        for _ in range(4):
            srv.must("constant", ["var<float32>:0"], [T("v_G")])
            rs = srv.raw(datagram, 8)
            assert [r.id for r in rs] == [str(7000 + i) for i in range(8)] and all(r.ok for r in rs)
            p = str(tmp_path / "v_G_out")
            srv.must("save", [T("v_G", "any"), f"var<string>:{p}"], [], author="")
            assert np.allclose(read_tensor(p)[0], want, rtol=1e-6, atol=0)
    finally:
        srv.close()
    assert srv.proc.returncode == 0


def test_fused_runs_equal_line_by_line(tmp_path):
    """Inside a batch, runs of float elementwise lines (an fp32 sum over the last axis among them) are
    launched as one kernel.  Bit for bit the tensors of a line-by-line execution, for: a run that is cut by a
    bfloat16 reduction and by an integer op, an fp32 reduction in the middle of a run, an in-place line whose old value an earlier line reads and whose
    new value a later line reads, bfloat16, a size that is not a whole number of vectors (not
    fused), a line that fails in the middle (its neighbours still run), and the same batch with
    fusion switched off."""
    rng = np.random.default_rng(91)
    shape = [64, 136]
    lines = [
        "add({a}, {b})->({c})", "mulscalar({c}, var<float32>:0.25)->({d})", "sub({d}, {a})->({a})",   # in place: a changes here
        "mul({a}, {c})->({e})", "exp({e})->({f})",
        "sum({f}, vector<int32>:[1], var<bool>:true)->({s})",                                          # not elementwise: cuts the run
        "rdivscalar(var<float32>:1, {s})->({t})", "sqrt({t})->({u})", "log({u})->({v})",               # [64,1] tensors: a run of their own
        "max({f}, {e})->({g})", "minscalar({g}, var<float32>:1.5)->({h})",
        "add({i1}, {i2})->({i3})",                                                                     # int32: never fused
        "div({h}, {b})->({k})", "rsubscalar(var<float32>:2, {k})->({m})",
    ]
    big = ["a", "b", "c", "d", "e", "f", "g", "h", "k", "m"]
    small = ["s", "t", "u", "v"]
    ints = ["i1", "i2", "i3"]

    def build(ex, prefix, dt):
        h = Host(ex, tmp_path)
        for n in big[2:]:
            h.run(f"newtensor({V(shape)})->({T(prefix + n, dt)})")
        for n in small:
            h.run(f"newtensor({V([shape[0], 1])})->({T(prefix + n, dt)})")
        h.run(f"newtensor({V(shape)})->({T(prefix + 'i3', 'int32')})")
        return h

    def fill(h, prefix, dt, data):
        stored = lambda x: x if dt == "float32" else H.to_storage(x.reshape(-1).astype(np.float64), dx.BF16).reshape(x.shape)
        h.put(prefix + "a", stored(data["a"]), dt)
        h.put(prefix + "b", stored(data["b"]), dt)
        h.put(prefix + "i1", data["i1"], "int32")
        h.put(prefix + "i2", data["i2"], "int32")

    for dt in ("float32", "bfloat16"):
        data = {"a": rng.uniform(0.5, 1.5, shape).astype(np.float32), "b": rng.uniform(0.5, 1.5, shape).astype(np.float32),
                "i1": rng.integers(-9, 9, shape).astype(np.int32), "i2": rng.integers(-9, 9, shape).astype(np.int32)}
        results = {}
        for mode in ("lines", "fused", "unfused"):
            ex = InProc()
            ex.set_fusion(mode == "fused")
            prefix = f"{mode}_{dt}_"
            h = build(ex, prefix, dt)
            fill(h, prefix, dt, data)
            names = {n: T(prefix + n, "int32" if n in ints else dt) for n in big + small + ints}
            text = [line.format(**names) + f" // author=miaobyte id={500 + i}" for i, line in enumerate(lines)]
            if mode == "lines":
                rs = [ex.execute(t) for t in text]
            else:
                rs = ex.execute_batch(text)
            assert all(r.split(" ")[1].startswith("ok") for r in rs), rs
            results[mode] = {n: h.get(prefix + n) for n in big + small + ["i3"]}
            if mode == "fused":
                # bfloat16: [add mulscalar sub mul exp] [rdivscalar sqrt log] [max minscalar] [div rsubscalar];
                # float32: the row sum joins its neighbours, [add ... exp sum rdivscalar sqrt log max minscalar] [div rsubscalar]
                want_stats = {"runs": 2, "lines": 13} if dt == "float32" else {"runs": 4, "lines": 12}
                assert {k: ex.fusion_stats()[k] for k in want_stats} == want_stats, ex.fusion_stats()
            else:
                assert ex.fusion_stats() == {"runs": 0, "lines": 0, "matmul_groups": 0, "matmul_lines": 0}
        for n in big + small + ["i3"]:
            want = results["lines"][n]
            for mode in ("fused", "unfused"):
                got = results[mode][n]
                assert got.dtype == want.dtype and np.array_equal(got.view(np.uint8), want.view(np.uint8)), (dt, mode, n)

    # a length that is not a whole number of 16-byte vectors is left to the separate kernels
    ex = InProc()
    h = Host(ex, tmp_path)
    for n in ("y", "z"):
        h.run(f"newtensor({V([3, 5])})->({T('odd_' + n)})")
    x = rng.uniform(-1, 1, [3, 5]).astype(np.float32)
    h.put("odd_x", x)
    rs = ex.execute_batch([f"mulscalar({T('odd_x')}, var<float32>:2)->({T('odd_y')}) // id=1", f"exp({T('odd_y')})->({T('odd_z')}) // id=2"])
    assert all(r.split(" ")[1].startswith("ok") for r in rs) and ex.fusion_stats()["runs"] == 0
    assert np.array_equal(h.get("odd_z"), np.exp((x * np.float32(2)).astype(np.float32)).astype(np.float32)) or np.allclose(h.get("odd_z"), np.exp(x * 2), rtol=1e-6)

    # a failing line (unknown tensor) between fusable ones: reported on its own, the rest runs
    ex = InProc()
    h = Host(ex, tmp_path)
    for n in ("p", "q", "r"):
        h.run(f"newtensor({V([8, 16])})->({T('e_' + n)})")
    x = rng.uniform(-1, 1, [8, 16]).astype(np.float32)
    h.put("e_x", x)
    rs = ex.execute_batch([f"addscalar({T('e_x')}, var<float32>:1)->({T('e_p')}) // id=1", f"mulscalar({T('e_p')}, var<float32>:3)->({T('e_q')}) // id=2",
                           f"add({T('e_q')}, {T('e_missing')})->({T('e_r')}) // id=3", f"sqrt({T('e_q')})->({T('e_r')}) // id=4"])
    assert [r.split(" ")[1][:2] for r in rs] == ["ok", "ok", "er", "ok"], rs
    assert np.array_equal(h.get("e_q"), (x + np.float32(1)) * np.float32(3))


def test_fused_in_place_run(tmp_path):
    """The SiLU gate as the front emits it for an in-place activation: five lines rewrite one tensor.
    As one launch only the last of them stores it; the result equals the line-by-line bits, and the
    tensors that the run only reads are untouched."""
    rng = np.random.default_rng(92)
    shape = [32, 264]
    g = H.to_storage(rng.standard_normal(shape[0] * shape[1]), dx.BF16).reshape(shape)
    u = H.to_storage(rng.standard_normal(shape[0] * shape[1]), dx.BF16).reshape(shape)
    b16 = "bfloat16"
    outs = {}
    for mode in ("lines", "fused"):
        ex = InProc()
        h = Host(ex, tmp_path)
        p = mode + "_"
        h.run(f"newtensor({V(shape)})->({T(p + 'sg', b16)})")
        h.put(p + "g", g, b16)
        h.put(p + "u", u, b16)
        n = lambda name: T(p + name, b16)
        text = [f"mulscalar({n('g')}, var<float32>:-1)->({n('sg')})", f"exp({n('sg')})->({n('sg')})", f"addscalar({n('sg')}, var<float32>:1)->({n('sg')})",
                f"rdivscalar(var<float32>:1, {n('sg')})->({n('sg')})", f"mul({n('g')}, {n('sg')})->({n('sg')})", f"mul({n('sg')}, {n('u')})->({n('sg')})"]
        text = [t + f" // author=miaobyte id={i + 1}" for i, t in enumerate(text)]
        rs = [ex.execute(t) for t in text] if mode == "lines" else ex.execute_batch(text)
        assert all(r.split(" ")[1].startswith("ok") for r in rs), rs
        if mode == "fused":
            assert {k: ex.fusion_stats()[k] for k in ("runs", "lines")} == {"runs": 1, "lines": 6}
        outs[mode] = {k: h.get(p + k) for k in ("sg", "g", "u")}
    for k in ("sg", "g", "u"):
        assert np.array_equal(outs["fused"][k], outs["lines"][k]), k
    assert np.array_equal(outs["fused"]["g"], g) and np.array_equal(outs["fused"]["u"], u)


def test_recorded_graph_notices_an_in_place_reshape(tmp_path):
    """A recorded batch freezes launch shapes.  An in-place reshape keeps a tensor's address, size and
    dtype but changes its dims: the next arrival of the same text must run with the new dims (be
    recorded again), not replay the old launch."""
    ex = InProc()
    ex.set_graphs(True)
    h = Host(ex, tmp_path)
    a = np.arange(32, dtype=np.float32).reshape(4, 8)
    h.put("rs_A", a)
    h.run(f"newtensor({V([32])})->({T('rs_C')})")
    h.run(f"newtensor({V([32])})->({T('rs_D')})")
    lines = [f"transpose({T('rs_A')}, {V([1, 0])})->({T('rs_C')}) // author=miaobyte id=7001",
             f"addscalar({T('rs_C')}, var<float32>:1)->({T('rs_D')}) // author=miaobyte id=7002"]
    for _ in range(3):  # eager, recorded, replayed
        assert all(r.split(" ")[1].startswith("ok") for r in ex.execute_batch(lines))
    assert np.array_equal(h.get("rs_C"), a.T.reshape(-1))
    assert ex.stats()["captures"] == 1 and ex.stats()["replays"] == 1
    h.run(f"reshape({T('rs_A')}, {V([8, 4])})->({T('rs_A')})")
    for _ in range(3):
        h.run(f"constant(var<float32>:0)->({T('rs_C')})")
        assert all(r.split(" ")[1].startswith("ok") for r in ex.execute_batch(lines))
        assert np.array_equal(h.get("rs_C"), a.reshape(8, 4).T.reshape(-1))
        assert np.array_equal(h.get("rs_D"), a.reshape(8, 4).T.reshape(-1) + 1)
    assert ex.stats()["captures"] == 2, ex.stats()


def test_config5_block_at_full_size_in_every_mode(tmp_path):
    """The whole BASELINE config-5 block (RMSNorm + gated MLP, 22 deepxIR ops) at its stated size,
    2048 rows, through the executor line by line, line by line with lines held back until their run is
    complete (DEEPX_DEFER), as one batch, as one batch with fused elementwise
    runs, and as a recorded graph without and with fused runs.  Every mode against a float64 numpy
    model of the same op sequence with bf16 rounding where the graph stores bf16 (rel 1e-2 per bf16
    rounding; 3e-2 of the output scale end to end, 1e-2 for the normalised activations), and every
    mode bit-identical to the line-by-line execution."""
    rng = np.random.default_rng(14)
    S, Hd, I = 2048, 896, 4864
    f2b, b2f = H.f32_to_bf16_bits, H.bf16_bits_to_f32
    x = f2b(rng.standard_normal((S, Hd)).astype(np.float32))
    w = f2b(np.ones(Hd, dtype=np.float32) + 0.1 * rng.standard_normal(Hd).astype(np.float32))
    Wg = f2b((rng.standard_normal((Hd, I)) * 0.02).astype(np.float32))
    Wu = f2b((rng.standard_normal((Hd, I)) * 0.02).astype(np.float32))
    Wd = f2b((rng.standard_normal((I, Hd)) * 0.02).astype(np.float32))
    # float64 model (front/py/deepx/nn/modules/norm/t5layernorm.py:17-22, mlp/gatedmlp.py:20-26)
    rb = lambda a: b2f(f2b(a.astype(np.float32))).astype(np.float64)
    xf = b2f(x).astype(np.float64)
    xn = xf * (1.0 / np.sqrt((xf ** 2).sum(-1, keepdims=True) / Hd + 1e-6))
    h_ref = rb(b2f(w).astype(np.float64) * xn)
    g = rb(h_ref @ b2f(Wg).astype(np.float64)); u = rb(h_ref @ b2f(Wu).astype(np.float64))
    act = rb(rb(g * rb(1.0 / rb(1.0 + rb(np.exp(rb(-g)))))) * u)
    Wd64 = b2f(Wd).astype(np.float64)
    y_ref = act @ Wd64
    y_mag = np.abs(act) @ np.abs(Wd64)

    b16, f32 = "bfloat16", "float32"
    n = lambda name, dt=f32: T("f5_" + name, dt)
    tensors = [("xf", [S, Hd], f32), ("sq", [S, Hd], f32), ("var", [S, 1], f32), ("rs", [S, Hd], f32), ("xn", [S, Hd], f32),
               ("wf1", [1, Hd], f32), ("wf", [S, Hd], f32), ("h", [S, Hd], b16), ("g", [S, I], b16), ("u", [S, I], b16),
               ("sg", [S, I], b16), ("y", [S, Hd], b16)]
    block = [f"todtype({n('x', b16)})->({n('xf')})",
             f"powscalar({n('xf')}, var<float32>:2)->({n('sq')})",
             f"sum({n('sq')}, {V([-1])}, var<bool>:True)->({n('var')})",
             f"divscalar({n('var')}, var<float32>:{Hd})->({n('var')})",
             f"addscalar({n('var')}, var<float32>:1e-06)->({n('var')})",
             f"sqrt({n('var')})->({n('var')})",
             f"rdivscalar(var<float32>:1, {n('var')})->({n('var')})",
             f"broadcastTo({n('var')}, {V([S, Hd])})->({n('rs')})",
             f"mul({n('xf')}, {n('rs')})->({n('xn')})",
             f"todtype({n('w', b16)})->({n('wf1')})",
             f"broadcastTo({n('wf1')}, {V([S, Hd])})->({n('wf')})",
             f"mul({n('wf')}, {n('xn')})->({n('xn')})",
             f"todtype({n('xn')})->({n('h', b16)})",
             f"matmul({n('h', b16)}, {n('Wg', b16)})->({n('g', b16)})",
             f"matmul({n('h', b16)}, {n('Wu', b16)})->({n('u', b16)})",
             f"mulscalar({n('g', b16)}, var<float32>:-1)->({n('sg', b16)})",
             f"exp({n('sg', b16)})->({n('sg', b16)})",
             f"addscalar({n('sg', b16)}, var<float32>:1)->({n('sg', b16)})",
             f"rdivscalar(var<float32>:1, {n('sg', b16)})->({n('sg', b16)})",
             f"mul({n('g', b16)}, {n('sg', b16)})->({n('sg', b16)})",
             f"mul({n('sg', b16)}, {n('u', b16)})->({n('sg', b16)})",
             f"matmul({n('sg', b16)}, {n('Wd', b16)})->({n('y', b16)})"]
    text = [f"{line} // author=miaobyte id={100 + i}" for i, line in enumerate(block)]
    kept = {}
    for mode, batched, fused, graphs in (("lines", 0, 0, 0), ("lines_deferred", 0, 1, 0), ("batch", 1, 0, 0), ("batch_fused", 1, 1, 0), ("graph", 1, 0, 1), ("graph_fused", 1, 1, 1)):
        ex = InProc()
        ex.set_graphs(bool(graphs))
        ex.set_fusion(bool(fused))
        ex.set_defer(mode == "lines_deferred")
        h = Host(ex, tmp_path)
        for name, arr in (("x", x), ("w", w.reshape(1, Hd)), ("Wg", Wg), ("Wu", Wu), ("Wd", Wd)):
            h.put("f5_" + name, arr, b16)
        for name, shape, dt in tensors:
            h.run(f"newtensor({V(shape)})->({T('f5_' + name, dt)})")
        for rep in range(3 if graphs else 1):  # a graph is recorded on the second arrival and replayed on the third
            if rep:
                h.run(f"constant(var<float32>:0)->({n('y', b16)})")
            rs = ex.execute_batch(text) if batched else [ex.execute(t) for t in text]
            assert all(r.split(" ")[1].startswith("ok") for r in rs), (mode, rs)
        if mode == "lines_deferred":
            assert ex.held() == 1  # the down projection waits for a product on the same activations
            ex.flush()
            assert ex.held() == 0 and ex.defer_stats()["held_lines"] == 22
        if graphs:
            st = ex.stats()
            assert st["captures"] == 1 and st["replays"] == 1 and st["rejects"] == 0, (mode, st)
        if fused:
            # the thirteen lines of the RMSNorm, its row sum included; the six of the gate
            fs = ex.fusion_stats()
            assert fs["runs"] == 2 * (2 if graphs else 1) and fs["lines"] == 19 * (2 if graphs else 1), (mode, fs)
            # the gate and the up projection share their activations: one call for the two lines
            assert fs["matmul_groups"] == (2 if graphs else 1) and fs["matmul_lines"] == 2 * (2 if graphs else 1), (mode, fs)
        kept[mode] = {k: h.get("f5_" + k) for k in ("y", "h", "sg", "xf", "sq", "var", "rs", "xn", "wf1", "wf", "g", "u")}
        y = b2f(kept[mode]["y"]).astype(np.float64)
        hh = b2f(kept[mode]["h"]).astype(np.float64)
        assert np.abs(y - y_ref).max() <= 3e-2 * np.abs(y_ref).max(), mode
        assert np.abs(hh - h_ref).max() <= 1e-2 * np.abs(h_ref).max(), mode
        # element by element as well: every output against the model within 1e-2 of the magnitude that
        # went into it (sum_k |act||Wd| for the GEMM, the value itself for the normalised activations) ...
        assert np.all(np.abs(y - y_ref) <= 1e-2 * y_mag), (mode, float(np.max(np.abs(y - y_ref) / y_mag)))
        assert np.all(np.abs(hh - h_ref) <= 1e-2 * np.abs(h_ref) + 1e-30), mode
        # ... and every stage against the model applied to the stage's own inputs as the device left them
        if mode == "lines":
            gd, ud, sgd = (b2f(kept[mode][k]).astype(np.float64) for k in ("g", "u", "sg"))
            Wg64, Wu64 = b2f(Wg).astype(np.float64), b2f(Wu).astype(np.float64)
            assert np.all(np.abs(gd - hh @ Wg64) <= 1e-2 * (np.abs(hh) @ np.abs(Wg64)))
            assert np.all(np.abs(ud - hh @ Wu64) <= 1e-2 * (np.abs(hh) @ np.abs(Wu64)))
            sg_model = rb(rb(gd * rb(1.0 / rb(1.0 + rb(np.exp(rb(-gd)))))) * ud)
            # five bf16 roundings; a 4-ulp exp or a double rounding may move one of them by one bf16 step
            assert np.all(np.abs(sgd - sg_model) <= 2.0 ** -6 * np.abs(sg_model) + 1e-37)
            assert np.all(np.abs(y - sgd @ Wd64) <= 1e-2 * (np.abs(sgd) @ np.abs(Wd64)))
        del ex
    for mode in ("lines_deferred", "batch", "batch_fused", "graph", "graph_fused"):
        for k in kept["lines"]:
            assert np.array_equal(kept[mode][k], kept["lines"][k]), (mode, k)


def test_random_batches_fused_equal_line_by_line(tmp_path):
    """Random batches over a pool of [rows, cols], [rows, 1] and [1, cols] tensors in float32,
    bfloat16 and float16: elementwise lines (in place or not), casts, squares, broadcastTo of the
    vectors and sums over the last axis, in random order.  Whatever runs the planner forms — one
    dtype, mixed, with row or column vectors, with a row sum inside, cut at a vector that would be
    overwritten while other lanes still read it — every tensor must end up with the bits of the
    line-by-line execution, and every line must get the reply it gets on its own.  The same lines sent
    one by one with runs held back (DEEPX_DEFER) must do the same, and so must the batch with independent
    lines spread over three side streams (DEEPX_STREAMS), fused and unfused: a random program is full of
    read-after-write, write-after-read and write-after-write pairs for the stream choice to get wrong."""
    rng = np.random.default_rng(20251)
    dts = ["float32", "bfloat16", "float16"]
    code = {"float32": dx.F32, "bfloat16": dx.BF16, "float16": dx.F16}
    fused_lines = held_lines = side_launches = 0
    for trial in range(72):
        rows, cols = [(16, 64), (5, 12), (64, 896), (3, 1000), (33, 260), (128, 32)][trial % 6]
        shapes = {"F": [rows, cols], "C": [rows, 1], "R": [1, cols]}
        pool = [(f"t{trial}_{k}{i}_{dt[:3]}{dt[-2:]}", k, dt) for k in shapes for i in range(3) for dt in dts]
        data = {name: H.to_storage(rng.uniform(0.25, 2.0, int(np.prod(shapes[k]))), code[dt]).reshape(shapes[k]) if dt != "float32"
                else rng.uniform(0.25, 2.0, shapes[k]).astype(np.float32) for name, k, dt in pool}
        def pick(k, dt):
            fits = [p for p in pool if p[1] == k and p[2] == dt]
            return fits[int(rng.integers(0, len(fits)))]
        lines = []
        for _ in range(int(rng.integers(10, 22))):
            kind = str(rng.choice(["bin", "bin", "scalar", "scalar", "sqrt", "todtype", "square", "broadcast", "sum"]))
            k, dt = str(rng.choice(["F", "F", "F", "C", "R"])), str(rng.choice(dts))
            a, b, c = pick(k, dt), pick(k, dt), pick(k, dt)
            if kind == "bin":
                lines.append(f"{rng.choice(['add', 'mul', 'sub', 'max', 'min', 'div'])}({T(a[0], dt)}, {T(b[0], dt)})->({T(c[0], dt)})")
            elif kind == "scalar":
                op = str(rng.choice(["addscalar", "mulscalar", "divscalar", "maxscalar", "rsubscalar", "rdivscalar"]))
                s = float(rng.choice([0.5, 2.0, 1.25, 3.0]))
                args = f"var<float32>:{s}, {T(a[0], dt)}" if op in ("rsubscalar", "rdivscalar") else f"{T(a[0], dt)}, var<float32>:{s}"
                lines.append(f"{op}({args})->({T(c[0], dt)})")
            elif kind == "sqrt":
                lines.append(f"sqrt({T(a[0], dt)})->({T(c[0], dt)})")
            elif kind == "todtype":
                d2 = str(rng.choice(dts))
                lines.append(f"todtype({T(a[0], dt)})->({T(pick(k, d2)[0], d2)})")
            elif kind == "square":
                a, c = pick(k, "float32"), pick(k, "float32")
                lines.append(f"powscalar({T(a[0])}, var<float32>:2)->({T(c[0])})")
            elif kind == "broadcast":
                v = pick(str(rng.choice(["C", "R"])), dt)
                lines.append(f"broadcastTo({T(v[0], dt)}, {V(shapes['F'])})->({T(pick('F', dt)[0], dt)})")
            else:
                dt = str(rng.choice(["float32", "float32", "bfloat16"]))
                lines.append(f"sum({T(pick('F', dt)[0], dt)}, {V([-1])}, var<bool>:true)->({T(pick('C', dt)[0], dt)})")
        text = [f"{line} // author=miaobyte id={900 + i}" for i, line in enumerate(lines)]
        results, replies = {}, {}
        for mode in ("lines", "fused", "held", "streams", "streams_unfused", "streams_lines"):
            ex = InProc()
            ex.set_fusion(mode not in ("lines", "streams_unfused", "streams_lines"))
            ex.set_defer(mode == "held")
            ex.set_streams(3 if mode.startswith("streams") else 1)
            h = Host(ex, tmp_path)
            for name, k, dt in pool:
                h.put(name, data[name], dt)
            replies[mode] = ex.execute_batch(text) if mode in ("fused", "streams", "streams_unfused") else [ex.execute(t) for t in text]
            if mode == "fused":
                fused_lines += ex.fusion_stats()["lines"]
            if mode == "held":
                held_lines += ex.defer_stats()["held_lines"]
            if mode.startswith("streams"):
                side_launches += ex.side_launches()
            results[mode] = {name: h.get(name) for name, _, _ in pool}
            ex.close()
        for mode in ("fused", "held", "streams", "streams_unfused", "streams_lines"):
            got, want = [r.split("//")[0] for r in replies[mode]], [r.split("//")[0] for r in replies["lines"]]
            differ = [(i, replies[mode][i], replies["lines"][i]) for i in range(min(len(got), len(want))) if got[i] != want[i]]
            assert got == want, (trial, mode, len(got), len(want), differ[:3], lines)
            for name, _, _ in pool:
                a, b = results["lines"][name], results[mode][name]
                same = np.array_equal(a.view(np.uint8), b.view(np.uint8))
                if not same and a.dtype.kind == "f":
                    same = np.array_equal(a, b, equal_nan=True)
                if not same:  # 16-bit floats come back as raw bits: NaN payloads aside they must agree
                    fa, fb = H.to_float(a.reshape(-1), code[[p for p in pool if p[0] == name][0][2]]), H.to_float(b.reshape(-1), code[[p for p in pool if p[0] == name][0][2]])
                    same = np.array_equal(fa, fb, equal_nan=True)
                assert same, (trial, mode, name, lines)
    assert fused_lines > 400 and held_lines > 400  # the batches did form runs, the single lines were held
    assert side_launches > 100  # and independent lines did leave the default stream


def test_square_view_row_sum_without_keepdims_fuses(tmp_path):
    """On a square [N, N] view the [N] result of a row sum without keepdims looks like a row by its shape
    and is a column to the run that produced it: lines that go on with it stay in the run (one launch)
    and leave the bits of the line-by-line execution."""
    ex = InProc()
    h = Host(ex, tmp_path)
    rng = np.random.default_rng(47)
    N = 128
    h.put("q_x", rng.standard_normal((N, N)).astype(np.float32))
    for name, shape in (("q_sq", [N, N]), ("q_s", [N]), ("q_m", [N]), ("q_r", [N])):
        h.run(f"newtensor({V(shape)})->({T(name)})")
    lines = [f"powscalar({T('q_x')}, var<float32>:2)->({T('q_sq')}) // author=miaobyte id=1",
             f"sum({T('q_sq')}, {V([-1])}, var<bool>:false)->({T('q_s')}) // author=miaobyte id=2",
             f"divscalar({T('q_s')}, var<float32>:{N})->({T('q_m')}) // author=miaobyte id=3",
             f"sqrt({T('q_m')})->({T('q_r')}) // author=miaobyte id=4",
             f"mul({T('q_r')}, {T('q_s')})->({T('q_r')}) // author=miaobyte id=5"]
    ex.set_fusion(False)
    assert all(r.split(" ")[1].startswith("ok") for r in ex.execute_batch(lines))
    want = {n: h.get(n) for n in ("q_sq", "q_s", "q_m", "q_r")}
    x = h.get("q_x").astype(np.float64)
    assert np.allclose(want["q_r"], np.sqrt((x ** 2).sum(-1) / N) * (x ** 2).sum(-1), rtol=1e-5)
    for n in want:
        h.run(f"constant(var<float32>:0)->({T(n)})")
    ex.set_fusion(True)
    before = ex.fusion_stats()
    assert all(r.split(" ")[1].startswith("ok") for r in ex.execute_batch(lines))
    after = ex.fusion_stats()
    assert after["runs"] - before["runs"] == 1 and after["lines"] - before["lines"] == 5, (before, after)
    for n in want:
        assert np.array_equal(h.get(n).view(np.uint32), want[n].view(np.uint32)), n


def test_recorded_graphs_return_their_counters(dxh, tmp_path):
    """Launches recorded under capture that finish inside one launch (strided-axis sum) own counters of
    the library's array while their graph lives: recording and destroying many graphs leaves none taken."""
    import ctypes as C
    import torch
    L = dxh
    used, cap = C.c_int64(), C.c_int64()
    dx.check(L.dxh_graph_counter_stats(C.byref(used), C.byref(cap)))
    start = used.value
    x = torch.randn(2048, 1024, device="cuda")
    out = torch.empty(1024, device="cuda")
    want = torch.empty(1024, device="cuda")
    shape, ax0 = dx.i32arr([2048, 1024]), dx.i32arr([0])
    need = C.c_size_t(0)
    dx.check(L.dxh_reduce_workspace_bytes(dx.F32, shape, 2, ax0, 1, C.byref(need)))
    ws = torch.empty(max(1, need.value), dtype=torch.uint8, device="cuda")
    p = lambda t: C.c_void_p(t.data_ptr())
    dx.check(L.dxh_sum(dx.F32, p(x), shape, 2, ax0, 1, p(want), p(ws), need.value, None))
    torch.cuda.synchronize()
    st = C.c_void_p()
    dx.check(L.dxh_stream_create(C.byref(st)))
    peak = 0
    for i in range(300):  # far more recordings than the array could serve without returns (32 Ki counters)
        dx.check(L.dxh_graph_begin_capture(st))
        for _ in range(4):
            dx.check(L.dxh_sum(dx.F32, p(x), shape, 2, ax0, 1, p(out), p(ws), need.value, st))
        g = C.c_void_p()
        dx.check(L.dxh_graph_end_capture(st, C.byref(g)))
        dx.check(L.dxh_graph_counter_stats(C.byref(used), C.byref(cap)))
        peak = max(peak, used.value - start)
        if i % 50 == 0:
            out.zero_()
            dx.check(L.dxh_graph_launch(g, st))
            dx.check(L.dxh_stream_sync(st))
            assert torch.equal(out, want)
        dx.check(L.dxh_graph_destroy(g))
        dx.check(L.dxh_graph_counter_stats(C.byref(used), C.byref(cap)))
        assert used.value == start, (i, used.value, start)
    assert 0 < peak <= 4 * 1024 and cap.value >= 32 * 1024
    dx.check(L.dxh_stream_destroy(st))


@pytest.mark.parametrize("dt,rows,cols", [("float32", 4096, 2048), ("bfloat16", 2048, 896), ("float16", 300, 1000), ("float32", 2048, 896)])
def test_softmax_lines_fuse_into_one_launch(tmp_path, dt, rows, cols):
    """The front's softmax (front/py/deepx/nn/functional/normalization.py:4-17) as the eight lines it sends
    once its tensors exist: one launch in a fused batch, every tensor with the bits of the line-by-line run,
    rows summing to one."""
    ex = InProc()
    h = Host(ex, tmp_path)
    rng = np.random.default_rng(53)
    x = rng.uniform(-3, 3, (rows, cols)).astype(np.float32)
    store = {"float32": lambda a: a, "bfloat16": H.f32_to_bf16_bits, "float16": H.f32_to_f16_bits}[dt]
    h.put("sm_t", store(x), dt)
    full, col = [rows, cols], [rows, 1]
    for name, shape in (("m", col), ("mb", full), ("d", full), ("e", full), ("s", col), ("e2", full), ("sb", full), ("y", full)):
        h.run(f"newtensor({V(shape)})->({T('sm_' + name, dt)})")
    n = lambda name: T("sm_" + name, dt)
    lines = [f"reducemax({n('t')}, {V([-1])}, var<bool>:true)->({n('m')})", f"broadcastTo({n('m')}, {V(full)})->({n('mb')})",
             f"sub({n('t')}, {n('mb')})->({n('d')})", f"exp({n('d')})->({n('e')})", f"sum({n('e')}, {V([-1])}, var<bool>:true)->({n('s')})",
             f"exp({n('d')})->({n('e2')})", f"broadcastTo({n('s')}, {V(full)})->({n('sb')})", f"div({n('e2')}, {n('sb')})->({n('y')})"]
    lines = [f"{l} // author=miaobyte id={i + 1}" for i, l in enumerate(lines)]
    names = ["m", "mb", "d", "e", "s", "e2", "sb", "y"]
    ex.set_fusion(False)
    assert all(r.split(" ")[1].startswith("ok") for r in ex.execute_batch(lines))
    want = {k: h.get("sm_" + k) for k in names}
    for k in names:
        h.run(f"constant(var<float32>:0)->({n(k)})")
    ex.set_fusion(True)
    before = ex.fusion_stats()
    assert all(r.split(" ")[1].startswith("ok") for r in ex.execute_batch(lines))
    after = ex.fusion_stats()
    assert after["runs"] - before["runs"] == 1 and after["lines"] - before["lines"] == 8, (before, after)
    for k in names:
        assert np.array_equal(h.get("sm_" + k).view(np.uint8), want[k].view(np.uint8)), k
    load = {"float32": lambda a: a.astype(np.float64), "bfloat16": lambda a: H.bf16_bits_to_f32(a).astype(np.float64),
            "float16": lambda a: H.f16_bits_to_f32(a).astype(np.float64)}[dt]
    y = load(want["y"]).reshape(rows, cols)
    assert np.allclose(y.sum(1), 1.0, atol=1e-5 if dt == "float32" else 3e-2)


def test_side_streams_keep_every_hazard_in_order(tmp_path):
    """DEEPX_STREAMS: independent lines of a batch run side by side on side streams.  On tensors large enough
    for launches to overlap for tens of microseconds, a batch that mixes independent lines with
    read-after-write, write-after-read and write-after-write pairs leaves the bits of in-order execution,
    ten times in a row; the independent lines did leave the default stream."""
    n = [4096, 4096]
    rng = np.random.default_rng(411)
    x, y = rng.uniform(0.5, 1.5, n).astype(np.float32), rng.uniform(0.5, 1.5, n).astype(np.float32)
    names = ["z", "w", "x2", "s0", "s1", "m0", "m1", "v"]
    lines = [
        "add({x}, {y})->({z})",                                                  # independent
        "mul({z}, {y})->({w})",                                                  # reads z: after line 1
        "add({x}, {y})->({x2})",                                                 # independent of what is in flight
        "sum({x}, vector<int32>:[1], var<bool>:false)->({s0})",                  # independent reductions of one tensor ...
        "reducemax({x}, vector<int32>:[1], var<bool>:false)->({m0})",
        "sum({x}, vector<int32>:[0], var<bool>:false)->({s1})",
        "reducemin({x}, vector<int32>:[0], var<bool>:false)->({m1})",
        "addscalar({x}, var<float32>:1)->({y})",                                 # ... then y is rewritten while lines 1-3 may still read it
        "mul({x}, {x})->({z})",                                                  # z rewritten: after lines 1 and 2
        "sub({z}, {y})->({v})",                                                  # reads both
        "mulscalar({v}, var<float32>:0.5)->({x})",                               # x rewritten: after every reader above
        "add({x}, {y})->({w})",
    ]
    results = {}
    for streams, batched in ((1, True), (3, True), (3, False)):
        ex = InProc()
        ex.set_fusion(False)
        ex.set_streams(streams)
        h = Host(ex, tmp_path)
        p = f"hz{streams}{int(batched)}_"
        for k in names:
            shape = n if k in ("z", "w", "x2", "v") else [4096]
            h.run(f"newtensor({V(shape)})->({T(p + k)})")
        tn = {k: T(p + k) for k in names + ["x", "y"]}
        text = [line.format(**tn) + f" // author=miaobyte id={i + 1}" for i, line in enumerate(lines)]
        runs = []
        for rep in range(10 if streams > 1 else 1):
            h.put(p + "x", x)
            h.put(p + "y", y)
            rs = ex.execute_batch(text) if batched else [ex.execute(t) for t in text]
            assert all(r.split(" ")[1].startswith("ok") for r in rs), rs
            runs.append({k: h.get(p + k) for k in names + ["x", "y"]})
        if streams > 1:
            assert ex.side_launches() >= 10 * 5
        else:
            assert ex.side_launches() == 0
        results[(streams, batched)] = runs
    want = results[(1, True)][0]
    for key in ((3, True), (3, False)):  # as one datagram, and sent line by line
        for rep, got in enumerate(results[key]):
            for k in want:
                assert np.array_equal(got[k].view(np.uint8), want[k].view(np.uint8)), (key, rep, k)


def attention_core_lines(n, V, S, heads, hd, dt, scale, allocate=False):
    """The core of the front's attention (front/py/deepx/nn/modules/transformer/attention.py:15-32 with normalization.py:4-17
    for the softmax) on [1, heads, S, hd] tensors: scores = q @ k.mT, times the scaling factor, softmax over the last axis,
    times v.  With `allocate`, every result is made by a `newtensor` line right before its op, as the front does."""
    sc, full, col, out = [1, heads, S, S], [1, heads, S, S], [1, heads, S, 1], [1, heads, S, hd]
    steps = [(("kT", [1, heads, hd, S]), f"transpose({n('k')}, {V([0, 1, 3, 2])})->({n('kT')})"),
             (("sc", sc), f"matmul({n('q')}, {n('kT')})->({n('sc')})"),
             (("a", full), f"mulscalar({n('sc')}, var<float32>:{scale})->({n('a')})"),
             (("m", col), f"reducemax({n('a')}, {V([-1])}, var<bool>:true)->({n('m')})"),
             (("mb", full), f"broadcastTo({n('m')}, {V(full)})->({n('mb')})"),
             (("d", full), f"sub({n('a')}, {n('mb')})->({n('d')})"),
             (("e", full), f"exp({n('d')})->({n('e')})"),
             (("s", col), f"sum({n('e')}, {V([-1])}, var<bool>:true)->({n('s')})"),
             (("e2", full), f"exp({n('d')})->({n('e2')})"),
             (("sb", full), f"broadcastTo({n('s')}, {V(full)})->({n('sb')})"),
             (("y", full), f"div({n('e2')}, {n('sb')})->({n('y')})"),
             (("o", out), f"matmul({n('y')}, {n('v')})->({n('o')})")]
    lines = []
    for (name, shape), line in steps:
        if allocate:
            lines.append(f"newtensor({V(shape)})->({n(name)})")
        lines.append(line)
    return [name for (name, _), _ in steps], [shape for (_, shape), _ in steps], lines


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_attention_core_one_launch_for_scale_and_softmax(dxh, tmp_path, dt):
    """q @ k.mT, the scaling, the softmax and the product with v as the front sends them, every result allocated right
    before its op: as one datagram and line by line with runs held back, the nine lines from the scaling to the division
    are one launch of the kernel compiled for them; every tensor has the bits of plain line-by-line execution, and the
    output agrees with a float64 model of the same roundings."""
    S, heads, hd = 256, 4, 64
    scale = hd ** -0.5
    rng = np.random.default_rng(61)
    store = {"float32": lambda a: a, "bfloat16": H.f32_to_bf16_bits}[dt]
    load = {"float32": lambda a: a.astype(np.float64), "bfloat16": lambda a: H.bf16_bits_to_f32(a).astype(np.float64)}[dt]
    q, k, v = (rng.standard_normal((1, heads, S, hd)).astype(np.float32) for _ in range(3))
    results = {}
    for mode in ("plain", "batch", "held"):
        ex = InProc()
        ex.set_defer(mode == "held")
        ex.set_fusion(mode != "plain")
        h = Host(ex, tmp_path)
        p = f"att_{mode}_{dt}_"
        n = lambda name: T(p + name, dt)
        for name, arr in (("q", q), ("k", k), ("v", v)):
            h.put(p + name, store(arr), dt)
        names, _, lines = attention_core_lines(n, V, S, heads, hd, dt, scale, allocate=True)
        lines = [f"{l} // author=miaobyte id={500 + i}" for i, l in enumerate(lines)]
        a0, b0 = C.c_int64(), C.c_int64()
        dxh.dxh_chain_stats(C.byref(a0), C.byref(b0))
        rs = ex.execute_batch(lines) if mode == "batch" else [ex.execute(l) for l in lines]
        assert all(r.split(" ")[1].startswith("ok") for r in rs), rs
        ex.flush()
        a1, b1 = C.c_int64(), C.c_int64()
        dxh.dxh_chain_stats(C.byref(a1), C.byref(b1))
        if mode != "plain":
            fs = ex.fusion_stats()
            assert fs["runs"] == 1 and fs["lines"] == 9, fs
            assert (a1.value - a0.value, b1.value - b0.value) == (1, 0), "the run did not take its compiled kernel"
        results[mode] = {name: h.get(p + name) for name in names}
    for mode in ("batch", "held"):
        for name in results["plain"]:
            assert np.array_equal(results[mode][name].view(np.uint8), results["plain"][name].view(np.uint8)), (mode, name)
    # float64 model with the storage type's rounding where a tensor is stored
    rt = (lambda a: a.astype(np.float32).astype(np.float64)) if dt == "float32" else (lambda a: H.bf16_bits_to_f32(H.f32_to_bf16_bits(a.astype(np.float32))).astype(np.float64))
    q64, k64, v64 = (rt(x.astype(np.float64)) for x in (q, k, v))
    a = rt(rt(q64 @ k64.transpose(0, 1, 3, 2)) * rt(np.float64(scale)))
    d = rt(a - a.max(-1, keepdims=True))
    e = rt(np.exp(d))
    y = rt(e / rt(e.sum(-1, keepdims=True)))
    o = y @ v64
    got = load(results["plain"]["o"]).reshape(o.shape)
    tol = 1e-4 if dt == "float32" else 3e-2
    assert np.all(np.abs(got - o) <= tol * (np.abs(y) @ np.abs(v64)) + 1e-6), float(np.max(np.abs(got - o)))
    assert np.allclose(load(results["plain"]["y"]).reshape(y.shape).sum(-1), 1.0, atol=1e-5 if dt == "float32" else 3e-2)


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_rmsnorm_lines_take_the_compiled_kernel_in_fp32_too(dxh, tmp_path, dt):
    """The thirteen lines of the front's RMSNorm on an activation and a weight kept in fp32 (the front's default dtype; the
    two casts are then copies) or in bf16: one launch of the compiled kernel, the bits of the lines run one by one, and
    the formula in float64."""
    S, Hd = 192, 896
    rng = np.random.default_rng(67)
    store = {"float32": lambda a: a, "bfloat16": H.f32_to_bf16_bits}[dt]
    load = {"float32": lambda a: a.astype(np.float64), "bfloat16": lambda a: H.bf16_bits_to_f32(a).astype(np.float64)}[dt]
    x, w = rng.standard_normal((S, Hd)).astype(np.float32), (1 + 0.1 * rng.standard_normal((1, Hd))).astype(np.float32)
    f32 = "float32"
    results = {}
    for mode in ("plain", "batch"):
        ex = InProc()
        ex.set_fusion(mode == "batch")
        h = Host(ex, tmp_path)
        p = f"rn_{mode}_{dt}_"
        n = lambda name, d=f32: T(p + name, d)
        h.put(p + "x", store(x), dt)
        h.put(p + "w", store(w), dt)
        for name, shape, d in (("xf", [S, Hd], f32), ("sq", [S, Hd], f32), ("var", [S, 1], f32), ("rs", [S, Hd], f32), ("xn", [S, Hd], f32), ("wf1", [1, Hd], f32),
                               ("wf", [S, Hd], f32), ("h", [S, Hd], dt)):
            h.run(f"newtensor({V(shape)})->({n(name, d)})")
        lines = [f"todtype({n('x', dt)})->({n('xf')})", f"powscalar({n('xf')}, var<float32>:2)->({n('sq')})", f"sum({n('sq')}, {V([-1])}, var<bool>:true)->({n('var')})",
                 f"divscalar({n('var')}, var<float32>:{Hd})->({n('var')})", f"addscalar({n('var')}, var<float32>:1e-06)->({n('var')})", f"sqrt({n('var')})->({n('var')})",
                 f"rdivscalar(var<float32>:1, {n('var')})->({n('var')})", f"broadcastTo({n('var')}, {V([S, Hd])})->({n('rs')})", f"mul({n('xf')}, {n('rs')})->({n('xn')})",
                 f"todtype({n('w', dt)})->({n('wf1')})", f"broadcastTo({n('wf1')}, {V([S, Hd])})->({n('wf')})", f"mul({n('wf')}, {n('xn')})->({n('xn')})",
                 f"todtype({n('xn')})->({n('h', dt)})"]
        lines = [f"{l} // author=miaobyte id={i + 1}" for i, l in enumerate(lines)]
        a0, b0 = C.c_int64(), C.c_int64()
        dxh.dxh_chain_stats(C.byref(a0), C.byref(b0))
        rs = ex.execute_batch(lines)
        assert all(r.split(" ")[1].startswith("ok") for r in rs), rs
        a1, b1 = C.c_int64(), C.c_int64()
        dxh.dxh_chain_stats(C.byref(a1), C.byref(b1))
        if mode == "batch":
            assert ex.fusion_stats()["runs"] == 1 and ex.fusion_stats()["lines"] == 13, ex.fusion_stats()
            assert (a1.value - a0.value, b1.value - b0.value) == (1, 0), "the run did not take its compiled kernel"
        results[mode] = {k: h.get(p + k) for k in ("xf", "sq", "var", "rs", "xn", "wf1", "wf", "h")}
        ex.close()
    for k in results["plain"]:
        assert np.array_equal(results["batch"][k].view(np.uint8), results["plain"][k].view(np.uint8)), k
    x64, w64 = load(store(x)), load(store(w))
    ref = w64 * (x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + 1e-6))
    got = load(results["plain"]["h"]).reshape(S, Hd)
    assert np.all(np.abs(got - ref) <= (1e-5 if dt == f32 else 1e-2) * np.abs(ref) + 1e-6)
