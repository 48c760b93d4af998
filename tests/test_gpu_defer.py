"""GPU: lines that arrive one per datagram, as the unmodified front sends them, held back until the run
they belong to is complete (DEEPX_DEFER=1) — answered at once, launched together.  Every tensor must end
up with the bits of plain line-by-line execution, a line that would fail must still be the one that
reports it, and nothing may stay unlaunched."""
import time

import numpy as np
import pytest

from deepx_amd import lib as dx
from tests import helpers as H
from tests.executor_client import InProc, UdpExecutor, read_tensor, write_tensor
from tests.test_gpu_batch import Host, T, V

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _torch_owns_the_hip_runtime(dxh):
    yield


LINES = [
    "add({a}, {b})->({c})", "mulscalar({c}, var<float32>:0.25)->({d})", "sub({d}, {a})->({a})",
    "mul({a}, {c})->({e})", "exp({e})->({f})",
    "sum({f}, vector<int32>:[1], var<bool>:true)->({s})",
    "rdivscalar(var<float32>:1, {s})->({t})", "sqrt({t})->({u})", "log({u})->({v})",
    "max({f}, {e})->({g})", "minscalar({g}, var<float32>:1.5)->({h})",
    "add({i1}, {i2})->({i3})",
    "div({h}, {b})->({k})", "rsubscalar(var<float32>:2, {k})->({m})",
]
BIG, SMALL, INTS = ["a", "b", "c", "d", "e", "f", "g", "h", "k", "m"], ["s", "t", "u", "v"], ["i1", "i2", "i3"]


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_held_lines_equal_line_by_line(tmp_path, dt):
    """Fourteen lines — float runs cut by a row sum, by an integer op and by an in-place line — one
    execute() per line with and without holding: same bits everywhere, the same launches as the lines
    sent as one batch, and every reply `ok` at once."""
    rng = np.random.default_rng(191)
    shape = [64, 136]
    data = {"a": rng.uniform(0.5, 1.5, shape).astype(np.float32), "b": rng.uniform(0.5, 1.5, shape).astype(np.float32),
            "i1": rng.integers(-9, 9, shape).astype(np.int32), "i2": rng.integers(-9, 9, shape).astype(np.int32)}
    stored = lambda x: x if dt == "float32" else H.to_storage(x.reshape(-1).astype(np.float64), dx.BF16).reshape(x.shape)
    results = {}
    for mode in ("plain", "held"):
        ex = InProc()
        ex.set_defer(mode == "held")
        h = Host(ex, tmp_path)
        p = f"{mode}_{dt}_"
        for n in BIG[2:]:
            h.run(f"newtensor({V(shape)})->({T(p + n, dt)})")
        for n in SMALL:
            h.run(f"newtensor({V([shape[0], 1])})->({T(p + n, dt)})")
        h.run(f"newtensor({V(shape)})->({T(p + 'i3', 'int32')})")
        h.put(p + "a", stored(data["a"]), dt)
        h.put(p + "b", stored(data["b"]), dt)
        h.put(p + "i1", data["i1"], "int32")
        h.put(p + "i2", data["i2"], "int32")
        names = {n: T(p + n, "int32" if n in INTS else dt) for n in BIG + SMALL + INTS}
        for i, line in enumerate(LINES):
            r = ex.execute(line.format(**names) + f" // author=miaobyte id={700 + i}")
            assert r.startswith(f"{700 + i} ok"), r
        if mode == "held":
            assert ex.held() == 2  # div, rsubscalar: nothing has ended their run yet
            ex.flush()
            assert ex.held() == 0
            want = {"runs": 2, "lines": 13} if dt == "float32" else {"runs": 4, "lines": 12}  # as the same lines in one batch
            assert {k: ex.fusion_stats()[k] for k in want} == want, ex.fusion_stats()
            assert ex.defer_stats()["held_lines"] == 13  # all but the integer add
        else:
            assert ex.fusion_stats()["runs"] == 0 and ex.defer_stats()["held_lines"] == 0
        results[mode] = {n: h.get(p + n) for n in BIG + SMALL + ["i3"]}
    for n in BIG + SMALL + ["i3"]:
        assert np.array_equal(results["held"][n].view(np.uint8), results["plain"][n].view(np.uint8)), n


def test_a_failing_line_is_never_held(tmp_path):
    """A line that names a missing tensor, or tensors that do not fit each other, is executed at once and
    reports its own error; what was held before it has run by then, what follows is held again."""
    rng = np.random.default_rng(192)
    ex = InProc()
    ex.set_defer(True)
    h = Host(ex, tmp_path)
    for n in ("p", "q", "r"):
        h.run(f"newtensor({V([8, 16])})->({T('dh_' + n)})")
    h.run(f"newtensor({V([4, 16])})->({T('dh_small')})")
    x = rng.uniform(-1, 1, [8, 16]).astype(np.float32)
    h.put("dh_x", x)
    lines = [f"addscalar({T('dh_x')}, var<float32>:1)->({T('dh_p')}) // id=1", f"mulscalar({T('dh_p')}, var<float32>:3)->({T('dh_q')}) // id=2",
             f"add({T('dh_q')}, {T('dh_missing')})->({T('dh_r')}) // id=3", f"add({T('dh_q')}, {T('dh_small')})->({T('dh_r')}) // id=4",
             f"sqrt({T('dh_q')})->({T('dh_r')}) // id=5", "nosuchop(var<int32>:1)->() // id=6"]
    held_after = []
    replies = []
    for line in lines:
        replies.append(ex.execute(line))
        held_after.append(ex.held())
    assert [r.split(" ")[1][:2] for r in replies] == ["ok", "ok", "er", "er", "ok", "er"], replies
    assert held_after == [1, 2, 0, 0, 1, 0], held_after
    assert np.array_equal(h.get("dh_q"), (x + np.float32(1)) * np.float32(3))
    assert np.array_equal(h.get("dh_r"), np.sqrt((x + np.float32(1)) * np.float32(3)))


def test_a_line_that_needs_results_launches_what_is_held(tmp_path):
    """save, print and every other op that is not part of a run come after the held lines: the file a
    save writes holds the values of the lines sent before it.  Turning the switch off launches too."""
    ex = InProc()
    ex.set_defer(True)
    h = Host(ex, tmp_path)
    x = np.arange(64, dtype=np.float32).reshape(4, 16)
    h.put("dn_x", x)
    h.run(f"newtensor({V([4, 16])})->({T('dn_y')})")
    h.run(f"newtensor({V([4, 16])})->({T('dn_z')})")
    assert ex.execute(f"mulscalar({T('dn_x')}, var<float32>:2)->({T('dn_y')}) // id=50").startswith("50 ok")
    assert ex.execute(f"addscalar({T('dn_y')}, var<float32>:1)->({T('dn_z')}) // id=51").startswith("51 ok")
    assert ex.held() == 2
    assert np.array_equal(h.get("dn_z"), x * 2 + 1)  # the save came after them
    assert ex.held() == 0
    assert ex.execute(f"mulscalar({T('dn_z')}, var<float32>:2)->({T('dn_y')}) // id=52").startswith("52 ok")
    assert ex.held() == 1
    ex.set_defer(False)
    assert ex.held() == 0
    assert np.array_equal(h.get("dn_y"), (x * 2 + 1) * 2)
    # a switch turned while lines are held: they still come before the next line
    ex.set_defer(True)
    assert ex.execute(f"addscalar({T('dn_y')}, var<float32>:1)->({T('dn_z')}) // id=60").startswith("60 ok")
    assert ex.held() == 1
    ex.set_sync(True)
    assert ex.execute(f"mulscalar({T('dn_z')}, var<float32>:3)->({T('dn_y')}) // id=61").startswith("61 ok")
    assert ex.held() == 0
    ex.set_sync(False)
    assert np.array_equal(h.get("dn_y"), (((x * 2 + 1) * 2) + 1) * 3)
    ex.set_defer(False)
    # deltensor of an operand of a held line: the line runs first, then the tensor goes
    ex.set_defer(True)
    assert ex.execute(f"mulscalar({T('dn_x')}, var<float32>:5)->({T('dn_z')}) // id=53").startswith("53 ok")
    assert ex.execute(f"deltensor()->({T('dn_x', 'any')}) // id=54").startswith("54 ok")
    assert np.array_equal(h.get("dn_z"), x * 5)


def test_server_launches_held_lines_when_the_sender_pauses(tmp_path):
    """Over UDP with DEEPX_DEFER=1, one line per datagram: the replies come at once, a pause of the
    sender longer than the grace period launches what is held, and a save right after a run sees its
    results."""
    ex = UdpExecutor(env={"DEEPX_DEFER": "1", "DEEPX_DEFER_US": "300"})
    try:
        x = np.linspace(-2, 2, 32 * 48, dtype=np.float32).reshape(32, 48)
        write_tensor(str(tmp_path / "ds_x"), x, "float32")
        ex.must("load", [f"var<string>:{tmp_path / 'ds_x'}"], [])
        for n in ("y", "z", "w"):
            ex.must("newtensor", [V([32, 48])], [T("ds_" + n)])
        ex.must("mulscalar", [T("ds_x"), "var<float32>:-1"], [T("ds_y")])
        ex.must("exp", [T("ds_y")], [T("ds_z")])
        ex.must("addscalar", [T("ds_z"), "var<float32>:1"], [T("ds_w")])
        time.sleep(0.05)  # far beyond the grace period: the three lines have been launched as one run by now
        ex.must("mul", [T("ds_w"), T("ds_x")], [T("ds_y")])
        ex.must("save", [T("ds_y", "any"), f"var<string>:{tmp_path / 'ds_out'}"], [])
        got = read_tensor(str(tmp_path / "ds_out"))[0]
        want = (np.exp(-x).astype(np.float32) + np.float32(1)) * x
        assert np.allclose(got, want, rtol=1e-6, atol=1e-6)
    finally:
        ex.close()


@pytest.mark.parametrize("mode", ["held", "batch"])
def test_allocations_do_not_end_a_run(tmp_path, mode):
    """The front allocates every result right before the line that computes it (newtensor, then the op).  Held line by
    line, or as one datagram, the compute lines between the allocations still go out as one launch, and every tensor
    has the bits of in-order execution."""
    S, Hd = 96, 256
    rng = np.random.default_rng(193)
    x = H.f32_to_bf16_bits(rng.standard_normal((S, Hd)).astype(np.float32))
    f32, b16 = "float32", "bfloat16"
    steps = [  # (allocation of the result, compute line)
        (("xf", [S, Hd], f32), "todtype({x})->({xf})"),
        (("sq", [S, Hd], f32), "powscalar({xf}, var<float32>:2)->({sq})"),
        (("var", [S, 1], f32), "sum({sq}, vector<int32>:[-1], var<bool>:true)->({var})"),
        (None, f"divscalar({{var}}, var<float32>:{Hd})->({{var}})"),
        (("ve", [S, 1], f32), "addscalar({var}, var<float32>:1e-06)->({ve})"),
        (("sd", [S, 1], f32), "sqrt({ve})->({sd})"),
        (("rs1", [S, 1], f32), "rdivscalar(var<float32>:1, {sd})->({rs1})"),
        (("rs", [S, Hd], f32), f"broadcastTo({{rs1}}, {V([S, Hd])})->({{rs}})"),
        (("xn", [S, Hd], f32), "mul({xf}, {rs})->({xn})"),
        (("h", [S, Hd], b16), "todtype({xn})->({h})"),
    ]
    names = ["xf", "sq", "var", "ve", "sd", "rs1", "rs", "xn", "h"]
    results = {}
    for m in ("plain", mode):
        ex = InProc()
        ex.set_defer(m == "held")
        h = Host(ex, tmp_path)
        p = f"al_{m}_"
        h.put(p + "x", x, b16)
        tn = {k: T(p + k, b16 if k in ("x", "h") else f32) for k in names + ["x"]}
        text = []
        for alloc, line in steps:
            if alloc:
                text.append(f"newtensor({V(alloc[1])})->({T(p + alloc[0], alloc[2])})")
            text.append(line.format(**tn))
        text = [f"{t} // author=miaobyte id={300 + i}" for i, t in enumerate(text)]
        if m == "batch":
            rs = ex.execute_batch(text)
        else:
            rs = [ex.execute(t) for t in text]
        assert [r.split(" ")[0] for r in rs] == [str(300 + i) for i in range(len(text))], rs  # replies in the order of the lines
        assert all(r.split(" ")[1].startswith("ok") for r in rs), rs
        ex.flush()
        fs = ex.fusion_stats()
        if m == "plain":
            assert fs["runs"] == 0
        else:
            assert fs["runs"] == 1 and fs["lines"] == len(steps), fs
        results[m] = {k: h.get(p + k) for k in names}
    for k in names:
        assert np.array_equal(results[mode][k].view(np.uint8), results["plain"][k].view(np.uint8)), k
