"""GPU: the whole drop-in path — deepxIR text over UDP into deepx-executor-hip, tensors loaded
from / saved to deepx tensor files, results compared with the CPU oracle."""
import os

import numpy as np
import pytest

from deepx_amd import lib as dx
from tests import helpers as H
from tests.executor_client import UdpExecutor, read_tensor, write_tensor
from tests.helpers import hp

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def srv():
    s = UdpExecutor()
    yield s
    s.close()
    assert s.proc.returncode == 0


def T(name, dt="float32"):
    return f"tensor<{dt}>:{name}"


def V(values):
    return "vector<int32>:[" + " ".join(str(v) for v in values) + "]"


def load(srv, tmp_path, name, arr, dtype_name):
    p = str(tmp_path / name)
    write_tensor(p, arr, dtype_name)
    srv.must("load", [f"var<string>:{p}"], [], author="")


def fetch(srv, tmp_path, name):
    p = str(tmp_path / (name + "_out"))
    srv.must("save", [T(name, "any"), f"var<string>:{p}"], [], author="")
    return read_tensor(p)


def test_tensor_lifecycle_and_init(srv, tmp_path):
    srv.must("newtensor", [V([3, 4])], [T("t0")], author="")
    a, meta = fetch(srv, tmp_path, "t0")
    assert meta == {"dtype": "float32", "dim": 2, "shape": [3, 4], "stride": [4, 1], "size": 12}
    assert a.dtype == np.float32 and np.all(a == 0)
    srv.must("constant", ["var<float32>:2.5"], [T("t0")])
    assert np.all(fetch(srv, tmp_path, "t0")[0] == 2.5)
    srv.must("arange", ["var<float32>:1", "var<float32>:0.5"], [T("t0")])
    assert np.array_equal(fetch(srv, tmp_path, "t0")[0].reshape(-1), 1 + 0.5 * np.arange(12, dtype=np.float32))
    srv.must("newtensor", [V([3, 4])], [T("t1")], author="")
    srv.must("copytensor", [T("t0")], [T("t1")], author="")
    assert np.array_equal(fetch(srv, tmp_path, "t1")[0], fetch(srv, tmp_path, "t0")[0])
    srv.must("renametensor", ["var<string>:t2"], [T("t1")], author="")
    assert srv.send("print", [T("t1")], []).message == "print t1 not found"
    assert fetch(srv, tmp_path, "t2")[1]["shape"] == [3, 4]
    srv.must("deltensor", [], [T("t2")], author="")
    assert srv.send("copytensor", [T("t0")], [T("t2")], author="").message == "tensor not found: t2"
    # int / bool / 16-bit tensors
    for dt in ["int64", "int32", "int16", "int8", "bool", "float16", "bfloat16", "float64"]:
        srv.must("newtensor", [V([5])], [T("n_" + dt, dt)], author="")
        arr, meta = fetch(srv, tmp_path, "n_" + dt)
        assert meta["dtype"] == dt and not arr.any()
    assert srv.send("newtensor", [V([5])], [T("f8", "float8e4m3")], author="").result == "error"
    srv.must("print", [T("t0")], [])
    srv.must("print", [T("t0"), "var<string>:%.2f"], [])


def test_random_init_distributions(srv, tmp_path):
    srv.must("newtensor", [V([1 << 16])], [T("r")], author="")
    srv.must("uniform", ["var<float32>:-1", "var<float32>:3", "var<int32>:7"], [T("r")])
    u = fetch(srv, tmp_path, "r")[0]
    assert u.min() >= -1 and u.max() < 3 and abs(u.mean() - 1.0) < 0.05 and abs(u.std() - 4 / np.sqrt(12)) < 0.05
    srv.must("uniform", ["var<float32>:-1", "var<float32>:3", "var<int32>:7"], [T("r")])
    assert np.array_equal(fetch(srv, tmp_path, "r")[0], u)  # same seed, same stream
    srv.must("normal", ["var<float32>:2", "var<float32>:0.5", "var<int32>:9"], [T("r")])
    g = fetch(srv, tmp_path, "r")[0]
    assert abs(g.mean() - 2.0) < 0.02 and abs(g.std() - 0.5) < 0.02
    srv.must("constant", ["var<float32>:1"], [T("r")])
    srv.must("dropout", ["var<float32>:0.25", "var<int32>:11"], [T("r")])
    d = fetch(srv, tmp_path, "r")[0]
    assert set(np.unique(d)) == {0.0, 1.0} and abs((d == 0).mean() - 0.25) < 0.02


def test_config1_chain_over_ir(srv, tmp_path, orc):
    """BASELINE config 1 expressed as deepxIR (abs composed from mulscalar+max), reduced size."""
    n = (512, 1024)
    A = np.random.default_rng(1).uniform(-1, 1, n).astype(np.float32)
    B = np.random.default_rng(2).uniform(-1, 1, n).astype(np.float32)
    load(srv, tmp_path, "A", A, "float32")
    load(srv, tmp_path, "B", B, "float32")
    for name in ["C", "D", "E", "F", "nB", "absB", "den", "G"]:
        srv.must("newtensor", [V(n)], [T(name)], author="")
    srv.must("add", [T("A"), T("B")], [T("C")])
    srv.must("mul", [T("C"), T("B")], [T("D")])
    srv.must("addscalar", [T("D"), "var<float32>:0.5"], [T("E")])
    srv.must("exp", [T("E")], [T("F")])
    srv.must("mulscalar", [T("B"), "var<float32>:-1"], [T("nB")])
    srv.must("max", [T("B"), T("nB")], [T("absB")])
    srv.must("addscalar", [T("absB"), "var<int32>:1"], [T("den")])
    srv.must("div", [T("F"), T("den")], [T("G")])
    C_ = A + B
    D_ = C_ * B
    E_ = D_ + np.float32(0.5)
    assert np.array_equal(fetch(srv, tmp_path, "C")[0], C_)
    assert np.array_equal(fetch(srv, tmp_path, "D")[0], D_)
    assert np.array_equal(fetch(srv, tmp_path, "E")[0], E_)
    Fw = np.empty_like(E_)
    assert orc.orc_exp(dx.F32, hp(E_), hp(Fw), E_.size) == 0
    Fg = fetch(srv, tmp_path, "F")[0]
    assert H.ulp_diff(Fg, Fw, dx.F32) <= 4
    den = np.abs(B) + np.float32(1)
    assert np.array_equal(fetch(srv, tmp_path, "den")[0], den)
    assert np.array_equal(fetch(srv, tmp_path, "G")[0], Fg / den)
    # in place: the same name on both sides (docs/design.md:18-21)
    srv.must("add", [T("A"), T("B")], [T("A")])
    assert np.array_equal(fetch(srv, tmp_path, "A")[0], C_)
    # scalar through float32: 0.1 is float(0.1), also for a float64 tensor (tf.hpp:119-123)
    load(srv, tmp_path, "d64", np.ones(8), "float64")
    srv.must("addscalar", [T("d64", "float64"), "var<float64>:0.1"], [T("d64", "float64")])
    assert np.all(fetch(srv, tmp_path, "d64")[0] == 1.0 + float(np.float32(0.1)))
    # r*scalar ops take (scalar, tensor) as registered and as the front sends them
    srv.must("rsubscalar", ["var<float32>:1", T("B")], [T("nB")])
    assert np.array_equal(fetch(srv, tmp_path, "nB")[0], np.float32(1) - B)
    srv.must("rdivscalar", ["var<float32>:1", T("den")], [T("nB")])
    assert np.array_equal(fetch(srv, tmp_path, "nB")[0], np.float32(1) / den)
    srv.must("powscalar", [T("den"), "var<float32>:2"], [T("nB")])
    assert H.ulp_diff(fetch(srv, tmp_path, "nB")[0], den * den, dx.F32) <= 1


def test_errors_do_not_kill_the_executor(srv, tmp_path):
    load(srv, tmp_path, "ea", np.zeros((2, 3), dtype=np.float32), "float32")
    load(srv, tmp_path, "eb", np.zeros((2, 3), dtype=np.int32), "int32")
    load(srv, tmp_path, "ec", np.zeros((4, 3), dtype=np.float32), "float32")
    assert srv.send("add", [T("ea"), T("eb", "int32")], [T("ea")]).message == "Type mismatch: float32 != int32 != float32"
    assert srv.send("add", [T("ea"), T("ec")], [T("ea")]).message.startswith("shape mismatch")
    assert srv.send("pow", [T("eb", "int32"), T("eb", "int32")], [T("eb", "int32")]).message == "Unsupported dtype for pow"
    assert srv.send("sum", [T("ea"), V([5]), "var<bool>:false"], [T("ea")]).message == "Dimension out of range in sum"
    assert srv.send("sum", [T("ea"), "vector<int32>:[]", "var<bool>:false"], [T("ea")]).result == "error"
    assert srv.send("sum", [T("ea"), V([1]), "var<bool>:maybe"], [T("ea")]).message == "Invalid bool value:maybe"
    assert srv.send("transpose", [T("ea"), V([0, 0])], [T("ea")]).result == "error"
    assert srv.send("broadcastTo", [T("ea"), V([5, 3])], [T("ec")]).message == "Broadcast shape mismatch"
    assert srv.send("matmul", [T("ea"), T("ea")], [T("ea")], author="cublas").message == "A[-1] must be equal to B[-2]"
    assert srv.send("load", ["var<string>:/nonexistent/t"], [], author="").result == "error"
    assert srv.send("greater", [T("ea"), T("ea")], [T("ea")]).result == "error"  # return must be tensor<bool>
    assert srv.proc.poll() is None


def test_config2_reductions_over_ir(srv, tmp_path):
    X = np.random.default_rng(3).standard_normal((256, 512)).astype(np.float32)
    P = np.random.default_rng(4).uniform(0.9, 1.1, (256, 64)).astype(np.float32)
    load(srv, tmp_path, "X", X, "float32")
    load(srv, tmp_path, "P", P, "float32")
    for keep in (True, False):
        kd = "True" if keep else "False"   # Python's str(bool), as the front sends it
        for op, axis, ref in [("sum", 1, X.astype(np.float64).sum(1)), ("sum", 0, X.astype(np.float64).sum(0)),
                              ("reducemax", 1, X.max(1)), ("reducemin", 1, X.min(1))]:
            oshape = ([256, 1] if axis == 1 else [1, 512]) if keep else ([256] if axis == 1 else [512])
            srv.must("newtensor", [V(oshape)], [T("red")], author="")
            srv.must(op, [T("X"), V([axis]), f"var<bool>:{kd}"], [T("red")])
            got, meta = fetch(srv, tmp_path, "red")
            assert meta["shape"] == oshape
            if op == "sum":
                assert np.allclose(got.reshape(-1), ref, rtol=0, atol=1e-5 * np.sqrt(512) * np.abs(X).max() * 4)
            else:
                assert np.array_equal(got.reshape(-1), ref)
            srv.must("deltensor", [], [T("red")], author="")
        oshape = [256, 1] if keep else [256]
        srv.must("newtensor", [V(oshape)], [T("pr")], author="")
        srv.must("prod", [T("P"), V([-1]), f"var<bool>:{kd}"], [T("pr")])
        assert np.allclose(fetch(srv, tmp_path, "pr")[0].reshape(-1), P.astype(np.float64).prod(1), rtol=1e-5)
        srv.must("deltensor", [], [T("pr")], author="")
    # all axes -> shape [1] (shape_reduce.cpp:68-72)
    srv.must("newtensor", [V([1])], [T("all")], author="")
    srv.must("sum", [T("X"), V([0, 1]), "var<bool>:false"], [T("all")])
    assert np.allclose(fetch(srv, tmp_path, "all")[0][0], X.astype(np.float64).sum(), atol=1e-2)
    # wrong output size is an error, not a fault
    assert srv.send("sum", [T("X"), V([0]), "var<bool>:false"], [T("all")]).message.startswith("Shape mismatch")


def test_config3_4_changeshape_over_ir(srv, tmp_path):
    rng = np.random.default_rng(5)
    t = rng.integers(0, 65536, size=(2, 64, 14, 64), dtype=np.uint16)
    load(srv, tmp_path, "t", t, "bfloat16")
    srv.must("newtensor", [V([2, 14, 64, 64])], [T("tt", "bfloat16")], author="")
    srv.must("transpose", [T("t", "bfloat16"), V([0, 2, 1, 3])], [T("tt", "bfloat16")])
    assert np.array_equal(fetch(srv, tmp_path, "tt")[0], t.transpose(0, 2, 1, 3))
    cs = [rng.integers(0, 65536, size=(4, 8 + i, 32), dtype=np.uint16) for i in range(3)]
    for i, c in enumerate(cs):
        load(srv, tmp_path, f"c{i}", c, "float16")
    srv.must("newtensor", [V([4, 27, 32])], [T("cc", "float16")], author="")
    srv.must("concat", ["listtensor<float16>:[c0 c1 c2]", "var<int32>:1"], [T("cc", "float16")])
    assert np.array_equal(fetch(srv, tmp_path, "cc")[0], np.concatenate(cs, axis=1))
    r = rng.integers(0, 65536, size=(1, 256), dtype=np.uint16)
    load(srv, tmp_path, "r", r, "bfloat16")
    srv.must("newtensor", [V([64, 256])], [T("rb", "bfloat16")], author="")
    srv.must("broadcastTo", [T("r", "bfloat16"), V([64, 256])], [T("rb", "bfloat16")])
    assert np.array_equal(fetch(srv, tmp_path, "rb")[0], np.broadcast_to(r, (64, 256)))
    # reshape: metadata of the output changes, data is copied
    srv.must("newtensor", [V([64 * 256])], [T("rs", "bfloat16")], author="")
    srv.must("reshape", [T("rb", "bfloat16"), V([128, 128])], [T("rs", "bfloat16")])
    got, meta = fetch(srv, tmp_path, "rs")
    assert meta["shape"] == [128, 128] and np.array_equal(got.reshape(-1), np.broadcast_to(r, (64, 256)).reshape(-1))
    # config 4: int32 max/min/greater/where(=switch) and the embedding gather, reduced size
    a = rng.integers(-2 ** 20, 2 ** 20, 100003).astype(np.int32)
    b = rng.integers(-2 ** 20, 2 ** 20, 100003).astype(np.int32)
    load(srv, tmp_path, "ia", a, "int32")
    load(srv, tmp_path, "ib", b, "int32")
    srv.must("newtensor", [V([100003])], [T("io", "int32")], author="")
    srv.must("newtensor", [V([100003])], [T("m", "bool")], author="")
    srv.must("max", [T("ia", "int32"), T("ib", "int32")], [T("io", "int32")])
    assert np.array_equal(fetch(srv, tmp_path, "io")[0], np.maximum(a, b))
    srv.must("min", [T("ia", "int32"), T("ib", "int32")], [T("io", "int32")])
    assert np.array_equal(fetch(srv, tmp_path, "io")[0], np.minimum(a, b))
    srv.must("greater", [T("ia", "int32"), T("ib", "int32")], [T("m", "bool")])
    assert np.array_equal(fetch(srv, tmp_path, "m")[0], (a > b).astype(np.uint8))
    srv.must("switch", ["listtensor<int32>:[ib ia]", T("m", "bool")], [T("io", "int32")])
    assert np.array_equal(fetch(srv, tmp_path, "io")[0], np.where(a > b, a, b))
    srv.must("invert", [T("m", "bool")], [T("m", "bool")])
    assert np.array_equal(fetch(srv, tmp_path, "m")[0], (~(a > b)).astype(np.uint8))
    E = rng.integers(0, 65536, size=(1000, 896), dtype=np.uint16)
    idx = rng.integers(0, 1000, size=(4, 16)).astype(np.int64)
    load(srv, tmp_path, "E", E, "bfloat16")
    load(srv, tmp_path, "idx", idx, "int64")
    srv.must("newtensor", [V([4, 16, 896])], [T("emb", "bfloat16")], author="")
    srv.must("indexselect", [T("E", "bfloat16"), T("idx", "int64"), "var<int32>:0"], [T("emb", "bfloat16")])
    assert np.array_equal(fetch(srv, tmp_path, "emb")[0], E[idx])
    srv.must("newtensor", [V([2000, 896 * 2])], [T("rep", "bfloat16")], author="")
    srv.must("repeat", [T("E", "bfloat16"), V([2, 2])], [T("rep", "bfloat16")])
    assert np.array_equal(fetch(srv, tmp_path, "rep")[0], np.repeat(np.repeat(E, 2, 0), 2, 1))


def test_config5_mlp_block_over_ir(srv, tmp_path):
    """Qwen2-0.5B-shaped MLP + RMSNorm block composed from deepxIR ops (reduced rows), bf16 storage,
    checked end to end against a float64 numpy model of the same op sequence; tolerance rel 1e-2 per
    op rounding (bf16), accumulated over the chain -> 3e-2 of the output scale."""
    rng = np.random.default_rng(14)
    S, Hd, I = 128, 896, 4864
    f2b, b2f = H.f32_to_bf16_bits, H.bf16_bits_to_f32
    x = f2b(rng.standard_normal((S, Hd)).astype(np.float32))
    w = f2b(np.ones(Hd, dtype=np.float32) + 0.1 * rng.standard_normal(Hd).astype(np.float32))
    Wg = f2b((rng.standard_normal((Hd, I)) * 0.02).astype(np.float32))
    Wu = f2b((rng.standard_normal((Hd, I)) * 0.02).astype(np.float32))
    Wd = f2b((rng.standard_normal((I, Hd)) * 0.02).astype(np.float32))
    for name, arr in [("q5_x", x), ("q5_w", w.reshape(1, Hd)), ("q5_Wg", Wg), ("q5_Wu", Wu), ("q5_Wd", Wd)]:
        load(srv, tmp_path, name, arr, "bfloat16")
    B16, F32 = "bfloat16", "float32"
    new = lambda name, shape, dt: srv.must("newtensor", [V(shape)], [T(name, dt)], author="")
    # RMSNorm in fp32 (front/py/deepx/nn/modules/norm/t5layernorm.py:17-22)
    new("q5_xf", [S, Hd], F32); srv.must("todtype", [T("q5_x", B16)], [T("q5_xf", F32)], author="")
    new("q5_sq", [S, Hd], F32); srv.must("powscalar", [T("q5_xf"), "var<float32>:2"], [T("q5_sq")])
    new("q5_var", [S, 1], F32); srv.must("sum", [T("q5_sq"), V([-1]), "var<bool>:True"], [T("q5_var")])
    srv.must("divscalar", [T("q5_var"), f"var<float32>:{Hd}"], [T("q5_var")])
    srv.must("addscalar", [T("q5_var"), "var<float32>:1e-06"], [T("q5_var")])
    srv.must("sqrt", [T("q5_var")], [T("q5_var")])
    srv.must("rdivscalar", ["var<float32>:1", T("q5_var")], [T("q5_var")])
    new("q5_rs", [S, Hd], F32); srv.must("broadcastTo", [T("q5_var"), V([S, Hd])], [T("q5_rs")])
    new("q5_xn", [S, Hd], F32); srv.must("mul", [T("q5_xf"), T("q5_rs")], [T("q5_xn")])
    new("q5_wf1", [1, Hd], F32); srv.must("todtype", [T("q5_w", B16)], [T("q5_wf1")], author="")
    new("q5_wf", [S, Hd], F32); srv.must("broadcastTo", [T("q5_wf1"), V([S, Hd])], [T("q5_wf")])
    srv.must("mul", [T("q5_wf"), T("q5_xn")], [T("q5_xn")])
    new("q5_h", [S, Hd], B16); srv.must("todtype", [T("q5_xn")], [T("q5_h", B16)], author="")
    # gated MLP (front/py/deepx/nn/modules/mlp/gatedmlp.py:20-26), SiLU = x * 1/(1+exp(-x)) (activite.py:11-18)
    new("q5_g", [S, I], B16); srv.must("matmul", [T("q5_h", B16), T("q5_Wg", B16)], [T("q5_g", B16)], author="cublas")
    new("q5_u", [S, I], B16); srv.must("matmul", [T("q5_h", B16), T("q5_Wu", B16)], [T("q5_u", B16)], author="cublas")
    new("q5_sg", [S, I], B16); srv.must("mulscalar", [T("q5_g", B16), "var<float32>:-1"], [T("q5_sg", B16)])
    srv.must("exp", [T("q5_sg", B16)], [T("q5_sg", B16)])
    srv.must("addscalar", [T("q5_sg", B16), "var<float32>:1"], [T("q5_sg", B16)])
    srv.must("rdivscalar", ["var<float32>:1", T("q5_sg", B16)], [T("q5_sg", B16)])
    srv.must("mul", [T("q5_g", B16), T("q5_sg", B16)], [T("q5_sg", B16)])
    srv.must("mul", [T("q5_sg", B16), T("q5_u", B16)], [T("q5_sg", B16)])
    new("q5_y", [S, Hd], B16); srv.must("matmul", [T("q5_sg", B16), T("q5_Wd", B16)], [T("q5_y", B16)], author="cublas")
    y = b2f(fetch(srv, tmp_path, "q5_y")[0]).astype(np.float64)
    # float64 model of the same graph, with bf16 rounding where the graph stores bf16
    rb = lambda a: b2f(f2b(a.astype(np.float32))).astype(np.float64)
    xf = b2f(x).astype(np.float64)
    xn = xf * (1.0 / np.sqrt((xf ** 2).sum(-1, keepdims=True) / Hd + 1e-6))
    h = rb(b2f(w).astype(np.float64) * xn)
    g = rb(h @ b2f(Wg).astype(np.float64)); u = rb(h @ b2f(Wu).astype(np.float64))
    act = rb(rb(g * rb(1.0 / rb(1.0 + rb(np.exp(rb(-g)))))) * u)
    yref = act @ b2f(Wd).astype(np.float64)
    assert np.abs(y - yref).max() <= 3e-2 * np.abs(yref).max()
    # element by element: within 1e-2 of the magnitude that went into each output
    ymag = np.abs(act) @ np.abs(b2f(Wd).astype(np.float64))
    assert np.all(np.abs(y - yref) <= 1e-2 * ymag), float(np.max(np.abs(y - yref) / ymag))
    hg = b2f(fetch(srv, tmp_path, "q5_h")[0]).astype(np.float64)
    assert np.abs(hg - h).max() <= 1e-2 * np.abs(h).max()
    assert np.all(np.abs(hg - h) <= 1e-2 * np.abs(h) + 1e-30)


def test_benchmark_repeat_and_timestamps(srv, tmp_path):
    load(srv, tmp_path, "ba", np.ones((256, 256), dtype=np.float32), "float32")
    r = srv.must("add", [T("ba"), T("ba")], [T("ba")], extra="benchmark.repeat=3")
    assert np.all(fetch(srv, tmp_path, "ba")[0] == 8.0)  # 1 -> 2 -> 4 -> 8
    assert r.times["recv_at"] <= r.times["start_at"] <= r.times["finish_at"]


def test_waiting_for_the_device_before_each_reply(tmp_path):
    """DEEPX_SYNC=1: every reply is sent after the kernels of its line have finished (the default
    replies at launch, as op-cuda does).  Same results either way; with the wait, finish_at of a
    long op lies after its start_at by at least the kernel's run time."""
    rng = np.random.default_rng(5)
    a = rng.uniform(-1, 1, (512, 512)).astype(np.float32)
    want = None
    for env in ({"DEEPX_SYNC": "1"}, {}):
        s = UdpExecutor(env=env)
        try:
            load(s, tmp_path, "sy_a", a, "float32")
            s.must("newtensor", [V([512, 512])], [T("sy_c")], author="")
            s.must("matmul", [T("sy_a"), T("sy_a")], [T("sy_c")], author="cublas")
            s.must("exp", [T("sy_c")], [T("sy_c")])
            got = fetch(s, tmp_path, "sy_c")[0]
        finally:
            s.close()
        assert s.proc.returncode == 0
        if want is None:
            want = got
            ref = np.exp(a.astype(np.float64) @ a.astype(np.float64))
            assert np.allclose(got, ref, rtol=1e-4)
        else:
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
