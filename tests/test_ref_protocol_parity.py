"""The executor's protocol layer against the REFERENCE's own code (oracle/_ref/libdeepxref.so, built
by oracle/ref.mk from deepxcore's tf.cpp / tffactory.cpp / dtype.hpp / shape_*.cpp): identical parse
results, dtype strings, match decisions and inferred shapes on hand-written and generated inputs.
Skipped where the reference build is absent (it needs the reference checkout at build time)."""
import itertools
import os
import random

import pytest

from tests.executor_client import REF_SO, InProc, Reference

pytestmark = pytest.mark.skipif(not os.path.exists(REF_SO), reason="oracle/_ref not built (make -C oracle -f ref.mk)")


@pytest.fixture(scope="module")
def ref():
    return Reference()


@pytest.fixture(scope="module")
def ex():
    return InProc()


PRECISIONS = ["float64", "float32", "float16", "bfloat16", "float8e5m2", "float8e4m3", "float4e2m1", "int64", "int32",
              "int16", "int8", "int4", "bool", "string", "any", "int", "float", "float8", "nonsense"]
CATEGORIES = ["tensor", "vector", "var", "listtensor", "tensor|var", "var|vector", "bogus"]


def test_typedef_strings_and_bits(ref, ex):
    for c, p in itertools.product(CATEGORIES, PRECISIONS):
        for text in (f"{c}<{p}>", c):
            assert ex.typedef(text) == ref.typedef(text), text
    for text in ["", "<float32>", "tensor<", "tensor>float32<", "tensor<float32", "tensor<>"]:
        assert ex.typedef(text) == ref.typedef(text), text


LINES = [
    "add(tensor<float32>:a, tensor<float32>:b)->(tensor<float32>:c) // author=miaobyte id=7 created_at=1744724799.0650852 sent_at=1744724799.0650952",
    "add (tensor<float32>:a, tensor<float32>:b) -> (tensor<float32>:c) // author=miaobyte  id=7  created_at=1744724799.0650852  sent_at=1744724799.0650952",
    "newtensor ( [3 4 5]) -> ( tensor_136144420556608) // id=1 created_at=1744724799.0650852 sent_at=1744724799.0650952",
    "newtensor (vector<int32>:[3 4 5]) -> (tensor<float32>:tensor_1) // id=1",
    "sum(tensor<float32>:x, vector<int32>:[0 -1], var<bool>:True)->(tensor<float32>:y)",
    "concat(listtensor<float16>:[a b c], var<int32>:1)->(tensor<float16>:r) // author=miaobyte",
    "save(tensor<any>:t, var<string>:/tmp/x:y/z)->()",
    "print(tensor<any>:t, var<string>:%.2f)->() // id=12 benchmark.repeat=4",
    "deltensor()->(tensor<any>:t)",
    "add(a, b)->(c)",
    "add a, b -> c",
    "argset(var<int32>:5)->(var<int32>:n)//id=3",
    "matmul(tensor<float64|float32>:A, tensor<float64|float32>:B)->(tensor<float64|float32>:C)",
    "x()->()",
    "  lead(tensor:a)->(tensor:b)",
    "op(tensor<float32>: spaced , var<int32>:  7 )->( tensor<float32>:out ) // junk noequals id=9 author=",
    "rsubscalar(var<float32>:1.5, tensor<float32>:0)->(tensor<float32>:1) // author=miaobyte id=2 recv_at=5",
    "no arrow at all",
    "",
]


def test_parse_and_print_identical(ref, ex):
    for line in LINES:
        assert ex.parse(line) == ref.parse(line), line


def test_parse_generated_lines(ref, ex):
    rnd = random.Random(1234)
    names = ["a", "t1", "tensor_99", "0", "w.x", "q5_Wg"]
    def param():
        kind = rnd.choice(["typed", "bare", "vec", "list", "num"])
        if kind == "typed":
            return f"{rnd.choice(CATEGORIES[:4])}<{rnd.choice(PRECISIONS[:15])}>:{rnd.choice(names)}"
        if kind == "bare":
            return rnd.choice(names)
        if kind == "vec":
            return "vector<int32>:[" + " ".join(str(rnd.randint(-3, 9)) for _ in range(rnd.randint(1, 4))) + "]"
        if kind == "list":
            return "listtensor<float32>:[" + " ".join(rnd.choice(names) for _ in range(rnd.randint(1, 3))) + "]"
        return f"var<float32>:{rnd.uniform(-5, 5):.3f}"
    for _ in range(400):
        args = ", ".join(param() for _ in range(rnd.randint(0, 4)))
        rets = ", ".join(param() for _ in range(rnd.randint(0, 2)))
        sep = rnd.choice(["", " "])
        meta = rnd.choice(["", f" // id={rnd.randint(1, 999)}", f" // author=miaobyte id={rnd.randint(1, 99)} created_at=17447247{rnd.randint(10, 99)}.5",
                           f" //benchmark.repeat={rnd.randint(1, 5)} id={rnd.randint(1, 9)}"])
        line = f"op{rnd.randint(0, 9)}{sep}({args}){sep}->{sep}({rets}){meta}"
        assert ex.parse(line) == ref.parse(line), line


def test_match_decisions_identical(ref, ex):
    """Feed the reference factory the same registrations this executor prints in its op table, then
    compare which signature each call resolves to."""
    rows = []
    for ln in ex.op_table().splitlines():
        if ln.startswith("| ") and not ln.startswith("| Operation"):
            parts = [x.strip() for x in ln.strip()[1:-1].split(" | ")]
            author = "" if parts[1] == "none" else parts[1]
            rows.append(f"{author}|{' | '.join(parts[3:]).strip()}")
    calls = [
        "add(tensor<float32>:a, tensor<float32>:b)->(tensor<float32>:c) // author=miaobyte",
        "add(tensor<float32>:a, tensor<float32>:b)->(tensor<float32>:c) // author=cublas",
        "add(tensor<float32>:a)->(tensor<float32>:c) // author=miaobyte",
        "add(var<float32>:1, tensor<float32>:b)->(tensor<float32>:c) // author=miaobyte",
        "add(a, b)->(c) // author=miaobyte",
        "invert(tensor<int32>:a)->(tensor<int32>:c) // author=miaobyte",
        "invert(tensor<float32>:a)->(tensor<float32>:c) // author=miaobyte",
        "invert(tensor<int>:a)->(tensor<int>:c) // author=miaobyte",
        "greater(tensor<int32>:a, tensor<int32>:b)->(tensor<bool>:m) // author=miaobyte",
        "greater(tensor<int32>:a, tensor<int32>:b)->(tensor<int32>:m) // author=miaobyte",
        "switch(listtensor<int32>:[b a], tensor<bool>:m)->(tensor<int32>:w) // author=miaobyte",
        "switch(listtensor<int32>:[b a], tensor<float32>:m)->(tensor<int32>:w) // author=miaobyte",
        "newtensor(vector<int32>:[2 3])->(tensor<float32>:t)",
        "newtensor(var<string>:s)->(tensor<float32>:t)",
        "newtensor(vector<int64>:[2 3])->(tensor<float32>:t)",
        "matmul(tensor<bfloat16>:a, tensor<bfloat16>:b)->(tensor<bfloat16>:c) // author=cublas",
        "matmul(tensor<bfloat16>:a, tensor<bfloat16>:b)->(tensor<bfloat16>:c) // author=miaobyte",
        "sum(tensor<float32>:x, vector<int32>:[0], var<bool>:true)->(tensor<float32>:y) // author=miaobyte",
        "sum(tensor<float32>:x, vector<float32>:[0], var<bool>:true)->(tensor<float32>:y) // author=miaobyte",
        "indexselect(tensor<bfloat16>:E, tensor<int64>:i, var<int32>:0)->(tensor<bfloat16>:o) // author=miaobyte",
        "indexselect(tensor<bfloat16>:E, tensor<int16>:i, var<int32>:0)->(tensor<bfloat16>:o) // author=miaobyte",
        "frobnicate(tensor<float32>:a)->(tensor<float32>:c)",
        "uniform(var<float32>:0, var<float32>:1, var<int32>:3)->(tensor<float32>:t) // author=miaobyte",
        "uniform(var<float32>:0, var<float32>:1, var<float32>:3)->(tensor<float32>:t) // author=miaobyte",
    ]
    for call in calls:
        want = ref.match(rows, call)
        got = ex.match(call)
        if want == "none":
            assert got.startswith("none"), (call, got)
        else:
            assert got.split("|", 1)[1] == want, (call, got, want)


def test_shape_inference_identical(ref, ex):
    rnd = random.Random(99)
    for _ in range(300):
        nd = rnd.randint(1, 5)
        shape = [rnd.randint(1, 6) for _ in range(nd)]
        order = list(range(nd))
        rnd.shuffle(order)
        assert ex.infer("transpose", shape, order) == ref.transpose_shape(shape, order)
        other = [rnd.choice([1, s]) for s in shape[rnd.randint(0, nd - 1):]]
        assert ex.infer("broadcast", shape, other) == ref.broadcast_shape(shape, other)
        bad = [s + 1 if s > 1 else s for s in shape]
        assert ex.infer("broadcast", shape, bad) == ref.broadcast_shape(shape, bad)
        idx = [rnd.randint(1, 4) for _ in range(rnd.randint(1, 3))]
        axis = rnd.randint(0, nd - 1)
        assert ex.infer("indexselect", shape, idx, axis) == ref.indexselect_shape(shape, idx, axis)
        reps = [rnd.randint(1, 3) for _ in range(nd)]
        assert ex.infer("repeat", shape, reps) == ref.repeat_shape(shape, reps)
        dims = [rnd.randint(-nd, nd - 1) for _ in range(rnd.randint(0, nd))]
        cd = ref.checked_dims(shape, dims)
        assert ex.infer("checked_dims", shape, dims) == cd
        checked = [int(x) for x in cd.split()] if cd else []
        for keep in (0, 1):
            assert ex.infer("reduced", shape, checked, keep) == ref.reduced_shape(shape, checked, keep)
    assert ex.infer("checked_dims", [2, 3], [2]).startswith("error") and ref.checked_dims([2, 3], [2]).startswith("error")
    assert ex.infer("repeat", [2, 3], [2]).startswith("error") and ref.repeat_shape([2, 3], [2]).startswith("error")
