"""The drop-in boundary without a GPU: deepxIR grammar, dtype vocabulary, op matching, the op table
against the reference's generated lists, tensor-file metadata, and error replies over real UDP."""
import json
import os
import re

import pytest
import yaml

from tests.executor_client import InProc, UdpExecutor

GOLD = os.path.join(os.path.dirname(__file__), "golden")


@pytest.fixture(scope="module")
def ex():
    return InProc()


# ---- dtype vocabulary ------------------------------------------------------------------------
def test_typedef_table_from_reference_test(ex):
    g = json.load(open(os.path.join(GOLD, "dtype_table.json")))
    for text, cat, prec in g["rows"]:
        back, cbits, pbits = ex.typedef(text).split(" ")
        assert int(cbits) == g["category_bits"][cat], text
        assert int(pbits) == g["precision_bits"][prec], text
        want = f"{cat}<{prec}>" if prec not in ("int",) else None
        if want:
            assert back == want, (text, back)
    # a union is not wire syntax: like the reference's precision() it reads as "any"
    assert ex.typedef("tensor<float64|float32>").split(" ")[0] == "tensor<any>"
    assert ex.typedef("tensor<int>").split(" ")[0] == "tensor<int64|int32|int16|int8|int4>"
    assert ex.typedef("listtensor<any>").split(" ")[:2] == ["listtensor<any>", "8"]
    assert ex.typedef("frob").split(" ")[1:] == ["0", "65535"]  # unknown category, precision any


# ---- grammar ---------------------------------------------------------------------------------
def test_parse_front_format(ex):
    # exactly what str(DeepxIR) produces: spaces around parens/arrow, double spaces in metadata
    line = "add (tensor<float32>:a, tensor<float32>:b) -> (tensor<float32>:c) // author=miaobyte  id=7  created_at=1744724799.0650852  sent_at=1744724799.0650952"
    out = ex.parse(line)
    assert out.startswith("add(tensor<float32>:a, tensor<float32>:b)->(tensor<float32>:c) //author=miaobyte id=7 ")
    assert "created_at=1744724799000" in out and "sent_at=1744724799000" in out
    # vectors, bools, strings, list of tensors, negative numbers
    out = ex.parse("sum(tensor<float32>:x, vector<int32>:[0 -1], var<bool>:True)->(tensor<float32>:y) // id=1")
    assert out.startswith("sum(tensor<float32>:x, vector<int32>:[0 -1], var<bool>:True)->(tensor<float32>:y)")
    out = ex.parse("concat(listtensor<float16>:[a b c], var<int32>:1)->(tensor<float16>:r)")
    assert out.startswith("concat(listtensor<float16>:[a b c], var<int32>:1)->(tensor<float16>:r)")
    out = ex.parse("save(tensor<any>:t, var<string>:/tmp/x/y)->()")
    assert out.startswith("save(tensor<any>:t, var<string>:/tmp/x/y)->()")
    # untyped params: category unknown, precision any
    assert ex.parse("add(a, b)->(c)").startswith("add(unknown<any>:a, unknown<any>:b)->(unknown<any>:c)")
    # the name may be followed by a space instead of '('
    assert ex.parse("newtensor (vector<int32>:[3 4 5]) -> (tensor<float32>:t1)").startswith("newtensor(vector<int32>:[3 4 5])->(tensor<float32>:t1)")
    assert ex.parse("deltensor()->(tensor<any>:t) // benchmark.repeat=3 id=2").endswith("id=2 benchmark.repeat=3 ")
    assert ex.parse("no arrow here") == "error: Invalid IR format: missing arrow"


# ---- matching --------------------------------------------------------------------------------
def test_matching_rules(ex):
    assert ex.match("add(tensor<float32>:a, tensor<float32>:b)->(tensor<float32>:c) // author=miaobyte").startswith("miaobyte|add(")
    # unknown author falls back to the first registered author
    assert ex.match("add(tensor<float32>:a, tensor<float32>:b)->(tensor<float32>:c) // author=nobody").startswith("miaobyte|add(")
    assert ex.match("matmul(tensor<bfloat16>:a, tensor<bfloat16>:b)->(tensor<bfloat16>:c) // author=cublas").startswith("cublas|matmul(")
    assert ex.match("matmul(tensor<float32>:a, tensor<float32>:b)->(tensor<float32>:c) // author=cblas").startswith("cblas|matmul(")
    # arity and category must fit
    assert ex.match("add(tensor<float32>:a)->(tensor<float32>:c)").startswith("none")
    assert ex.match("add(var<float32>:1, tensor<float32>:b)->(tensor<float32>:c)").startswith("none")
    # precision subset: invert is registered for ints and bool only
    assert ex.match("invert(tensor<int32>:a)->(tensor<int32>:c)").startswith("miaobyte|invert(")
    assert ex.match("invert(tensor<float32>:a)->(tensor<float32>:c)").startswith("none")
    assert ex.match("greater(tensor<int32>:a, tensor<int32>:b)->(tensor<bool>:m)").startswith("miaobyte|greater(")
    assert ex.match("greater(tensor<int32>:a, tensor<int32>:b)->(tensor<int32>:m)").startswith("none")
    assert ex.match("switch(listtensor<int32>:[b a], tensor<bool>:m)->(tensor<int32>:w)").startswith("miaobyte|switch(")
    # newtensor has two signatures: vector<int32> shape or var<string>
    assert "vector<int32>:shape" in ex.match("newtensor(vector<int32>:[2 3])->(tensor<float32>:t)")
    assert "var<string>:shape" in ex.match("newtensor(var<string>:s)->(tensor<float32>:t)")
    assert ex.match("frobnicate(tensor<float32>:a)->(tensor<float32>:c)").startswith("none: <op> frobnicate not found")


def rows_of(md):
    rows, sect = [], None
    for ln in md.splitlines():
        if ln.startswith("### "):
            sect = ln[4:].strip()
        elif ln.startswith("| ") and not ln.startswith("| Operation"):
            parts = [x.strip() for x in ln.strip()[1:-1].split(" | ")]
            rows.append({"tftype": sect, "name": parts[0], "author": parts[1], "formula": parts[2], "ir": " | ".join(parts[3:]).strip()})
    return rows


def sig_shape(ir):
    """(op, [arg categories], [return categories]) of an IR signature string"""
    name = ir[:ir.index("(")]
    a, r = ir[ir.index("(") + 1:].split(")->(")
    cats = lambda s: [p.strip().split("<")[0] for p in s.rstrip(")").split(", ") if p.strip()]
    return name, cats(a), cats(r)


@pytest.mark.parametrize("ref", ["op-mem-cuda", "op-mem-ompsimd"])
def test_op_table_covers_reference_lists(ex, ref):
    """Every row of the reference's generated op list has a registered op here with the same name,
    tftype, arity and parameter categories; every call the reference row accepts resolves."""
    gold = json.load(open(os.path.join(GOLD, f"op_table_{ref}.json")))["rows"]
    mine = rows_of(ex.op_table())
    assert mine[0].keys() == gold[0].keys()
    by_name = {}
    for r in mine:
        by_name.setdefault(r["name"], []).append(r)
    for g in gold:
        assert g["name"] in by_name, g["name"]
        cands = by_name[g["name"]]
        assert any(c["tftype"] == g["tftype"] for c in cands), g
        assert any(sig_shape(c["ir"])[1:] == sig_shape(g["ir"])[1:] for c in cands), (g["ir"], [c["ir"] for c in cands])
        # a concrete call built from the reference signature (first precision of each union) resolves
        call = re.sub(r"<([a-z0-9]+)\|[^>]*>", r"<\1>", g["ir"]).replace("<any>", "<float32>").replace("listtensor<float32>", "listtensor<float32>")
        author = g["author"] if g["author"] != "none" else ""
        assert not ex.match(call + (f" // author={author}" if author else "")).startswith("none"), call


def test_op_table_markdown_layout(ex):
    md = ex.op_table("op-mem-hip")
    assert md.startswith("## op-mem-hip 支持算子列表 \n\n本页面由 `executor/op-mem-hip 生成，请勿手动修改 \n\n### ")
    assert "| Operation | Author |  Math Formula | IR Instruction |\n|-----------|--------|--------------|----------------|\n" in md
    assert "| add | miaobyte | T3=T1+T2 | add(tensor<any>:a, tensor<any>:b)->(tensor<any>:c) |" in md
    assert "| deltensor |  none  | del->T1 | deltensor()->(tensor<any>:t) |" in md


# ---- tensor metadata ---------------------------------------------------------------------------
def test_shape_yaml_is_the_reference_layout(ex):
    text = "dtype: float32\ndim: 3\nshape: [2, 3, 4]\nstride: [12, 4, 1]\nsize: 24\n"  # PyYAML flow style
    out = ex.shape_yaml(text)
    assert yaml.safe_load(out) == {"dtype": "float32", "dim": 3, "shape": [2, 3, 4], "stride": [12, 4, 1], "size": 24}
    assert list(yaml.safe_load(out).keys()) == ["dtype", "dim", "shape", "stride", "size"]
    block = "dtype: bfloat16\ndim: 2\nshape:\n  - 5\n  - 7\nstride:\n  - 7\n  - 1\nsize: 35\n"  # yaml-cpp block style
    assert yaml.safe_load(ex.shape_yaml(block)) == {"dtype": "bfloat16", "dim": 2, "shape": [5, 7], "stride": [7, 1], "size": 35}
    assert ex.shape_yaml("dtype: float32\ndim: 2\nshape: [2, 3]\nstride: [1, 2]\nsize: 6\n") == "error: Shape::fromYaml: strides mismatch"
    assert ex.shape_yaml("dtype: float32\ndim: 2\nshape: [2, 3]\nstride: [3, 1]\nsize: 7\n") == "error: Shape::fromYaml: size mismatch"


# ---- replies -----------------------------------------------------------------------------------
def test_inproc_error_replies(ex):
    r = ex.execute("frobnicate(tensor<float32>:a)->(tensor<float32>:c) // id=3")
    assert re.fullmatch(r"3 error// recv_at=\d+ start_at=\d+ finish_at=\d+ opfrobnicate not found", r), r
    assert ex.execute("garbage").endswith("Invalid IR format: missing arrow")
    assert ex.execute("add(tensor<float32>:a, tensor<float32>:b)->(tensor<float32>:c) // id=4").endswith("tensor not found: a")
    assert re.fullmatch(r"6 ok// recv_at=\d+ start_at=\d+ finish_at=\d+", ex.execute("argset(var<int32>:5)->(var<int32>:n) // id=6"))
    assert ex.execute("vecset(vector<int32>:[1 2 3])->(vector<int32>:v) // id=7").startswith("7 ok//")
    assert ex.execute("argset(var<int32>:5)->(tensor<int32>:n) // id=8").startswith("8 error//")
    assert "id" not in ex.execute("sum(tensor<float32>:x, vector<int32>:[], var<bool>:false)->(tensor<float32>:y) // id=x9")[:4]  # bad id is an error reply, not a crash


def test_print_format_from_the_wire_is_validated(ex):
    """`print(t, format)` hands its format to snprintf with one value: exactly one conversion of the
    value's kind is accepted; %n, %s, '*', several conversions or none are refused (an error reply)."""
    for fmt in ["%f", "%.4f", "%8.3e", "%g", "%-10.2F", "%+.1f", "x=%f;", "%lf", "100%% %f"]:
        assert ex.print_format_ok(fmt, True), fmt
    for fmt in ["%d", "%5d", "%x", "%lld", "%ld", "%hhd", "%08X", "%i", "%u", "[%o]"]:
        assert ex.print_format_ok(fmt, False), fmt
    for fmt in ["%s", "%n", "%f%f", "%*d", "%.*f", "%d %d", "", "plain", "%", "%5", "%c", "%p", "%f%n", "%ls", "%Lf", "%" + "9" * 80 + "f"]:
        assert not ex.print_format_ok(fmt, True), fmt
        assert not ex.print_format_ok(fmt, False), fmt
    assert not ex.print_format_ok("%d", True) and not ex.print_format_ok("%f", False)


def test_udp_server_error_paths_and_framing():
    srv = UdpExecutor()
    try:
        r = srv.send("frobnicate", ["tensor<float32>:a"], ["tensor<float32>:c"])
        assert r.result == "error" and r.message == "opfrobnicate not found"
        assert set(r.times) == {"recv_at", "start_at", "finish_at"} and r.times["recv_at"] <= r.times["finish_at"]
        r = srv.send("add", ["tensor<float32>:a", "tensor<float32>:b"], ["tensor<float32>:c"])
        assert r.result == "error" and r.message == "tensor not found: a"
        assert srv.send("argset", ["var<float32>:0.5"], ["var<float32>:half"], author="").ok
        # several newline-separated instructions in one datagram: one reply each, in order
        rs = srv.raw("argset(var<int32>:1)->(var<int32>:a) // id=101\nargset(var<int32>:2)->(var<int32>:b) // id=102\n\nbogus // id=103", 3)
        assert [x.id for x in rs] == ["101", "102", "0"] and [x.result for x in rs] == ["ok", "ok", "error"]
        # a datagram longer than the reference's 1024-byte buffer is handled, not overflowed
        long_name = "n" * 3000
        r = srv.raw(f"argset(var<int32>:7)->(var<int32>:{long_name}) // id=104")[0]
        assert r.id == "104" and r.ok
        # the process survived all of it
        assert srv.proc.poll() is None
        assert srv.send("argset", ["var<int32>:3"], ["var<int32>:still_alive"], author="").ok
    finally:
        srv.close()
    assert srv.proc.returncode == 0


def test_inproc_batch_replies_in_order(ex):
    """A datagram's lines as one batch: one reply per line, in order, each line failing or
    succeeding on its own (same replies as when the lines are sent one by one)."""
    lines = ["argset(var<int32>:1)->(var<int32>:ba) // id=201", "frobnicate(tensor<float32>:a)->(tensor<float32>:c) // id=202",
             "garbage", "add(tensor<float32>:nope, tensor<float32>:b)->(tensor<float32>:c) // id=204",
             "vecset(vector<int32>:[4 5])->(vector<int32>:bv) // id=205"]
    before = ex.stats()["batches"]
    rs = ex.execute_batch(lines)
    assert len(rs) == 5
    assert rs[0].startswith("201 ok//") and rs[4].startswith("205 ok//")
    assert rs[1].startswith("202 error//") and rs[1].endswith("opfrobnicate not found")
    assert rs[2].endswith("Invalid IR format: missing arrow")
    assert rs[3].startswith("204 error//") and rs[3].endswith("tensor not found: nope")
    assert ex.stats()["batches"] == before + 1
    # a batch of one line is the plain path
    assert ex.execute_batch(["argset(var<int32>:9)->(var<int32>:bz) // id=206"])[0].startswith("206 ok//")
    assert ex.stats()["batches"] == before + 1


def test_mutated_instructions_never_take_the_process_down(ex):
    """Seeded mutations (deletions, insertions, substitutions of separator and digit characters) of
    valid instructions and short random strings: every one gets a reply line and the process lives
    (the reference unwinds out of its receiver thread on the first malformed line)."""
    import random
    rng = random.Random(1234)
    seeds = ["add(tensor<float32>:a, tensor<float32>:b)->(tensor<float32>:c) // author=miaobyte id=1 created_at=1.5 sent_at=2.5",
             "sum(tensor<float32>:x, vector<int32>:[0 1], var<bool>:true)->(tensor<float32>:y) // id=2",
             "argset(var<int32>:5)->(var<int32>:n) // id=4", "vecset(vector<int32>:[1 2 3])->(vector<int32>:v) // id=5",
             "concat(listtensor<float32>:[a b c], var<int32>:1)->(tensor<float32>:o) // id=6",
             "transpose(tensor<any>:a, vector<int32>:[1 0])->(tensor<any>:b) // benchmark.repeat=3 id=7",
             "load(var<string>:/nonexistent/path)->() // id=8", "print(tensor<any>:zzz, var<string>:%f)->() // id=9"]
    alphabet = "()<>[],:->/= \t|abcxyz0123456789.-+eE%\"'\\"
    for _ in range(3000):
        if rng.randrange(4) == 0:
            s = "".join(rng.choice(alphabet) for _ in range(rng.randrange(0, 80)))
        else:
            chars = list(rng.choice(seeds))
            for _ in range(rng.randrange(1, 6)):
                pos = rng.randrange(len(chars)) if chars else 0
                kind = rng.randrange(3)
                if kind == 0 and chars:
                    del chars[pos]
                elif kind == 1:
                    chars.insert(pos, rng.choice(alphabet))
                elif chars:
                    chars[pos] = rng.choice(alphabet)
            s = "".join(chars)
        reply = ex.execute(s)
        assert " ok//" in reply or " error//" in reply, (s, reply)
    assert ex.execute("argset(var<int32>:1)->(var<int32>:alive) // id=99").startswith("99 ok//")
