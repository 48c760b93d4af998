"""Heap-tensor store (the reference's heapmem: one hash per tensor, a list of JSON lifecycle
commands — executor/heapmem-cuda/README.md:13-34): control plane on the CPU, with host-backed
allocations; first on the in-process key-value backend, then through the store's own RESP client
against a stand-in Redis server over TCP."""
import json
import os
import subprocess
import sys

import pytest

from tests.heapmem_client import FakeRedis, HeapStore, RespClient

FIELDS = ["dtype", "shape", "ctime", "node", "device", "bytes", "ipc_handle", "refcount", "owner_pid", "state"]


def cmd(op, name, **kw):
    return json.dumps(dict({"op": op, "name": name}, **kw))


@pytest.fixture(params=["memory", "resp"])
def store(request):
    server = None
    if request.param == "memory":
        s = HeapStore("memory", "host")
    else:
        server = FakeRedis()
        s = HeapStore(f"127.0.0.1:{server.port}", "host")
    yield s
    s.close()
    if server:
        server.close()


def test_create_get_delete_refcounts(store):
    # the README's own example command: shape as a JSON array, short dtype name
    assert store.command('{"op":"create", "name":"X", "dtype":"f32", "shape":[2,3], "device":0, "pid":123, "node":"n1"}') == 1
    m = store.meta("X")
    assert list(m) == FIELDS
    assert m["dtype"] == "f32" and m["shape"] == "[2,3]" and m["bytes"] == "24" and m["node"] == "n1" and m["device"] == "0"
    assert m["refcount"] == "1" and m["state"] == "ready" and int(m["owner_pid"]) == os.getpid() and int(m["ctime"]) > 0
    assert len(m["ipc_handle"]) == 128 and store.pointer("X") != 0 and store.owned() == 1
    assert store.command(cmd("get", "X", pid=7)) == 1 and store.meta("X")["refcount"] == "2"
    assert store.command(cmd("create", "X", dtype="f32", shape=[2, 3], node="n1")) == 1   # create of a known name = one more reference
    assert store.meta("X")["refcount"] == "3" and store.owned() == 1
    for left in ("2", "1"):
        assert store.command(cmd("delete", "X")) == 1 and store.meta("X")["refcount"] == left
    assert store.command(cmd("delete", "X")) == 1
    assert store.meta("X") is None and store.pointer("X") == 0 and store.owned() == 0


def test_sizes_and_shape_spellings(store):
    cases = [("float64", "[4]", 32), ("bfloat16", "[2, 3, 4]", 48), ("int8", "[5 7]", 35), ("bool", "[]", 1), ("i64", "[3,1]", 24),
             ("float16", "[0,8]", 0)]
    for i, (dt, shape, nbytes) in enumerate(cases):
        raw = '{"op":"create","name":"t%d","dtype":"%s","shape":"%s","node":"n"}' % (i, dt, shape)
        assert store.command(raw) == 1, store.last_error()
        assert store.meta("t%d" % i)["bytes"] == str(nbytes)
    assert store.owned() == len(cases)


def test_bad_commands_are_reported_not_fatal(store):
    assert store.command(cmd("create", "bad", dtype="complex64", shape=[2])) == -1 and "unknown dtype" in store.last_error()
    assert store.command(cmd("create", "bad", dtype="f32", shape="[2,x]")) == -1 and "malformed shape" in store.last_error()
    assert store.command(cmd("get", "nope")) == -1 and store.last_error() == "tensor not found: nope"
    assert store.command(cmd("delete", "nope")) == -1
    assert store.command(cmd("frobnicate", "x")) == -1 and "unknown op" in store.last_error()
    assert store.command("not json at all") == -1 and "malformed command" in store.last_error()
    assert store.run_once(0) == 0                      # nothing queued
    assert store.command(cmd("create", "ok", dtype="f32", shape=[1], node="n")) == 1
    assert store.meta("bad") is None and store.owned() == 1


def test_create_refuses_what_cannot_be_shared(store):
    """A shared allocation stays under 2 GiB (larger IPC handles do not open), and a shape whose
    element count overflows is refused instead of wrapping into a small or huge request."""
    assert store.command(cmd("create", "big", dtype="f32", shape=[1 << 29], node="n")) == -1 and "too large" in store.last_error()
    assert store.command(cmd("create", "big", dtype="int8", shape=[1 << 31], node="n")) == -1 and "too large" in store.last_error()
    assert store.command(cmd("create", "big", dtype="f64", shape=[1 << 20, 1 << 20, 1 << 20, 1 << 20], node="n")) == -1 and "too large" in store.last_error()
    assert store.command('{"op":"create","name":"big","dtype":"f32","shape":"[99999999999999999999999]","node":"n"}') == -1
    assert "too large" in store.last_error()
    assert store.meta("big") is None and store.owned() == 0
    assert store.command(cmd("create", "empty", dtype="f32", shape=[1 << 40, 0], node="n")) == 1   # empty whatever the other extent says
    assert store.meta("empty")["bytes"] == "0"
    assert store.command(cmd("create", "edge", dtype="int8", shape=[4096], node="n")) == 1 and store.owned() == 2


def test_sweep_keeps_referenced_tensors_of_live_owners(store):
    for name in ("a", "b"):
        assert store.command(cmd("create", name, dtype="f32", shape=[8], node="here")) == 1
    assert store.command(cmd("create", "c", dtype="f32", shape=[8], node="elsewhere")) == 1
    assert store.sweep("here") == 0 and store.owned() == 3      # all referenced, owner alive
    assert store.sweep("nowhere") == 0


def test_compute_process_view_over_resp():
    """A compute process never links the store: it pushes JSON on the list and reads the hash with
    plain Redis commands.  Also: tensors whose owner died are swept."""
    server = FakeRedis()
    store = HeapStore(f"127.0.0.1:{server.port}", "host")
    client = RespClient(server.port)
    try:
        assert client.call("PING") == "PONG"
        assert client.call("LPUSH", "tensor_lifecycle", cmd("create", "W", dtype="bf16", shape=[4, 4], device=0, pid=1, node="n1")) == 1
        assert store.run_once(2) == 1
        flat = client.call("HGETALL", "tensor:W")
        h = dict(zip(flat[::2], flat[1::2]))
        assert h[b"dtype"] == b"bf16" and h[b"bytes"] == b"32" and h[b"refcount"] == b"1" and h[b"state"] == b"ready"
        assert client.call("LPUSH", "tensor_lifecycle", cmd("get", "W", pid=2)) == 1
        assert store.run_once(2) == 1 and client.call("HGETALL", "tensor:W")[flat.index(b"refcount") + 1] in (b"2",)
        # an entry left behind by a process that no longer exists
        dead = subprocess.Popen([sys.executable, "-c", "pass"])
        dead.wait()
        client.call("HSET", "tensor:orphan", "node", "n1", "refcount", "1", "owner_pid", str(dead.pid), "bytes", "0", "state", "ready")
        client.call("HSET", "tensor:other_node", "node", "n2", "refcount", "0", "owner_pid", "1")
        assert store.sweep("n1") == 1
        assert client.call("HGETALL", "tensor:orphan") == [] and client.call("HGETALL", "tensor:other_node") != []
        assert store.meta("W")["refcount"] == "2"
    finally:
        client.close()
        store.close()
        server.close()
