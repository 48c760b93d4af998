"""GPU: heap tensors in device memory.  The store allocates through the C ABI and exports the IPC
handle into the tensor's hash; a second process (the role of an op executor) opens the handle it
reads from the hash, sees the bytes the first process wrote and writes back through the same
mapping."""
import ctypes as C
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from deepx_amd import lib as dx
from tests.heapmem_client import HeapStore

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CONSUMER = r"""
import ctypes as C, sys
import numpy as np
import torch  # first, like the test process: both sides must run on the same copy of the HIP runtime
sys.path.insert(0, sys.argv[1])
from deepx_amd import lib as dx
L = dx.load()
dx.check(L.dxh_set_device(0), "set_device")
handle = bytes.fromhex(sys.argv[2]); n = int(sys.argv[3])
buf = C.create_string_buffer(handle, 64)
ptr = C.c_void_p()
dx.check(L.dxh_ipc_open(buf, C.byref(ptr)), "open")
host = np.empty(n, dtype=np.float32)
dx.check(L.dxh_memcpy_d2h(host.ctypes.data_as(C.c_void_p), ptr, n * 4, None), "d2h")
assert np.array_equal(host, 1.0 + 0.5 * np.arange(n, dtype=np.float32)), host[:8]
dx.check(L.dxh_mulscalar(dx.F32, ptr, dx.scalar(2.0), ptr, n, None), "mulscalar")   # in place, through the shared mapping
dx.check(L.dxh_device_sync(), "sync")
dx.check(L.dxh_ipc_close(ptr), "close")
print("consumer ok")
"""


def test_heap_tensor_shared_with_a_second_process(dxh):
    store = HeapStore("memory", "hip")
    try:
        n = 1024 * 256
        assert store.command(json.dumps({"op": "create", "name": "H", "dtype": "float32", "shape": [1024, 256], "device": 0, "node": "n1"})) == 1, store.last_error()
        m = store.meta("H")
        assert m["bytes"] == str(n * 4) and m["state"] == "ready" and len(m["ipc_handle"]) == 128 and set(m["ipc_handle"]) != {"0"}
        ptr = C.c_void_p(store.pointer("H"))
        assert ptr.value
        dx.check(dxh.dxh_arange(dx.F32, ptr, n, dx.scalar(1.0), dx.scalar(0.5), None))
        dx.check(dxh.dxh_device_sync())
        assert store.command(json.dumps({"op": "get", "name": "H", "pid": 4242})) == 1 and store.meta("H")["refcount"] == "2"
        r = subprocess.run([sys.executable, "-c", CONSUMER, ROOT, m["ipc_handle"], str(n)], capture_output=True, text=True, timeout=120)
        assert r.returncode == 0 and "consumer ok" in r.stdout, r.stdout + r.stderr
        host = np.empty(n, dtype=np.float32)
        dx.check(dxh.dxh_memcpy_d2h(host.ctypes.data_as(C.c_void_p), ptr, n * 4, None))
        assert np.array_equal(host, 2.0 * (1.0 + 0.5 * np.arange(n, dtype=np.float32)))   # the consumer's write is visible here
        assert store.command(json.dumps({"op": "delete", "name": "H"})) == 1 and store.meta("H")["refcount"] == "1"
        assert store.command(json.dumps({"op": "delete", "name": "H"})) == 1
        assert store.meta("H") is None and store.owned() == 0
    finally:
        store.close()


def test_many_heap_tensors_and_reuse_of_names(dxh):
    store = HeapStore("memory", "hip")
    try:
        for round_no in range(3):
            for i in range(16):
                assert store.command(json.dumps({"op": "create", "name": f"t{i}", "dtype": "bfloat16", "shape": [64, 1 << (i % 8)], "node": "n"})) == 1
            assert store.owned() == 16
            ptrs = {store.pointer(f"t{i}") for i in range(16)}
            assert len(ptrs) == 16 and 0 not in ptrs
            for i in range(16):
                assert store.command(json.dumps({"op": "delete", "name": f"t{i}"})) == 1
            assert store.owned() == 0
    finally:
        store.close()
