"""Test-side clients of the executor: the in-process C API (libdxexec.so) and the UDP binary.

The UDP client formats requests exactly like front/py/deepx/nn/deepxir.py:133-159 prints a DeepxIR
and reads replies like DeepxIRResp (:161-204)."""
import ctypes as C
import os
import socket
import subprocess
import tempfile
import time

import numpy as np
import yaml

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXEC_DIR = os.path.join(ROOT, "deepx_amd", "executor")
BIN = os.path.join(EXEC_DIR, "deepx-executor-hip")
LIB = os.path.join(EXEC_DIR, "libdxexec.so")


class InProc:
    def __init__(self):
        L = C.CDLL(LIB)
        L.dxe_create.restype = C.c_void_p
        L.dxe_destroy.argtypes = [C.c_void_p]
        for name, args in [("dxe_execute", [C.c_void_p, C.c_char_p]), ("dxe_execute_batch", [C.c_void_p, C.c_char_p]), ("dxe_stats", [C.c_void_p]),
                           ("dxe_fusion_stats", [C.c_void_p]), ("dxe_defer_stats", [C.c_void_p]),
                           ("dxe_parse", [C.c_char_p]), ("dxe_match", [C.c_void_p, C.c_char_p]),
                           ("dxe_op_table", [C.c_void_p, C.c_char_p]), ("dxe_typedef_roundtrip", [C.c_char_p]),
                           ("dxe_tensor_yaml", [C.c_void_p, C.c_char_p]), ("dxe_shape_yaml_roundtrip", [C.c_char_p])]:
            fn = getattr(L, name)
            fn.argtypes = args + [C.c_char_p, C.c_size_t]
            fn.restype = C.c_size_t
        L.dxe_infer_shape.argtypes = [C.c_char_p, C.POINTER(C.c_int), C.c_int, C.POINTER(C.c_int), C.c_int, C.c_int, C.c_char_p, C.c_size_t]
        L.dxe_infer_shape.restype = C.c_size_t
        for name in ("dxe_data_write", "dxe_data_read"):
            getattr(L, name).argtypes = [C.c_char_p, C.c_char_p, C.c_size_t, C.c_char_p, C.c_size_t]
            getattr(L, name).restype = C.c_size_t
        L.dxe_set_graphs.argtypes = [C.c_void_p, C.c_int]
        L.dxe_set_fusion.argtypes = [C.c_void_p, C.c_int]
        L.dxe_print_format_ok.argtypes = [C.c_char_p, C.c_int]
        L.dxe_set_sync.argtypes = [C.c_void_p, C.c_int]
        L.dxe_set_defer.argtypes = [C.c_void_p, C.c_int]
        L.dxe_set_streams.argtypes = [C.c_void_p, C.c_int]
        L.dxe_set_pool.argtypes = [C.c_int]
        L.dxe_set_zero_later.argtypes = [C.c_void_p, C.c_int]
        L.dxe_side_launches.argtypes = [C.c_void_p]
        L.dxe_side_launches.restype = C.c_size_t
        L.dxe_flush.argtypes = [C.c_void_p]
        L.dxe_held.argtypes = [C.c_void_p]
        L.dxe_held.restype = C.c_size_t
        self.L = L
        self.ex = L.dxe_create()
        assert self.ex

    def _call(self, fn, *args):
        buf = C.create_string_buffer(1 << 18)
        fn(*args, buf, len(buf))
        return buf.value.decode("utf-8")

    def close(self):
        """destroys the executor (its tensors, side streams and recorded graphs); tests that make hundreds of executors call it"""
        if self.ex:
            self.L.dxe_destroy(self.ex)
            self.ex = None

    def execute(self, line): return self._call(self.L.dxe_execute, self.ex, line.encode())
    def execute_batch(self, lines): return self._call(self.L.dxe_execute_batch, self.ex, "\n".join(lines).encode()).split("\n")
    def set_graphs(self, on): self.L.dxe_set_graphs(self.ex, int(on))
    def set_fusion(self, on): self.L.dxe_set_fusion(self.ex, int(on))
    def set_sync(self, on): self.L.dxe_set_sync(self.ex, int(on))
    def set_defer(self, on): self.L.dxe_set_defer(self.ex, int(on))
    def set_streams(self, n): self.L.dxe_set_streams(self.ex, int(n))
    def set_zero_later(self, on): self.L.dxe_set_zero_later(self.ex, int(on))
    def set_pool(self, on): self.L.dxe_set_pool(int(on))  # process-wide: tensors made from now on
    def side_launches(self): return int(self.L.dxe_side_launches(self.ex))
    def flush(self): self.L.dxe_flush(self.ex)
    def held(self): return int(self.L.dxe_held(self.ex))

    def defer_stats(self):
        held, flushes = (int(x) for x in self._call(self.L.dxe_defer_stats, self.ex).split())
        return {"held_lines": held, "flushes": flushes}

    def fusion_stats(self):
        runs, lines, groups, group_lines = (int(x) for x in self._call(self.L.dxe_fusion_stats, self.ex).split())
        return {"runs": runs, "lines": lines, "matmul_groups": groups, "matmul_lines": group_lines}

    def stats(self):
        b, c, r, j = (int(x) for x in self._call(self.L.dxe_stats, self.ex).split())
        return {"batches": b, "captures": c, "replays": r, "rejects": j}

    def data_write(self, path, data):
        """raw bytes to `path` through the writer behind `save`; returns an empty string or 'error: ...'"""
        return self._call(self.L.dxe_data_write, path.encode(), bytes(data), len(data))

    def data_read(self, path, nbytes):
        """(status, bytes) through the reader behind `load` / `loadtensordata`, which wants exactly nbytes"""
        buf = C.create_string_buffer(max(1, nbytes))
        status = self._call(self.L.dxe_data_read, path.encode(), buf, nbytes)
        return status, buf.raw[:nbytes]

    def parse(self, line): return self._call(self.L.dxe_parse, line.encode())
    def match(self, line): return self._call(self.L.dxe_match, self.ex, line.encode())
    def op_table(self, name="op-mem-hip"): return self._call(self.L.dxe_op_table, self.ex, name.encode())
    def typedef(self, text): return self._call(self.L.dxe_typedef_roundtrip, text.encode())
    def tensor_yaml(self, name): return self._call(self.L.dxe_tensor_yaml, self.ex, name.encode())
    def shape_yaml(self, text): return self._call(self.L.dxe_shape_yaml_roundtrip, text.encode())

    def print_format_ok(self, fmt, is_float): return bool(self.L.dxe_print_format_ok(fmt.encode(), int(is_float)))

    def infer(self, op, a, b=(), extra=0):
        A = (C.c_int * max(1, len(a)))(*a)
        B = (C.c_int * max(1, len(b)))(*b)
        return self._call(self.L.dxe_infer_shape, op.encode(), A, len(a), B, len(b), extra)


REF_SO = os.path.join(ROOT, "oracle", "_ref", "libdeepxref.so")


class Reference:
    """The reference's own deepxcore code (IR parser, dtype strings, factory, shape inference),
    compiled by oracle/ref.mk from the reference checkout.  Test-side only."""

    def __init__(self):
        L = C.CDLL(REF_SO)
        ip = C.POINTER(C.c_int)
        sigs = {"ref_parse": [C.c_char_p], "ref_typedef": [C.c_char_p], "ref_match": [C.c_char_p, C.c_char_p],
                "ref_transpose_shape": [ip, C.c_int, ip], "ref_broadcast_shape": [ip, C.c_int, ip, C.c_int],
                "ref_indexselect_shape": [ip, C.c_int, ip, C.c_int, C.c_int], "ref_repeat_shape": [ip, C.c_int, ip, C.c_int],
                "ref_checked_dims": [ip, C.c_int, ip, C.c_int], "ref_reduced_shape": [ip, C.c_int, ip, C.c_int, C.c_int],
                "ref_fs_save": [C.c_char_p, C.c_char_p, C.c_size_t], "ref_fs_load": [C.c_char_p, C.c_char_p, C.c_size_t],
                "ref_fs_load_any": [C.c_char_p, C.c_char_p, C.c_size_t], "ref_fs_filename": [C.c_char_p]}
        for name, args in sigs.items():
            fn = getattr(L, name)
            fn.argtypes = args + [C.c_char_p, C.c_size_t]
            fn.restype = C.c_size_t
        self.L = L

    def _call(self, fn, *args):
        buf = C.create_string_buffer(1 << 16)
        fn(*args, buf, len(buf))
        return buf.value.decode("utf-8")

    @staticmethod
    def _arr(v):
        return (C.c_int * max(1, len(v)))(*v)

    def parse(self, line): return self._call(self.L.ref_parse, line.encode())
    def typedef(self, text): return self._call(self.L.ref_typedef, text.encode())
    def match(self, registered_rows, call): return self._call(self.L.ref_match, "\n".join(registered_rows).encode(), call.encode())
    def transpose_shape(self, s, o): return self._call(self.L.ref_transpose_shape, self._arr(s), len(s), self._arr(o))
    def broadcast_shape(self, a, b): return self._call(self.L.ref_broadcast_shape, self._arr(a), len(a), self._arr(b), len(b))
    def indexselect_shape(self, a, b, axis): return self._call(self.L.ref_indexselect_shape, self._arr(a), len(a), self._arr(b), len(b), axis)
    def repeat_shape(self, a, b): return self._call(self.L.ref_repeat_shape, self._arr(a), len(a), self._arr(b), len(b))
    def checked_dims(self, s, d): return self._call(self.L.ref_checked_dims, self._arr(s), len(s), self._arr(d), len(d))
    def reduced_shape(self, s, d, keep): return self._call(self.L.ref_reduced_shape, self._arr(s), len(s), self._arr(d), len(d), int(keep))
    def fs_save(self, path, data): return self._call(self.L.ref_fs_save, path.encode(), bytes(data), len(data))
    def fs_filename(self, path): return self._call(self.L.ref_fs_filename, path.encode())

    def fs_load(self, path, nbytes):
        buf = C.create_string_buffer(max(1, nbytes))
        status = self._call(self.L.ref_fs_load, path.encode(), buf, nbytes)
        return status, buf.raw[:nbytes]

    def fs_load_any(self, path, room):
        buf = C.create_string_buffer(max(1, room))
        status = self._call(self.L.ref_fs_load_any, path.encode(), buf, room)
        return status, buf.raw[:room]


def free_port():
    s = socket.socket(socket.AF_INET, socket.SOCK_DGRAM)
    s.bind(("127.0.0.1", 0))
    p = s.getsockname()[1]
    s.close()
    return p


class Resp:
    """'<id> ok// recv_at=.. start_at=.. finish_at=.. [message]' as DeepxIRResp splits it"""

    def __init__(self, text):
        self.text = text
        front, _, extra = text.partition("//")
        parts = front.strip().split(" ", 2)
        self.id = parts[0] if parts else None
        self.result = parts[1] if len(parts) > 1 else ""
        self.times, msg = {}, []
        for tok in extra.strip().split(" "):
            k, eq, v = tok.partition("=")
            if eq and k in ("recv_at", "start_at", "finish_at") and not msg:
                self.times[k] = int(v)
            elif tok:
                msg.append(tok)
        self.message = " ".join(msg)

    @property
    def ok(self): return self.result == "ok"


class UdpExecutor:
    """Runs deepx-executor-hip as a child process and talks deepxIR to it over UDP."""

    def __init__(self, env=None):
        self.port = free_port()
        e = dict(os.environ, DEEPX_PORT=str(self.port))
        e.update(env or {})
        # what the server prints goes to a file, not a pipe: nobody reads a pipe here, and a server that has printed
        # a pipe's worth of messages (one per line that fails) would block in its next write
        self.log = tempfile.TemporaryFile()
        self.proc = subprocess.Popen([BIN], env=e, stdout=self.log, stderr=subprocess.STDOUT)
        self.sock = socket.socket(socket.AF_INET, socket.SOCK_DGRAM)
        self.sock.settimeout(60)
        self._id = 0
        deadline = time.time() + 120
        while True:  # wait until it answers
            try:
                self.sock.settimeout(1)
                self.sock.sendto(b"argset(var<int32>:1)->(var<int32>:__ready) // id=0", ("127.0.0.1", self.port))
                self.sock.recvfrom(65536)
                break
            except socket.timeout:
                if self.proc.poll() is not None or time.time() > deadline:
                    self.log.seek(0)
                    raise RuntimeError("executor did not start: " + self.log.read().decode(errors="replace"))
        self.sock.settimeout(60)

    def raw(self, text, nreplies=1):
        self.sock.sendto(text.encode("utf-8"), ("127.0.0.1", self.port))
        return [Resp(self.sock.recvfrom(65536)[0].decode("utf-8")) for _ in range(nreplies)]

    def send(self, op, args, returns, author="miaobyte", extra=""):
        """format like str(DeepxIR): 'name (a, b) -> (c) // author=x  id=n  created_at=t  sent_at=t'"""
        self._id += 1
        now = time.time()
        meta = []
        if author:
            meta.append(f"author={author}")
        meta += [f" id={self._id}", f" created_at={now}", f" sent_at={now}"]
        if extra:
            meta.append(" " + extra)
        line = " ".join([op, "(" + ", ".join(args) + ")", "->", "(" + ", ".join(returns) + ")", "//", " ".join(meta)])
        r = self.raw(line)[0]
        assert r.id == str(self._id), (r.text, self._id)
        return r

    def must(self, op, args, returns, author="miaobyte", extra=""):
        r = self.send(op, args, returns, author, extra)
        assert r.ok, f"{op}: {r.text}"
        return r

    def close(self):
        try:
            self.sock.sendto(b"__quit__", ("127.0.0.1", self.port))
            self.proc.wait(timeout=10)
        except Exception:
            self.proc.kill()
        self.sock.close()
        self.log.close()


# ---- deepx tensor files (the format of front/py/deepxutil/numpy/io.py and shape.cpp:93-101) ------
NP_OF = {"float64": np.float64, "float32": np.float32, "float16": np.uint16, "bfloat16": np.uint16, "int64": np.int64,
         "int32": np.int32, "int16": np.int16, "int8": np.int8, "bool": np.uint8}


def write_tensor(path, arr, dtype_name):
    arr = np.ascontiguousarray(arr)
    strides, s = [], 1
    for d in reversed(arr.shape):
        strides.insert(0, s)
        s *= d
    with open(path + ".shape", "w") as f:  # what PyYAML writes for the front (shape.py:185-191)
        yaml.safe_dump({"dtype": dtype_name, "dim": arr.ndim, "shape": list(arr.shape), "stride": strides, "size": int(arr.size)}, f)
    arr.tofile(path + ".data")


def read_tensor(path):
    meta = yaml.safe_load(open(path + ".shape"))
    data = np.fromfile(path + ".data", dtype=NP_OF[meta["dtype"]])
    assert data.size == meta["size"]
    return data.reshape(meta["shape"]), meta
