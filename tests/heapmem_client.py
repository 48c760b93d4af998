"""Test-side helpers for the heap-tensor store: the ctypes view of libdxheap.so and a tiny RESP2
server that stands in for Redis (the handful of commands the store uses), so the store's own RESP
client is exercised over a real TCP connection."""
import ctypes as C
import os
import socket
import threading
import time

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "deepx_amd", "heapmem", "libdxheap.so")


class HeapStore:
    def __init__(self, backend="memory", device="hip"):
        L = C.CDLL(LIB)
        L.dxm_create.restype = C.c_void_p
        L.dxm_create.argtypes = [C.c_char_p, C.c_char_p]
        L.dxm_destroy.argtypes = [C.c_void_p]
        L.dxm_push.argtypes = [C.c_void_p, C.c_char_p]
        L.dxm_run_once.argtypes = [C.c_void_p, C.c_int]
        L.dxm_last_error.argtypes = [C.c_void_p, C.c_char_p, C.c_size_t]
        L.dxm_meta.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p, C.c_size_t]
        L.dxm_pointer.argtypes = [C.c_void_p, C.c_char_p]
        L.dxm_pointer.restype = C.c_ulonglong
        L.dxm_owned.argtypes = [C.c_void_p]
        L.dxm_owned.restype = C.c_longlong
        L.dxm_sweep.argtypes = [C.c_void_p, C.c_char_p]
        L.dxm_sweep.restype = C.c_longlong
        self.L = L
        self.h = L.dxm_create(backend.encode(), device.encode())
        assert self.h, f"cannot create store on {backend}"

    def close(self):
        if self.h:
            self.L.dxm_destroy(self.h)
            self.h = None

    def push(self, json_text): assert self.L.dxm_push(self.h, json_text.encode()) == 0
    def run_once(self, timeout=1): return self.L.dxm_run_once(self.h, timeout)

    def command(self, json_text):
        """push + handle, like a compute process and the store would between them"""
        self.push(json_text)
        return self.run_once()

    def last_error(self):
        buf = C.create_string_buffer(4096)
        self.L.dxm_last_error(self.h, buf, len(buf))
        return buf.value.decode()

    def meta(self, name):
        buf = C.create_string_buffer(4096)
        self.L.dxm_meta(self.h, name.encode(), buf, len(buf))
        text = buf.value.decode()
        return dict(line.split("=", 1) for line in text.split("\n")) if text else None

    def pointer(self, name): return self.L.dxm_pointer(self.h, name.encode())
    def owned(self): return self.L.dxm_owned(self.h)
    def sweep(self, node): return self.L.dxm_sweep(self.h, node.encode())


class FakeRedis:
    """RESP2 over TCP: PING HGETALL HSET HINCRBY DEL KEYS LPUSH BRPOP, one thread per connection."""

    def __init__(self):
        self.hashes, self.lists = {}, {}
        self.cv = threading.Condition()
        self.sock = socket.socket(socket.AF_INET, socket.SOCK_STREAM)
        self.sock.setsockopt(socket.SOL_SOCKET, socket.SO_REUSEADDR, 1)
        self.sock.bind(("127.0.0.1", 0))
        self.sock.listen(8)
        self.port = self.sock.getsockname()[1]
        self.alive = True
        threading.Thread(target=self._accept, daemon=True).start()

    def close(self):
        self.alive = False
        try:
            self.sock.close()
        except OSError:
            pass

    def _accept(self):
        while self.alive:
            try:
                conn, _ = self.sock.accept()
            except OSError:
                return
            threading.Thread(target=self._serve, args=(conn,), daemon=True).start()

    @staticmethod
    def _bulk(b): return b"$%d\r\n%s\r\n" % (len(b), b)

    def _serve(self, conn):
        f = conn.makefile("rb")
        try:
            while True:
                head = f.readline()
                if not head:
                    return
                assert head[:1] == b"*", head
                args = []
                for _ in range(int(head[1:])):
                    n = int(f.readline()[1:])
                    args.append(f.read(n + 2)[:-2])
                conn.sendall(self._run(args))
        except (OSError, AssertionError, ValueError):
            pass
        finally:
            conn.close()

    def _run(self, a):
        cmd = a[0].upper()
        with self.cv:
            if cmd == b"PING":
                return b"+PONG\r\n"
            if cmd == b"HGETALL":
                h = self.hashes.get(a[1], {})
                return b"*%d\r\n" % (2 * len(h)) + b"".join(self._bulk(k) + self._bulk(v) for k, v in h.items())
            if cmd == b"HSET":
                h = self.hashes.setdefault(a[1], {})
                added = 0
                for k, v in zip(a[2::2], a[3::2]):
                    added += k not in h
                    h[k] = v
                return b":%d\r\n" % added
            if cmd == b"HINCRBY":
                h = self.hashes.setdefault(a[1], {})
                h[a[2]] = b"%d" % (int(h.get(a[2], b"0")) + int(a[3]))
                return b":" + h[a[2]] + b"\r\n"
            if cmd == b"DEL":
                return b":%d\r\n" % sum(self.hashes.pop(k, None) is not None for k in a[1:])
            if cmd == b"KEYS":
                prefix = a[1].rstrip(b"*")
                ks = [k for k in self.hashes if k.startswith(prefix)]
                return b"*%d\r\n" % len(ks) + b"".join(self._bulk(k) for k in ks)
            if cmd == b"LPUSH":
                self.lists.setdefault(a[1], []).insert(0, a[2])
                self.cv.notify_all()
                return b":%d\r\n" % len(self.lists[a[1]])
            if cmd == b"BRPOP":
                deadline = time.time() + float(a[2])
                while not self.lists.get(a[1]):
                    left = deadline - time.time()
                    if left <= 0 or not self.cv.wait(left):
                        if not self.lists.get(a[1]):
                            return b"*-1\r\n"
                return b"*2\r\n" + self._bulk(a[1]) + self._bulk(self.lists[a[1]].pop())
        return b"-ERR unknown command\r\n"


class RespClient:
    """what a compute process does: raw RESP requests from Python"""

    def __init__(self, port):
        self.s = socket.create_connection(("127.0.0.1", port))
        self.f = self.s.makefile("rb")

    def call(self, *args):
        req = b"*%d\r\n" % len(args) + b"".join(FakeRedis._bulk(x if isinstance(x, bytes) else str(x).encode()) for x in args)
        self.s.sendall(req)
        return self._read()

    def _read(self):
        line = self.f.readline()
        t, rest = line[:1], line[1:-2]
        if t in (b"+", b"-"):
            return rest.decode()
        if t == b":":
            return int(rest)
        if t == b"$":
            n = int(rest)
            return None if n < 0 else self.f.read(n + 2)[:-2]
        n = int(rest)
        return None if n < 0 else [self._read() for _ in range(n)]

    def close(self):
        self.s.close()
