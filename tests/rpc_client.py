"""Test client of the ggml RPC wire protocol 4.1.0: the helpers of the reference's own test program
(third_party/llama.cpp/patches/0002-rpc-add-direct-peer-tensor-transfers.patch:1174-1487 -- framing, HELLO, buffer and tensor
helpers, REGISTER_PEER, PUSH_TENSOR_TO_PEER) restated in Python, plus a process wrapper that starts a server the way
test_rpc_server does (`-H 127.0.0.1 -p PORT`, :1286-1331)."""
import os
import socket
import struct
import subprocess
import time

(ALLOC_BUFFER, GET_ALIGNMENT, GET_MAX_SIZE, BUFFER_GET_BASE, FREE_BUFFER, BUFFER_CLEAR, SET_TENSOR, SET_TENSOR_HASH, GET_TENSOR,
 COPY_TENSOR, GRAPH_COMPUTE, GET_DEVICE_MEMORY, INIT_TENSOR, GET_ALLOC_SIZE, HELLO, DEVICE_COUNT, GRAPH_RECOMPUTE, SET_TENSOR_GGUF,
 REGISTER_PEER, PUSH_TENSOR_TO_PEER, PEER_TENSOR_DATA, CMD_COUNT) = range(22)

# rpc_tensor, 296 bytes packed (patches/0002:1070-1085)
TENSOR_FMT = "<QIQ4I4II16ii10QQQQ64s4s"
TENSOR_SIZE = struct.calcsize(TENSOR_FMT)
assert TENSOR_SIZE == 296


def pick_free_port():
    s = socket.socket()
    s.bind(("127.0.0.1", 0))
    port = s.getsockname()[1]
    s.close()
    return port


def tensor(buffer, data, ne, nb, ttype=0, name=b"test"):
    ne = list(ne) + [1] * (4 - len(ne))
    return struct.pack(TENSOR_FMT, 0, ttype, buffer, *ne, *nb, 0, *([0] * 16), 0, *([0] * 10), 0, 0, data, name, b"")


def f32_tensor(buffer, base, n, name=b"test"):
    """make_f32_tensor of the reference's test (patches/0002:1392-1415)."""
    return tensor(buffer, base, [n], [4, 4 * n, 4 * n, 4 * n], 0, name)


class ConnectionClosed(Exception):
    pass


class Client:
    def __init__(self, port, hello=True):
        self.sock = socket.create_connection(("127.0.0.1", port), timeout=30)
        self.sock.setsockopt(socket.IPPROTO_TCP, socket.TCP_NODELAY, 1)
        self.version = None
        if hello:
            self.version = self.hello()

    def close(self):
        self.sock.close()

    def _recv(self, n):
        out = bytearray()
        while len(out) < n:
            chunk = self.sock.recv(min(n - len(out), 1 << 20))
            if not chunk:
                raise ConnectionClosed()
            out += chunk
        return bytes(out)

    def send(self, cmd, payload=b""):
        self.sock.sendall(bytes([cmd]) + struct.pack("<Q", len(payload)) + payload)

    def reply(self):
        (n,) = struct.unpack("<Q", self._recv(8))
        return self._recv(n)

    def call(self, cmd, payload=b""):
        self.send(cmd, payload)
        return self.reply()

    def closed_by_server(self, timeout=5.0):
        """True when the server has ended the connection (what a failed validation does)."""
        self.sock.settimeout(timeout)
        try:
            return self.sock.recv(1) == b""
        except (ConnectionResetError, BrokenPipeError):
            return True
        except socket.timeout:
            return False

    # ---- commands
    def hello(self):
        rsp = self.call(HELLO, bytes(24))
        assert len(rsp) == 28
        return tuple(rsp[:3])

    def device_count(self):
        return struct.unpack("<I", self.call(DEVICE_COUNT))[0]

    def device_memory(self, dev=0):
        return struct.unpack("<QQ", self.call(GET_DEVICE_MEMORY, struct.pack("<I", dev)))

    def alignment(self, dev=0):
        return struct.unpack("<Q", self.call(GET_ALIGNMENT, struct.pack("<I", dev)))[0]

    def max_size(self, dev=0):
        return struct.unpack("<Q", self.call(GET_MAX_SIZE, struct.pack("<I", dev)))[0]

    def alloc_buffer(self, size, dev=0):
        return struct.unpack("<QQ", self.call(ALLOC_BUFFER, struct.pack("<IQ", dev, size)))

    def buffer_get_base(self, handle):
        return struct.unpack("<Q", self.call(BUFFER_GET_BASE, struct.pack("<Q", handle)))[0]

    def free_buffer(self, handle):
        return self.call(FREE_BUFFER, struct.pack("<Q", handle)) == b""

    def buffer_clear(self, handle, value):
        return self.call(BUFFER_CLEAR, struct.pack("<QB", handle, value)) == b""

    def set_tensor(self, t, offset, data):
        self.send(SET_TENSOR, t + struct.pack("<Q", offset) + bytes(data))      # no reply

    def get_tensor(self, t, offset, size):
        rsp = self.call(GET_TENSOR, t + struct.pack("<QQ", offset, size))
        assert len(rsp) == size
        return rsp

    def register_peer(self, peer_id, endpoint):
        ep = endpoint.encode()[:127]
        return self.call(REGISTER_PEER, struct.pack("<I128s", peer_id, ep))[0]

    def push_tensor_to_peer(self, peer_id, src, dst, offset, size):
        return self.call(PUSH_TENSOR_TO_PEER, struct.pack("<I", peer_id) + src + dst + struct.pack("<QQ", offset, size))[0]

    def set_tensor_gguf(self, t, offset=0):
        return self.call(SET_TENSOR_GGUF, t + struct.pack("<Q", offset))[0]


class ServerProcess:
    def __init__(self, binary, port=None, extra=(), env=None):
        self.port = port or pick_free_port()
        self.endpoint = "127.0.0.1:%d" % self.port
        self.output = None
        e = dict(os.environ)
        e.update(env or {})
        self.proc = subprocess.Popen([binary, "-H", "127.0.0.1", "-p", str(self.port), *extra], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=e)
        deadline = time.time() + 60
        while time.time() < deadline:
            if self.proc.poll() is not None:
                raise RuntimeError("rpc-server exited: " + self.proc.stdout.read().decode(errors="replace"))
            try:
                socket.create_connection(("127.0.0.1", self.port), timeout=1).close()
                return
            except OSError:
                time.sleep(0.05)
        self.stop()
        raise RuntimeError("rpc-server did not start listening")

    def stop(self):
        """Ends the server; returns everything it printed."""
        if self.output is not None:
            return self.output
        if self.proc.poll() is None:
            self.proc.terminate()           # SIGTERM, as mesh-llm's launcher does (launch.rs:390-402)
            try:
                self.proc.wait(timeout=10)
            except subprocess.TimeoutExpired:
                self.proc.kill()
                self.proc.wait()
        self.output = self.proc.stdout.read().decode(errors="replace")
        self.proc.stdout.close()
        return self.output

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.stop()
