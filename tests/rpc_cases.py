"""The cases of the reference's server-to-server transfer test program
(third_party/llama.cpp/patches/0002-rpc-add-direct-peer-tensor-transfers.patch:1553-1927), written once and run against the
host-memory build on any machine and against the HIP build on the GPU box."""
import numpy as np

from rpc_client import Client, ServerProcess, f32_tensor, pick_free_port


def peer_registration(binary):
    """Test 1 (:1553-1611): registration round trip, empty endpoint refused, re-registration, a nearly full endpoint field."""
    with ServerProcess(binary) as a, ServerProcess(binary) as b:
        ca, cb = Client(a.port), Client(b.port)
        assert ca.register_peer(1, b.endpoint) == 1
        assert cb.register_peer(0, a.endpoint) == 1
        assert ca.register_peer(99, "") == 0
        assert ca.register_peer(1, b.endpoint) == 1
        assert ca.register_peer(50, "a" * 120 + ":12345") == 1
        # malformed endpoints of register_peer's own validation (:487-491): no colon, empty host, empty port
        assert ca.register_peer(51, "localhost") == 0
        assert ca.register_peer(52, ":123") == 0
        assert ca.register_peer(53, "host:") == 0
        ca.close()
        cb.close()


def direct_push(binary):
    """Test 2 (:1616-1745): 4096 bytes i & 0xFF pushed A -> B, a partial push (offset 1024, size 2048) into a zeroed
    destination, and the reverse direction with 0xFF - (i & 0xFF)."""
    size, n = 4096, 1024
    with ServerProcess(binary) as a, ServerProcess(binary) as b:
        ca, cb = Client(a.port), Client(b.port)
        assert ca.register_peer(1, b.endpoint) == 1 and cb.register_peer(0, a.endpoint) == 1
        buf_a, act_a = ca.alloc_buffer(size)
        buf_b, act_b = cb.alloc_buffer(size)
        assert buf_a and buf_b and act_a >= size and act_b >= size
        base_a, base_b = ca.buffer_get_base(buf_a), cb.buffer_get_base(buf_b)
        assert base_a and base_b
        src = bytes(i & 0xFF for i in range(size))
        ta, tb = f32_tensor(buf_a, base_a, n), f32_tensor(buf_b, base_b, n)
        ca.set_tensor(ta, 0, src)
        assert ca.push_tensor_to_peer(1, ta, tb, 0, size) == 1
        assert cb.get_tensor(tb, 0, size) == src
        # partial
        cb.set_tensor(tb, 0, bytes(size))
        # SET_TENSOR has no reply and the push reaches B on another connection: a command with a reply on this
        # connection first, so that the zeroing has been processed before the push can arrive
        assert cb.get_tensor(tb, 0, 16) == bytes(16)
        assert ca.push_tensor_to_peer(1, ta, tb, 1024, 2048) == 1
        got = cb.get_tensor(tb, 0, size)
        assert got[:1024] == bytes(1024) and got[1024:3072] == src[1024:3072] and got[3072:] == bytes(1024)
        # reverse
        rev = bytes(0xFF - (i & 0xFF) for i in range(size))
        cb.set_tensor(tb, 0, rev)
        assert cb.push_tensor_to_peer(0, tb, ta, 0, size) == 1
        assert ca.get_tensor(ta, 0, size) == rev
        assert ca.free_buffer(buf_a) and cb.free_buffer(buf_b)
        ca.close()
        cb.close()


def large_push(binary):
    """Test 3 (:1750-1801): 16 MiB of (i * 7 + 13) & 0xFF."""
    size = 16 * 1024 * 1024
    with ServerProcess(binary) as a, ServerProcess(binary) as b:
        ca, cb = Client(a.port), Client(b.port)
        assert ca.register_peer(1, b.endpoint) == 1
        buf_a, _ = ca.alloc_buffer(size)
        buf_b, _ = cb.alloc_buffer(size)
        assert buf_a and buf_b
        base_a, base_b = ca.buffer_get_base(buf_a), cb.buffer_get_base(buf_b)
        data = ((np.arange(size, dtype=np.uint64) * 7 + 13) & 0xFF).astype(np.uint8).tobytes()
        ta, tb = f32_tensor(buf_a, base_a, size // 4), f32_tensor(buf_b, base_b, size // 4)
        ca.set_tensor(ta, 0, data)
        assert ca.push_tensor_to_peer(1, ta, tb, 0, size) == 1
        assert cb.get_tensor(tb, 0, size) == data
        assert ca.free_buffer(buf_a) and cb.free_buffer(buf_b)
        ca.close()
        cb.close()


def fallback_on_failed_push(binary):
    """Test 4 (:1806-1880): a peer registered at an endpoint nobody listens on -> the push answers 0 (the command itself
    succeeds) and the client relays with GET_TENSOR + SET_TENSOR."""
    size = 1024
    with ServerProcess(binary) as a, ServerProcess(binary) as b:
        ca, cb = Client(a.port), Client(b.port)
        assert ca.register_peer(1, "127.0.0.1:%d" % pick_free_port()) == 1
        buf_a, _ = ca.alloc_buffer(size)
        buf_b, _ = cb.alloc_buffer(size)
        base_a, base_b = ca.buffer_get_base(buf_a), cb.buffer_get_base(buf_b)
        data = bytes(i & 0xFF for i in range(size))
        ta, tb = f32_tensor(buf_a, base_a, size // 4), f32_tensor(buf_b, base_b, size // 4)
        ca.set_tensor(ta, 0, data)
        assert ca.push_tensor_to_peer(1, ta, tb, 0, size) == 0
        assert ca.push_tensor_to_peer(77, ta, tb, 0, size) == 0          # a peer never registered
        relay = ca.get_tensor(ta, 0, size)
        cb.set_tensor(tb, 0, relay)
        assert cb.get_tensor(tb, 0, size) == data
        ca.free_buffer(buf_a)
        cb.free_buffer(buf_b)
        ca.close()
        cb.close()


def rapid_connect_disconnect(binary, iterations=100):
    """Test 5 (:1885-1917): 100 connect + HELLO + close cycles, at least 90 % succeed, the server answers afterwards."""
    with ServerProcess(binary) as s:
        ok = 0
        for _ in range(iterations):
            try:
                c = Client(s.port)
                ok += c.version[0] == 4
                c.close()
            except OSError:
                pass
        assert ok >= iterations * 9 // 10
        c = Client(s.port)
        assert c.version[0] == 4
        c.close()
