"""rpc-server-compatible front end: wire protocol 4.1.0 against the host-memory build (no GPU needed).

The five cases of the reference's own test program (tests/rpc_cases.py) plus the commands and failure behaviour the launcher
and llama-server's RPC backend rely on: HELLO first, device listing and `-d <unknown>` probe, buffer life cycle, bounds
checks, SET_TENSOR_GGUF by tensor name, the REGISTER_PEER frame mesh-llm's tunnel rewrites."""
import os
import struct
import subprocess
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import gguf_util as G
import rpc_cases
import rpc_client as R
from rpc_client import Client, ServerProcess, f32_tensor, tensor
from util import mesh

Q4_K, Q6_K, F32 = 12, 14, 0


@pytest.fixture(scope="session")
def server_bin(tmp_path_factory):
    mesh()                                      # imports the package (and its build module)
    from mesh_llm_amd import build
    return build.build_rpc_server_hostmem(str(tmp_path_factory.mktemp("rpc") / "rpc-server-hostmem"))


# ---- the reference's five tests
def test_peer_registration(server_bin):
    rpc_cases.peer_registration(server_bin)


def test_direct_push(server_bin):
    rpc_cases.direct_push(server_bin)


def test_large_push(server_bin):
    rpc_cases.large_push(server_bin)


def test_fallback_on_failed_push(server_bin):
    rpc_cases.fallback_on_failed_push(server_bin)


def test_rapid_connect_disconnect(server_bin):
    rpc_cases.rapid_connect_disconnect(server_bin)


# ---- launcher contract (mesh-llm/src/inference/launch.rs)
def parse_available_devices(output):
    """parse_available_devices of launch.rs:743-765: lines after 'available devices:', name = text before the first ':',
    ASCII alphanumeric only."""
    devices, inside = [], False
    for line in output.splitlines():
        t = line.strip()
        if t == "available devices:":
            inside = True
            continue
        if not inside or not t or ":" not in t:
            continue
        name = t.split(":", 1)[0]
        if name.isascii() and name.isalnum():
            devices.append(name)
    return devices


def test_device_probe_lists_devices_and_fails(server_bin):
    """probe_available_devices (launch.rs:768-782) runs `-d __mesh_llm_probe_invalid__ -p 0` and reads stdout + stderr."""
    r = subprocess.run([server_bin, "-d", "__mesh_llm_probe_invalid__", "-p", "0"], capture_output=True, text=True, timeout=30)
    assert r.returncode != 0
    assert parse_available_devices(r.stdout + "\n" + r.stderr) == ["ROCm0", "ROCm1"]


def test_launcher_argv_device_port_gguf(server_bin, tmp_path):
    """`-d DEV -p PORT --gguf PATH` (launch.rs:920-932) with both spellings of an AMD device (launch.rs:812-823); the port is
    open well inside the launcher's 15 s and the process ends on SIGTERM."""
    path = str(tmp_path / "m.gguf")
    G.write_gguf(path, [("general.architecture", G.T_STR, "llama")], [("a", F32, (8,), np.arange(8, dtype=np.float32))])
    for dev in ("ROCm1", "HIP0"):
        port = R.pick_free_port()
        p = subprocess.Popen([server_bin, "-d", dev, "-p", str(port), "--gguf", path], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                             env=dict(os.environ, MESH_LLM_OWNER_PID=str(os.getpid()), MESH_LLM_RUNTIME_DIR=str(tmp_path)))
        try:
            for _ in range(200):
                try:
                    c = Client(port)
                    break
                except OSError:
                    import time
                    time.sleep(0.05)
            assert c.version == (4, 1, 0)
            assert c.device_count() == 1            # only the device named on the command line is exposed
            c.close()
        finally:
            p.terminate()
            assert p.wait(timeout=10) is not None
            p.stdout.close()


def test_bad_arguments_exit_nonzero(server_bin):
    for argv in (["-p", "0"], ["-p", "70000"], ["--no-such-flag"], ["-d"]):
        r = subprocess.run([server_bin, *argv], capture_output=True, text=True, timeout=30)
        assert r.returncode != 0, argv


# ---- protocol
def test_hello_is_4_1_0_and_must_come_first(server_bin):
    with ServerProcess(server_bin) as s:
        c = Client(s.port, hello=False)
        rsp = c.call(R.HELLO, bytes(24))
        assert len(rsp) == 28 and tuple(rsp[:3]) == (4, 1, 0)      # minor >= 1 announces the peer commands (patches/0002:25-28)
        assert rsp[4:] == bytes(24)                                 # no extra transport capabilities
        c.close()
        c = Client(s.port, hello=False)
        c.send(R.DEVICE_COUNT)
        assert c.closed_by_server()
        c.close()
        c = Client(s.port)
        c.send(200)                                                 # not a command
        assert c.closed_by_server()
        c.close()


def test_device_queries(server_bin):
    with ServerProcess(server_bin) as s:
        c = Client(s.port)
        assert c.device_count() == 2
        free, total = c.device_memory(1)
        assert 0 < free <= total
        assert c.alignment() >= 32 and c.alignment() & (c.alignment() - 1) == 0
        assert c.max_size() >= 1 << 30
        c.send(R.GET_DEVICE_MEMORY, struct.pack("<I", 5))           # no such device
        assert c.closed_by_server()
        c.close()


def test_buffer_life_cycle_and_clear(server_bin):
    with ServerProcess(server_bin) as s:
        c = Client(s.port)
        h, size = c.alloc_buffer(1000, dev=1)
        assert h and size >= 1000
        base = c.buffer_get_base(h)
        assert base and base % c.alignment() == 0
        t = tensor(h, base, [1000], [1, 1000, 1000, 1000], ttype=24)      # I8
        assert c.buffer_clear(h, 0xA5)
        assert c.get_tensor(t, 0, 1000) == bytes([0xA5]) * 1000
        c.set_tensor(t, 10, b"hello")
        got = c.get_tensor(t, 0, 1000)
        assert got[10:15] == b"hello" and got[:10] == bytes([0xA5]) * 10 and got[15:] == bytes([0xA5]) * 985
        assert c.get_tensor(t, 12, 3) == b"llo"
        assert c.free_buffer(h)
        c.send(R.BUFFER_GET_BASE, struct.pack("<Q", h))              # freed handle
        assert c.closed_by_server()
        c.close()
        c = Client(s.port)
        h0, size0 = c.alloc_buffer(1 << 40)                           # cannot be had: answers 0 / 0, connection stays
        assert h0 == 0 and size0 == 0
        assert c.device_count() == 2
        c.close()


def test_bounds_are_enforced(server_bin):
    """A request outside its buffer ends the connection and changes nothing (the reference's region checks,
    patches/0002:572-585 and patches/0001:229-240)."""
    with ServerProcess(server_bin) as s:
        c = Client(s.port)
        h, _ = c.alloc_buffer(4096)
        base = c.buffer_get_base(h)
        good = f32_tensor(h, base, 1024)
        c.set_tensor(good, 0, bytes(4096))
        cases = [
            lambda k: k.set_tensor(good, 4000, bytes(200)),                                 # runs past the tensor
            lambda k: k.set_tensor(f32_tensor(h, base + 2048, 1024), 0, bytes(16)),         # descriptor leaves the buffer
            lambda k: k.set_tensor(f32_tensor(h, base - 64, 16), 0, bytes(16)),             # starts before it
            lambda k: k.set_tensor(f32_tensor(h + 8, base, 16), 0, bytes(16)),              # not a buffer handle
            lambda k: k.set_tensor(f32_tensor(0, base, 16), 0, bytes(16)),                  # no buffer
            lambda k: k.send(R.GET_TENSOR, good + struct.pack("<QQ", 4095, 2)),
            lambda k: k.send(R.GET_TENSOR, good + struct.pack("<QQ", 2 ** 63, 2 ** 63)),    # offset + size wraps
            lambda k: k.set_tensor(tensor(h, base, [16], [4, 64, 64, 64], ttype=99), 0, bytes(16)),   # unknown type
        ]
        for bad in cases:
            k = Client(s.port)
            bad(k)
            assert k.closed_by_server()
            k.close()
        assert c.get_tensor(good, 0, 4096) == bytes(4096)
        # the push reports 0 instead (it has a result byte) and the connection stays
        assert c.push_tensor_to_peer(1, f32_tensor(h, base + 4000, 1024), good, 0, 4096) == 0
        assert c.device_count() == 2
        c.close()


def test_set_tensor_hash_copy_init_alloc_size(server_bin):
    with ServerProcess(server_bin) as s:
        c = Client(s.port)
        h, _ = c.alloc_buffer(8192)
        base = c.buffer_get_base(h)
        a, b = f32_tensor(h, base, 1024), f32_tensor(h, base + 4096, 1024)
        # no tensor cache: the hash is never known, so the client sends the bytes (result 0)
        assert c.call(R.SET_TENSOR_HASH, a + struct.pack("<QQ", 0, 0x1234))[0] == 0
        data = np.random.Generator(np.random.PCG64(1)).integers(0, 256, 4096, dtype=np.uint8).tobytes()
        c.set_tensor(a, 0, data)
        assert c.call(R.COPY_TENSOR, a + b)[0] == 1
        assert c.get_tensor(b, 0, 4096) == data
        assert c.call(R.COPY_TENSOR, a + f32_tensor(h, base + 4096, 512))[0] == 0      # sizes differ
        assert c.call(R.INIT_TENSOR, a) == b""
        # GET_ALLOC_SIZE: device, tensor, 10 source descriptors; a 4096 x 512 Q4_K matrix is 512 * 16 * 144 bytes
        q = tensor(0, 0, [4096, 512], [144, 16 * 144, 512 * 16 * 144, 512 * 16 * 144], ttype=Q4_K)
        rsp = c.call(R.GET_ALLOC_SIZE, struct.pack("<I", 0) + q + bytes(296 * 10))
        assert struct.unpack("<Q", rsp)[0] == 512 * 16 * 144
        c.close()


def test_register_peer_frame_of_the_tunnel(server_bin):
    """The exact frame mesh-llm's tunnel parses and rewrites (mesh-llm/src/network/rewrite.rs:221-232: command 18, payload
    size 132 = peer_id u32 + endpoint[128])."""
    with ServerProcess(server_bin) as s:
        c = Client(s.port)
        endpoint = b"127.0.0.1:49502"
        payload = bytearray(132)
        payload[:4] = (7).to_bytes(4, "little")
        payload[4:4 + len(endpoint)] = endpoint
        c.sock.sendall(bytes([18]) + (132).to_bytes(8, "little") + bytes(payload))
        assert c.reply() == b"\x01"
        c.sock.sendall(bytes([18]) + (131).to_bytes(8, "little") + bytes(131))           # malformed size (rewrite.rs:262-283)
        assert c.closed_by_server()
        c.close()


# ---- GRAPH_COMPUTE / GRAPH_RECOMPUTE (patches/0002:443-459, patches/0001:163-174)
def _fake_weights(layers, E=64, H=2, HK=1, hd=32, FF=96, extra=None, drop=()):
    """GGUF names and shapes of decoder layers (shapes only: the host-memory build's stand-in runner never reads weights)."""
    w = {}
    for il in layers:
        p = "blk.%d." % il
        w.update({p + "attn_norm.weight": (F32, [E]), p + "attn_q.weight": (Q4_K, [E * 4, H * hd]), p + "attn_k.weight": (Q4_K, [E * 4, HK * hd]),
                  p + "attn_v.weight": (Q6_K, [E * 4, HK * hd]), p + "attn_output.weight": (Q4_K, [H * hd * 4, E]), p + "ffn_norm.weight": (F32, [E]),
                  p + "ffn_gate.weight": (Q4_K, [E * 4, FF]), p + "ffn_up.weight": (Q4_K, [E * 4, FF]), p + "ffn_down.weight": (Q6_K, [FF * 8 // 3, E])})
    # (row lengths of the quantised matrices are multiples of 256 so that their descriptors are well-formed; the attention
    # norm fixes the hidden size the recogniser reads)
    for k in drop:
        del w[k]
    w.update(extra or {})
    return w


def _graph_case(c, layers, T=3, device=0, **kw):
    import rpc_graph_util as GU
    h, _ = c.alloc_buffer(8 << 20, device)
    base = c.buffer_get_base(h)
    gb = GU.GraphBuilder(h, base, device)
    weights = kw.pop("weights", None) or _fake_weights(layers)
    inp, pos, out = GU.layer_range_graph(gb, weights, layers, T, 2, 1, 32, 128, **kw)
    return gb, inp, pos, out


def _expected(x, pos, b, e, rows):
    T, E = x.shape
    cols = np.arange(rows) % E
    return x[:, cols] + np.asarray(pos, np.float32)[:, None] + 100.0 * b + 10000.0 * e


def _any_gguf(tmp_path):
    path = str(tmp_path / "m.gguf")
    G.write_gguf(path, [("general.architecture", G.T_STR, "llama")], [("a", F32, (8,), np.arange(8, dtype=np.float32))])
    return path


def test_graph_compute_runs_a_layer_range_and_recompute_replays_it(server_bin, tmp_path):
    """The decoder sub-graph of layers 1-2 is parsed, recognised by its weight names and handed to the runner (here the
    host-memory stand-in, whose result shows which range ran on which data); GRAPH_RECOMPUTE replays the stored graph on
    the inputs as they are then; a second device keeps its own stored graph."""
    with ServerProcess(server_bin, extra=["--gguf", _any_gguf(tmp_path)]) as s:
        c = Client(s.port)
        gb, inp, pos, out = _graph_case(c, [1, 2], T=3)
        rng = np.random.Generator(np.random.PCG64(1))
        x = rng.standard_normal((3, 64)).astype(np.float32)
        c.set_tensor(gb.descriptor(inp), 0, x.tobytes())
        c.set_tensor(gb.descriptor(pos), 0, np.array([7, 8, 9], np.int32).tobytes())
        c.send(R.GRAPH_COMPUTE, gb.payload())                    # no reply
        got = np.frombuffer(c.get_tensor(gb.descriptor(out), 0, 3 * 64 * 4), np.float32).reshape(3, 64)
        assert np.array_equal(got, _expected(x, [7, 8, 9], 1, 3, 64).astype(np.float32))
        # new data, same graph
        x2 = rng.standard_normal((3, 64)).astype(np.float32)
        c.set_tensor(gb.descriptor(inp), 0, x2.tobytes())
        c.set_tensor(gb.descriptor(pos), 0, np.array([10, 11, 12], np.int32).tobytes())
        c.send(R.GRAPH_RECOMPUTE, struct.pack("<I", 0))
        got = np.frombuffer(c.get_tensor(gb.descriptor(out), 0, 3 * 64 * 4), np.float32).reshape(3, 64)
        assert np.array_equal(got, _expected(x2, [10, 11, 12], 1, 3, 64).astype(np.float32))
        # the other device: its own graph (one layer, one token, logits out), and the first device's stored graph is untouched
        gb1, inp1, pos1, out1 = _graph_case(c, [3], T=1, device=1, with_output=True,
                                            weights=_fake_weights([3], extra={"output_norm.weight": (F32, [64]), "output.weight": (Q6_K, [256, 80])}))
        x3 = rng.standard_normal((1, 64)).astype(np.float32)
        c.set_tensor(gb1.descriptor(inp1), 0, x3.tobytes())
        c.set_tensor(gb1.descriptor(pos1), 0, np.array([5], np.int32).tobytes())
        c.send(R.GRAPH_COMPUTE, gb1.payload())
        got = np.frombuffer(c.get_tensor(gb1.descriptor(out1), 0, 80 * 4), np.float32).reshape(1, 80)
        assert np.array_equal(got, _expected(x3, [5], 3, 4, 80).astype(np.float32))
        c.send(R.GRAPH_RECOMPUTE, struct.pack("<I", 0))
        got = np.frombuffer(c.get_tensor(gb.descriptor(out), 0, 3 * 64 * 4), np.float32).reshape(3, 64)
        assert np.array_equal(got, _expected(x2, [10, 11, 12], 1, 3, 64).astype(np.float32))
        c.close()


def test_graph_of_a_mixture_of_experts_range_with_biases_and_head_norms(server_bin, tmp_path):
    w = _fake_weights([0, 1], drop=["blk.%d.ffn_%s.weight" % (il, k) for il in (0, 1) for k in ("gate", "up", "down")])
    for il in (0, 1):
        p = "blk.%d." % il
        w.update({p + "ffn_gate_inp.weight": (F32, [64, 4]), p + "ffn_gate_exps.weight": (Q4_K, [256, 32, 4]), p + "ffn_up_exps.weight": (Q4_K, [256, 32, 4]),
                  p + "ffn_down_exps.weight": (Q6_K, [256, 64, 4]), p + "attn_q.bias": (F32, [64]), p + "attn_k.bias": (F32, [32]), p + "attn_v.bias": (F32, [32]),
                  p + "attn_q_norm.weight": (F32, [32]), p + "attn_k_norm.weight": (F32, [32])})
    with ServerProcess(server_bin, extra=["--gguf", _any_gguf(tmp_path)]) as s:
        c = Client(s.port)
        gb, inp, pos, out = _graph_case(c, [0, 1], T=2, weights=w)
        x = np.arange(128, dtype=np.float32).reshape(2, 64)
        c.set_tensor(gb.descriptor(inp), 0, x.tobytes())
        c.set_tensor(gb.descriptor(pos), 0, np.array([0, 1], np.int32).tobytes())
        c.send(R.GRAPH_COMPUTE, gb.payload())
        got = np.frombuffer(c.get_tensor(gb.descriptor(out), 0, 2 * 64 * 4), np.float32).reshape(2, 64)
        assert np.array_equal(got, _expected(x, [0, 1], 0, 2, 64).astype(np.float32))
        c.close()


@pytest.mark.parametrize("case", ["empty", "truncated", "trailing", "dangling-source", "duplicate-id", "not-a-layer-graph", "layers-1-and-3", "fused-qkv",
                                  "layer-without-ffn", "result-outside-buffer", "row-selection", "two-inputs", "recompute-without-a-graph", "no-model-file"])
def test_graphs_this_build_cannot_run_end_the_connection_with_a_reason(server_bin, tmp_path, case):
    """A malformed payload, a graph that is not the decoder sub-graph of one contiguous layer range, or one that needs
    something the stage has no kernel for: the request fails, which ends the connection (what a failing request does in
    the reference), and the log says why."""
    import rpc_graph_util as GU
    extra = [] if case == "no-model-file" else ["--gguf", _any_gguf(tmp_path)]
    with ServerProcess(server_bin, extra=extra) as s:
        c = Client(s.port)
        reason = None
        if case == "empty":
            payload, reason = struct.pack("<II", 0, 0), "malformed"
        elif case == "recompute-without-a-graph":
            c.send(R.GRAPH_RECOMPUTE, struct.pack("<I", 0))
            payload, reason = None, "no stored graph"
        elif case == "not-a-layer-graph":
            h, _ = c.alloc_buffer(1 << 16)
            gb = GU.GraphBuilder(h, c.buffer_get_base(h))
            a, b = gb.leaf("a", F32, [8]), gb.leaf("b", F32, [8])
            gb.node("sum", "ADD", [8], [a, b])
            payload, reason = gb.payload(), "not a decoder layer sub-graph"
        else:
            kw, layers = {}, [1, 2]
            if case == "layers-1-and-3":
                layers, reason = [1, 3], "contiguous"
            if case == "fused-qkv":
                kw["weights"], reason = _fake_weights(layers, extra={"blk.1.attn_qkv.weight": (Q4_K, [256, 128])}), "no kernel for this weight"
            if case == "layer-without-ffn":
                kw["weights"], reason = _fake_weights(layers, drop=["blk.2.ffn_up.weight"]), "feed-forward"
            gb, inp, pos, out = _graph_case(c, layers, T=3, **kw) if case not in ("fused-qkv", "layer-without-ffn") else (None, None, None, None)
            if gb is None:
                # these two cannot be built by the layer builder (it would dereference the odd weight set): assemble by hand
                h, _ = c.alloc_buffer(8 << 20)
                gb = GU.GraphBuilder(h, c.buffer_get_base(h))
                w = {n: gb.leaf(n, t, d) for n, (t, d) in kw["weights"].items()}
                x = gb.leaf("RPC0#l_out-0#0", F32, [64, 3])
                gb.leaf("RPC0#inp_pos#0", GU.I32, [3])
                cur = x
                for n, wid in w.items():
                    cur = gb.node("use-" + n, "MUL_MAT", [64, 3], [wid, cur])
            payload = gb.payload()
            if case == "truncated":
                payload, reason = payload[:-100], "malformed"
            elif case == "trailing":
                payload, reason = payload + b"\0" * 8, "malformed"
            elif case == "dangling-source":
                payload, reason = gb.payload(drop=[inp]), "malformed"
            elif case == "duplicate-id":
                first = next(iter(gb.tensors.values()))
                payload = gb.payload()
                payload = payload[:-len(first)] + first                    # the last descriptor replaced by a copy of the first
                reason = "malformed"
            elif case == "result-outside-buffer":
                t = list(struct.unpack(R.TENSOR_FMT, gb.tensors[out]))
                t[-3] += 64 << 20
                gb.tensors[out] = struct.pack(R.TENSOR_FMT, *t)
                payload, reason = gb.payload(), "does not lie inside its buffer"
            elif case == "row-selection":
                t = list(struct.unpack(R.TENSOR_FMT, gb.tensors[out]))
                t[4] = 1                                                    # ne[1]: one output row for three tokens
                gb.tensors[out] = struct.pack(R.TENSOR_FMT, *t)
                payload, reason = gb.payload(), "row selection"
            elif case == "two-inputs":
                extra_in = gb.leaf("RPC0#other#0", F32, [64, 3])
                gb.node("mix", "ADD", [64, 3], [extra_in, out])
                payload, reason = gb.payload(), "candidates for the hidden-state input"
            elif case == "no-model-file":
                reason = "--gguf"
        if payload is not None:
            c.send(R.GRAPH_COMPUTE, payload)
        assert c.closed_by_server(), case
        c.close()
        log = s.stop()
        assert reason in log, (case, log[-600:])


# ---- SET_TENSOR_GGUF (patches/0001:179-266)
def write_small_model(path):
    rng = np.random.Generator(np.random.PCG64(7))
    tensors = [
        ("blk.0.attn_norm.weight", F32, (512,), rng.standard_normal(512).astype(np.float32).view(np.uint8)),
        ("blk.0.attn_q.weight", Q4_K, (512, 64), rng.integers(0, 256, 64 * 2 * 144, dtype=np.uint8)),
        ("blk.0.ffn_down.weight", Q6_K, (256, 32), rng.integers(0, 256, 32 * 210, dtype=np.uint8)),
    ]
    G.write_gguf(path, [("general.architecture", G.T_STR, "llama")], tensors)
    return {n: (t, d, b.tobytes()) for n, t, d, b in tensors}


def test_set_tensor_gguf_loads_by_name(server_bin, tmp_path):
    path = str(tmp_path / "w.gguf")
    model = write_small_model(path)
    with ServerProcess(server_bin, extra=["--gguf", path]) as s:
        c = Client(s.port)
        h, _ = c.alloc_buffer(1 << 16)
        base = c.buffer_get_base(h)
        at = base
        for name, (ttype, dims, raw) in model.items():
            if ttype == F32:
                t = tensor(h, at, dims, [4, 4 * dims[0]] + [4 * dims[0]] * 2, ttype, name.encode())
            else:
                bb = {Q4_K: 144, Q6_K: 210}[ttype]
                row = dims[0] // 256 * bb
                t = tensor(h, at, dims, [bb, row, row * dims[1], row * dims[1]], ttype, name.encode())
            assert c.set_tensor_gguf(t) == 1, name
            assert c.get_tensor(t, 0, len(raw)) == raw, name
            at += (len(raw) + 255) // 256 * 256
        name, (ttype, dims, raw) = "blk.0.attn_norm.weight", model["blk.0.attn_norm.weight"]
        # absent name, wrong size, wrong type: result 0 and the client falls back to sending the bytes (patches/0001:73-91)
        assert c.set_tensor_gguf(tensor(h, base, dims, [4, 2048, 2048, 2048], F32, b"blk.9.attn_norm.weight")) == 0
        assert c.set_tensor_gguf(tensor(h, base, (256,), [4, 1024, 1024, 1024], F32, name.encode())) == 0
        assert c.set_tensor_gguf(tensor(h, base, dims, [2, 1024, 1024, 1024], 1, name.encode())) == 0
        # destination outside the buffer
        assert c.set_tensor_gguf(tensor(h, base + (1 << 16) - 64, dims, [4, 2048, 2048, 2048], F32, name.encode())) == 0
        assert c.device_count() == 2
        c.close()


def test_set_tensor_gguf_without_a_model_file(server_bin):
    with ServerProcess(server_bin) as s:
        c = Client(s.port)
        h, _ = c.alloc_buffer(4096)
        base = c.buffer_get_base(h)
        assert c.set_tensor_gguf(f32_tensor(h, base, 512, b"blk.0.attn_norm.weight")) == 0
        c.close()


def test_two_clients_share_buffers_and_peers(server_bin):
    """Server state is per process, not per connection (patches/0002:2309-2329): a buffer allocated on one connection is
    addressable from another, which is what a pushed PEER_TENSOR_DATA relies on."""
    with ServerProcess(server_bin) as s:
        c1, c2 = Client(s.port), Client(s.port)
        h, _ = c1.alloc_buffer(256)
        base = c1.buffer_get_base(h)
        t = f32_tensor(h, base, 64)
        c1.set_tensor(t, 0, bytes(range(256)))
        c1.device_count()                       # SET_TENSOR has no reply: a later reply orders it before the other connection reads
        assert c2.get_tensor(t, 0, 256) == bytes(range(256))
        c1.close()
        assert c2.get_tensor(t, 0, 256) == bytes(range(256))      # the buffer outlives the connection that made it
        c2.close()
