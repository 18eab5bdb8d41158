"""The rpc-server binary on a real GPU: the reference's transfer cases and a local-GGUF load with buffers in HBM."""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import rpc_cases
from rpc_client import Client, ServerProcess, tensor
from test_rpc_server import parse_available_devices, write_small_model, F32, Q4_K, Q6_K

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "mesh-llm_amd", "rpc-server")


@pytest.fixture(scope="module")
def server_bin():
    assert os.access(BINARY, os.X_OK), "mesh-llm_amd/rpc-server is not built (run __graft_entry__.build())"
    return BINARY


def test_device_probe_names_the_gpu(server_bin):
    import subprocess
    r = subprocess.run([server_bin, "-d", "__mesh_llm_probe_invalid__", "-p", "0"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "ROCm0" in parse_available_devices(r.stdout + "\n" + r.stderr)


def test_direct_push_between_two_servers(server_bin):
    rpc_cases.direct_push(server_bin)


def test_large_push_between_two_servers(server_bin):
    rpc_cases.large_push(server_bin)


def test_fallback_on_failed_push(server_bin):
    rpc_cases.fallback_on_failed_push(server_bin)


def test_device_memory_and_gguf_load_into_hbm(server_bin, tmp_path):
    path = str(tmp_path / "w.gguf")
    model = write_small_model(path)
    with ServerProcess(server_bin, extra=["-d", "ROCm0", "--gguf", path]) as s:
        c = Client(s.port)
        assert c.version == (4, 1, 0) and c.device_count() == 1
        free, total = c.device_memory(0)
        assert total > (200 << 30) and 0 < free <= total           # 288 GB of HBM3E
        h, _ = c.alloc_buffer(1 << 20)
        base = c.buffer_get_base(h)
        assert c.buffer_clear(h, 0)
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
        assert c.free_buffer(h)
        c.close()


@pytest.mark.parametrize("name,lb,le,with_output", [("tiny-llama", 1, 3, False), ("tiny-qwen2", 1, 3, True), ("tiny-moe", 0, 2, False)])
def test_graph_compute_of_a_layer_range_equals_the_stage_library(server_bin, tmp_path, name, lb, le, with_output):
    """GRAPH_COMPUTE with the decoder sub-graph of a layer range, tensors in HBM buffers of the server: a 5-token prompt
    chunk, then single-token steps replayed with GRAPH_RECOMPUTE (same graph, new input and position).  The hidden states
    (or, through the last layer, the logits) the client reads back are bit for bit what mesh_stage_decode of the same
    range returns, and within the stage tolerance of the CPU oracle."""
    import models
    import rpc_graph_util as GU
    from oracle.stage import StageOracle
    from util import mesh
    m = mesh()
    cfg = models.CONFIGS[name]
    path = str(tmp_path / (name + ".gguf"))
    extra = ("output",) if with_output else ()
    tensors = models.write_model(path, cfg, range(lb, le), seed=11, **({"with_output": True} if with_output else {}))
    E, n_ctx = cfg["n_embd"], 64
    weights = {n: (t, list(d)) for n, (t, d, _) in tensors.items() if n.startswith("blk.") or (with_output and n in ("output_norm.weight", "output.weight", "token_embd.weight"))}
    if with_output and "output.weight" in weights:
        weights.pop("token_embd.weight", None)
    st = m.Stage(path, lb, le, n_ctx=n_ctx, n_seq_max=1, n_batch_max=512)
    ses = st.session()
    orc = StageOracle(cfg, tensors, lb, le, n_ctx)
    rng = np.random.Generator(np.random.PCG64(5))
    with ServerProcess(server_bin, extra=["-d", "ROCm0", "--gguf", path]) as s:
        c = Client(s.port)
        steps = [(5, 0), (1, 5), (1, 6)]
        graphs = {}
        for T, p0 in steps:
            if T not in graphs:
                h, _ = c.alloc_buffer(64 << 20)
                gb = GU.GraphBuilder(h, c.buffer_get_base(h))
                graphs[T] = (gb,) + GU.layer_range_graph(gb, weights, list(range(lb, le)), T, cfg["n_head"], cfg["n_head_kv"], cfg["head_dim"], n_ctx,
                                                         with_output=with_output)
                fresh = True
            else:
                fresh = False
            gb, inp, pos, out = graphs[T]
            x = rng.standard_normal((T, E)).astype(np.float32)
            positions = np.arange(p0, p0 + T, dtype=np.int32)
            c.set_tensor(gb.descriptor(inp), 0, x.tobytes())
            c.set_tensor(gb.descriptor(pos), 0, positions.tobytes())
            if fresh:
                c.send(R_GRAPH_COMPUTE, gb.payload())
            else:
                c.send(R_GRAPH_RECOMPUTE, (0).to_bytes(4, "little"))
            rows = struct_ne0(gb.descriptor(out))
            got = np.frombuffer(c.get_tensor(gb.descriptor(out), 0, T * rows * 4), np.float32).reshape(T, rows)
            want = ses.decode(x, positions, out_fmt=m.LOGITS if with_output else m.F32).view(np.float32).reshape(T, rows)
            assert np.array_equal(got, want), (T, p0)
            ref = orc.logits(orc.forward(x, positions)) if with_output else orc.forward(x, positions)
            rel = float(np.linalg.norm(got.astype(np.float64) - ref) / np.linalg.norm(ref))
            assert rel <= 1e-2, (T, p0, rel)
        c.close()
        log = s.stop()
        assert "opened as a stage" in log
    ses.close(); st.close()


def test_graph_recompute_step_through_the_server_costs_little_more_than_the_library_call(server_bin, tmp_path):
    """What the front end adds to a decode step: two real-shape layers (Llama-3-8B shape), single-token steps as a client
    drives them -- SET_TENSOR of the hidden state and of the position, GRAPH_RECOMPUTE, GET_TENSOR of the result -- against
    mesh_stage_decode of the same layers on host buffers in this process.  Bit-identical results; the difference in wall
    time per step is the four messages over loopback, their handling in the server and this Python client."""
    import time
    import models
    import rpc_graph_util as GU
    from util import mesh
    m = mesh()
    name, lb, le = "llama3-8b", 3, 5
    cfg = models.CONFIGS[name]
    path = str(tmp_path / (name + ".gguf"))
    tensors = models.write_model(path, cfg, range(lb, le), seed=11)
    E, n_ctx = cfg["n_embd"], 256
    weights = {n: (t, list(d)) for n, (t, d, _) in tensors.items() if n.startswith("blk.")}
    st = m.Stage(path, lb, le, n_ctx=n_ctx, n_seq_max=1, n_batch_max=16)
    ses = st.session()
    rng = np.random.Generator(np.random.PCG64(6))
    n_steps = 120
    xs = rng.standard_normal((n_steps, 1, E)).astype(np.float32)
    with ServerProcess(server_bin, extra=["-d", "ROCm0", "--gguf", path]) as s:
        c = Client(s.port)
        h, _ = c.alloc_buffer(512 << 20)       # (the graph's weight leaves lie in the client's buffer too: 2 x 218 MB)
        gb = GU.GraphBuilder(h, c.buffer_get_base(h))
        inp, pos, out = GU.layer_range_graph(gb, weights, list(range(lb, le)), 1, cfg["n_head"], cfg["n_head_kv"], cfg["head_dim"], n_ctx)
        d_in, d_pos, d_out = gb.descriptor(inp), gb.descriptor(pos), gb.descriptor(out)
        got, want = [], []
        t_rpc = t_lib = 0.0
        for i in range(n_steps):
            p = np.array([i], np.int32)
            t0 = time.perf_counter()
            c.set_tensor(d_in, 0, xs[i].tobytes())
            c.set_tensor(d_pos, 0, p.tobytes())
            if i == 0:
                c.send(R_GRAPH_COMPUTE, gb.payload())
            else:
                c.send(R_GRAPH_RECOMPUTE, (0).to_bytes(4, "little"))
            try:
                r = c.get_tensor(d_out, 0, E * 4)
            except ConnectionError:
                raise AssertionError("the server closed the connection: " + s.stop()[-2000:])
            t1 = time.perf_counter()
            w = ses.decode(xs[i], p).copy()
            t2 = time.perf_counter()
            got.append(np.frombuffer(r, np.float32))
            want.append(w.view(np.float32).reshape(-1))
            if i >= 20:                     # (the first steps open the stage and warm both paths)
                t_rpc += t1 - t0
                t_lib += t2 - t1
        c.close()
        s.stop()
    for i, (a, b) in enumerate(zip(got, want)):
        assert np.array_equal(a, b), i
    n = n_steps - 20
    print("[rpc] decode step of 2 real-shape layers: %.1f us through rpc-server (4 messages), %.1f us through the library; the front end adds %.1f us"
          % (t_rpc / n * 1e6, t_lib / n * 1e6, (t_rpc - t_lib) / n * 1e6))
    assert (t_rpc - t_lib) / n < 2e-3          # a loose bound: loopback round trips and a Python client, not a regression gate for microseconds
    ses.close(); st.close()


R_GRAPH_COMPUTE, R_GRAPH_RECOMPUTE = 10, 16


def struct_ne0(descriptor):
    import struct
    from rpc_client import TENSOR_FMT
    return struct.unpack(TENSOR_FMT, descriptor)[3]
