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
