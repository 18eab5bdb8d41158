"""mesh-stage-plugin with the stage open on a real GPU: the endpoint's stage route returns what the library returns."""
import json
import os
import sys
import urllib.request

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import models
import oracle
from oracle.stage import StageOracle
from plugin_host import PB, PluginHost
from util import mesh

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "mesh-llm_amd", "mesh-stage-plugin")


def test_stage_route_matches_library_and_oracle(tmp_path):
    assert os.access(BINARY, os.X_OK), "mesh-llm_amd/mesh-stage-plugin is not built (run __graft_entry__.build())"
    m = mesh()
    cfg = models.CONFIGS["tiny-llama"]
    path = str(tmp_path / "tiny.gguf")
    tensors = models.write_model(path, cfg, [1, 2], seed=3)
    host = PluginHost(BINARY, ["--gguf", path, "--layers", "1:3", "-d", "ROCm0", "-c", "64", "--batch", "16"], tmp_path, name="stage-b")
    init = host.initialize().initialize_response
    assert json.loads(init.server_info_json)["stage_open"] is True
    address = init.manifest.endpoints[0].address
    assert host.request(health_request=PB["HealthRequest"]()).health_response.status == 1
    E = cfg["n_embd"]
    rng = np.random.Generator(np.random.PCG64(4))
    x = rng.standard_normal((5, E)).astype(np.float32)
    packed_in = oracle.quantize_q8_0(x.reshape(-1)).tobytes()
    req = urllib.request.Request(address + "/stage/decode", data=packed_in, method="POST",
                                 headers={"X-Mesh-Tokens": "5", "X-Mesh-Pos0": "0", "X-Mesh-In-Format": "q8_0", "X-Mesh-Out-Format": "q8_0",
                                          "Content-Type": "application/octet-stream"})
    with urllib.request.urlopen(req, timeout=60) as r:
        assert r.status == 200
        got = r.read()
    # the same call through the library in this process
    st = m.Stage(path, 1, 3, n_ctx=64, n_seq_max=1, n_batch_max=16)
    ses = st.session()
    direct = ses.decode(np.frombuffer(packed_in, np.uint8), np.arange(5), in_fmt=m.Q8_0, out_fmt=m.Q8_0)
    assert got == direct.tobytes()
    # and the oracle on the dequantised input
    xin = oracle.dequantize(oracle.Q8_0, np.frombuffer(packed_in, np.uint8), x.size).reshape(5, E)
    want = StageOracle(cfg, tensors, 1, 3, 64).forward(xin, np.arange(5))
    got_f = oracle.dequantize(oracle.Q8_0, np.frombuffer(got, np.uint8), want.size)
    assert np.linalg.norm(got_f - want.reshape(-1)) / np.linalg.norm(want) < 1.5e-2      # q8_0 boundary rounding included
    # a second step continues the sequence; a wrong body size is refused
    req = urllib.request.Request(address + "/stage/decode", data=packed_in[:34 * (E // 32)], method="POST",
                                 headers={"X-Mesh-Tokens": "1", "X-Mesh-Pos0": "5"})
    with urllib.request.urlopen(req, timeout=60) as r:
        assert r.status == 200 and len(r.read()) == 34 * (E // 32)
    req = urllib.request.Request(address + "/stage/decode", data=b"123", method="POST", headers={"X-Mesh-Tokens": "1", "X-Mesh-Pos0": "6"})
    with pytest.raises(urllib.error.HTTPError) as err:
        urllib.request.urlopen(req, timeout=60)
    assert err.value.code == 400
    assert host.request(shutdown_request=PB["ShutdownRequest"](reason="done")).WhichOneof("payload") == "shutdown_response"
    host.close()
    assert host.proc.returncode == 0
    ses.close()
    st.close()
