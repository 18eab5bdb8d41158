"""mesh-stage-plugin against a stand-in plugin host (no GPU needed with --no-stage): the initialize / health / shutdown
exchange of mesh-llm/src/plugin/runtime.rs:237-290, the endpoint manifest an `inference::provider` emits
(plugin/src/dsl.rs:469-476, plugin/src/manifest.rs:378-395), and the GET <address>/models probe with which the host
decides that the endpoint is healthy and which models it serves (src/plugin/mod.rs:1633-1711)."""
import json
import os
import sys
import urllib.error
import urllib.request

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import gguf_util as G
import models
from plugin_host import PB, PluginHost
from util import mesh


@pytest.fixture(scope="session")
def plugin_bin(tmp_path_factory):
    mesh()
    from mesh_llm_amd import build
    return build.build_plugin(str(tmp_path_factory.mktemp("plugin") / "mesh-stage-plugin"))


def endpoint_models_url(address):
    """endpoint_models_url of src/plugin/mod.rs:1693-1711."""
    from urllib.parse import urlsplit, urlunsplit
    u = urlsplit(address)
    path = u.path.rstrip("/") or "/v1"
    if not path.endswith("/models"):
        path += "/models" if path.endswith("/v1") or path.endswith("/api/v1") else "/v1/models"
    return urlunsplit((u.scheme, u.netloc, path, "", ""))


def small_model(tmp_path):
    path = str(tmp_path / "tiny-llama-q4km.gguf")
    models.write_model(path, models.CONFIGS["tiny-llama"], [0, 1], seed=5)
    return path


def test_initialize_manifest_health_models_shutdown(plugin_bin, tmp_path):
    host = PluginHost(plugin_bin, ["--gguf", small_model(tmp_path), "--layers", "0:2", "--no-stage"], tmp_path, name="stage-a")
    rsp = host.initialize()
    assert rsp.WhichOneof("payload") == "initialize_response"
    init = rsp.initialize_response
    assert init.plugin_id == "stage-a" and init.plugin_protocol_version == 2          # what runtime.rs:274-288 checks
    info = json.loads(init.server_info_json)
    assert info["model"] == "tiny-llama-q4km" and info["layers"] == [0, 2] and info["n_embd"] == 256
    assert len(init.manifest.endpoints) == 1
    ep = init.manifest.endpoints[0]
    assert (ep.kind, ep.transport_kind, ep.protocol) == (1, 1, "openai_compatible")   # INFERENCE over HTTP: the pair probe_endpoint handles
    assert ep.managed_by_plugin and ep.endpoint_id == "stage" and ep.address.startswith("http://127.0.0.1:")
    # the host's health probe
    with urllib.request.urlopen(endpoint_models_url(ep.address), timeout=3) as r:
        assert r.status == 200
        ids = [e["id"] for e in json.load(r)["data"]]
    assert ids == ["tiny-llama-q4km"]
    # health and an unknown request
    h = host.request(health_request=PB["HealthRequest"]())
    assert h.WhichOneof("payload") == "health_response" and h.health_response.status == 1
    e = host.request(rpc_request=PB["RpcRequest"](method="tools/list", params_json="{}"))
    assert e.WhichOneof("payload") == "error_response" and e.error_response.code == -32601
    # the OpenAI routes a stage cannot serve, and the stage route without an open stage
    for path, code in (("/chat/completions", 501), ("/stage/decode", 503), ("/nothing", 404)):
        req = urllib.request.Request(ep.address + path, data=b"{}", method="POST")
        with pytest.raises(urllib.error.HTTPError) as err:
            urllib.request.urlopen(req, timeout=3)
        assert err.value.code == code and "error" in json.load(err.value)
    s = host.request(shutdown_request=PB["ShutdownRequest"](reason="test over"))
    assert s.WhichOneof("payload") == "shutdown_response"
    host.close()
    assert host.proc.returncode == 0


def test_plugin_leaves_when_the_host_goes_away(plugin_bin, tmp_path):
    host = PluginHost(plugin_bin, ["--gguf", small_model(tmp_path), "--no-stage"], tmp_path)
    host.initialize()
    host.close()                             # no ShutdownRequest: the socket just closes
    assert host.proc.returncode == 0


def test_oversized_and_malformed_frames_end_the_plugin(plugin_bin, tmp_path):
    import struct
    host = PluginHost(plugin_bin, ["--gguf", small_model(tmp_path), "--no-stage"], tmp_path)
    host.conn.sendall(struct.pack("<I", 16 * 1024 * 1024 + 1))        # io.rs:178-180: "Plugin frame too large"
    out = host.close()
    assert host.proc.returncode == 1 and "16 MiB" in out
    host = PluginHost(plugin_bin, ["--gguf", small_model(tmp_path), "--no-stage"], tmp_path)
    host.send_raw(b"\x52\xff\xff\xff\xff\x0f")                         # a length-delimited field that claims more bytes than the frame has
    out = host.close()
    assert host.proc.returncode == 1 and "malformed" in out


def test_startup_failures(plugin_bin, tmp_path):
    import subprocess
    env = {k: v for k, v in os.environ.items() if not k.startswith("MESH_LLM_PLUGIN_")}
    r = subprocess.run([plugin_bin, "--gguf", small_model(tmp_path), "--no-stage"], env=env, capture_output=True, text=True, timeout=30)
    assert r.returncode == 1 and "MESH_LLM_PLUGIN_ENDPOINT is not set" in r.stderr      # io.rs:119-120
    r = subprocess.run([plugin_bin, "--gguf", str(tmp_path / "missing.gguf"), "--no-stage"], env=env, capture_output=True, text=True, timeout=30)
    assert r.returncode == 1
    r = subprocess.run([plugin_bin], env=env, capture_output=True, text=True, timeout=30)
    assert r.returncode == 2
