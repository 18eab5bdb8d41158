"""Kernel-selection switches: one table, set as text when a stage is opened and by name on a session.  The parsing runs
before any device call, so its refusals are checked without a GPU; the session side is checked on one."""
import os
import re

import numpy as np
import pytest

import models
from util import ROOT, mesh


def documented_switches():
    """name -> default, from the comment of mesh_session_set_option in the header."""
    text = open(os.path.join(ROOT, "include", "mesh_stage.h")).read()
    block = text[text.index("Kernel-selection switches."):text.index("int mesh_session_set_option(")]
    return {n: int(v) for n, v in re.findall(r"\b([a-z][a-z0-9_]+)=(\d+)\b", block) if n not in ("name",)}


def table_switches():
    text = open(os.path.join(ROOT, "mesh-llm_amd", "csrc", "tuning.cpp")).read()
    return re.findall(r'\{"([a-z0-9_]+)", &Tuning::\1,', text)


def test_header_documents_every_switch_of_the_table():
    doc, table = documented_switches(), table_switches()
    assert len(table) >= 20
    assert sorted(doc) == sorted(table)
    text = open(os.path.join(ROOT, "mesh-llm_amd", "csrc", "tuning.hpp")).read()
    for name, default in doc.items():
        assert re.search(r"\bint %s = %d;" % (name, default), text), "default of %s differs between header and table" % name


def test_nothing_else_reads_the_environment_for_tuning():
    src = os.path.join(ROOT, "mesh-llm_amd", "csrc")
    seen = []
    for d, _, files in os.walk(src):
        for f in files:
            if f.endswith((".hip", ".cpp", ".hpp", ".inc")):
                for var in re.findall(r'getenv\("(MESH_[A-Z0-9_]+)"\)', open(os.path.join(d, f)).read()):
                    seen.append((f, var))
    assert sorted(seen) == [("plugin_main.cpp", "MESH_LLM_PLUGIN_ENDPOINT"), ("plugin_main.cpp", "MESH_LLM_PLUGIN_NAME"),
                            ("plugin_main.cpp", "MESH_LLM_PLUGIN_TRANSPORT"), ("tuning.cpp", "MESH_TUNING")]


@pytest.mark.parametrize("text,fragment", [
    ("skinny_f17=1", "no switch named 'skinny_f17'"),
    ("skinny_f16=2", "outside [0, 1]"),
    ("gemm_min_tokens=0", "outside [1,"),
    ("skinny_f16", "not name=integer"),
    ("skinny_f16=", "not name=integer"),
    ("=1", "not name=integer"),
    ("skinny_f16=1x", "not name=integer"),
    ("graphs=1,moe_group=-1", "moe_group=-1 outside"),
])
def test_bad_tuning_text_is_refused_before_any_device_call(tmp_path, text, fragment):
    m = mesh()
    cfg = models.CONFIGS["tiny-llama"]
    path = os.path.join(str(tmp_path), "t.gguf")
    models.write_model(path, cfg, [0], seed=1)
    with pytest.raises(m.MeshError) as e:
        m.Stage(path, 0, 1, n_ctx=32, tuning=text)
    assert e.value.code == m.ERR_INVALID, e.value.message
    assert "mesh_stage_opts.tuning" in e.value.message and fragment in e.value.message, e.value.message


def test_environment_string_is_read_once_per_process_and_checked(tmp_path):
    """MESH_TUNING holds the same text as mesh_stage_opts.tuning; a bad one makes mesh_stage_open fail with a message that
    names the variable (a process of its own: the library reads it once)."""
    import subprocess
    import sys
    cfg = models.CONFIGS["tiny-llama"]
    path = os.path.join(str(tmp_path), "t.gguf")
    models.write_model(path, cfg, [0], seed=1)
    prog = ("import sys; sys.path.insert(0, %r); sys.path.insert(0, %r)\n"
            "from util import mesh\n"
            "m = mesh()\n"
            "try:\n"
            "    m.Stage(%r, 0, 1, n_ctx=32)\n"
            "    print('opened')\n"
            "except m.MeshError as e:\n"
            "    print(e.code, e.message)\n") % (ROOT, os.path.join(ROOT, "tests"), path)
    for text, expect in (("skinny_f16=3", "MESH_TUNING: tuning: skinny_f16=3 outside [0, 1]"), ("nonsense", "MESH_TUNING: 'nonsense' is not name=integer")):
        out = subprocess.run([sys.executable, "-c", prog], env=dict(os.environ, MESH_TUNING=text), capture_output=True, text=True, timeout=120).stdout
        assert out.startswith("-1 ") and expect in out, out
    # a good one gets past the parser: what stops the call on a machine without a GPU is the device, not the text
    out = subprocess.run([sys.executable, "-c", prog], env=dict(os.environ, MESH_TUNING=" graphs=1 , skinny_f16=0 "), capture_output=True, text=True, timeout=120).stdout
    assert "MESH_TUNING" not in out, out


@pytest.mark.gpu
def test_session_options_round_trip_and_levels(tmp_path):
    m = mesh()
    cfg = models.CONFIGS["tiny-llama"]
    path = os.path.join(str(tmp_path), "t.gguf")
    models.write_model(path, cfg, [0, 1], seed=1)
    st = m.Stage(path, 0, 2, n_ctx=64, n_seq_max=4, n_batch_max=32, tuning=" skinny_f16 = 0, gemm_min_tokens=20 ")
    ses = st.session()
    doc = documented_switches()
    for name, default in doc.items():
        want = {"skinny_f16": 0, "gemm_min_tokens": 20}.get(name, default)
        assert ses.get_option(name) == want, name
    # a session-level switch changes for this session only
    ses.set_option("skinny_f16", 1)
    other = st.session()
    assert ses.get_option("skinny_f16") == 1 and other.get_option("skinny_f16") == 0
    # stage-level switches decide allocations and are refused on a session; unknown names and bad values too
    for name, value in (("gemm_min_tokens", 17), ("gemm_layout", 0), ("skinny_min_tokens", 8), ("nope", 1), ("graphs", 7)):
        with pytest.raises(m.MeshError) as e:
            ses.set_option(name, value)
        assert e.value.code == m.ERR_INVALID
    assert ses.get_option("gemm_min_tokens") == 20
    # switching between calls takes effect on the next call: 8 tokens through the integer and the f16 skinny kernels
    # differ in rounding, and each equals a fresh session created with that value
    E = cfg["n_embd"]
    x = np.random.Generator(np.random.PCG64(4)).standard_normal((8, E)).astype(np.float32)
    seqs = [0, 1, 2, 3, 0, 1, 2, 3]
    pos = [0, 0, 0, 0, 1, 1, 1, 1]
    a16 = ses.decode(x, pos, seq=seqs).copy()
    ses.set_option("skinny_f16", 0)
    a8 = ses.decode(x, pos, seq=seqs).copy()
    b8 = other.decode(x, pos, seq=seqs).copy()
    fresh16 = st.session(skinny_f16=1)
    b16 = fresh16.decode(x, pos, seq=seqs).copy()
    assert np.array_equal(a8, b8) and np.array_equal(a16, b16)
    for s in (ses, other, fresh16):
        s.close()
    st.close()
