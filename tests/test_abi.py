"""CPU-only checks of the drop-in boundary: the library loads and exports every symbol of include/mesh_stage.h,
and the entry points that need no GPU behave as documented."""
import os
import re

import numpy as np
import pytest

from util import ROOT, mesh


def header_symbols():
    text = open(os.path.join(ROOT, "include", "mesh_stage.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mesh_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    m = mesh()
    L = m.lib()
    syms = header_symbols()
    assert len(syms) >= 9
    for s in syms:
        assert hasattr(L, s), "libmeshstage.so does not export %s" % s
        assert s in m.SIGNATURES, "binding has no signature for %s" % s
    assert sorted(m.SIGNATURES) == syms


def test_packed_size_is_ggml_nbytes():
    m = mesh()
    assert m.act_packed_size(m.Q8_0, 4096, 4096) == 4096 * 4096 // 32 * 34
    assert m.act_packed_size(m.Q8_0, 1, 896) == 28 * 34
    assert m.act_packed_size(m.F16, 512, 4096) == 512 * 4096 * 2
    assert m.act_packed_size(m.F32, 16, 4096) == 16 * 4096 * 4
    assert m.act_packed_size(m.Q8_0, 3, 100) == 0      # rows must be whole blocks
    assert m.act_packed_size(m.Q4_K, 1, 4096) == 0     # not an activation format
    assert m.act_packed_size(m.Q8_0, -1, 4096) == 0


def test_errors_are_codes_plus_message_not_exceptions():
    m = mesh()
    x = np.zeros(33, np.float32)
    with pytest.raises(m.MeshError) as e:
        m.act_pack(m.Q8_0, x)
    assert e.value.code == m.ERR_INVALID and "whole number of blocks" in e.value.message
    with pytest.raises(m.MeshError) as e:
        m.act_pack(m.Q4_K, np.zeros(256, np.float32))
    assert e.value.code == m.ERR_INVALID
    with pytest.raises(m.MeshError) as e:
        m.device_select("Vulkan0")
    assert e.value.code == m.ERR_INVALID
    with pytest.raises(m.MeshError) as e:
        m.hbm_read_probe(1024, 0, 1)        # below a megabyte: refused before any device call
    assert e.value.code == m.ERR_INVALID
    # zero elements is a no-op, not an error, and touches no device
    assert m.act_pack(m.Q8_0, np.zeros(0, np.float32)).size == 0
