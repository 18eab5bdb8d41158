"""mesh_act_pack_noalloc (the entry point that allocates no GPU memory: its device staging is a fixed array inside
the library) against mesh_act_pack, through the C ABI: bit-exact for every activation format, on calls in a row that
shrink and grow (the array keeps the previous call's contents), and refused with a clear error beyond its limit."""
import numpy as np
import pytest

from util import codec_input, mesh

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

LIMIT = 1 << 20


def test_noalloc_pack_equals_allocating_pack_on_consecutive_calls():
    m = mesh()
    rng = np.random.Generator(np.random.PCG64(404))
    big = codec_input(200).reshape(-1)                     # 200 x 4096 elements with the x50 outlier channels
    small = (rng.standard_normal(16 * 4096) * 3).astype(np.float32)
    tiny = np.array([0.0, -0.0, 1e-8, -65504.0, 70000.0, np.inf, -np.inf, np.nan] * 4, np.float32)
    full = rng.standard_normal(LIMIT).astype(np.float32)   # exactly the limit
    for fmt in (m.Q8_0, m.F16, m.F32):
        # a large call, then smaller ones, then the largest allowed, then small again
        for x in (big, small, tiny, full, small[:4096]):
            got = m.act_pack_noalloc(fmt, x)
            want = m.act_pack(fmt, x)
            assert got.size == m.act_packed_size(fmt, 1, x.size)
            assert np.array_equal(got, want), (fmt, x.size)


def test_noalloc_pack_limits_and_errors():
    m = mesh()
    x = np.zeros(LIMIT + 32, np.float32)
    with pytest.raises(m.MeshError) as e:
        m.act_pack_noalloc(m.Q8_0, x)
    assert e.value.code == m.ERR_INVALID and "exceed" in e.value.message
    with pytest.raises(m.MeshError) as e:
        m.act_pack_noalloc(m.Q8_0, x[:33])                 # not a whole number of blocks
    assert e.value.code == m.ERR_INVALID
    with pytest.raises(m.MeshError) as e:
        m.act_pack_noalloc(m.Q4_K, x[:256])                # not an activation format
    assert e.value.code == m.ERR_INVALID
    assert m.act_pack_noalloc(m.F16, x[:0]).size == 0
    # and the call still works after the refusals
    y = np.arange(64, dtype=np.float32)
    assert np.array_equal(m.act_pack_noalloc(m.Q8_0, y), m.act_pack(m.Q8_0, y))
