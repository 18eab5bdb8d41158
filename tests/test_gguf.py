"""CPU-only tests of the GGUF reader behind the C ABI, mirroring the reference's own reader tests
(mesh-client/src/models/gguf.rs:621-758: hostile array nesting, negative / excessive counts) and the
tensor-by-name lookup of rpc_server::set_tensor_gguf (patches/0001:203-209,228-239)."""
import os
import struct

import numpy as np
import pytest

import gguf_util as G
import models
from util import mesh


def _write(tmp_path, name, data):
    p = os.path.join(str(tmp_path), name)
    with open(p, "wb") as f:
        f.write(data)
    return p


def test_probe_reads_hparams_and_skips_arrays(tmp_path):
    m = mesh()
    cfg = models.CONFIGS["tiny-llama"]
    path = os.path.join(str(tmp_path), "tiny.gguf")
    tensors = models.write_model(path, cfg, range(cfg["n_layer"]), with_embd=True, with_output=True)
    info = m.gguf_probe(path)
    assert info.arch == b"llama"
    assert (info.n_layer, info.n_embd, info.n_head, info.n_head_kv, info.head_dim, info.n_ff) == (4, 256, 4, 2, 64, 512)
    assert info.n_vocab == 512 and info.rope_mode == 0 and info.n_rot == 64
    assert abs(info.rms_eps - 1e-5) < 1e-12 and info.rope_freq_base == 1e4
    assert info.gguf_version == 3 and info.alignment == 32 and info.n_tensors == len(tensors)
    assert info.data_offset % 32 == 0 and info.file_size == os.path.getsize(path)


def test_tensor_lookup_matches_file_bytes(tmp_path):
    m = mesh()
    cfg = models.CONFIGS["tiny-llama"]
    path = os.path.join(str(tmp_path), "tiny.gguf")
    tensors = models.write_model(path, cfg, [1, 2])
    raw = np.fromfile(path, dtype=np.uint8)
    for name, (ttype, dims, data) in tensors.items():
        ti = m.gguf_tensor(path, name)
        assert ti.type == ttype and ti.n_dims == len(dims) and list(ti.ne[:len(dims)]) == list(dims)
        assert ti.nbytes == data.nbytes and ti.file_offset % 32 == 0
        assert np.array_equal(raw[ti.file_offset:ti.file_offset + ti.nbytes], data.reshape(-1))
    with pytest.raises(m.MeshError) as e:
        m.gguf_tensor(path, "blk.0.attn_q.weight")     # layer 0 was not written
    assert e.value.code == m.ERR_INVALID and "not found" in e.value.message


def test_tensor_outside_file_is_rejected(tmp_path):
    m = mesh()
    cfg = models.CONFIGS["tiny-llama"]
    path = os.path.join(str(tmp_path), "trunc.gguf")
    models.write_model(path, cfg, [0])
    size = os.path.getsize(path)
    with open(path, "r+b") as f:
        f.truncate(size - 4096)
    with pytest.raises(m.MeshError) as e:
        m.gguf_tensor(path, "blk.0.ffn_down.weight")
    assert e.value.code == m.ERR_FORMAT and "outside the file" in e.value.message


def _head(n_tensors, n_kv, version=2):
    return b"GGUF" + struct.pack("<Iqq", version, n_tensors, n_kv)


def _arch_kvs():
    return b"".join(G.kv_bytes(*kv) for kv in [
        ("general.architecture", G.T_STR, "llama"), ("llama.block_count", G.T_U32, 2),
        ("llama.embedding_length", G.T_U32, 256), ("llama.attention.head_count", G.T_U32, 4)])


def test_rejects_what_the_reference_reader_rejects(tmp_path):
    m = mesh()

    def code(data):
        with pytest.raises(m.MeshError) as e:
            m.gguf_probe(_write(tmp_path, "bad.gguf", data))
        return e.value.code, e.value.message

    assert code(b"GGML" + b"\0" * 64)[0] == m.ERR_FORMAT                       # magic
    assert code(_head(0, 0, version=1) + b"\0" * 8)[0] == m.ERR_FORMAT         # version < 2
    assert code(_head(0, -1) + b"\0" * 8)[0] == m.ERR_FORMAT                   # negative KV count
    assert code(_head(1_000_001, 0) + b"\0" * 8)[0] == m.ERR_FORMAT            # excessive tensor count
    assert code(b"GGUF")[0] == m.ERR_FORMAT                                    # too short
    # array nested deeper than 64
    nested = _head(0, 1) + G._s("general.architecture") + struct.pack("<I", G.T_ARR)
    for _ in range(65):
        nested += struct.pack("<IQ", G.T_ARR, 1)
    nested += struct.pack("<IQ", G.T_U8, 1) + b"\0"
    c, msg = code(nested)
    assert c == m.ERR_FORMAT and "nesting too deep" in msg
    # array longer than 1e6 elements
    c, msg = code(_head(0, 1) + G._s("x") + struct.pack("<IIQ", G.T_ARR, G.T_U8, 1_000_001))
    assert c == m.ERR_FORMAT and "array too long" in msg
    # string longer than 1e6 bytes
    c, msg = code(_head(0, 1) + struct.pack("<Q", 1_000_001))
    assert c == m.ERR_FORMAT and "string too long" in msg
    # truncated in the middle of the KV table
    assert code(_head(0, 4) + _arch_kvs()[:-3])[0] == m.ERR_FORMAT
    # negative Int32 where an unsigned value is expected
    kv = G.kv_bytes("general.architecture", G.T_STR, "llama") + G.kv_bytes("llama.block_count", G.T_I32, -1)
    c, msg = code(_head(0, 2) + kv + b"\0" * 32)
    assert c == m.ERR_FORMAT and "block_count" in msg
    # tensor with more than 8 dimensions
    ti = G._s("t") + struct.pack("<I", 9)
    assert code(_head(1, 4) + _arch_kvs() + ti + b"\0" * 128)[0] == m.ERR_FORMAT
    # unknown architecture is UNSUPPORTED, not FORMAT
    kv = G.kv_bytes("general.architecture", G.T_STR, "mamba")
    assert code(_head(0, 1) + kv + b"\0" * 32)[0] == m.ERR_UNSUPPORTED
    with pytest.raises(m.MeshError) as e:
        m.gguf_probe(os.path.join(str(tmp_path), "missing.gguf"))
    assert e.value.code == m.ERR_IO


def test_alignment_key_moves_the_data_section(tmp_path):
    m = mesh()
    kvs = [("general.architecture", G.T_STR, "llama"), ("general.alignment", G.T_U32, 256), ("llama.block_count", G.T_U32, 1),
           ("llama.embedding_length", G.T_U32, 256), ("llama.attention.head_count", G.T_U32, 4)]
    data = np.arange(64, dtype=np.float32).view(np.uint8)
    path = os.path.join(str(tmp_path), "al.gguf")
    G.write_gguf(path, kvs, [("a", 0, (64,), data), ("b", 0, (64,), data)], alignment=256)
    info = m.gguf_probe(path)
    assert info.alignment == 256 and info.data_offset % 256 == 0
    tb = m.gguf_tensor(path, "b")
    assert tb.file_offset == info.data_offset + 256


def test_stage_open_without_gpu_or_with_bad_range_fails_cleanly(tmp_path):
    m = mesh()
    cfg = models.CONFIGS["tiny-llama"]
    path = os.path.join(str(tmp_path), "tiny.gguf")
    models.write_model(path, cfg, [0, 1])
    with pytest.raises(m.MeshError) as e:
        m.Stage(path, 3, 2)
    assert e.value.code == m.ERR_INVALID
    if m.device_count() == 0:
        with pytest.raises(m.MeshError) as e:
            m.Stage(path, 0, 2)
        assert e.value.code == m.ERR_DEVICE      # no CPU fallback: the product path fails loudly without a GPU
