"""The persistent single-launch decode kernel against the oracle and against the per-projection kernels.

Batches of up to four single-token sequences on a dense K-quant stage with head_dim 128 run every layer in one
cooperative launch (csrc/decode_mega.hip) when the session is created with MESH_STAGE_PERSISTENT=1.  The same
steps are replayed on a default session (per-projection kernels) and on the CPU oracle; `persistent_steps` proves which path ran.
Graph: rpc_server::graph_compute, third_party/llama.cpp/patches/0002-rpc-add-direct-peer-tensor-transfers.patch:443-451.
"""
import os

import numpy as np
import pytest

import models
from oracle.stage import StageOracle
from util import mesh

torch = pytest.importorskip("torch")     # before the library loads: torch brings its own HIP runtime of the same soname
pytestmark = pytest.mark.gpu


def rel_l2(a, b):
    a = np.asarray(a, np.float64).reshape(-1)
    b = np.asarray(b, np.float64).reshape(-1)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def _sessions(tmp_path, name, n_ctx, n_seq, seed=5):
    m = mesh()
    cfg = models.CONFIGS[name]
    nl = min(cfg["n_layer"], 2)
    # the first two layers; under the Q4_K_M map at least one of them carries q6_K attn_v / ffn_down
    path = os.path.join(str(tmp_path), name + ".gguf")
    tensors = models.write_model(path, cfg, range(nl), seed=seed)
    st = m.Stage(path, 0, nl, n_ctx=n_ctx, n_seq_max=n_seq, n_batch_max=16)
    os.unlink(path)
    os.environ["MESH_STAGE_PERSISTENT"] = "1"
    try:
        fast = st.session()
    finally:
        del os.environ["MESH_STAGE_PERSISTENT"]
    plain = st.session()
    orc = StageOracle(cfg, tensors, 0, nl, n_ctx, n_seq_max=n_seq)
    return m, cfg, nl, st, fast, plain, orc


def _seed_kv(rng, cfg, nl, sessions, orc, n_seq, depth):
    hk, hd = cfg["n_head_kv"], cfg["head_dim"]
    for il in range(nl):
        for s in range(n_seq):
            k = (rng.standard_normal((depth, hk, hd)) * 0.5).astype(np.float16).view(np.uint16)
            v = (rng.standard_normal((depth, hk, hd)) * 0.5).astype(np.float16).view(np.uint16)
            for ses in sessions:
                ses.kv_write(il, s, 0, k, v)
            orc.k[il, s, :, :depth] = k.transpose(1, 0, 2)
            orc.v[il, s, :, :depth] = v.transpose(1, 0, 2)


@pytest.mark.parametrize("name,depth", [("tiny-qwen2", 0), ("tiny-qwen2", 700), ("tiny-g5", 150), ("tiny-g8", 257),
                                        ("tiny-g2", 64), ("tiny-g7", 33)])
def test_persistent_decode_matches_oracle_and_plain_path(tmp_path, name, depth):
    n_ctx, n_seq = 1024, 4
    m, cfg, nl, st, fast, plain, orc = _sessions(tmp_path, name, n_ctx, n_seq)
    E = cfg["n_embd"]
    rng = np.random.Generator(np.random.PCG64(21))
    if depth:
        _seed_kv(rng, cfg, nl, (fast, plain), orc, n_seq, depth)
    expected_steps = 0
    # batches of 1..4 distinct sequences, at ragged positions; then a second round that reads what the first appended
    nxt = [depth] * n_seq
    for rnd in range(2):
        for T in (1, 2, 3, 4):
            seqs = [(rnd + i) % n_seq for i in range(T)]
            pos = [nxt[s] for s in seqs]
            for s in seqs:
                nxt[s] += 1
            x = rng.standard_normal((T, E)).astype(np.float32)
            got = fast.decode(x, pos, seq=seqs).view(np.float32).reshape(T, E)
            alt = plain.decode(x, pos, seq=seqs).view(np.float32).reshape(T, E)
            ref = orc.forward(x, pos, seq=seqs)
            expected_steps += 1
            assert fast.persistent_steps == expected_steps, "the persistent kernel did not take this batch"
            assert rel_l2(got, ref) <= 1e-3, (name, rnd, T)
            # the default session runs batches of three and more through the skinny MFMA GEMM (f16 activations)
            assert rel_l2(got, alt) <= (2e-4 if T < 3 else 3e-3), (name, rnd, T)
    assert plain.persistent_steps == 0
    # both paths appended the same keys and values (f16 of nearly equal f32 numbers)
    for il in range(nl):
        for s in range(n_seq):
            n_new = nxt[s] - depth
            k1, v1 = fast.kv_read(il, s, depth, n_new)
            k2, v2 = plain.kv_read(il, s, depth, n_new)
            ko = orc.k[il, s, :, depth:depth + n_new].transpose(1, 0, 2)
            f = lambda a: np.asarray(a).view(np.float16).astype(np.float32)
            assert rel_l2(f(k1), f(k2)) <= 3e-3 and rel_l2(f(v1), f(v2)) <= 3e-3
            assert rel_l2(f(k1), f(ko)) <= 2e-3
    fast.close()
    plain.close()
    st.close()


def test_persistent_kernel_is_skipped_when_a_sequence_repeats_or_batch_is_wide(tmp_path):
    """Two tokens of one sequence in a batch (causal within the batch) and batches over four tokens stay on the
    per-projection kernels; results still match the oracle."""
    m, cfg, nl, st, fast, plain, orc = _sessions(tmp_path, "tiny-qwen2", 64, 4)
    E = cfg["n_embd"]
    rng = np.random.Generator(np.random.PCG64(22))
    x = rng.standard_normal((2, E)).astype(np.float32)
    got = fast.decode(x, [0, 1], seq=[0, 0]).view(np.float32).reshape(2, E)
    assert fast.persistent_steps == 0
    assert rel_l2(got, orc.forward(x, [0, 1], seq=[0, 0])) <= 1e-3
    x = rng.standard_normal((5, E)).astype(np.float32)
    pos, seq = [2, 0, 0, 0, 3], [0, 1, 2, 3, 0]
    got = fast.decode(x, pos, seq=seq).view(np.float32).reshape(5, E)
    assert fast.persistent_steps == 0
    assert rel_l2(got, orc.forward(x, pos, seq=seq)) <= 1e-3
    x = rng.standard_normal((1, E)).astype(np.float32)
    got = fast.decode(x, [4], seq=[0]).view(np.float32)
    assert fast.persistent_steps == 1
    assert rel_l2(got, orc.forward(x, [4], seq=[0])) <= 1e-3
    fast.close()
    plain.close()
    st.close()


def test_persistent_decode_boundary_formats_and_queued_steps(tmp_path):
    """q8_0 in / q8_0 out through the persistent path is the bit-exact codec around the same f32 stage output, and
    steps queued back to back on the device stream (no host wait in between) keep the grid barrier's epoch in step."""
    import oracle
    m, cfg, nl, st, fast, plain, orc = _sessions(tmp_path, "tiny-qwen2", 128, 2)
    E = cfg["n_embd"]
    rng = np.random.Generator(np.random.PCG64(23))
    x = rng.standard_normal((2, E)).astype(np.float32)
    packed = oracle.quantize_q8_0(x.reshape(-1))
    out = fast.decode(packed, [0, 0], seq=[0, 1], in_fmt=m.Q8_0, out_fmt=m.Q8_0)
    f32 = plain.decode(packed, [0, 0], seq=[0, 1], in_fmt=m.Q8_0, out_fmt=m.F32).view(np.float32)
    x_eff = oracle.dequantize(oracle.Q8_0, packed, x.size).reshape(2, E)
    assert rel_l2(oracle.dequantize(oracle.Q8_0, out, f32.size), orc.forward(x_eff, [0, 0], seq=[0, 1])) <= 1.5e-2
    assert rel_l2(oracle.dequantize(oracle.Q8_0, out, f32.size), f32) <= 1.5e-2
    # 40 queued single-token steps feeding each output back in, against the same loop with a host wait per step
    dev = torch.device("cuda:0")
    h = rng.standard_normal((1, E)).astype(np.float32)
    a = torch.from_numpy(h.copy()).to(dev)
    b = torch.empty_like(a)
    torch.cuda.synchronize()
    ext = torch.cuda.ExternalStream(fast.stream)
    with torch.cuda.stream(ext):
        for i in range(40):
            fast.decode_dev(a.data_ptr(), [1 + i], b.data_ptr(), E * 4, seq=[0])
            a, b = b, a
    fast.synchronize()
    got = a.cpu().numpy()
    cur = h
    for i in range(40):
        cur = plain.decode(cur, [1 + i], seq=[0]).view(np.float32).reshape(1, E)
    assert fast.persistent_steps == 41
    assert np.isfinite(got).all()
    assert rel_l2(got, cur) <= 5e-3          # 40 chained steps: rounding differences of the two paths compound
    fast.close()
    plain.close()
    st.close()
