"""GPU parity of the single-launch one-token decode step (the layer graph sharded over the compute dies) through the C
ABI: against the CPU oracle (relative L2 <= 1e-3, the f32-activation bar of the stage tests), against the
launch-per-projection path (<= 1e-3: the same arithmetic in another summation order, so the 16-bit activation roundings of
the two fall differently; measured 1e-4..4e-4, what each is away from the oracle), run-to-run bit equality, and the KV
rows it appends."""
import os

import numpy as np
import pytest

import models
from oracle.stage import StageOracle
from util import mesh

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def rel_l2(a, b):
    a = np.asarray(a, np.float64).reshape(-1)
    b = np.asarray(b, np.float64).reshape(-1)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def _open(tmp_path, layers, n_ctx, n_seq):
    m = mesh()
    cfg = models.CONFIGS["llama3-8b"]
    path = os.path.join(str(tmp_path), "llama3-8b.gguf")
    tensors = models.write_model(path, cfg, layers, seed=5)
    st = m.Stage(path, layers[0], layers[-1] + 1, n_ctx=n_ctx, n_seq_max=n_seq, n_batch_max=8)
    os.unlink(path)
    return m, cfg, tensors, st


def _fill(ses_list, orc, layers, n_seq, n_past, rng):
    for il in layers:
        for s in range(n_seq):
            k = (rng.standard_normal((n_past, 8, 128)) * 0.5).astype(np.float16).view(np.uint16)
            v = (rng.standard_normal((n_past, 8, 128)) * 0.5).astype(np.float16).view(np.uint16)
            for ses in ses_list:
                ses.kv_write(il, s, 0, k, v)
            if orc is not None:
                orc.k[il - layers[0], s, :, :n_past] = k.transpose(1, 0, 2)
                orc.v[il - layers[0], s, :, :n_past] = v.transpose(1, 0, 2)


def test_single_launch_steps_match_oracle_and_projection_path(tmp_path, monkeypatch):
    """Three real-shape layers (Q6_K attn_v / ffn_down on the first, all Q4_K after), KV depth 300 in two sequences,
    then: steps at depth 300.. in one sequence, a step into an empty sequence (one key), steps at depths 1..4 (fewer
    keys than key ranges)."""
    layers = [3, 4, 5]
    m, cfg, tensors, st = _open(tmp_path, layers, 512, 4)
    assert tensors["blk.3.ffn_down.weight"][0] == models.Q6_K and tensors["blk.4.ffn_down.weight"][0] == models.Q4_K
    monkeypatch.setenv("MESH_DECODE_DIE", "1")
    ses = st.session()
    monkeypatch.setenv("MESH_DECODE_DIE", "0")
    ses_ref = st.session()
    orc = StageOracle(cfg, tensors, 3, 6, 512, n_seq_max=4)
    rng = np.random.Generator(np.random.PCG64(21))
    n_past = 300
    _fill([ses, ses_ref], orc, layers, 2, n_past, rng)
    steps = [(n_past, 1), (n_past + 1, 1), (n_past, 0), (0, 2), (1, 2), (2, 2), (3, 2), (4, 2), (n_past + 2, 1), (0, 3)]
    worst_o = worst_p = 0.0
    for pos, seq in steps:
        x = rng.standard_normal((1, 4096)).astype(np.float32)
        got = ses.decode(x, [pos], seq=[seq]).view(np.float32)
        alt = ses_ref.decode(x, [pos], seq=[seq]).view(np.float32)
        ref = orc.forward(x, [pos], seq=[seq])
        assert np.isfinite(got).all()
        worst_o = max(worst_o, rel_l2(got, ref))
        worst_p = max(worst_p, rel_l2(got, alt))
    print("single-launch step: worst rel-L2 vs oracle %.3g, vs launch-per-projection path %.3g" % (worst_o, worst_p))
    assert ses.single_launch_steps == len(steps) and ses_ref.single_launch_steps == 0
    assert worst_o <= 1e-3
    assert worst_p <= 1e-3
    # the rows both paths appended to the cache: f16 of values that differ in the last bits at most
    for il in layers:
        for seq, p0, n in ((1, n_past, 3), (2, 0, 5), (3, 0, 1), (0, n_past, 1)):
            ka, va = ses.kv_read(il, seq, p0, n)
            kb, vb = ses_ref.kv_read(il, seq, p0, n)
            for a, b in ((ka, kb), (va, vb)):
                fa, fb = a.view(np.float16).astype(np.float32), b.view(np.float16).astype(np.float32)
                assert a.any() and np.abs(fa - fb).max() <= 2e-3 * max(np.abs(fb).max(), 1e-6)
                if il == layers[0]:      # same inputs: only the summation order differs
                    assert (a != b).mean() <= 0.02
    ses.close(); ses_ref.close(); st.close()


def test_single_launch_steps_are_reproducible_and_mix_with_batches(tmp_path, monkeypatch):
    """The same steps in two fresh sessions give the same bits (every reduction has a fixed order); one-token steps
    interleave with multi-token calls of the launch-per-projection path on the same cache."""
    layers = [3, 4]
    monkeypatch.setenv("MESH_DECODE_DIE", "1")
    m, cfg, tensors, st = _open(tmp_path, layers, 256, 3)
    orc = StageOracle(cfg, tensors, 3, 5, 256, n_seq_max=3)
    rng = np.random.Generator(np.random.PCG64(22))
    xs = [rng.standard_normal((T, 4096)).astype(np.float32) for T in (5, 1, 1, 3, 1, 1)]
    runs = []
    for _ in range(2):
        ses = st.session()
        outs, nxt = [], 0
        for x in xs:
            T = x.shape[0]
            outs.append(ses.decode(x, list(range(nxt, nxt + T)), seq=[1] * T).view(np.float32).copy())
            nxt += T
        assert ses.single_launch_steps == 4
        runs.append(outs)
        ses.close()
    for a, b in zip(*runs):
        assert np.array_equal(a, b)
    nxt = 0
    for x, got in zip(xs, runs[0]):
        T = x.shape[0]
        ref = orc.forward(x, list(range(nxt, nxt + T)), seq=[1] * T)
        nxt += T
        assert rel_l2(got, ref) <= 3e-3
    st.close()
