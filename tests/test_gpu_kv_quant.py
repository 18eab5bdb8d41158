"""Quantised KV cache tiers (K q8_0 / V q4_0 and q4_0 / q4_0: KvCacheQuant::for_model_size,
mesh-llm/src/inference/launch.rs:568-591) against the CPU oracle: the cache rows bit-exactly, the stage output within
the stage tolerance (1e-2 rel-L2; the quantisation itself is part of both sides)."""
import os
import sys

import numpy as np
import pytest

torch = pytest.importorskip("torch")

import models
import oracle
from oracle.stage import StageOracle
from util import mesh

pytestmark = pytest.mark.gpu


def rel_l2(a, b):
    a = np.asarray(a, np.float64).reshape(-1)
    b = np.asarray(b, np.float64).reshape(-1)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))

PAIRS = [(oracle.Q8_0, oracle.Q4_0), (oracle.Q4_0, oracle.Q4_0)]
# A prefill chunk that starts an EMPTY sequence over a quantised cache, whole chunk and worst token.  The f16-activation
# GEMMs move the K / V rows entering the cache by ~1e-3 relative, which lands a fraction of a percent of the 4-bit codes
# on the neighbouring step (an eighth of the block maximum); the first tokens of a sequence attend to a handful of rows,
# so nothing averages that out: measured 1.3e-2 (q8_0 / q4_0) and 2.1e-2 (q4_0 / q4_0) for the chunk, 3.9e-2 for its worst token.  This bound is
# therefore about the quantiser's discontinuity, not the kernels: those are held to 2e-3 by the same test with the
# device's own cache rows handed to the oracle (measured 8e-4, worst token 9e-4), and the codes that moved are counted.
CHUNK_TOL, CHUNK_TOL_TOKEN = 3e-2, 6e-2


def _open(tmp_path, name, layers, lb, le, kv_types, n_ctx=64, n_seq=2, n_batch=16, seed=5):
    m = mesh()
    cfg = models.CONFIGS[name]
    path = os.path.join(str(tmp_path), name + ".gguf")
    tensors = models.write_model(path, cfg, layers, seed=seed)
    st = m.Stage(path, lb, le, n_ctx=n_ctx, n_seq_max=n_seq, n_batch_max=n_batch, kv_types=kv_types)
    os.unlink(path)
    return m, cfg, tensors, st


def _f16(x):
    return x.view(np.float16).astype(np.float32)


@pytest.mark.parametrize("kv_types", PAIRS)
@pytest.mark.parametrize("name", ["tiny-llama", "tiny-qwen2"])      # head_dim 64 and 128
def test_cache_rows_quantise_bit_exactly(tmp_path, name, kv_types):
    """kv_write quantises f16 rows into the cache type, kv_read returns the dequantised values rounded to f16: both
    must equal the oracle's quantise -> dequantise of the same rows, bit for bit (ties in magnitude, zero rows and tiny
    values included)."""
    m, cfg, tensors, st = _open(tmp_path, name, [0], 0, 1, kv_types, n_ctx=64)
    ses = st.session()
    hk, hd = cfg["n_head_kv"], cfg["head_dim"]
    rng = np.random.Generator(np.random.PCG64(21))
    n = 40
    k = rng.standard_normal((n, hk, hd)).astype(np.float32)
    v = (rng.standard_normal((n, hk, hd)) * 3).astype(np.float32)
    k[0] = 0.0
    v[1] = 0.0
    k[2, :, 5], k[2, :, 9] = 4.0, -4.0          # equal magnitudes: the first one decides q4_0's sign
    v[2, :, 9], v[2, :, 5] = 4.5, -4.5
    k[3] *= 1e-5                                # scale is an fp16 subnormal
    v[3] *= 1e-5
    kh, vh = k.astype(np.float16).view(np.uint16), v.astype(np.float16).view(np.uint16)
    ses.kv_write(0, 1, 3, kh, vh)
    gk, gv = ses.kv_read(0, 1, 3, n)
    wk = oracle.kv_round(kv_types[0], _f16(kh)).astype(np.float16).view(np.uint16)
    wv = oracle.kv_round(kv_types[1], _f16(vh)).astype(np.float16).view(np.uint16)
    assert np.array_equal(gk, wk)
    assert np.array_equal(gv, wv)
    # other positions of the sequence and the other sequence stay zero
    zk, zv = ses.kv_read(0, 0, 0, 64)
    assert not _f16(zk).any() and not _f16(zv).any()
    zk, _ = ses.kv_read(0, 1, 0, 3)
    assert not _f16(zk).any()
    ses.close()
    st.close()


@pytest.mark.parametrize("kv_types", PAIRS)
@pytest.mark.parametrize("name", ["tiny-llama", "tiny-qwen2", "tiny-odd"])
def test_stage_with_quantised_kv_matches_oracle(tmp_path, name, kv_types):
    cfg = models.CONFIGS[name]
    nl = cfg["n_layer"]
    m, cfg, tensors, st = _open(tmp_path, name, range(nl), 0, nl, kv_types)
    ses = st.session()
    orc = StageOracle(cfg, tensors, 0, nl, 64, n_seq_max=2, kv_types=kv_types)
    rng = np.random.Generator(np.random.PCG64(7))
    E = cfg["n_embd"]
    x = rng.standard_normal((7, E)).astype(np.float32)
    got = ses.decode(x, np.arange(7), seq=np.ones(7, np.int32)).view(np.float32).reshape(7, E)
    ref = orc.forward(x, np.arange(7), seq=np.ones(7, np.int32))
    assert rel_l2(got, ref) <= 1e-2
    for step in range(3):
        x1 = rng.standard_normal((1, E)).astype(np.float32)
        got = ses.decode(x1, [7 + step], seq=[1]).view(np.float32)
        ref = orc.forward(x1, [7 + step], seq=[1])
        assert rel_l2(got, ref) <= 1e-2
    xm = rng.standard_normal((5, E)).astype(np.float32)
    pos, seq = [0, 10, 1, 11, 2], [0, 1, 0, 1, 0]
    got = ses.decode(xm, pos, seq=seq).view(np.float32).reshape(5, E)
    ref = orc.forward(xm, pos, seq=seq)
    assert rel_l2(got, ref) <= 1e-2
    # first layer's cache: its inputs agree on both sides up to GEMV rounding, so the rows agree up to a quant step in
    # a few elements and the low bits of the block scales
    k, v = ses.kv_read(0, 1, 0, 12)
    ko = orc.k[0, 1, :, :12].transpose(1, 0, 2)
    vo = orc.v[0, 1, :, :12].transpose(1, 0, 2)
    assert rel_l2(_f16(k), ko) <= 2e-2 and rel_l2(_f16(v), vo) <= 2e-2
    ses.close()
    st.close()


@pytest.mark.parametrize("kv_types", PAIRS)
def test_llama3_8b_shaped_layers_quantised_kv_all_paths(tmp_path, kv_types):
    """Two real-shape layers over a 300-deep quantised cache: split-KV decode at batch 1 and 4, the batched (skinny
    GEMM) path at batch 9, and a 200-token prefill chunk through the matrix-core attention kernel."""
    name = "llama3-8b"
    m, cfg, tensors, st = _open(tmp_path, name, [3, 4], 3, 5, kv_types, n_ctx=512, n_seq=10, n_batch=208)
    ses = st.session()
    orc = StageOracle(cfg, tensors, 3, 5, 512, n_seq_max=10, kv_types=kv_types)
    rng = np.random.Generator(np.random.PCG64(11))
    n_past = 300
    for il in (3, 4):
        for s in range(9):
            k = (rng.standard_normal((n_past, 8, 128)) * 0.5).astype(np.float16)
            v = (rng.standard_normal((n_past, 8, 128)) * 0.5).astype(np.float16)
            ses.kv_write(il, s, 0, k.view(np.uint16), v.view(np.uint16))
            orc.k[il - 3, s, :, :n_past] = oracle.kv_round(kv_types[0], k.astype(np.float32)).transpose(1, 0, 2)
            orc.v[il - 3, s, :, :n_past] = oracle.kv_round(kv_types[1], v.astype(np.float32)).transpose(1, 0, 2)
    x = rng.standard_normal((1, 4096)).astype(np.float32)
    got = ses.decode(x, [n_past], seq=[2]).view(np.float32)
    ref = orc.forward(x, [n_past], seq=[2])
    assert rel_l2(got, ref) <= 1e-2
    x4 = rng.standard_normal((4, 4096)).astype(np.float32)
    pos, seq = [n_past, n_past, n_past + 1, n_past], [0, 1, 2, 3]
    got = ses.decode(x4, pos, seq=seq).view(np.float32).reshape(4, 4096)
    ref = orc.forward(x4, pos, seq=seq)
    assert rel_l2(got, ref) <= 1e-2
    x9 = rng.standard_normal((9, 4096)).astype(np.float32)
    pos, seq = [n_past + 1, n_past + 1, n_past + 2, n_past + 1, n_past, n_past, n_past, n_past, n_past], list(range(9))
    got = ses.decode(x9, pos, seq=seq).view(np.float32).reshape(9, 4096)
    ref = orc.forward(x9, pos, seq=seq)
    assert rel_l2(got, ref) <= 1e-2
    # prefill chunk of 200 tokens into the empty sequence 9.  The prefill GEMMs run on f16 activations, so the K / V
    # rows entering the cache differ from the oracle's by ~1e-3 relative; that moves a fraction of a percent of the
    # 4-bit quants by one step (an eighth of the block maximum), which is the error floor seen here: the bound is the
    # stage tolerance times 3, with the f16-cache prefill test holding the kernels themselves to 3e-3.
    T = 200
    xp = rng.standard_normal((T, 4096)).astype(np.float32)
    got = ses.decode(xp, np.arange(T), seq=np.full(T, 9, np.int32)).view(np.float32).reshape(T, 4096)
    ref = orc.forward(xp, np.arange(T), seq=np.full(T, 9, np.int32))
    r, r_tok = rel_l2(got, ref), max(rel_l2(got[i], ref[i]) for i in range(T))
    # (a) the rows the chunk left in the cache against the oracle's: the same blocks up to a few codes that sat near a
    # decision threshold; (b) the oracle run again with the device's rows in its cache: what is left is the arithmetic
    dev_rows = {}
    for il in (3, 4):
        kd, vd = ses.kv_read(il, 9, 0, T)
        dev_rows[il - 3] = (_f16(kd), _f16(vd))
        ko, vo = orc.k[il - 3, 9, :, :T].transpose(1, 0, 2), orc.v[il - 3, 9, :, :T].transpose(1, 0, 2)
        for name, d_, o_, typ in (("K", dev_rows[il - 3][0], ko, kv_types[0]), ("V", dev_rows[il - 3][1], vo, kv_types[1])):
            blk_max = np.abs(o_).reshape(-1, 32).max(axis=1, keepdims=True) + 1e-30
            step = blk_max / (7.0 if typ == oracle.Q4_0 else 127.0)
            off = np.abs(d_.reshape(-1, 32) - o_.reshape(-1, 32)) / step
            moved = float((off > 0.5).mean())
            print("[kv-quant] layer %d %s rows: %.3f%% of the codes differ from the oracle's, largest distance %.2f steps" % (il, name, 100 * moved, off.max()),
                  file=sys.stderr, flush=True)
            # the first layer's rows come from identical inputs: a code and, rarely, a block scale's rounding on top.  (The
            # next layer's input already carries the first layer's moved codes, so its rows are only reported.)
            if il == 3:
                assert moved <= 0.03 and off.max() <= 2.6
    ref_same = orc.forward(xp, np.arange(T), seq=np.full(T, 9, np.int32), kv_rows=dev_rows)
    r_same, r_same_tok = rel_l2(got, ref_same), max(rel_l2(got[i], ref_same[i]) for i in range(T))
    print("[kv-quant] %s prefill chunk of 200: rel-L2 %.3e, worst token %.3e; with the device's cache rows in the oracle %.3e, %.3e"
          % (kv_types, r, r_tok, r_same, r_same_tok), file=sys.stderr, flush=True)
    assert r_same <= 2e-3 and r_same_tok <= 3e-3
    assert r <= CHUNK_TOL
    assert r_tok <= CHUNK_TOL_TOKEN
    # a second chunk on top of the first (136 tokens at positions 200 .. 335): chunks this long decode the cache rows
    # they attend to once, into an f16 scratch, before the walk; that has to cover the first chunk's rows too
    T2 = 136
    xp2 = rng.standard_normal((T2, 4096)).astype(np.float32)
    got2 = ses.decode(xp2, np.arange(T, T + T2), seq=np.full(T2, 9, np.int32)).view(np.float32).reshape(T2, 4096)
    ref2 = orc.forward(xp2, np.arange(T, T + T2), seq=np.full(T2, 9, np.int32))
    r2 = rel_l2(got2, ref2)
    print("[kv-quant] %s second chunk of 136: rel-L2 %.3e" % (kv_types, r2), file=sys.stderr, flush=True)
    assert r2 <= CHUNK_TOL
    ses.close()
    # the same two chunks with the scratch switched off (every query tile decodes the rows itself): the same values
    # reach the matrix cores in the same order, so the hidden states are bit-identical
    ses = st.session(chunk_kv16=0)
    got_b = ses.decode(xp, np.arange(T), seq=np.full(T, 9, np.int32)).view(np.float32).reshape(T, 4096)
    got2_b = ses.decode(xp2, np.arange(T, T + T2), seq=np.full(T2, 9, np.int32)).view(np.float32).reshape(T2, 4096)
    assert np.array_equal(got_b.view(np.uint32), got.view(np.uint32))
    assert np.array_equal(got2_b.view(np.uint32), got2.view(np.uint32))
    ses.close()
    st.close()


def test_unsupported_kv_pairs_are_refused(tmp_path):
    m = mesh()
    cfg = models.CONFIGS["tiny-llama"]
    path = os.path.join(str(tmp_path), "t.gguf")
    models.write_model(path, cfg, [0], seed=5)
    for pair in [(oracle.F16, oracle.Q4_0), (oracle.Q8_0, oracle.Q8_0), (oracle.Q4_K, oracle.Q4_0), (oracle.Q4_0, oracle.Q8_0)]:
        with pytest.raises(m.MeshError):
            m.Stage(path, 0, 1, kv_types=pair)
    # K type alone picks the tier's V type
    st = m.Stage(path, 0, 1, n_ctx=32, kv_types=(oracle.Q8_0, 0))
    st.close()
