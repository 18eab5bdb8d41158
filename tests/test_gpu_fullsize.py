"""Parity of the stage executor ON THE CONFIGURATIONS THE TOLERANCE IS STATED ON: relative L2 <= 1e-2 between the
GPU stage's output hidden state and the CPU oracle's on identical seeded weights and inputs.

  C3  Llama-3-8B-shaped stage, ALL 16 layers (0-15 of 32), 4096-token KV context filled to depth 4095: decode at batch
      1, 4 and 16 (mat-vec kernels, skinny MFMA GEMM, matrix-core decode attention); a 2048-token prefill through two
      real-shape layers and a 256-token prefill through all 16 (large-tile MFMA GEMM, chunk attention).
  C4  Qwen2.5-32B-shaped layers (hidden 5120, 40 / 8 heads, FFN 27648, q/k/v bias): decode batch 24 and 32 (f16 skinny
      GEMM with two blocks of 16 activation columns per pass), a 320-token prefill (large-tile GEMM, chunk attention with
      5 query heads per KV head), over f16 and over q8_0 / q4_0 caches; decode at KV depth 8191 of 8192 on all cache tiers.
  C5  Qwen3-30B-A3B-shaped 64-expert shard layer, router logits ~ N(0,1) + Zipf(1.1) expert bias, batch 16 on top of a
      filled KV cache.
Every test prints the figure it measured.  The oracle's projections of prefill-sized calls go through numpy's float64
matmul over the dequantised weights (StageOracle(blas=True)), the definition its C loop is pinned to.
"""
import os
import sys

import numpy as np
import pytest

import models
import oracle
from oracle.stage import StageOracle
from util import mesh

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

NORTH_STAR = 1e-2


def rel_l2(a, b):
    a = np.asarray(a, np.float64).reshape(-1)
    b = np.asarray(b, np.float64).reshape(-1)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def report(what, value):
    print("[fullsize] %s: rel-L2 %.3e" % (what, value), file=sys.stderr, flush=True)


def random_kv(rng, n_pos, n_kv=8, hd=128, scale=0.5):
    return (rng.standard_normal((n_pos, n_kv, hd)) * scale).astype(np.float16).view(np.uint16)


@pytest.fixture(scope="module")
def c3_model(tmp_path_factory):
    """The 16-layer stage file of the benchmark (same generator, same seed)."""
    cfg = models.CONFIGS["llama3-8b"]
    path = os.path.join(models.tmp_dir(), "mesh_test_c3_%d.gguf" % os.getpid())
    tensors = models.write_model(path, cfg, range(16), seed=42, fast=True)
    yield cfg, tensors, path
    if os.path.exists(path):
        os.unlink(path)


def test_c3_sixteen_layer_stage_decode_at_kv_depth_4095(c3_model):
    m = mesh()
    cfg, tensors, path = c3_model
    n_ctx, n_seq, depth = 4096, 16, 4095
    st = m.Stage(path, 0, 16, n_ctx=n_ctx, n_seq_max=n_seq, n_batch_max=16)
    assert st.weight_bytes == 2093219840          # the stage the roofline is quoted on
    ses = st.session()
    orc = StageOracle(cfg, tensors, 0, 16, n_ctx, n_seq_max=n_seq)
    rng = np.random.Generator(np.random.PCG64(4095))
    for il in range(16):
        # every sequence holds its own context (a sequence-index mix-up in a batched kernel must show): sequence s is the
        # layer's random rows rotated by 251 s positions, K and V in opposite directions
        k, v = random_kv(rng, depth), random_kv(rng, depth)
        for s in range(n_seq):
            ks, vs = np.roll(k, 251 * s, axis=0), np.roll(v, -251 * s, axis=0)
            ses.kv_write(il, s, 0, ks, vs)
            orc.k[il, s, :, :depth] = ks.transpose(1, 0, 2)
            orc.v[il, s, :, :depth] = vs.transpose(1, 0, 2)
    for seqs in ([0], [1, 2, 3, 4], list(range(16))):
        T = len(seqs)
        x = rng.standard_normal((T, 4096)).astype(np.float32)
        pos = [depth] * T
        got = ses.decode(x, pos, seq=seqs).view(np.float32).reshape(T, 4096)
        ref = orc.forward(x, pos, seq=seqs)
        r = rel_l2(got, ref)
        report("C3 16 layers, KV depth 4095, decode batch %d" % T, r)
        assert r <= NORTH_STAR, T
        assert max(rel_l2(got[i], ref[i]) for i in range(T)) <= NORTH_STAR
        # the q8_0 boundary activation of the same step is the codec applied to that output
        packed = ses.decode(x, pos, seq=seqs, out_fmt=m.Q8_0)
        assert np.array_equal(packed, oracle.quantize_q8_0(got.reshape(-1)))
    ses.close(); st.close()


def test_c3_prefill_2048_tokens_two_layers(c3_model):
    m = mesh()
    cfg, tensors, path = c3_model
    T = 2048
    st = m.Stage(path, 3, 5, n_ctx=T + 8, n_seq_max=1, n_batch_max=T)
    ses = st.session()
    orc = StageOracle(cfg, tensors, 3, 5, T + 8, blas=True)
    rng = np.random.Generator(np.random.PCG64(2048))
    x = rng.standard_normal((T, 4096)).astype(np.float32)
    got = ses.decode(x, np.arange(T)).view(np.float32).reshape(T, 4096)
    ref = orc.forward(x, np.arange(T))
    r = rel_l2(got, ref)
    report("C3 layers 3-4, prefill 2048 tokens", r)
    assert r <= NORTH_STAR
    assert max(rel_l2(got[i], ref[i]) for i in range(T)) <= NORTH_STAR
    # launches that fill the chip with 256 x 128 tiles take the big-tile kernel; with gemm_big=0 all keep the
    # 128 x 128 one.  Same fragments, same order along K: the same bits.
    ses.set_option("gemm_big", 0)
    small = ses.decode(x, np.arange(T)).view(np.float32).reshape(T, 4096)
    ses.set_option("gemm_big", 1)
    assert np.array_equal(got, small)
    # one decode token on top of the 2048 cached positions
    x1 = rng.standard_normal((1, 4096)).astype(np.float32)
    r1 = rel_l2(ses.decode(x1, [T]).view(np.float32), orc.forward(x1, [T]))
    report("C3 layers 3-4, decode on the prefilled cache", r1)
    assert r1 <= NORTH_STAR
    ses.close(); st.close()


def test_c3_prefill_256_tokens_sixteen_layers(c3_model):
    m = mesh()
    cfg, tensors, path = c3_model
    T = 256
    st = m.Stage(path, 0, 16, n_ctx=T + 8, n_seq_max=1, n_batch_max=T)
    ses = st.session()
    orc = StageOracle(cfg, tensors, 0, 16, T + 8, blas=True)
    rng = np.random.Generator(np.random.PCG64(256))
    x = rng.standard_normal((T, 4096)).astype(np.float32)
    got = ses.decode(x, np.arange(T)).view(np.float32).reshape(T, 4096)
    ref = orc.forward(x, np.arange(T))
    r = rel_l2(got, ref)
    report("C3 16 layers, prefill 256 tokens", r)
    assert r <= NORTH_STAR
    assert max(rel_l2(got[i], ref[i]) for i in range(T)) <= NORTH_STAR
    x1 = rng.standard_normal((1, 4096)).astype(np.float32)
    r1 = rel_l2(ses.decode(x1, [T]).view(np.float32), orc.forward(x1, [T]))
    report("C3 16 layers, decode on the prefilled cache", r1)
    assert r1 <= NORTH_STAR
    ses.close(); st.close()


def test_c4_long_prefill_takes_the_big_tile_with_biases(tmp_path):
    """1664 tokens through one Qwen2.5-32B-shaped layer: every projection launch has enough 256-row tiles to fill the chip,
    so the fused q / k / v launch (three matrices, biases, 40 + 8 + 8 row blocks) and the q6_K down projection run on the
    256 x 128 tile; against the oracle, and bit for bit against the 128 x 128 kernel."""
    m = mesh()
    cfg = models.CONFIGS["qwen2.5-32b"]
    path = os.path.join(str(tmp_path), "c4l.gguf")
    tensors = models.write_model(path, cfg, [7], seed=42, fast=True)
    T, E = 1664, 5120
    st = m.Stage(path, 7, 8, n_ctx=T, n_seq_max=1, n_batch_max=T)
    os.unlink(path)
    ses = st.session()
    orc = StageOracle(cfg, tensors, 7, 8, T, blas=True)
    rng = np.random.Generator(np.random.PCG64(1664))
    x = rng.standard_normal((T, E)).astype(np.float32)
    got = ses.decode(x, np.arange(T)).view(np.float32).reshape(T, E)
    ref = orc.forward(x, np.arange(T))
    r = rel_l2(got, ref)
    report("C4 layer 7, prefill 1664 tokens (big tile)", r)
    assert r <= NORTH_STAR
    ses.set_option("gemm_big", 0)
    small = ses.decode(x, np.arange(T)).view(np.float32).reshape(T, E)
    assert np.array_equal(got, small)
    ses.close(); st.close()


@pytest.mark.parametrize("kv", ["f16", "q8_0/q4_0"])
def test_c4_qwen25_32b_layers_wide_batches_and_prefill(tmp_path, kv):
    """Layers 7 (q6_K attn_v / ffn_down) and 8 (all q4_K) of the 64-layer model."""
    m = mesh()
    cfg = models.CONFIGS["qwen2.5-32b"]
    path = os.path.join(str(tmp_path), "c4.gguf")
    tensors = models.write_model(path, cfg, [7, 8], seed=42, fast=True)
    assert tensors["blk.7.ffn_down.weight"][0] == models.Q6_K and tensors["blk.8.ffn_down.weight"][0] == models.Q4_K
    n_ctx, n_seq, depth, E = 512, 32, 100, 5120
    kv_m = {"f16": (m.F16, m.F16), "q8_0/q4_0": (m.Q8_0, m.Q4_0)}[kv]
    kv_o = {"f16": None, "q8_0/q4_0": (oracle.Q8_0, oracle.Q4_0)}[kv]
    st = m.Stage(path, 7, 9, n_ctx=n_ctx, n_seq_max=n_seq, n_batch_max=320, kv_types=kv_m)
    os.unlink(path)
    ses = st.session()
    orc = StageOracle(cfg, tensors, 7, 9, n_ctx, n_seq_max=n_seq, kv_types=kv_o, blas=True)
    rng = np.random.Generator(np.random.PCG64(32))
    for il in (7, 8):
        for s in range(1, n_seq):
            k, v = random_kv(rng, depth), random_kv(rng, depth)
            ses.kv_write(il, s, 0, k, v)
            kf, vf = k.view(np.float16).astype(np.float32), v.view(np.float16).astype(np.float32)
            if kv_o:
                orc.k[il - 7, s, :, :depth] = oracle.kv_round(kv_o[0], kf).transpose(1, 0, 2)
                orc.v[il - 7, s, :, :depth] = oracle.kv_round(kv_o[1], vf).transpose(1, 0, 2)
            else:
                orc.k[il - 7, s, :, :depth] = k.transpose(1, 0, 2)
                orc.v[il - 7, s, :, :depth] = v.transpose(1, 0, 2)
    # 320-token prefill chunk of sequence 0 (5 query heads per KV head in the chunk attention kernel), then a second chunk
    for pos0, T in ((0, 320), (320, 100)):
        x = rng.standard_normal((T, E)).astype(np.float32)
        pos = np.arange(pos0, pos0 + T)
        got = ses.decode(x, pos).view(np.float32).reshape(T, E)
        ref = orc.forward(x, pos)
        r = rel_l2(got, ref)
        report("C4 layers 7-8, %s KV, prefill chunk of %d tokens at %d" % (kv, T, pos0), r)
        assert r <= NORTH_STAR
    # decode batches of 24 and 32 single-token sequences at KV depth 100 / 101: large-tile GEMM, K split over workgroups
    nxt = [420] + [depth] * (n_seq - 1)
    for seqs in (list(range(1, 25)), list(range(32))):
        T = len(seqs)
        pos = [nxt[q] for q in seqs]
        for q in seqs:
            nxt[q] += 1
        x = rng.standard_normal((T, E)).astype(np.float32)
        got = ses.decode(x, pos, seq=seqs).view(np.float32).reshape(T, E)
        ref = orc.forward(x, pos, seq=seqs)
        r = rel_l2(got, ref)
        report("C4 layers 7-8, %s KV, decode batch %d" % (kv, T), r)
        assert r <= NORTH_STAR, T
    ses.close(); st.close()


@pytest.mark.parametrize("kv", ["f16", "q8_0/q4_0", "q4_0/q4_0"])
def test_c4_decode_at_kv_depth_8191(tmp_path, kv):
    """The context the Qwen2.5-32B-shaped configuration is stated on: layers 7 (q6_K attn_v / ffn_down) and 8 at KV depth
    8191 of an 8192-token context, decode batch 1, 8 and 32, every sequence with its own cache rows, over an f16 cache and
    over the two quantised tiers the reference's launcher picks by model size (mesh-llm/src/inference/launch.rs:568-591:
    K q8_0 / V q4_0, and q4_0 / q4_0).  5 query heads per KV head, 32 key splits at batch 1."""
    m = mesh()
    cfg = models.CONFIGS["qwen2.5-32b"]
    path = os.path.join(str(tmp_path), "c4d.gguf")
    tensors = models.write_model(path, cfg, [7, 8], seed=42, fast=True)
    n_ctx, n_seq, depth, E = 8192, 32, 8191, 5120
    kv_m = {"f16": (m.F16, m.F16), "q8_0/q4_0": (m.Q8_0, m.Q4_0), "q4_0/q4_0": (m.Q4_0, m.Q4_0)}[kv]
    kv_o = {"f16": None, "q8_0/q4_0": (oracle.Q8_0, oracle.Q4_0), "q4_0/q4_0": (oracle.Q4_0, oracle.Q4_0)}[kv]
    st = m.Stage(path, 7, 9, n_ctx=n_ctx, n_seq_max=n_seq, n_batch_max=32, kv_types=kv_m)
    os.unlink(path)
    ses = st.session()
    orc = StageOracle(cfg, tensors, 7, 9, n_ctx, n_seq_max=n_seq, kv_types=kv_o)
    rng = np.random.Generator(np.random.PCG64(8191))
    for il in (7, 8):
        k, v = random_kv(rng, depth), random_kv(rng, depth)
        if kv_o:
            kq = oracle.kv_round(kv_o[0], k.view(np.float16).astype(np.float32))
            vq = oracle.kv_round(kv_o[1], v.view(np.float16).astype(np.float32))
        for s in range(n_seq):
            ks, vs = np.roll(k, 509 * s, axis=0), np.roll(v, -509 * s, axis=0)
            ses.kv_write(il, s, 0, ks, vs)
            if kv_o:        # (a row's quantisation depends on that row alone, so rounding commutes with the rotation)
                orc.k[il - 7, s, :, :depth] = np.roll(kq, 509 * s, axis=0).transpose(1, 0, 2)
                orc.v[il - 7, s, :, :depth] = np.roll(vq, -509 * s, axis=0).transpose(1, 0, 2)
            else:
                orc.k[il - 7, s, :, :depth] = ks.transpose(1, 0, 2)
                orc.v[il - 7, s, :, :depth] = vs.transpose(1, 0, 2)
    for seqs in ([5], list(range(8, 16)), list(range(32))):
        T = len(seqs)
        x = rng.standard_normal((T, E)).astype(np.float32)
        pos = [depth] * T
        got = ses.decode(x, pos, seq=seqs).view(np.float32).reshape(T, E)
        ref = orc.forward(x, pos, seq=seqs)
        r = rel_l2(got, ref)
        report("C4 layers 7-8, %s KV, depth 8191, decode batch %d" % (kv, T), r)
        assert r <= NORTH_STAR, T
        assert max(rel_l2(got[i], ref[i]) for i in range(T)) <= NORTH_STAR, T
    ses.close(); st.close()


def test_c5_expert_shard_layer_zipf_router_on_filled_cache(tmp_path):
    """A 64-expert shard layer of the 128-expert model, router logits ~ N(0,1) + Zipf(1.1) expert bias (models.py),
    decode batch 16 at KV depth 200 and one more step on top."""
    m = mesh()
    cfg = dict(models.CONFIGS["qwen3-30b-a3b"])
    path = os.path.join(str(tmp_path), "shard.gguf")
    tensors = models.write_model(path, cfg, [5, 6], seed=9, n_expert_local=64, fast=True, router="zipf")
    n_ctx, depth, E = 256, 200, 2048
    st = m.Stage(path, 5, 7, n_ctx=n_ctx, n_seq_max=16, n_batch_max=16)
    os.unlink(path)
    ses = st.session()
    orc = StageOracle(cfg, tensors, 5, 7, n_ctx, n_seq_max=16)
    rng = np.random.Generator(np.random.PCG64(55))
    for il in (5, 6):
        for s in range(16):
            k, v = random_kv(rng, depth, n_kv=4), random_kv(rng, depth, n_kv=4)
            ses.kv_write(il, s, 0, k, v)
            orc.k[il - 5, s, :, :depth] = k.transpose(1, 0, 2)
            orc.v[il - 5, s, :, :depth] = v.transpose(1, 0, 2)
    distinct = []
    for step in range(2):
        x = models.zipf_hidden_state(rng, 16, E)
        pos, seq = np.full(16, depth + step, np.int32), np.arange(16, dtype=np.int32)
        got = ses.decode(x, pos, seq=seq).view(np.float32).reshape(16, E)
        ref = orc.forward(x, pos, seq=seq)
        r = rel_l2(got - x, ref - x)              # what the layers add (the carrier channel would dominate the norm)
        report("C5 shard layers 5-6, Zipf router, batch 16 at KV depth %d (of the layers' contribution)" % (depth + step), r)
        assert r <= NORTH_STAR
        ids = ses.moe_last_ids(16)
        assert np.array_equal(np.sort(ids, axis=1), np.sort(np.stack(orc.last_expert_ids), axis=1))
        distinct.append(len(set(ids.reshape(-1))))
    # the bias concentrates the batch on the popular experts: far fewer than the ~56 of 64 a uniform router touches
    print("[fullsize] C5 distinct experts touched by 16 tokens x top-8: %s" % distinct, file=sys.stderr, flush=True)
    assert max(distinct) <= 44
    ses.close(); st.close()


@pytest.mark.parametrize("expert_gemm", ["1", "0"])
def test_c5_expert_shard_prefill_and_wide_batch_on_matrix_cores(tmp_path, expert_gemm):
    """The same shard with enough tokens per expert for the matrix cores (from four pairs per expert on average: 32
    tokens x top-8 over 64 experts): a 96-token prompt chunk of one sequence, then a decode batch of 40 sequences, Zipf
    router, against the oracle; routing decisions identical.  Once with the expert products as tiles of the large-tile
    f16 GEMM (the default), once through the 16-pair integer kernel (moe_gemm=0)."""
    m = mesh()
    cfg = dict(models.CONFIGS["qwen3-30b-a3b"])
    path = os.path.join(str(tmp_path), "shard.gguf")
    tensors = models.write_model(path, cfg, [5, 6], seed=9, n_expert_local=64, fast=True, router="zipf")
    n_ctx, E = 128, 2048
    st = m.Stage(path, 5, 7, n_ctx=n_ctx, n_seq_max=40, n_batch_max=96)
    os.unlink(path)
    ses = st.session(moe_gemm=int(expert_gemm))
    orc = StageOracle(cfg, tensors, 5, 7, n_ctx, n_seq_max=40)
    rng = np.random.Generator(np.random.PCG64(56))
    # prompt chunk
    T = 96
    x = models.zipf_hidden_state(rng, T, E)
    pos = np.arange(T, dtype=np.int32)
    got = ses.decode(x, pos).view(np.float32).reshape(T, E)
    ref = orc.forward(x, pos)
    r = rel_l2(got - x, ref - x)
    report("C5 shard layers 5-6, 96-token prefill (matrix-core expert products, moe_gemm=%s; of the layers' contribution)" % expert_gemm, r)
    assert r <= NORTH_STAR
    assert np.array_equal(np.sort(ses.moe_last_ids(T), axis=1), np.sort(np.stack(orc.last_expert_ids), axis=1))
    # wide decode batch: sequence 0 continues its prompt, the others start
    T = 40
    x = models.zipf_hidden_state(rng, T, E)
    pos = np.zeros(T, np.int32)
    pos[0] = 96
    seq = np.arange(T, dtype=np.int32)
    got = ses.decode(x, pos, seq=seq).view(np.float32).reshape(T, E)
    ref = orc.forward(x, pos, seq=seq)
    r = rel_l2(got - x, ref - x)
    report("C5 shard layers 5-6, decode batch 40 (matrix-core expert products, moe_gemm=%s)" % expert_gemm, r)
    assert r <= NORTH_STAR
    assert np.array_equal(np.sort(ses.moe_last_ids(T), axis=1), np.sort(np.stack(orc.last_expert_ids), axis=1))
    ses.close(); st.close()


def test_c5_expert_shard_long_prefill_as_expert_gemm_tiles(tmp_path):
    """The same shard with a 272-token prompt chunk (34 pairs per expert on average; ragged: 272 = 2 * 128 + 16): the
    pairs are sorted by expert and the expert products run as tiles of the large-tile f16 GEMM.  Against the oracle, the
    routing decisions identical; then a second chunk on top; then the first chunk again through the 16-pair
    integer matrix-core kernel (moe_gemm=0), which has to agree to within both paths' distance from the oracle."""
    m = mesh()
    cfg = dict(models.CONFIGS["qwen3-30b-a3b"])
    path = os.path.join(str(tmp_path), "shard.gguf")
    tensors = models.write_model(path, cfg, [5, 6], seed=9, n_expert_local=64, fast=True, router="zipf")
    n_ctx, E = 640, 2048
    st = m.Stage(path, 5, 7, n_ctx=n_ctx, n_seq_max=2, n_batch_max=520)
    os.unlink(path)
    ses = st.session()
    orc = StageOracle(cfg, tensors, 5, 7, n_ctx, n_seq_max=2)
    rng = np.random.Generator(np.random.PCG64(57))
    T = 272
    x = models.zipf_hidden_state(rng, T, E)
    pos = np.arange(T, dtype=np.int32)
    got = ses.decode(x, pos).view(np.float32).reshape(T, E)
    ref = orc.forward(x, pos)
    r = rel_l2(got - x, ref - x)
    report("C5 shard layers 5-6, 272-token prefill (expert products as large-tile GEMM tiles; of the layers' contribution)", r)
    assert r <= NORTH_STAR
    assert max(rel_l2(got[i] - x[i], ref[i] - x[i]) for i in range(T)) <= 3 * NORTH_STAR
    assert np.array_equal(np.sort(ses.moe_last_ids(T), axis=1), np.sort(np.stack(orc.last_expert_ids), axis=1))
    T2 = 150
    x2 = models.zipf_hidden_state(rng, T2, E)
    pos2 = np.arange(T, T + T2, dtype=np.int32)
    got2 = ses.decode(x2, pos2).view(np.float32).reshape(T2, E)
    ref2 = orc.forward(x2, pos2)
    r2 = rel_l2(got2 - x2, ref2 - x2)
    report("C5 shard layers 5-6, second chunk of 150 tokens on top (same path)", r2)
    assert r2 <= NORTH_STAR
    # a 520-token chunk of the other sequence (from 512 tokens the router runs as small workgroups, one per token)
    T3 = 520
    x3 = models.zipf_hidden_state(rng, T3, E)
    pos3 = np.arange(T3, dtype=np.int32)
    got3 = ses.decode(x3, pos3, seq=np.ones(T3, np.int32)).view(np.float32).reshape(T3, E)
    ref3 = orc.forward(x3, pos3, seq=np.ones(T3, np.int32))
    r3 = rel_l2(got3 - x3, ref3 - x3)
    report("C5 shard layers 5-6, 520-token prefill of a second sequence (same path)", r3)
    assert r3 <= NORTH_STAR
    assert np.array_equal(np.sort(ses.moe_last_ids(T3), axis=1), np.sort(np.stack(orc.last_expert_ids), axis=1))
    ses.close()
    ses = st.session(moe_gemm=0)
    alt = ses.decode(x, pos).view(np.float32).reshape(T, E)
    ra = rel_l2(alt - x, ref - x)
    report("C5 shard layers 5-6, the same 272 tokens through the 16-pair integer kernel", ra)
    assert ra <= NORTH_STAR
    assert rel_l2(got - x, alt - x) <= r + ra
    ses.close(); st.close()


def test_c5_combine_step_quantises_for_the_next_layer_bit_identically(tmp_path):
    """Decode batch 16 over three shard layers: the combine step at the end of a mixture-of-experts layer also writes the
    quantised activations the next layer's q / k / v launch reads.  The same bits as with the two separate launches
    (moe_fuse_quant=0), step after step."""
    m = mesh()
    cfg = dict(models.CONFIGS["qwen3-30b-a3b"])
    path = os.path.join(str(tmp_path), "shard.gguf")
    models.write_model(path, cfg, [5, 6, 7], seed=9, n_expert_local=64, fast=True, router="zipf")
    E = 2048
    st = m.Stage(path, 5, 8, n_ctx=64, n_seq_max=16, n_batch_max=16)
    os.unlink(path)
    rng = np.random.Generator(np.random.PCG64(58))
    xs = [models.zipf_hidden_state(rng, 16, E) for _ in range(3)]
    outs = []
    for fuse in ("1", "0"):
        ses = st.session(moe_fuse_quant=int(fuse))
        got = []
        for step, x in enumerate(xs):
            got.append(ses.decode(x, np.full(16, step, np.int32), seq=np.arange(16, dtype=np.int32)).view(np.uint32).copy())
        outs.append(got)
        ses.close()
    for a, b in zip(*outs):
        assert np.array_equal(a, b)
    st.close()
