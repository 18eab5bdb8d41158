"""GPU parity of the stage executor (GEMV, RoPE/KV, attention, layer loop) through the C ABI against the CPU
oracle.  Floating point: tolerance is relative L2 <= 1e-3 for f32-activation paths (the north-star bar for a
whole stage is 1e-2), stated per test."""
import os

import numpy as np
import pytest

import models
import oracle
from oracle.stage import StageOracle
from util import mesh

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def rel_l2(a, b):
    a = np.asarray(a, np.float64).reshape(-1)
    b = np.asarray(b, np.float64).reshape(-1)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


@pytest.mark.parametrize("type_", [models.Q4_K, models.Q6_K])
@pytest.mark.parametrize("M,K", [(16, 256), (40, 512), (1000, 1024)])
def test_tiled_layout_round_trip(type_, M, K):
    m = mesh()
    rng = np.random.Generator(np.random.PCG64(M + K))
    be, bb = models.BLOCK[type_]
    data = rng.integers(0, 256, M * K // be * bb, dtype=np.uint8)
    w = m.Weight(type_, data, M, K)
    assert w.nbytes == data.size
    assert np.array_equal(w.download(), data)
    w.close()


@pytest.mark.parametrize("type_", [models.Q4_K, models.Q6_K, models.Q8_0, models.Q5_0, models.F16, models.F32])
@pytest.mark.parametrize("M,K", [(48, 512), (1024, 4096), (72, 14336)])
def test_mul_mat_vs_oracle(type_, M, K):
    m = mesh()
    rng = np.random.Generator(np.random.PCG64(type_ * 131 + M))
    data = models.random_tensor(rng, type_, M, K)
    w = m.Weight(type_, data, M, K)
    for T in (1, 2, 3, 4, 7):
        x = rng.standard_normal((T, K)).astype(np.float32)
        xd = torch.from_numpy(x).cuda()
        yd = torch.full((T, M), np.nan, dtype=torch.float32, device="cuda")
        w.mul_mat_dev(xd.data_ptr(), T, yd.data_ptr(), torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        ref = oracle.mul_mat(type_, data, M, K, x)
        # K-quant kernels round activations to 16-bit fixed point per 32-block (error ~2e-5); the others stay f32
        tol = 1e-4 if type_ in (models.Q4_K, models.Q6_K) else 2e-6
        assert rel_l2(yd.cpu().numpy(), ref) <= tol, (type_, M, K, T)
    w.close()


def cfg_layers(name):
    return models.CONFIGS[name]["n_layer"]


def _open(tmp_path, name, layers, lb, le, n_ctx=64, n_seq=2, n_batch=16, seed=5, **kw):
    m = mesh()
    cfg = models.CONFIGS[name]
    path = os.path.join(str(tmp_path), name + ".gguf")
    tensors = models.write_model(path, cfg, layers, seed=seed, **kw)
    st = m.Stage(path, lb, le, n_ctx=n_ctx, n_seq_max=n_seq, n_batch_max=n_batch)
    os.unlink(path)
    return m, cfg, tensors, st


@pytest.mark.parametrize("name", ["tiny-llama", "tiny-qwen2", "tiny-qwen3", "tiny-odd"])
def test_stage_prefill_then_decode_matches_oracle(tmp_path, name):
    cfg = models.CONFIGS[name]
    nl = cfg["n_layer"]
    lb, le = (1, nl) if nl > 2 else (0, nl)
    m, cfg, tensors, st = _open(tmp_path, name, range(lb, le), lb, le)
    assert st.weight_bytes == sum(d.nbytes for _, _, d in tensors.values())
    ses = st.session()
    orc = StageOracle(cfg, tensors, lb, le, 64, n_seq_max=2)
    rng = np.random.Generator(np.random.PCG64(7))
    E = cfg["n_embd"]
    # prefill 7 tokens of sequence 1, then three single-token steps, then a mixed batch over both sequences
    x = rng.standard_normal((7, E)).astype(np.float32)
    got = ses.decode(x, np.arange(7), seq=np.ones(7, np.int32)).view(np.float32).reshape(7, E)
    ref = orc.forward(x, np.arange(7), seq=np.ones(7, np.int32))
    assert rel_l2(got, ref) <= 1e-3
    for step in range(3):
        x1 = rng.standard_normal((1, E)).astype(np.float32)
        got = ses.decode(x1, [7 + step], seq=[1]).view(np.float32)
        ref = orc.forward(x1, [7 + step], seq=[1])
        assert rel_l2(got, ref) <= 1e-3
    xm = rng.standard_normal((5, E)).astype(np.float32)
    pos, seq = [0, 10, 1, 11, 2], [0, 1, 0, 1, 0]
    got = ses.decode(xm, pos, seq=seq).view(np.float32).reshape(5, E)
    ref = orc.forward(xm, pos, seq=seq)
    assert rel_l2(got, ref) <= 1e-3
    # the KV cache holds what the oracle's holds (f16 of nearly equal f32 values: compare as numbers)
    for il in range(lb, le):
        k, v = ses.kv_read(il, 1, 0, 12)
        ko = orc.k[il - lb, 1, :, :12].transpose(1, 0, 2)
        vo = orc.v[il - lb, 1, :, :12].transpose(1, 0, 2)
        assert rel_l2(k.view(np.float16).astype(np.float32), ko.view(np.float16).astype(np.float32)) <= 2e-3
        assert rel_l2(v.view(np.float16).astype(np.float32), vo.view(np.float16).astype(np.float32)) <= 2e-3
    ses.close()
    st.close()


@pytest.mark.parametrize("fmt_name", ["f16", "q8_0"])
def test_stage_boundary_formats(tmp_path, fmt_name):
    m, cfg, tensors, st = _open(tmp_path, "tiny-llama", range(0, 2), 0, 2)
    fmt = {"f16": m.F16, "q8_0": m.Q8_0}[fmt_name]
    ses = st.session()
    orc = StageOracle(cfg, tensors, 0, 2, 64)
    rng = np.random.Generator(np.random.PCG64(9))
    E = cfg["n_embd"]
    x = rng.standard_normal((4, E)).astype(np.float32)
    if fmt == m.F16:
        packed_in = oracle.fp32_to_fp16(x.reshape(-1))
        x_eff = oracle.fp16_to_fp32(packed_in).reshape(4, E)
    else:
        packed_in = oracle.quantize_q8_0(x.reshape(-1))
        x_eff = oracle.dequantize(oracle.Q8_0, packed_in, x.size).reshape(4, E)
    out = ses.decode(packed_in, np.arange(4), in_fmt=fmt, out_fmt=fmt)
    assert out.size == m.act_packed_size(fmt, 4, E)
    ref = orc.forward(x_eff, np.arange(4))
    if fmt == m.F16:
        got = oracle.fp16_to_fp32(out.view(np.uint16))
        assert rel_l2(got, ref) <= 1e-3
    else:
        got = oracle.dequantize(oracle.Q8_0, out, ref.size)
        assert rel_l2(got, ref) <= 1.5e-2        # one q8_0 rounding of the output
        # and the packing itself is the bit-exact codec applied to the stage's own f32 output
        f32_out = ses.decode(packed_in, np.arange(4), in_fmt=fmt, out_fmt=m.F32).view(np.float32)
        assert np.array_equal(out, oracle.quantize_q8_0(f32_out))
    ses.close()
    st.close()


def test_llama3_8b_shaped_layers_decode_with_long_kv(tmp_path):
    """Two real-shape layers (one with Q6_K attn_v/ffn_down, one all Q4_K), batch 1, 4 and 3 at KV depth 300+."""
    name = "llama3-8b"
    m, cfg, tensors, st = _open(tmp_path, name, [3, 4], 3, 5, n_ctx=512, n_seq=4, n_batch=8)
    assert tensors["blk.3.ffn_down.weight"][0] == models.Q6_K and tensors["blk.4.ffn_down.weight"][0] == models.Q4_K
    ses = st.session()
    orc = StageOracle(cfg, tensors, 3, 5, 512, n_seq_max=4)
    rng = np.random.Generator(np.random.PCG64(11))
    n_past = 300
    for il in (3, 4):
        for s in range(4):
            k = (rng.standard_normal((n_past, 8, 128)) * 0.5).astype(np.float16).view(np.uint16)
            v = (rng.standard_normal((n_past, 8, 128)) * 0.5).astype(np.float16).view(np.uint16)
            ses.kv_write(il, s, 0, k, v)
            orc.k[il - 3, s, :, :n_past] = k.transpose(1, 0, 2)
            orc.v[il - 3, s, :, :n_past] = v.transpose(1, 0, 2)
    x = rng.standard_normal((1, 4096)).astype(np.float32)
    got = ses.decode(x, [n_past], seq=[2]).view(np.float32)
    ref = orc.forward(x, [n_past], seq=[2])
    assert rel_l2(got, ref) <= 1e-3
    x4 = rng.standard_normal((4, 4096)).astype(np.float32)
    pos, seq = [n_past, n_past, n_past + 1, n_past], [0, 1, 2, 3]
    got = ses.decode(x4, pos, seq=seq).view(np.float32).reshape(4, 4096)
    ref = orc.forward(x4, pos, seq=seq)
    assert rel_l2(got, ref) <= 3e-3        # four tokens: the batched MFMA GEMM (f16 activations)
    # three tokens: the 3-column mat-vec kernels
    x3 = rng.standard_normal((3, 4096)).astype(np.float32)
    pos, seq = [n_past + 1, n_past + 1, n_past], [0, 1, 3]
    got = ses.decode(x3, pos, seq=seq).view(np.float32).reshape(3, 4096)
    ref = orc.forward(x3, pos, seq=seq)
    assert rel_l2(got, ref) <= 1e-3
    ses.close()
    st.close()


def test_qwen25_32b_shaped_layer_all_decode_paths(tmp_path):
    """One real-shape Qwen2.5-32B layer (hidden 5120 = 20 super-blocks, 40 heads / 8 KV heads = 5 per group, FFN 27648, q/k/v
    bias, NEOX rope): batch 1 on the mat-vec kernel, 4, 16 and a ragged 11 on the skinny MFMA GEMM, at KV depth 100."""
    name = "qwen2.5-32b"
    m, cfg, tensors, st = _open(tmp_path, name, [7], 7, 8, n_ctx=128, n_seq=16, n_batch=16)
    ses = st.session()
    orc = StageOracle(cfg, tensors, 7, 8, 128, n_seq_max=16)
    rng = np.random.Generator(np.random.PCG64(14))
    n_past = 100
    for s_ in range(16):
        k = (rng.standard_normal((n_past, 8, 128)) * 0.5).astype(np.float16).view(np.uint16)
        v = (rng.standard_normal((n_past, 8, 128)) * 0.5).astype(np.float16).view(np.uint16)
        ses.kv_write(7, s_, 0, k, v)
        orc.k[0, s_, :, :n_past] = k.transpose(1, 0, 2)
        orc.v[0, s_, :, :n_past] = v.transpose(1, 0, 2)
    nxt = [n_past] * 16
    for seqs, tol in (([3], 1e-3), ([0, 5, 9, 12], 3e-3), ([2, 6, 14], 1e-3), (list(range(16)), 3e-3), ([1, 2, 3, 4, 6, 7, 8, 10, 11, 13, 15], 3e-3)):
        T = len(seqs)
        pos = [nxt[q] for q in seqs]
        for q in seqs:
            nxt[q] += 1
        x = rng.standard_normal((T, 5120)).astype(np.float32)
        got = ses.decode(x, pos, seq=seqs).view(np.float32).reshape(T, 5120)
        ref = orc.forward(x, pos, seq=seqs)
        assert rel_l2(got, ref) <= tol, T
    ses.close(); st.close()


def test_decode_argument_errors(tmp_path):
    m, cfg, tensors, st = _open(tmp_path, "tiny-llama", range(0, 2), 0, 2, n_ctx=32, n_seq=1, n_batch=4)
    ses = st.session()
    x = np.zeros((5, 256), np.float32)
    for pos, seq, n in [([40], [0], 1), ([0], [3], 1), ([-1], [0], 1), (np.arange(5), None, 5)]:
        with pytest.raises(m.MeshError) as e:
            ses.decode(x[:n], pos, seq=seq)
        assert e.value.code == m.ERR_INVALID
    with pytest.raises(m.MeshError) as e:
        ses.decode(np.zeros(1, np.int32), [0], in_fmt=m.TOKENS)      # file has no token_embd
    assert e.value.code == m.ERR_INVALID
    with pytest.raises(m.MeshError):
        ses.decode(x[:1], [0], out_fmt=m.LOGITS)
    ses.close()
    st.close()


def test_moe_stage_matches_oracle_with_and_without_mask(tmp_path):
    m, cfg, tensors, st = _open(tmp_path, "tiny-moe", range(0, 2), 0, 2)
    ses = st.session()
    rng = np.random.Generator(np.random.PCG64(21))
    E = cfg["n_embd"]
    x = rng.standard_normal((6, E)).astype(np.float32)
    orc = StageOracle(cfg, tensors, 0, 2, 64)
    got = ses.decode(x, np.arange(6)).view(np.float32).reshape(6, E)
    ref = orc.forward(x, np.arange(6))
    assert rel_l2(got, ref) <= 1e-3
    assert np.array_equal(np.sort(ses.moe_last_ids(6), axis=1), np.sort(np.stack(orc.last_expert_ids), axis=1))
    # expert mask: only 3 of the 8 experts allowed (0 / -inf added to the selection probabilities)
    allowed = np.zeros(8, bool)
    allowed[[1, 4, 6]] = True
    ses2 = st.session()
    ses2.set_expert_mask(allowed)
    orc2 = StageOracle(cfg, tensors, 0, 2, 64, expert_mask=np.where(allowed, 0.0, -np.inf).astype(np.float32))
    got = ses2.decode(x, np.arange(6)).view(np.float32).reshape(6, E)
    ref2 = orc2.forward(x, np.arange(6))
    assert rel_l2(got, ref2) <= 1e-3
    assert set(ses2.moe_last_ids(6).reshape(-1)) <= {1, 4, 6}
    assert rel_l2(ref2, ref) > 1e-2            # the mask really changed the result
    with pytest.raises(m.MeshError) as e:
        ses2.set_expert_mask(np.ones(5, bool))
    assert e.value.code == m.ERR_INVALID
    ses2.set_expert_mask(None)
    ses.close(); ses2.close(); st.close()


def test_moe_pairs_grouped_by_expert_equal_pair_by_pair(tmp_path):
    """The expert launches walk (token, slot) pairs grouped by expert, up to four pairs of an expert per pass over its
    weights (mat-vec kernel, fewer than 5 tokens) or up to sixteen (matrix-core kernel); the switch moe_group=0 runs every pair
    as its own product.  A column's arithmetic does not depend on its neighbours, so the mat-vec groups give the same
    bits as pair-by-pair, whatever the group sizes (8 experts, top-2: 1 to 30 tokens make groups of every size and
    experts with more than one group)."""
    m, cfg, tensors, st = _open(tmp_path, "tiny-moe", range(0, 2), 0, 2, n_ctx=64, n_batch=64)
    E = cfg["n_embd"]
    rng = np.random.Generator(np.random.PCG64(77))
    ses = st.session()
    ses0 = st.session(moe_group=0)
    orc = StageOracle(cfg, tensors, 0, 2, 64)
    pos0 = 0
    for T in (1, 2, 4, 3, 5, 23, 26):           # the bit-exact cases first: afterwards the two caches differ in the last bits
        x = rng.standard_normal((T, E)).astype(np.float32)
        pos = np.arange(pos0, pos0 + T)
        a = ses.decode(x, pos).view(np.float32).reshape(T, E)
        b = ses0.decode(x, pos).view(np.float32).reshape(T, E)
        if T < 5:
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), T
        else:
            # from 5 tokens on the grouped launches run on the matrix cores (16 pairs of an expert per pass): 16-bit
            # fixed-point activations and exact integer dot products like the mat-vec kernel, f32 sums in another order
            assert rel_l2(a, b) <= 5e-5, T
        assert np.array_equal(ses.moe_last_ids(T), ses0.moe_last_ids(T))
        assert rel_l2(a, orc.forward(x, pos)) <= 1e-3
        pos0 += T
    ses.close(); ses0.close(); st.close()


def test_qwen3_30b_a3b_shaped_expert_shard_layer(tmp_path):
    """One real-shape MoE layer of a 64-expert shard (of 128), decode batch 16, top-8 routing."""
    m = mesh()
    cfg = dict(models.CONFIGS["qwen3-30b-a3b"])
    path = os.path.join(str(tmp_path), "shard.gguf")
    tensors = models.write_model(path, cfg, [5], seed=9, n_expert_local=64, fast=True)
    st = m.Stage(path, 5, 6, n_ctx=64, n_seq_max=16, n_batch_max=16)
    os.unlink(path)
    assert st.info.n_expert == 64 and st.info.n_expert_used == 8
    ses = st.session()
    orc = StageOracle(cfg, tensors, 5, 6, 64, n_seq_max=16)
    rng = np.random.Generator(np.random.PCG64(31))
    x = rng.standard_normal((16, 2048)).astype(np.float32)
    pos, seq = np.zeros(16, np.int32), np.arange(16, dtype=np.int32)
    got = ses.decode(x, pos, seq=seq).view(np.float32).reshape(16, 2048)
    ref = orc.forward(x, pos, seq=seq)
    assert rel_l2(got, ref) <= 1e-3
    ids = ses.moe_last_ids(16)
    assert np.array_equal(np.sort(ids, axis=1), np.sort(np.stack(orc.last_expert_ids), axis=1))
    assert len(set(ids.reshape(-1))) > 8
    ses.close()
    # the router launch's last-arriving workgroup routes and groups the pairs (the default), or a second launch does
    # (moe_router_tail=0): the same bits and the same routing, step after step (the arrival counter returns to zero)
    runs = []
    for tail in (1, 0):
        q = st.session(moe_router_tail=tail)
        r2 = np.random.Generator(np.random.PCG64(32))
        outs = []
        for step, T in enumerate((16, 11, 6, 16, 1, 16)):
            xs = r2.standard_normal((T, 2048)).astype(np.float32)
            outs.append((q.decode(xs, np.full(T, step, np.int32), seq=np.arange(T, dtype=np.int32)).copy(), q.moe_last_ids(T).copy()))
        runs.append(outs)
        q.close()
    for (a, ia), (b, ib) in zip(*runs):
        assert np.array_equal(ia, ib)
        assert np.array_equal(a, b)
    st.close()


@pytest.mark.parametrize("name,T", [("tiny-llama", 192), ("tiny-llama", 257), ("tiny-qwen2", 256), ("tiny-qwen3", 300), ("tiny-g7", 193)])
def test_prefill_gemm_token_counts_and_head_layouts(tmp_path, name, T):
    """Prefill-sized calls at and around the 128-token tile edges, over the small models: head_dim 64 and 128, K / V
    projections of 128 and 256 rows (q and k fused with and without v), q/k norms, biases, odd head groups."""
    m, cfg, tensors, st = _open(tmp_path, name, range(cfg_layers(name)), 0, cfg_layers(name), n_ctx=320, n_seq=1, n_batch=304)
    E = cfg["n_embd"]
    x = np.random.Generator(np.random.PCG64(T)).standard_normal((T, E)).astype(np.float32)
    ses = st.session()
    got = ses.decode(x, np.arange(T)).view(np.float32).reshape(T, E)
    orc = StageOracle(cfg, tensors, 0, cfg_layers(name), 320, n_seq_max=1)
    ref = orc.forward(x, np.arange(T))
    assert rel_l2(got, ref) <= 3e-3
    assert max(rel_l2(got[i], ref[i]) for i in range(T)) <= 1e-2
    # one more token on top of the prefilled cache, through the mat-vec path
    x1 = np.random.Generator(np.random.PCG64(1)).standard_normal((1, E)).astype(np.float32)
    got1 = ses.decode(x1, [T]).view(np.float32)
    assert rel_l2(got1, orc.forward(x1, [T])) <= 3e-3
    ses.close(); st.close()


@pytest.mark.parametrize("name,layers", [("llama3-8b", [3, 4]), ("tiny-qwen2", [0, 1, 2]), ("tiny-llama", [0, 1])])
def test_prefill_gemm_variants_agree(tmp_path, name, layers):
    """Stages that can take prefill-sized calls keep a second copy of their projections arranged for the GEMM's
    staging threads, with the per-sub-block f16 scale products precomputed; the stage switch gemm_layout=0 makes the GEMM read the
    mat-vec tiles instead.  Same arithmetic on the same values: bit-identical outputs (q4_K and q6_K matrices, row
    counts that are and are not multiples of the 128-row tile), both when the matrix-core waves take their activation
    fragments straight from the k8-major layout and when row-major activations are staged through LDS
    (gemm_xdirect=0).  Across producers of the f16 activations -- the two activation layouts, or the SwiGLU
    epilogue of the fused gate / up launch against the separate kernel (gemm_fused=0) -- the f32 expressions are
    the same but compiled in different kernels, so a few values differ by an f16 rounding step: those agree to 1e-3."""
    m = mesh()
    cfg = models.CONFIGS[name]
    path = os.path.join(str(tmp_path), name + ".gguf")
    models.write_model(path, cfg, layers, seed=5)
    lb, le = layers[0], layers[-1] + 1
    st1 = m.Stage(path, lb, le, n_ctx=256, n_seq_max=1, n_batch_max=208)
    st0 = m.Stage(path, lb, le, n_ctx=256, n_seq_max=1, n_batch_max=208, tuning={"gemm_layout": 0})
    os.unlink(path)
    E = cfg["n_embd"]
    T = 200
    x = np.random.Generator(np.random.PCG64(3)).standard_normal((T, E)).astype(np.float32)

    def run(st, **options):
        ses = st.session(**options)
        out = ses.decode(x, np.arange(T)).view(np.uint32)
        ses.close()
        return out

    fused = run(st1)
    split = run(st1, gemm_fused=0)
    assert np.array_equal(split, run(st0))
    staged = run(st1, gemm_fused=0, gemm_xdirect=0)
    assert np.array_equal(staged, run(st0, gemm_xdirect=0))
    f = lambda a: a.view(np.float32)
    assert rel_l2(f(fused), f(split)) <= 1e-3
    assert rel_l2(f(staged), f(split)) <= 1e-3
    st1.close(); st0.close()


def test_prefill_mfma_path_matches_oracle_and_decode_path(tmp_path):
    """Calls with >= 17 tokens take the large-tile MFMA GEMM (f16 activations, f32 accumulate): compare it with the
    oracle and with the same tokens fed 16 at a time (skinny GEMM), then keep decoding on top of the prefilled cache."""
    m, cfg, tensors, st = _open(tmp_path, "llama3-8b", [3, 4], 3, 5, n_ctx=256, n_seq=2, n_batch=208)
    E = cfg["n_embd"]
    rng = np.random.Generator(np.random.PCG64(41))
    T = 200                                     # at least 17 tokens take the large-tile GEMM; not a multiple of its 128-token tile
    x = rng.standard_normal((T, E)).astype(np.float32)
    ses = st.session()
    got = ses.decode(x, np.arange(T)).view(np.float32).reshape(T, E)
    orc = StageOracle(cfg, tensors, 3, 5, 256, n_seq_max=2)
    ref = orc.forward(x, np.arange(T))
    assert rel_l2(got, ref) <= 3e-3             # f16 GEMM inputs
    # same tokens 16 at a time (the skinny MFMA GEMM of batched decode, f16 activations as well), into the other sequence
    ses2 = st.session()
    parts = [ses2.decode(x[i:i + 16], np.arange(i, min(i + 16, T)), seq=np.ones(min(16, T - i), np.int32)).view(np.float32)
             for i in range(0, T, 16)]
    step = np.concatenate(parts).reshape(T, E)
    assert rel_l2(got, step) <= 3e-3
    assert rel_l2(step, ref) <= 3e-3
    # decode one more token on top of the prefilled cache
    x1 = rng.standard_normal((1, E)).astype(np.float32)
    got1 = ses.decode(x1, [T]).view(np.float32)
    ref1 = orc.forward(x1, [T])
    assert rel_l2(got1, ref1) <= 3e-3
    ses.close(); ses2.close(); st.close()


def test_prefill_path_small_model_with_bias_and_neox(tmp_path):
    m, cfg, tensors, st = _open(tmp_path, "tiny-qwen2", range(0, 3), 0, 3, n_ctx=512, n_seq=2, n_batch=208)
    E = cfg["n_embd"]
    rng = np.random.Generator(np.random.PCG64(43))
    orc = StageOracle(cfg, tensors, 0, 3, 512, n_seq_max=2)
    ses = st.session()
    # large-tile GEMM + chunk attention from position 0, a second chunk on top of the first (ragged: 200 = 6 * 32 + 8),
    # then the skinny GEMM (one ragged 16-column pass) on the other sequence and calls of 27 and 47 tokens on top of it
    # (large-tile GEMM again, K split over workgroups: few row blocks x one token block)
    for T, pos0, seq in ((200, 0, 0), (200, 200, 0), (13, 0, 1), (27, 13, 1), (47, 40, 1)):
        x = rng.standard_normal((T, E)).astype(np.float32)
        sq = np.full(T, seq, np.int32)
        pos = np.arange(pos0, pos0 + T)
        got = ses.decode(x, pos, seq=sq).view(np.float32).reshape(T, E)
        ref = orc.forward(x, pos, seq=sq)
        assert rel_l2(got, ref) <= 3e-3, (T, pos0)
    ses.close(); st.close()


def test_long_chunk_with_an_odd_number_of_head_rows(tmp_path):
    """2816 tokens of a model with three KV heads of four query heads: the chunk attention launch has 88 query tiles x 3
    head rows = 264 workgroups, between one and two per CU, an even count with an odd number of rows -- the shape for
    which a launch must not hand the second half of its workgroups their tiles in forward order (half the launch would
    not be whole rows, and tiles would be computed twice or not at all)."""
    T = 2816
    m, cfg, tensors, st = _open(tmp_path, "tiny-kv3", [0], 0, 1, n_ctx=T, n_seq=1, n_batch=T)
    E = cfg["n_embd"]
    rng = np.random.Generator(np.random.PCG64(44))
    orc = StageOracle(cfg, tensors, 0, 1, T, n_seq_max=1)
    ses = st.session()
    x = rng.standard_normal((T, E)).astype(np.float32)
    got = ses.decode(x, np.arange(T)).view(np.float32).reshape(T, E)
    ref = orc.forward(x, np.arange(T))
    assert rel_l2(got, ref) <= 3e-3
    assert max(rel_l2(got[i], ref[i]) for i in range(0, T, 29)) <= 1e-2
    ses.close(); st.close()


def test_short_chunks_on_a_long_history_split_their_key_walks(tmp_path):
    """A chunk with few query tiles and a long history splits every tile's walk over several workgroups and merges the
    partials (the split-KV combine kernel): 96 tokens on top of 448 (two splits), then 48 on top of 2000 (eight splits;
    the last split holds the diagonal, where the chunk's earlier queries see no key at all).  Against the oracle, and
    against the same calls with the splitting switched off."""
    n_ctx = 2112
    m, cfg, tensors, st = _open(tmp_path, "tiny-qwen2", [0], 0, 1, n_ctx=n_ctx, n_seq=1, n_batch=1024)
    E = cfg["n_embd"]
    rng = np.random.Generator(np.random.PCG64(46))
    orc = StageOracle(cfg, tensors, 0, 1, n_ctx, n_seq_max=1)
    calls = [(448, 0), (96, 448), (976, 544), (480, 1520), (48, 2000)]
    xs = [rng.standard_normal((T, E)).astype(np.float32) for T, _ in calls]
    outs = {}
    for mode in ("1", "0"):
        ses = st.session(attn_chunk_ksplit=int(mode))
        outs[mode] = [ses.decode(x, np.arange(p0, p0 + T)).view(np.float32).reshape(T, E).copy() for x, (T, p0) in zip(xs, calls)]
        ses.close()
    for x, (T, p0), got, alt in zip(xs, calls, outs["1"], outs["0"]):
        ref = orc.forward(x, np.arange(p0, p0 + T))
        assert rel_l2(got, ref) <= 3e-3, (T, p0)
        assert max(rel_l2(got[i], ref[i]) for i in range(T)) <= 1e-2, (T, p0)
        assert rel_l2(got, alt) <= 2e-3, (T, p0)
    st.close()


def test_key_split_boundary_inside_a_query_tile(tmp_path):
    """Chunks whose first position is not a multiple of 32: a key split then begins strictly inside a query tile's
    position range, so that in the split's first step the tile's earlier queries still see no key while the later ones
    do.  40 tokens on top of 3560 (eight splits of 512 keys; the last begins at key 3584, inside positions 3560..3591)
    and 512 tokens on top of 10; finite, against the oracle, and against the same calls with the splitting switched off."""
    n_ctx = 3712
    m, cfg, tensors, st = _open(tmp_path, "tiny-qwen2", [0], 0, 1, n_ctx=n_ctx, n_seq=2, n_batch=1024)
    E = cfg["n_embd"]
    rng = np.random.Generator(np.random.PCG64(3560))
    orc = StageOracle(cfg, tensors, 0, 1, n_ctx, n_seq_max=2)
    hist = {0: 3560, 1: 10}
    kv = {}
    for s, n_past in hist.items():
        k = (rng.standard_normal((n_past, 1, 128)) * 0.5).astype(np.float16).view(np.uint16)
        v = (rng.standard_normal((n_past, 1, 128)) * 0.5).astype(np.float16).view(np.uint16)
        kv[s] = (k, v)
        orc.k[0, s, :, :n_past] = np.ascontiguousarray(k.transpose(1, 0, 2))
        orc.v[0, s, :, :n_past] = np.ascontiguousarray(v.transpose(1, 0, 2))
    calls = [(40, 3560, 0), (512, 10, 1)]
    xs = [rng.standard_normal((T, E)).astype(np.float32) for T, _, _ in calls]
    outs = {}
    for mode in ("1", "0"):
        ses = st.session(attn_chunk_ksplit=int(mode))
        for s, (k, v) in kv.items():
            ses.kv_write(0, s, 0, k, v)
        outs[mode] = [ses.decode(x, np.arange(p0, p0 + T), seq=[s] * T).view(np.float32).reshape(T, E).copy() for x, (T, p0, s) in zip(xs, calls)]
        ses.close()
    for x, (T, p0, s), got, alt in zip(xs, calls, outs["1"], outs["0"]):
        assert np.isfinite(got).all(), (T, p0)
        ref = orc.forward(x, np.arange(p0, p0 + T), seq=[s] * T)
        assert rel_l2(got, ref) <= 3e-3, (T, p0)
        assert max(rel_l2(got[i], ref[i]) for i in range(T)) <= 1e-2, (T, p0)
        assert rel_l2(got, alt) <= 2e-3, (T, p0)
    st.close()


def test_prefill_chunks_of_a_model_with_one_query_head_per_kv_head(tmp_path):
    """Groups of fewer than four query heads fill a chunk attention workgroup with several consecutive query tiles (four for
    one head per KV head): 300 tokens from position 0 (ragged: 9 full tiles + 12 tokens, so the last workgroup has a tile
    without queries), a second chunk of 100 on top, against the oracle."""
    m, cfg, tensors, st = _open(tmp_path, "tiny-mha", [0], 0, 1, n_ctx=512, n_seq=1, n_batch=300)
    E = cfg["n_embd"]
    rng = np.random.Generator(np.random.PCG64(45))
    orc = StageOracle(cfg, tensors, 0, 1, 512, n_seq_max=1)
    ses = st.session()
    for T, pos0 in ((300, 0), (100, 300)):
        x = rng.standard_normal((T, E)).astype(np.float32)
        pos = np.arange(pos0, pos0 + T)
        got = ses.decode(x, pos).view(np.float32).reshape(T, E)
        ref = orc.forward(x, pos)
        assert rel_l2(got, ref) <= 3e-3, (T, pos0)
        assert max(rel_l2(got[i], ref[i]) for i in range(T)) <= 1e-2, (T, pos0)
    ses.close(); st.close()


def test_batched_decode_skinny_gemm_matches_oracle_and_gemv_path(tmp_path):
    """Decode batches of 4..16 tokens run their projections on the matrix cores (gemm_skinny_f16.hip, gemm_skinny.hip).  Real-shape layers
    (one with q6_K attn_v / ffn_down, so q/k/v mix two weight types: one pair launch, or two launches), 16 sequences at KV depth 300, full and ragged
    batches; against the oracle and against the same steps fed three at a time through the mat-vec kernel."""
    name = "llama3-8b"
    m, cfg, tensors, st = _open(tmp_path, name, [3, 4], 3, 5, n_ctx=512, n_seq=16, n_batch=16)
    ses, ses4 = st.session(), st.session()
    ses_two = st.session(skinny_pair=0)        # q/k (q4_K) and v (q6_K) as two launches instead of one: the same bits
    int_one, int_two = st.session(skinny_f16=0), st.session(skinny_f16=0, skinny_pair=0)      # the same for the integer kernel
    orc = StageOracle(cfg, tensors, 3, 5, 512, n_seq_max=16)
    rng = np.random.Generator(np.random.PCG64(12))
    n_past = 300
    for il in (3, 4):
        for s in range(16):
            k = (rng.standard_normal((n_past, 8, 128)) * 0.5).astype(np.float16).view(np.uint16)
            v = (rng.standard_normal((n_past, 8, 128)) * 0.5).astype(np.float16).view(np.uint16)
            for x_ in (ses, ses4, ses_two, int_one, int_two):
                x_.kv_write(il, s, 0, k, v)
            orc.k[il - 3, s, :, :n_past] = k.transpose(1, 0, 2)
            orc.v[il - 3, s, :, :n_past] = v.transpose(1, 0, 2)
    nxt = [n_past] * 16
    for seqs in (list(range(16)), [1, 3, 4, 7, 8, 9, 10, 12, 15], [0, 2, 5, 6, 11]):
        T = len(seqs)
        pos = [nxt[s] for s in seqs]
        for s in seqs:
            nxt[s] += 1
        x = rng.standard_normal((T, 4096)).astype(np.float32)
        got = ses.decode(x, pos, seq=seqs).view(np.float32).reshape(T, 4096)
        ref = orc.forward(x, pos, seq=seqs)
        alt = np.concatenate([ses4.decode(x[i:i + 3], pos[i:i + 3], seq=seqs[i:i + 3]).view(np.float32) for i in range(0, T, 3)]).reshape(T, 4096)
        assert rel_l2(got, ref) <= 3e-3, T
        assert rel_l2(got, alt) <= 3e-3, T
        two = ses_two.decode(x, pos, seq=seqs).view(np.float32).reshape(T, 4096)
        assert np.array_equal(got, two), T
        if T >= 5:                          # (the integer kernel takes batches from five tokens on)
            i1 = int_one.decode(x, pos, seq=seqs).view(np.float32).reshape(T, 4096)
            i2 = int_two.decode(x, pos, seq=seqs).view(np.float32).reshape(T, 4096)
            assert np.array_equal(i1, i2), T
            assert rel_l2(i1, ref) <= 5e-4, T
        for q, p_ in ((seqs[0], pos[0]), (seqs[-1], pos[-1])):
            for il in (3, 4):
                ka, va = ses.kv_read(il, q, p_, 1)
                kb, vb = ses_two.kv_read(il, q, p_, 1)
                assert np.array_equal(ka, kb) and np.array_equal(va, vb)
    ses.close(); ses4.close(); ses_two.close(); int_one.close(); int_two.close(); st.close()


def test_wide_decode_batch_takes_large_tile_gemm(tmp_path):
    """From 17 tokens a call takes the large-tile MFMA GEMM whatever its shape: here 70 single-token sequences at ragged
    positions (not a prefill chunk, so the split-KV decode attention runs behind the GEMM's q/k/v).  One token block
    and 32..224 row blocks per projection: the launches split K over workgroups and add the slices in a second
    kernel.  Real-shape layers, against the oracle, against the same tokens fed 16 at a time (skinny GEMM) and against
    the unsplit launches (gemm_splitk=0: same products, another summation order)."""
    name = "llama3-8b"
    m, cfg, tensors, st = _open(tmp_path, name, [3, 4], 3, 5, n_ctx=64, n_seq=70, n_batch=70)
    ses, ses16 = st.session(), st.session()
    ses_whole = st.session(gemm_splitk=0)
    orc = StageOracle(cfg, tensors, 3, 5, 64, n_seq_max=70)
    rng = np.random.Generator(np.random.PCG64(21))
    depth = [int(d) for d in rng.integers(1, 40, size=70)]
    for il in (3, 4):
        for s in range(70):
            k = (rng.standard_normal((depth[s], 8, 128)) * 0.5).astype(np.float16).view(np.uint16)
            v = (rng.standard_normal((depth[s], 8, 128)) * 0.5).astype(np.float16).view(np.uint16)
            for x_ in (ses, ses16, ses_whole):
                x_.kv_write(il, s, 0, k, v)
            orc.k[il - 3, s, :, :depth[s]] = k.transpose(1, 0, 2)
            orc.v[il - 3, s, :, :depth[s]] = v.transpose(1, 0, 2)
    seqs = list(range(70))
    x = rng.standard_normal((70, 4096)).astype(np.float32)
    got = ses.decode(x, depth, seq=seqs).view(np.float32).reshape(70, 4096)
    ref = orc.forward(x, depth, seq=seqs)
    alt = np.concatenate([ses16.decode(x[i:i + 16], depth[i:i + 16], seq=seqs[i:i + 16]).view(np.float32) for i in range(0, 70, 16)]).reshape(70, 4096)
    whole = ses_whole.decode(x, depth, seq=seqs).view(np.float32).reshape(70, 4096)
    assert rel_l2(got, ref) <= 3e-3
    assert rel_l2(got, alt) <= 3e-3
    assert rel_l2(got, whole) <= 1e-3 and rel_l2(whole, ref) <= 3e-3
    # the appended K / V rows are the same f16 values on both paths up to one rounding step of the f16 activations
    for s in (0, 33, 69):
        ka, va = ses.kv_read(4, s, depth[s], 1)
        kb, vb = ses16.kv_read(4, s, depth[s], 1)
        assert rel_l2(ka.view(np.float16).astype(np.float32), kb.view(np.float16).astype(np.float32)) <= 3e-3
        assert rel_l2(va.view(np.float16).astype(np.float32), vb.view(np.float16).astype(np.float32)) <= 3e-3
    ses.close(); ses16.close(); ses_whole.close(); st.close()


def test_skinny_gemm_norms_ride_in_the_neighbouring_launches(tmp_path):
    """Batches of 4 to 16 tokens on the f16 skinny GEMM: the output projection and the down projection also write their
    result times the next RMS norm's weight as f16 plus per-workgroup sums of squares, and q/k/v and gate/up divide their
    products by the token's rms -- W . (y w / rms) = (W . (y w)) / rms -- instead of a norm launch in between
    (skinny_norm_fused=0).  Three real-shape layers (the middle one with q6_K attn_v / ffn_down), with a x40 outlier
    channel in one step so that the unnormalised f16 values are large: both ways against the oracle and against each
    other; the rounding points differ (f16 of y w against f16 of y w / rms), nothing else."""
    m, cfg, tensors, st = _open(tmp_path, "llama3-8b", [2, 3, 4], 2, 5, n_ctx=64, n_seq=16, n_batch=16)
    E = cfg["n_embd"]
    fused, plain = st.session(), st.session(skinny_norm_fused=0)
    assert fused.get_option("skinny_norm_fused") == 1
    orc = StageOracle(cfg, tensors, 2, 5, 64, n_seq_max=16)
    rng = np.random.Generator(np.random.PCG64(91))
    nxt = [0] * 16
    for step, T in enumerate((16, 5, 9, 16, 4, 13)):
        x = rng.standard_normal((T, E)).astype(np.float32)
        if step == 2:
            x[:, 1234] *= 40.0
        seqs = list(range(T))
        pos = [nxt[q] for q in seqs]
        for q in seqs:
            nxt[q] += 1
        a = fused.decode(x, pos, seq=seqs).view(np.float32).reshape(T, E)
        b = plain.decode(x, pos, seq=seqs).view(np.float32).reshape(T, E)
        ref = orc.forward(x, pos, seq=seqs)
        ra, rb, rab = rel_l2(a, ref), rel_l2(b, ref), rel_l2(a, b)
        print("[skinny norms] step %d, %d tokens: fused %.3e, separate %.3e of the oracle, %.3e apart" % (step, T, ra, rb, rab))
        assert np.isfinite(a).all()
        assert ra <= 3e-3 and rb <= 3e-3 and rab <= 3e-3, (step, T)
        assert max(rel_l2(a[i], ref[i]) for i in range(T)) <= 1e-2
    assert fused.f16_saturations() == 0
    fused.close(); plain.close(); st.close()


def test_decode_batches_of_17_to_32_stay_on_the_skinny_gemm(tmp_path):
    """Batches of 17 to 32 decode steps: one pass of the f16 skinny GEMM over the weights multiplies with two blocks of 16
    activation columns (the activation fragments of one super-block are held and refilled behind the MFMAs that used
    them), RoPE / KV append and the norm hand-over as for smaller batches.  Three real-shape layers (the middle one
    with q6_K attn_v / ffn_down) at ragged KV depths, a x40 outlier channel in one step: against the oracle, against the
    large-tile GEMM (skinny_f16_wide=0) and against norm launches of their own (skinny_norm_fused=0); then a smaller batch
    on the same sessions, so that the hand-over buffers of a 32-column call are followed by a 16-column one."""
    m, cfg, tensors, st = _open(tmp_path, "llama3-8b", [2, 3, 4], 2, 5, n_ctx=64, n_seq=32, n_batch=32)
    E = cfg["n_embd"]
    wide, gemm, plain = st.session(), st.session(skinny_f16_wide=0), st.session(skinny_norm_fused=0)
    two = st.session(skinny_pair=0)            # one launch per weight type in the q/k/v group: the same bits
    assert wide.get_option("skinny_f16_wide") == 1 and gemm.get_option("skinny_f16_wide") == 0
    orc = StageOracle(cfg, tensors, 2, 5, 64, n_seq_max=32)
    rng = np.random.Generator(np.random.PCG64(177))
    depth = [int(d) for d in rng.integers(0, 30, size=32)]
    for il in (2, 3, 4):
        for q in range(32):
            if depth[q] == 0:
                continue
            k = (rng.standard_normal((depth[q], 8, 128)) * 0.5).astype(np.float16).view(np.uint16)
            v = (rng.standard_normal((depth[q], 8, 128)) * 0.5).astype(np.float16).view(np.uint16)
            for x_ in (wide, gemm, plain, two):
                x_.kv_write(il, q, 0, k, v)
            orc.k[il - 2, q, :, :depth[q]] = k.transpose(1, 0, 2)
            orc.v[il - 2, q, :, :depth[q]] = v.transpose(1, 0, 2)
    nxt = list(depth)
    for step, T in enumerate((32, 17, 25, 32, 9, 20)):
        seqs = [int(q) for q in sorted(rng.permutation(32)[:T])]
        x = rng.standard_normal((T, E)).astype(np.float32)
        if step == 2:
            x[:, 1234] *= 40.0
        pos = [nxt[q] for q in seqs]
        for q in seqs:
            nxt[q] += 1
        a = wide.decode(x, pos, seq=seqs).view(np.float32).reshape(T, E)
        b = gemm.decode(x, pos, seq=seqs).view(np.float32).reshape(T, E)
        c = plain.decode(x, pos, seq=seqs).view(np.float32).reshape(T, E)
        assert np.array_equal(a, two.decode(x, pos, seq=seqs).view(np.float32).reshape(T, E)), (step, T)
        ref = orc.forward(x, pos, seq=seqs)
        ra, rb, rc = rel_l2(a, ref), rel_l2(b, ref), rel_l2(c, ref)
        print("[wide skinny] step %d, %d tokens: %.3e (large-tile GEMM %.3e, own norm launches %.3e) of the oracle, %.3e / %.3e apart"
              % (step, T, ra, rb, rc, rel_l2(a, b), rel_l2(a, c)))
        assert np.isfinite(a).all()
        assert ra <= 3e-3 and rb <= 3e-3 and rc <= 3e-3, (step, T)
        assert rel_l2(a, b) <= 3e-3 and rel_l2(a, c) <= 3e-3, (step, T)
        assert max(rel_l2(a[i], ref[i]) for i in range(T)) <= 1e-2
        # the K / V rows this step appended, last layer: both paths round the same f32 values to f16
        for q, p_ in ((seqs[0], pos[0]), (seqs[-1], pos[-1])):
            ka, va = wide.kv_read(4, q, p_, 1)
            kb, vb = gemm.kv_read(4, q, p_, 1)
            assert rel_l2(ka.view(np.float16).astype(np.float32), kb.view(np.float16).astype(np.float32)) <= 5e-3
            assert rel_l2(va.view(np.float16).astype(np.float32), vb.view(np.float16).astype(np.float32)) <= 5e-3
    assert wide.f16_saturations() == 0
    wide.close(); gemm.close(); plain.close(); two.close(); st.close()


def test_rope_in_projection_epilogue_equals_rope_kernel(tmp_path):
    """Llama-style (neighbouring-pair) RoPE and the KV append ride in the q/k/v projection's epilogue at batches of
    1-3 tokens (mat-vec kernels) and of 4+ tokens (batched MFMA GEMM); with gemv_rope=0 the separate kernel does
    them.  Outputs and cache contents must agree bit for bit (the arithmetic is the same), through the single-type
    and the mixed q4_K/q6_K launches."""
    for name, layers in (("llama3-8b", [3, 4]), ("tiny-llama", [0, 1])):
        m, cfg, tensors, st = _open(tmp_path, name, layers, layers[0], layers[-1] + 1, n_ctx=64, n_seq=9, n_batch=16)
        E = cfg["n_embd"]
        rng = np.random.Generator(np.random.PCG64(3))
        xs = [rng.standard_normal((T, E)).astype(np.float32) for T in (1, 2, 3, 4, 1, 6, 9, 5)]
        runs = []
        for flag in ("1", "0"):
            ses = st.session(gemv_rope=int(flag))
            outs, nxt = [], [0] * 9
            for x in xs:
                T = x.shape[0]
                seqs = list(range(T))
                pos = [nxt[q] for q in seqs]
                for q in seqs:
                    nxt[q] += 1
                outs.append(ses.decode(x, pos, seq=seqs).copy())
            kv = [ses.kv_read(il, q, 0, 8) for il in layers for q in range(9)]
            runs.append((outs, kv))
            ses.close()
        for a, b in zip(runs[0][0], runs[1][0]):
            assert np.array_equal(a, b)
        for (ka, va), (kb, vb) in zip(runs[0][1], runs[1][1]):
            assert np.array_equal(ka, kb) and np.array_equal(va, vb)
            assert ka.any() and va.any()
        st.close()


def test_ffn_vector_quantised_by_its_producer_equals_the_f32_hand_over(tmp_path):
    """At one token per call the gate / up launch leaves the FFN vector in the 16-bit fixed-point form the down projection
    consumes (whole 32-element blocks per workgroup), and the down projection copies it instead of quantising the f32
    vector in every workgroup.  The same arithmetic on the same values: bit-identical outputs with the hand-over switched
    off, through a q6_K and a q4_K down projection (real shape) and on a small model whose FFN rows do not split into
    whole blocks per workgroup (where the hand-over must not be taken)."""
    for name, layers in (("llama3-8b", [3, 4]), ("tiny-llama", [0, 1])):
        m, cfg, tensors, st = _open(tmp_path, name, layers, layers[0], layers[-1] + 1, n_ctx=64, n_seq=2, n_batch=4)
        E = cfg["n_embd"]
        rng = np.random.Generator(np.random.PCG64(77))
        xs = [rng.standard_normal((1, E)).astype(np.float32) * (50.0 if i == 2 else 1.0) for i in range(4)]
        runs = []
        for flag in ("1", "0"):
            ses = st.session(xq_handover=int(flag))
            runs.append([ses.decode(x, [i]).copy() for i, x in enumerate(xs)])
            ses.close()
        for a, b in zip(*runs):
            assert np.isfinite(a.view(np.float32)).all()
            assert np.array_equal(a, b)
        st.close()


@pytest.mark.parametrize("name,layers,wide", [("llama3-8b", [3, 4], 1), ("llama3-8b", [3, 4], 0), ("tiny-qwen2", [0, 1, 2], 1), ("tiny-moe", [0, 1], 1)])
def test_graph_replays_equal_eager_launches(tmp_path, name, layers, wide):
    """Decode-sized batches replay their layer launches from a captured graph (first use of a shape eager, second
    captured, then replays).  Every replay must give the bits the eager launches give: two sessions, graphs on and
    off, walk the same sequence of steps -- repeated shapes, other shapes and host synchronisations in between, KV
    depth growing past a change of the split count."""
    m, cfg, tensors, st = _open(tmp_path, name, layers, layers[0], layers[-1] + 1, n_ctx=256, n_seq=20, n_batch=32)
    E = cfg["n_embd"]
    rng = np.random.Generator(np.random.PCG64(17))
    # (20 tokens on real-shape layers: the f16 skinny GEMM with two column blocks; with skinny_f16_wide=0, and on the small
    # models, the large-tile GEMM with K split over workgroups, two kernels per projection, inside a graph)
    plan = [1, 1, 1, 4, 1, 4, 6, 1, 4, 6, 6, 1, 20, 1, 20] + [1] * 70 + [4, 4, 1, 6, 20]
    xs = [rng.standard_normal((T, E)).astype(np.float32) for T in plan]
    chunk_xs = [rng.standard_normal((25, E)).astype(np.float32) for _ in range(8)]
    runs = []
    for flag in ("1", "0"):
        ses = st.session(graphs=int(flag), skinny_f16_wide=wide)
        nxt = [0] * 20
        outs = []
        for x in xs:
            T = x.shape[0]
            seqs = list(range(T))
            pos = [nxt[q] for q in seqs]
            for q in seqs:
                nxt[q] += 1
            outs.append(ses.decode(x, pos, seq=seqs).copy())      # the host-pointer entry synchronises after every call
        # prefill chunks of one sequence, three in a row with the same token count (17..32 tokens: the chunk attention
        # kernel takes its first position as a launch argument, so these must never be replayed from a capture), with
        # a 20-sequence decode batch of the same token count in between
        for T, kind in ((20, "chunk"), (20, "chunk"), (20, "batch"), (20, "chunk"), (25, "chunk"), (25, "chunk"), (20, "batch"), (25, "chunk")):
            x = chunk_xs[len(outs) - len(xs)]
            if kind == "chunk":
                seqs, pos = [19] * T, list(range(nxt[19], nxt[19] + T))
                nxt[19] += T
            else:
                seqs = list(range(T))
                pos = [nxt[q] for q in seqs]
                for q in seqs:
                    nxt[q] += 1
            outs.append(ses.decode(x[:T], pos, seq=seqs).copy())
        runs.append((outs, [ses.kv_read(layers[0], q, 0, 8) for q in range(6)]))
        # shapes seen at least twice were captured and replayed; with graphs off nothing is
        assert (ses.graph_replays > 40) if flag == "1" else (ses.graph_replays == 0), ses.graph_replays
        ses.close()
    for i, (a, b) in enumerate(zip(runs[0][0], runs[1][0])):
        assert np.array_equal(a, b), "step %d (T=%d)" % (i, a.size // (4 * E))
    for (ka, va), (kb, vb) in zip(runs[0][1], runs[1][1]):
        assert np.array_equal(ka, kb) and np.array_equal(va, vb)
    st.close()
