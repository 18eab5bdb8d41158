"""Synthetic GGUF models of the benchmark shapes, generated directly in the block domain (no f32 -> K-quant
quantiser is needed): random quants and sub-scales, super-scales chosen so the dequantized tensor has sigma ~0.02.

  q4_K: qs uniform bytes; sub-scale sc uniform in [8,63], min m = sc, dmin = 7.5*d  =>  w = d*sc*(q - 7.5)
  q6_K: ql/qh uniform; sub-scale uniform in [16,127]; d ~ 1.38e-5 is an fp16 SUBNORMAL, as in real files
  q5_0 / q8_0 (fallback types of 896-wide rows): uniform quants, d = 0.02 / rms(q)
The distribution is a uniform mixture, not Gaussian.
"""
import os

import numpy as np

import gguf_util as G

F32, F16, Q5_0, Q8_0, Q4_K, Q6_K = 0, 1, 6, 8, 12, 14
BLOCK = {F32: (1, 4), F16: (1, 2), Q5_0: (32, 22), Q8_0: (32, 34), Q4_K: (256, 144), Q6_K: (256, 210)}


def pack_scales_k4(sc, m):
    """sc, m: uint8 [n, 8] six-bit values -> uint8 [n, 12]."""
    q = np.zeros((sc.shape[0], 12), np.uint8)
    q[:, 0:4] = sc[:, 0:4] | ((sc[:, 4:8] >> 4) << 6)
    q[:, 4:8] = m[:, 0:4] | ((m[:, 4:8] >> 4) << 6)
    q[:, 8:12] = (sc[:, 4:8] & 0xF) | ((m[:, 4:8] & 0xF) << 4)
    return q


_BASE_BYTES = {}


def _random_bytes(rng, n, variant):
    """n uniform random bytes.  variant None: drawn from rng.  Otherwise: one cached draw per size (seeded by the
    size), XOR-ed with a byte derived from `variant` -- still uniform, distinct per tensor, and ~10x cheaper, which
    matters when a benchmark model holds gigabytes."""
    if variant is None:
        return rng.bit_generator.random_raw((n + 7) // 8).view(np.uint8)[:n].copy()
    if n not in _BASE_BYTES:
        g = np.random.Generator(np.random.PCG64(n))
        _BASE_BYTES[n] = g.bit_generator.random_raw((n + 7) // 8).view(np.uint8)[:n]
    return _BASE_BYTES[n] ^ np.uint8((variant * 37 + 11) & 0xFF)


def random_tensor(rng, ttype, n_rows, row_len, sigma=0.02, variant=None):
    """uint8 array holding n_rows x row_len elements of `ttype` blocks."""
    be, bb = BLOCK[ttype]
    assert row_len % be == 0, (ttype, row_len)
    nblk = n_rows * row_len // be
    if ttype == F32:
        return (rng.standard_normal(n_rows * row_len) * sigma).astype(np.float32).view(np.uint8)
    if ttype == F16:
        return (rng.standard_normal(n_rows * row_len) * sigma).astype(np.float16).view(np.uint8)
    raw = _random_bytes(rng, nblk * bb, variant).reshape(nblk, bb)
    if ttype == Q4_K:
        sc = rng.integers(8, 64, size=(nblk, 8), dtype=np.uint8)
        d = np.float16(sigma / (4.61 * 39.0))
        raw[:, 0:2] = np.frombuffer(d.tobytes(), np.uint8)
        raw[:, 2:4] = np.frombuffer(np.float16(7.5 * float(d)).tobytes(), np.uint8)
        raw[:, 4:16] = pack_scales_k4(sc, sc)
    elif ttype == Q6_K:
        raw[:, 192:208] = rng.integers(16, 128, size=(nblk, 16), dtype=np.uint8)
        raw[:, 208:210] = np.frombuffer(np.float16(sigma / (18.5 * 78.5)).tobytes(), np.uint8)
    elif ttype == Q5_0:
        raw[:, 0:2] = np.frombuffer(np.float16(sigma / 9.23).tobytes(), np.uint8)
    elif ttype == Q8_0:
        raw[:, 0:2] = np.frombuffer(np.float16(sigma / 73.9).tobytes(), np.uint8)
    return raw.reshape(-1)


def use_more_bits(i, n):
    return i < n // 8 or i >= 7 * n // 8 or (i - n // 8) % 3 == 2


def q4km_type(name, i_layer, n_layer, row_len):
    """Tensor -> type map of a Q4_K_M file: attn_v and ffn_down get Q6_K on 'more bits' layers, output Q6_K;
    rows that are not a multiple of 256 fall back Q4_K -> Q5_0 and Q6_K -> Q8_0."""
    t = Q4_K
    if name in ("attn_v", "ffn_down", "ffn_down_exps") and use_more_bits(i_layer, n_layer):
        t = Q6_K
    if name in ("output", "token_embd_tied"):
        t = Q6_K
    if row_len % 256:
        t = Q5_0 if t == Q4_K else Q8_0
    return t


CONFIGS = {
    # name: arch, n_layer, n_embd, n_head, n_head_kv, head_dim, n_ff, vocab, eps, rope base
    "qwen2.5-0.5b": dict(arch="qwen2", n_layer=24, n_embd=896, n_head=14, n_head_kv=2, head_dim=64, n_ff=4864, n_vocab=151936, eps=1e-6, rope=1e6, bias=True, tied=True),
    "llama3-8b": dict(arch="llama", n_layer=32, n_embd=4096, n_head=32, n_head_kv=8, head_dim=128, n_ff=14336, n_vocab=128256, eps=1e-5, rope=5e5),
    "qwen2.5-32b": dict(arch="qwen2", n_layer=64, n_embd=5120, n_head=40, n_head_kv=8, head_dim=128, n_ff=27648, n_vocab=152064, eps=1e-6, rope=1e6, bias=True),
    "qwen3-30b-a3b": dict(arch="qwen3moe", n_layer=48, n_embd=2048, n_head=32, n_head_kv=4, head_dim=128, n_ff=6144, n_vocab=151936, eps=1e-6, rope=1e6, n_expert=128, n_expert_used=8, n_ff_exp=768, qk_norm=True),
    # small shapes for fast parity tests
    "tiny-llama": dict(arch="llama", n_layer=4, n_embd=256, n_head=4, n_head_kv=2, head_dim=64, n_ff=512, n_vocab=512, eps=1e-5, rope=1e4),
    "tiny-qwen2": dict(arch="qwen2", n_layer=3, n_embd=512, n_head=4, n_head_kv=1, head_dim=128, n_ff=768, n_vocab=768, eps=1e-6, rope=1e6, bias=True, tied=True),
    "tiny-qwen3": dict(arch="qwen3", n_layer=2, n_embd=256, n_head=8, n_head_kv=4, head_dim=64, n_ff=768, n_vocab=256, eps=1e-6, rope=1e6, qk_norm=True),
    "tiny-moe": dict(arch="qwen3moe", n_layer=2, n_embd=512, n_head=4, n_head_kv=2, head_dim=128, n_ff=0, n_vocab=256, eps=1e-6, rope=1e6, n_expert=8, n_expert_used=2, n_ff_exp=256, qk_norm=True),
    # head_dim 128 shapes with 5, 8, 2 and 7 query heads per KV head
    "tiny-g5": dict(arch="qwen2", n_layer=2, n_embd=1280, n_head=10, n_head_kv=2, head_dim=128, n_ff=1536, n_vocab=256, eps=1e-6, rope=1e6, bias=True),
    "tiny-g8": dict(arch="llama", n_layer=2, n_embd=1024, n_head=8, n_head_kv=1, head_dim=128, n_ff=1024, n_vocab=256, eps=1e-5, rope=5e5),
    # three KV heads of four query heads: an odd number of head rows in the chunk attention launch
    "tiny-kv3": dict(arch="llama", n_layer=1, n_embd=1536, n_head=12, n_head_kv=3, head_dim=128, n_ff=768, n_vocab=256, eps=1e-5, rope=1e4),
    # one query head per KV head (row lengths a multiple of 256, so that every projection is a K-quant)
    "tiny-mha": dict(arch="llama", n_layer=1, n_embd=512, n_head=4, n_head_kv=4, head_dim=128, n_ff=512, n_vocab=256, eps=1e-5, rope=1e4),
    "tiny-g2": dict(arch="llama", n_layer=2, n_embd=512, n_head=4, n_head_kv=2, head_dim=128, n_ff=512, n_vocab=256, eps=1e-5, rope=1e4),
    "tiny-g7": dict(arch="qwen2", n_layer=2, n_embd=1792, n_head=14, n_head_kv=2, head_dim=128, n_ff=2048, n_vocab=256, eps=1e-6, rope=1e6, bias=True),
    "tiny-odd": dict(arch="qwen2", n_layer=2, n_embd=320, n_head=5, n_head_kv=1, head_dim=64, n_ff=640, n_vocab=96, eps=1e-6, rope=1e4, bias=True, tied=True),
}


ZIPF_CHANNEL, ZIPF_LEVEL = 0, 8.0


def zipf_expert_bias(n_expert, n_local, seed, s=1.1):
    """Log-popularity of the experts a node holds when expert popularity follows Zipf(s): rank r (1 = most popular, a
    seeded permutation of the model's experts) has p ~ r^-s, bias = ln p.  A node that holds n_local < n_expert
    experts gets every (n_expert / n_local)-th pick of a snake draft over the ranking (node 0's share in
    mesh-llm/src/inference/moe.rs:597-643), renumbered in ascending rank."""
    ranks = np.arange(1, n_expert + 1)
    if n_local and n_local < n_expert:
        n_nodes = n_expert // n_local
        picks = [r for i, r in enumerate(ranks) if (i % (2 * n_nodes)) in (0, 2 * n_nodes - 1)]
        ranks = np.array(picks[:n_local])
    bias = -s * np.log(ranks.astype(np.float64))
    order = np.random.Generator(np.random.PCG64(seed)).permutation(len(bias))
    return bias[order].astype(np.float32)


def zipf_hidden_state(rng, T, E):
    """Hidden-state rows for a model built with router="zipf": N(0,1) with the carrier channel held at ZIPF_LEVEL (real
    models carry such constant 'massive activation' channels too)."""
    x = rng.standard_normal((T, E)).astype(np.float32)
    x[:, ZIPF_CHANNEL] = ZIPF_LEVEL
    return x


def build_tensors(cfg, layers, seed=42, with_embd=False, with_output=False, n_expert_local=None, fast=False, router=None):
    """Returns (kvs, tensors) for write_gguf; tensors only for `layers` (absolute indices).
    router="zipf" (mixture-of-experts models): router logits ~ N(0,1) plus a Zipf(1.1) expert bias.  The architecture has
    no router bias tensor, so the bias rides on one channel of the hidden state that the inputs hold at a constant
    level (zipf_hidden_state): router rows are N(0, 1/n_embd) (unit-variance logits on RMS-normalised inputs), and
    their weight on the carrier channel is bias_e divided by the channel's normalised level."""
    c = cfg
    a = c["arch"]
    E, H, HK, HD, FF = c["n_embd"], c["n_head"], c["n_head_kv"], c["head_dim"], c["n_ff"]
    kvs = [("general.architecture", G.T_STR, a), ("general.alignment", G.T_U32, 32),
           (a + ".block_count", G.T_U32, c["n_layer"]), (a + ".embedding_length", G.T_U32, E),
           (a + ".feed_forward_length", G.T_U32, FF), (a + ".attention.head_count", G.T_U32, H),
           (a + ".attention.head_count_kv", G.T_U32, HK), (a + ".attention.layer_norm_rms_epsilon", G.T_F32, c["eps"]),
           (a + ".rope.freq_base", G.T_F32, c["rope"]), (a + ".vocab_size", G.T_U32, c["n_vocab"]),
           ("tokenizer.ggml.tokens", G.T_ARR, (G.T_STR, ["<a>", "<b>"]))]   # an array the reader has to skip
    if E // H != HD:
        kvs += [(a + ".attention.key_length", G.T_U32, HD), (a + ".attention.value_length", G.T_U32, HD)]
    moe = a == "qwen3moe"
    NE = c.get("n_expert", 0)
    NEL = n_expert_local or NE
    if moe:
        kvs += [(a + ".expert_count", G.T_U32, NEL), (a + ".expert_used_count", G.T_U32, c["n_expert_used"]),
                (a + ".expert_feed_forward_length", G.T_U32, c["n_ff_exp"])]
    tensors = []

    counter = [0]

    def add(name, ttype, rows, cols, rng, kind="w", n_e=1):
        counter[0] += 1
        var = counter[0] if fast else None
        if kind == "norm":
            data = (1.0 + 0.02 * rng.standard_normal(cols)).astype(np.float32).view(np.uint8)
            tensors.append((name, F32, (cols,), data))
        elif kind == "bias":
            data = (0.02 * rng.standard_normal(cols)).astype(np.float32).view(np.uint8)
            tensors.append((name, F32, (cols,), data))
        elif n_e > 1:
            tensors.append((name, ttype, (cols, rows, n_e), random_tensor(rng, ttype, rows * n_e, cols, variant=var)))
        else:
            tensors.append((name, ttype, (cols, rows), random_tensor(rng, ttype, rows, cols, variant=var)))

    for il in layers:
        def rng_for(j):
            return np.random.Generator(np.random.PCG64(seed + 16 * il + j))
        p = "blk.%d." % il
        nl = c["n_layer"]
        add(p + "attn_norm.weight", F32, 1, E, rng_for(0), "norm")
        add(p + "attn_q.weight", q4km_type("attn_q", il, nl, E), H * HD, E, rng_for(1))
        add(p + "attn_k.weight", q4km_type("attn_k", il, nl, E), HK * HD, E, rng_for(2))
        add(p + "attn_v.weight", q4km_type("attn_v", il, nl, E), HK * HD, E, rng_for(3))
        add(p + "attn_output.weight", q4km_type("attn_output", il, nl, H * HD), E, H * HD, rng_for(4))
        if c.get("bias"):
            add(p + "attn_q.bias", F32, 1, H * HD, rng_for(9), "bias")
            add(p + "attn_k.bias", F32, 1, HK * HD, rng_for(10), "bias")
            add(p + "attn_v.bias", F32, 1, HK * HD, rng_for(11), "bias")
        if c.get("qk_norm"):
            add(p + "attn_q_norm.weight", F32, 1, HD, rng_for(12), "norm")
            add(p + "attn_k_norm.weight", F32, 1, HD, rng_for(13), "norm")
        add(p + "ffn_norm.weight", F32, 1, E, rng_for(5), "norm")
        if not moe:
            add(p + "ffn_gate.weight", q4km_type("ffn_gate", il, nl, E), FF, E, rng_for(6))
            add(p + "ffn_up.weight", q4km_type("ffn_up", il, nl, E), FF, E, rng_for(7))
            add(p + "ffn_down.weight", q4km_type("ffn_down", il, nl, FF), E, FF, rng_for(8))
        else:
            FE = c["n_ff_exp"]
            r = rng_for(14)
            if router == "zipf":
                Wr = (r.standard_normal((NEL, E)) / np.sqrt(E)).astype(np.float32)
                # the carrier channel after the RMS norm: level / rms(row) with rms^2 = ((E - 1) + level^2) / E, times its norm weight
                level = ZIPF_LEVEL / np.sqrt(((E - 1) + ZIPF_LEVEL ** 2) / E)
                nw = tensors[[n for n, *_ in tensors].index(p + "ffn_norm.weight")][3].view(np.float32)[ZIPF_CHANNEL]
                Wr[:, ZIPF_CHANNEL] = zipf_expert_bias(NE, NEL, seed + il) / (level * nw)
                tensors.append((p + "ffn_gate_inp.weight", F32, (E, NEL), Wr.reshape(-1).view(np.uint8)))
            else:
                tensors.append((p + "ffn_gate_inp.weight", F32, (E, NEL), (r.standard_normal(NEL * E) * 0.02).astype(np.float32).view(np.uint8)))
            add(p + "ffn_gate_exps.weight", q4km_type("ffn_gate_exps", il, nl, E), FE, E, rng_for(6), n_e=NEL)
            add(p + "ffn_up_exps.weight", q4km_type("ffn_up_exps", il, nl, E), FE, E, rng_for(7), n_e=NEL)
            add(p + "ffn_down_exps.weight", q4km_type("ffn_down_exps", il, nl, FE), E, FE, rng_for(8), n_e=NEL)
    V = c["n_vocab"]
    if with_embd or (with_output and c.get("tied")):
        t = q4km_type("token_embd_tied" if c.get("tied") else "token_embd", 0, 1, E)
        # sigma 1/sqrt(E)-ish embeddings would be tiny after the first norm anyway; use sigma 0.02 like the rest
        add("token_embd.weight", t, V, E, np.random.Generator(np.random.PCG64(seed + 100000)))
    if with_output:
        add("output_norm.weight", F32, 1, E, np.random.Generator(np.random.PCG64(seed + 100001)), "norm")
        if not c.get("tied"):
            add("output.weight", q4km_type("output", 0, 1, E), V, E, np.random.Generator(np.random.PCG64(seed + 100002)))
    return kvs, tensors


def write_model(path, cfg, layers, **kw):
    kvs, tensors = build_tensors(cfg, layers, **kw)
    G.write_gguf(path, kvs, tensors)
    return {name: (ttype, dims, data) for name, ttype, dims, data in tensors}


def tmp_dir():
    d = os.environ.get("MESH_TEST_TMP") or ("/dev/shm" if os.path.isdir("/dev/shm") else "/tmp")
    return d
