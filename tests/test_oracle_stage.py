"""Invariants that pin the oracle's layer composition (oracle/stage.py) without reference code:
prefill equals token-by-token decode, sequences do not interact, and two stages chained through any boundary
format reproduce the unsplit model (exactly for f32, within the codec's error for f16 / q8_0)."""
import numpy as np
import pytest

import models
import oracle
from oracle.stage import StageOracle


def _model(name, seed=3):
    cfg = models.CONFIGS[name]
    kvs, tensors = models.build_tensors(cfg, range(cfg["n_layer"]), seed=seed, with_embd=True, with_output=True)
    return cfg, {n: (t, d, x) for n, t, d, x in tensors}


@pytest.mark.parametrize("name", ["tiny-llama", "tiny-qwen2", "tiny-qwen3"])
def test_prefill_equals_stepwise_decode(name):
    cfg, tensors = _model(name)
    rng = np.random.Generator(np.random.PCG64(1))
    T = 6
    x = rng.standard_normal((T, cfg["n_embd"])).astype(np.float32)
    a = StageOracle(cfg, tensors, 0, cfg["n_layer"], 16)
    ya = a.forward(x, np.arange(T))
    b = StageOracle(cfg, tensors, 0, cfg["n_layer"], 16)
    yb = np.concatenate([b.forward(x[t:t + 1], [t]) for t in range(T)])
    assert np.allclose(ya, yb, rtol=1e-5, atol=1e-5)
    assert np.array_equal(a.k, b.k) and np.array_equal(a.v, b.v)


def test_sequences_do_not_interact():
    cfg, tensors = _model("tiny-llama")
    rng = np.random.Generator(np.random.PCG64(2))
    x = rng.standard_normal((8, cfg["n_embd"])).astype(np.float32)
    solo = StageOracle(cfg, tensors, 0, 2, 16, n_seq_max=1)
    y_solo = solo.forward(x[:4], [0, 1, 2, 3])
    both = StageOracle(cfg, tensors, 0, 2, 16, n_seq_max=2)
    inter = np.empty_like(x)
    inter[0::2], inter[1::2] = x[:4], x[4:]
    y = both.forward(inter, [0, 0, 1, 1, 2, 2, 3, 3], seq=[0, 1, 0, 1, 0, 1, 0, 1])
    assert np.allclose(y[0::2], y_solo, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("fmt", ["f32", "f16", "q8_0"])
def test_split_stages_reproduce_the_unsplit_model(fmt):
    cfg, tensors = _model("tiny-llama")
    rng = np.random.Generator(np.random.PCG64(4))
    T = 5
    x = rng.standard_normal((T, cfg["n_embd"])).astype(np.float32)
    pos = np.arange(T)
    full = StageOracle(cfg, tensors, 0, 4, 16).forward(x, pos)
    h = StageOracle(cfg, tensors, 0, 2, 16).forward(x, pos)
    if fmt == "f16":
        h = oracle.fp16_to_fp32(oracle.fp32_to_fp16(h))
    elif fmt == "q8_0":
        h = oracle.dequantize(oracle.Q8_0, oracle.quantize_q8_0(h.reshape(-1)), h.size).reshape(h.shape)
    out = StageOracle(cfg, tensors, 2, 4, 16).forward(h, pos)
    rel = np.linalg.norm(out - full) / np.linalg.norm(full)
    assert rel <= {"f32": 0.0, "f16": 2e-3, "q8_0": 2e-2}[fmt], rel


def test_logits_and_embedding_round_trip():
    cfg, tensors = _model("tiny-qwen2")
    st = StageOracle(cfg, tensors, 0, cfg["n_layer"], 8)
    ids = np.array([1, 5, 700], np.int32)
    x = st.embed(ids)
    assert x.shape == (3, cfg["n_embd"])
    lg = st.logits(st.forward(x, [0, 1, 2]))
    assert lg.shape == (3, cfg["n_vocab"]) and np.isfinite(lg).all()
