"""Two-stage greedy decoding of the Qwen2.5-0.5B-shaped model (24 layers split at 12, boundary packed to q8_0),
for the oracle and for the GPU stages."""
import numpy as np

import models
import oracle
from oracle.stage import StageOracle

CFG_NAME = "qwen2.5-0.5b"
N_PROMPT, N_DECODE, SPLIT = 128, 64, 12


def build(seed):
    cfg = models.CONFIGS[CFG_NAME]
    kvs, tl = models.build_tensors(cfg, range(cfg["n_layer"]), seed=seed, with_embd=True, with_output=True, fast=True)
    return cfg, kvs, tl


def prompt_tokens(cfg):
    return np.random.Generator(np.random.PCG64(7)).integers(0, cfg["n_vocab"], N_PROMPT).astype(np.int32)


def oracle_greedy(cfg, tensors, forced=None):
    """Returns (tokens[N_DECODE], margins[N_DECODE], logits_std).  forced: tokens to feed instead of its own argmax."""
    n_ctx = N_PROMPT + N_DECODE
    s0 = StageOracle(cfg, tensors, 0, SPLIT, n_ctx)
    s1 = StageOracle(cfg, tensors, SPLIT, cfg["n_layer"], n_ctx)

    def step(ids, pos):
        h = s0.forward(s0.embed(ids), pos)
        packed = oracle.quantize_q8_0(h.reshape(-1))                      # the q8_0 boundary activation
        h = oracle.dequantize(oracle.Q8_0, packed, h.size).reshape(h.shape)
        h = s1.forward(h, pos)
        return s1.logits(h[-1:])[0]

    toks, margins = [], []
    lg = step(prompt_tokens(cfg), np.arange(N_PROMPT))
    std = float(lg.std())
    for i in range(N_DECODE):
        order = np.argpartition(-lg, 2)[:2]
        order = order[np.argsort(-lg[order])]
        toks.append(int(order[0]))
        margins.append(float(lg[order[0]] - lg[order[1]]))
        nxt = toks[-1] if forced is None else int(forced[i])
        if i + 1 < N_DECODE:
            lg = step(np.array([nxt], np.int32), [N_PROMPT + i])
    return np.array(toks), np.array(margins), std
