"""End-to-end check on the reference's own CPU-runnable configuration: Qwen2.5-0.5B-shaped random-init model
(24 layers, hidden 896 -> Q5_0/Q8_0 fallback types, 14/2 heads, tied Q8_0 embeddings over a 151936 vocabulary),
split into two stages at layer 12 with the boundary hidden state packed to q8_0; 128 seeded prompt tokens, then
greedy decoding of 64 tokens.  The GPU stages must pick the same 64 tokens as the CPU oracle.

Random-init logits are nearly flat, so identity is only meaningful with a margin: the model seed was chosen (by an
oracle-only scan) so that the smallest top-1/top-2 gap over the 64 steps is 0.30 logit standard deviations, three
orders of magnitude above the GPU/oracle logit difference; both numbers are asserted below."""
import os

import numpy as np
import pytest

import gguf_util as G
import greedy_util as U
from util import mesh

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

SEED = 2


def test_two_stage_greedy_decode_is_token_identical(tmp_path):
    m = mesh()
    cfg, kvs, tl = U.build(SEED)
    tensors = {n: (t, d, x) for n, t, d, x in tl}
    path = os.path.join(str(tmp_path), "qwen05.gguf")
    G.write_gguf(path, kvs, tl)
    n_ctx = U.N_PROMPT + U.N_DECODE
    st0 = m.Stage(path, 0, U.SPLIT, n_ctx=n_ctx, n_seq_max=1, n_batch_max=U.N_PROMPT)
    st1 = m.Stage(path, U.SPLIT, cfg["n_layer"], n_ctx=n_ctx, n_seq_max=1, n_batch_max=U.N_PROMPT)
    os.unlink(path)
    s0, s1 = st0.session(), st1.session()

    def step(ids, pos):
        boundary = s0.decode(np.asarray(ids, np.int32), pos, in_fmt=m.TOKENS, out_fmt=m.Q8_0)
        assert boundary.size == len(ids) * cfg["n_embd"] // 32 * 34
        lg = s1.decode(boundary, pos, in_fmt=m.Q8_0, out_fmt=m.LOGITS).view(np.float32)
        return lg.reshape(len(ids), cfg["n_vocab"])[-1]

    gpu_tokens, gpu_logits = [], []
    lg = step(U.prompt_tokens(cfg), np.arange(U.N_PROMPT))
    for i in range(U.N_DECODE):
        gpu_logits.append(lg)
        gpu_tokens.append(int(np.argmax(lg)))
        if i + 1 < U.N_DECODE:
            lg = step([gpu_tokens[-1]], [U.N_PROMPT + i])

    ref_tokens, margins, std = U.oracle_greedy(cfg, tensors)
    assert list(ref_tokens) == gpu_tokens
    assert margins.min() / std > 0.25, "seed no longer gives a safe top-1 margin"
    # the GPU's own top-1/top-2 gap matches the oracle's at every step, far inside the margin
    gpu_margins = np.array([np.partition(-l, 1)[:2] for l in gpu_logits])
    gpu_margins = -(gpu_margins[:, 0] - gpu_margins[:, 1])
    assert np.max(np.abs(gpu_margins - margins)) / std < 2e-2
    for s in (s0, s1):
        s.close()
    st0.close(); st1.close()
