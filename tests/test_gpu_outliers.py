"""Activation range of the projection paths.  The mat-vec kernels (calls of up to 4 tokens) and the integer-MFMA skinny
GEMM quantise activations to 16-bit fixed point per 32-element block with an f32 block scale: any f32 magnitude is
representable, and an outlier channel costs precision only inside its own block.  The f16 skinny GEMM (calls of 4 to 16
tokens and batches of up to 32 decode steps, the default) and the large-tile GEMM (longer calls, prefill chunks) round activations to f16: relative precision 2^-11 whatever the
magnitude, up to +-65504, beyond which the producers SATURATE (a finite, wrong-by-clamping value) rather than emit an
infinity that the next norm would turn into NaN for the whole token, and count the value in the session's saturation
counter.

Checked here against the oracle: hidden states with the boundary codec's x50 outlier channels through every path, and
SwiGLU products beyond the f16 range (exact on the decode paths, finite on the f16 path)."""
import os

import numpy as np
import pytest

import gguf_util as G
import models
from oracle.stage import StageOracle
from util import mesh

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def rel_l2(a, b):
    a = np.asarray(a, np.float64).reshape(-1)
    b = np.asarray(b, np.float64).reshape(-1)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def outlier_input(rng, T, E):
    """N(0,1) rows with 0.1 % of the channels (fixed indices) scaled x50, as in the codec benchmark."""
    x = rng.standard_normal((T, E)).astype(np.float32)
    ch = np.random.Generator(np.random.PCG64(1234)).choice(E, size=int(np.ceil(E * 0.001)), replace=False)
    x[:, ch] *= 50
    return x


def _stage(tmp_path, scale_ffn_norm=None, n_seq=24, n_batch=208):
    m = mesh()
    cfg = models.CONFIGS["llama3-8b"]
    kvs, tl = models.build_tensors(cfg, [3, 4], seed=5)
    if scale_ffn_norm:
        tl = [(n, t, d, (x.view(np.float32) * scale_ffn_norm).view(np.uint8) if n == "blk.3.ffn_norm.weight" else x) for n, t, d, x in tl]
    path = os.path.join(str(tmp_path), "o.gguf")
    G.write_gguf(path, kvs, tl)
    st = m.Stage(path, 3, 5, n_ctx=256, n_seq_max=n_seq, n_batch_max=n_batch)
    os.unlink(path)
    return m, cfg, {n: (t, d, x) for n, t, d, x in tl}, st


@pytest.mark.parametrize("skinny", ["f16", "integer"])
def test_outlier_channels_through_every_projection_path(tmp_path, skinny):
    """Batches of 5..16 tokens once on the f16 matrix cores (the default: f16 activations, one rounding per weight) and once
    on the integer ones (16-bit fixed-point activations, the session switch skinny_f16=0)."""
    m, cfg, tensors, st = _stage(tmp_path)
    E = cfg["n_embd"]
    ses = st.session(skinny_f16=int(skinny == "f16"))
    orc = StageOracle(cfg, tensors, 3, 5, 256, n_seq_max=24, blas=True)
    rng = np.random.Generator(np.random.PCG64(50))
    nxt = {}
    # 200-token prefill chunk (large-tile GEMM, f16 activations), then decode batches on top of it and on fresh sequences
    for T, seqs, what in ((200, [0] * 200, "prefill 200 (f16 large-tile GEMM)"), (1, [0], "decode 1 (mat-vec)"), (3, [0, 1, 2], "decode 3 (mat-vec)"),
                          (8, list(range(8)), "decode 8 (%s skinny GEMM)" % skinny), (16, list(range(16)), "decode 16 (%s skinny GEMM)" % skinny),
                          (24, list(range(24)), "decode 24 (f16 skinny GEMM, two column blocks)" if skinny == "f16" else "decode 24 (f16 large-tile GEMM, split K)")):
        x = outlier_input(rng, T, E)
        pos = []
        for q in seqs:                      # every sequence continues where it stands
            pos.append(nxt.get(q, 0))
            nxt[q] = nxt.get(q, 0) + 1
        got = ses.decode(x, pos, seq=seqs).view(np.float32).reshape(T, E)
        ref = orc.forward(x, pos, seq=seqs)
        r = rel_l2(got, ref)
        print("[outliers] %s: rel-L2 %.3e" % (what, r))
        assert np.isfinite(got).all()
        assert r <= (3e-3 if "f16" in what else 5e-4), what
    ses.close(); st.close()


def test_swiglu_products_beyond_the_f16_range(tmp_path):
    """ffn_norm weights x300 in one layer: gate and up reach several hundred, silu(gate) * up ~1e5 > 65504."""
    m, cfg, tensors, st = _stage(tmp_path, scale_ffn_norm=300.0)
    E = cfg["n_embd"]
    ses = st.session()
    orc = StageOracle(cfg, tensors, 3, 5, 256, n_seq_max=24, blas=True)
    rng = np.random.Generator(np.random.PCG64(51))
    # the oracle's own SwiGLU output of this layer does exceed the f16 range
    x = rng.standard_normal((8, E)).astype(np.float32)
    import oracle as O
    n = O.rms_norm(x, tensors["blk.3.ffn_norm.weight"][2].view(np.float32), cfg["eps"])
    t, d, w = tensors["blk.3.ffn_gate.weight"]
    g = O.mul_mat(t, w, d[1], d[0], n)
    t, d, w = tensors["blk.3.ffn_up.weight"]
    u = O.mul_mat(t, w, d[1], d[0], n)
    assert np.abs(O.swiglu(g, u)).max() > 65504
    def run(ses, T, pos0, seq0):
        xs = rng.standard_normal((T, E)).astype(np.float32)
        seqs = [seq0 + i for i in range(T)] if pos0 == 0 else [seq0] * T
        pos = [0] * T if pos0 == 0 else list(range(pos0, pos0 + T))
        got = ses.decode(xs, pos, seq=seqs).view(np.float32).reshape(T, E)
        return got, rel_l2(got, orc.forward(xs, pos, seq=seqs))

    # integer paths (the single-token mat-vec, and the 16-bit fixed-point matrix-core kernel for small batches): exact
    # arithmetic range, same tolerance as ever, and nothing counted as saturated
    ses_int = st.session(skinny_f16=0)
    for T in (1, 8):
        got, r = run(ses_int, T, 0, 0)
        print("[outliers] SwiGLU beyond f16, decode %d (integer kernels): rel-L2 %.3e" % (T, r))
        assert r <= 5e-4, T
    assert ses_int.f16_saturations() == 0
    ses_int.close()
    # f16 paths: saturate, stay finite (and are therefore off by what the clamp removed), and say so through the counter
    got, r = run(ses, 1, 0, 0)
    assert r <= 5e-4 and ses.f16_saturations() == 0
    seen = 0
    for T, pos0, seq0, what in ((8, 0, 8, "f16 skinny GEMM"), (24, 0, 0, "f16 skinny GEMM, two column blocks"), (64, 1, 20, "prefill")):
        got, r = run(ses, T, pos0, seq0)
        n = ses.f16_saturations()
        print("[outliers] SwiGLU beyond f16, %s of %d tokens (saturating f16): rel-L2 %.3e, %d values clamped so far" % (what, T, r, n))
        assert np.isfinite(got).all()
        assert n > seen, what
        seen = n
    ses.close(); st.close()
