"""Single graph nodes on the GPU against the oracle's primitives: RMS norm into the two activation layouts of the batched
paths, SwiGLU, and decode attention over a session's KV cache (both kernels, all three cache tiers)."""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import models
import oracle
from util import mesh

pytestmark = pytest.mark.gpu

XQ_LEVELS = 32512.0


def decode_q16(raw, T, n):
    """f32 values and block scales out of the q16 layout (include/mesh_stage.h: mesh_op_rms_norm_q16_dev)."""
    nblk = (T + 15) // 16
    raw = raw.reshape(nblk, 36 * n)
    rec = raw[:, :32 * n].reshape(nblk, n // 8, 16, 16)                     # [block][group][token][hi x 8, lo x 8]
    hi = rec[..., :8].view(np.int8).astype(np.int32)
    lo = rec[..., 8:].view(np.int8).astype(np.int32)
    q = (hi * 256 + lo).transpose(0, 2, 1, 3).reshape(nblk * 16, n)        # [token][k]
    d = raw[:, 32 * n:34 * n].copy().view(np.float32).reshape(nblk, n // 32, 16).transpose(0, 2, 1).reshape(nblk * 16, n // 32)
    sx = raw[:, 34 * n:36 * n].copy().view(np.float32).reshape(nblk, n // 32, 16).transpose(0, 2, 1).reshape(nblk * 16, n // 32)
    return q[:T], d[:T], sx[:T]


def decode_k8(raw16, T, n):
    nblk = (T + 15) // 16
    a = raw16.reshape(nblk, n // 8, 16, 8).transpose(0, 2, 1, 3).reshape(nblk * 16, n)
    return a[:T].astype(np.float32), a[T:]


@pytest.mark.parametrize("T,n", [(1, 256), (5, 4096), (16, 4096), (37, 5120), (16, 14336)])
def test_rms_norm_q16(T, n):
    import torch
    m = mesh()
    rng = np.random.Generator(np.random.PCG64(T * 1000 + n))
    x = (rng.standard_normal((T, n)) * 3).astype(np.float32)
    x[:, [3, n // 2]] *= 50                                               # outlier channels
    w = (1 + 0.1 * rng.standard_normal(n)).astype(np.float32)
    eps = 1e-5
    xd, wd = torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda()
    out = torch.zeros(m.op_q16_bytes(T, n), dtype=torch.uint8, device="cuda")
    m.op_rms_norm_q16_dev(xd.data_ptr(), wd.data_ptr(), eps, T, n, out.data_ptr())
    torch.cuda.synchronize()
    q, d, sx = decode_q16(out.cpu().numpy(), T, n)
    want = oracle.rms_norm(x, w, eps)
    got = q.reshape(T, n // 32, 32) * d[:, :, None]
    blocks = want.reshape(T, n // 32, 32)
    amax = np.abs(blocks).max(axis=2)
    # 16-bit fixed point per 32-element block: the step is amax / 32512, the error at most half a step (+ f32 rounding of the norm)
    assert np.all(np.abs(got - blocks) <= amax[:, :, None] * (0.5 / XQ_LEVELS + 2e-6) + 1e-30)
    assert np.allclose(d, amax / XQ_LEVELS, rtol=2e-6, atol=0)
    assert np.allclose(sx, got.sum(axis=2), rtol=1e-5, atol=1e-6 * amax.max())   # the block sums the q4_K minimum term uses
    assert np.abs(q).max() <= 32512


def test_quantise_without_norm_and_zero_rows():
    import torch
    m = mesh()
    T, n = 3, 512
    x = np.zeros((T, n), np.float32)
    x[1] = np.linspace(-7, 7, n)
    xd = torch.from_numpy(x).cuda()
    out = torch.zeros(m.op_q16_bytes(T, n), dtype=torch.uint8, device="cuda")
    m.op_rms_norm_q16_dev(xd.data_ptr(), None, 0.0, T, n, out.data_ptr())
    torch.cuda.synchronize()
    q, d, sx = decode_q16(out.cpu().numpy(), T, n)
    got = (q.reshape(T, n // 32, 32) * d[:, :, None]).reshape(T, n)
    assert np.all(got[0] == 0) and np.all(got[2] == 0) and np.all(d[0] == 0)
    assert np.abs(got[1] - x[1]).max() <= 7 * 0.5 / XQ_LEVELS + 1e-6


@pytest.mark.parametrize("T,n", [(1, 256), (17, 4096), (200, 5120)])
def test_rms_norm_f16_k8(T, n):
    import torch
    m = mesh()
    rng = np.random.Generator(np.random.PCG64(T + n))
    x = rng.standard_normal((T, n)).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(n)).astype(np.float32)
    xd, wd = torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda()
    out = torch.full(((T + 15) // 16 * 16 * n,), 7.0, dtype=torch.float16, device="cuda")
    m.op_rms_norm_f16k8_dev(xd.data_ptr(), wd.data_ptr(), 1e-6, T, n, out.data_ptr())
    torch.cuda.synchronize()
    got, pad = decode_k8(out.cpu().numpy(), T, n)
    want = oracle.rms_norm(x, w, 1e-6)
    # one f16 rounding of an f32 result: half a unit in the 11-bit significand (+ the f32 norm's own rounding)
    assert np.all(np.abs(got - want) <= np.abs(want) * (2.0 ** -11 + 4e-6) + 2.0 ** -25)
    assert np.all(pad == 0)


@pytest.mark.parametrize("T,n", [(1, 512), (17, 14336), (130, 768)])
def test_swiglu_f16_k8(T, n):
    import torch
    m = mesh()
    rng = np.random.Generator(np.random.PCG64(T * 7 + n))
    g = (rng.standard_normal((T, n)) * 4).astype(np.float32)
    u = (rng.standard_normal((T, n)) * 4).astype(np.float32)
    g[0, :4] = [1e4, -1e4, 300.0, -300.0]                                  # silu saturates both ways; 1e4 * u leaves the f16 range
    u[0, :4] = [100.0, 100.0, 300.0, 300.0]
    gd, ud = torch.from_numpy(g).cuda(), torch.from_numpy(u).cuda()
    out = torch.full(((T + 15) // 16 * 16 * n,), 7.0, dtype=torch.float16, device="cuda")
    m.op_swiglu_f16k8_dev(gd.data_ptr(), ud.data_ptr(), T, n, out.data_ptr())
    torch.cuda.synchronize()
    got, pad = decode_k8(out.cpu().numpy(), T, n)
    want = np.clip(oracle.swiglu(g, u), -65504.0, 65504.0)                 # the f16 producers saturate instead of writing inf
    assert np.all(np.isfinite(got))
    assert np.all(np.abs(got - want) <= np.abs(want) * (2.0 ** -11 + 1e-5) + 1e-6)
    assert got[0, 0] == 65504.0
    assert np.all(pad == 0)


@pytest.mark.parametrize("kv", ["f16", "q8_0/q4_0", "q4_0/q4_0"])
@pytest.mark.parametrize("name", ["tiny-g2", "tiny-g5", "tiny-g8"])
@pytest.mark.parametrize("matrix_cores", [False, True])
def test_decode_attention(tmp_path, name, kv, matrix_cores):
    """Three sequences at different depths (one key, a few hundred, the whole cache), every head, vs the oracle's
    attention over the values the cache tier holds."""
    import torch
    m = mesh()
    cfg = models.CONFIGS[name]
    H, HK, HD = cfg["n_head"], cfg["n_head_kv"], cfg["head_dim"]
    n_ctx = 600
    path = str(tmp_path / "a.gguf")
    models.write_model(path, cfg, [1], seed=1)
    kv_types = {"f16": (m.F16, m.F16), "q8_0/q4_0": (m.Q8_0, m.Q4_0), "q4_0/q4_0": (m.Q4_0, m.Q4_0)}[kv]
    okv = {m.F16: None, m.Q8_0: oracle.Q8_0, m.Q4_0: oracle.Q4_0}
    st = m.Stage(path, 1, 2, n_ctx=n_ctx, n_seq_max=3, n_batch_max=8, kv_types=kv_types)
    ses = st.session()
    rng = np.random.Generator(np.random.PCG64(11))
    depth = [0, 333, n_ctx - 1]
    kc = np.zeros((3, HK, n_ctx, HD), np.float32)
    vc = np.zeros((3, HK, n_ctx, HD), np.float32)
    for s_, dpt in enumerate(depth):
        k = rng.standard_normal((dpt + 1, HK, HD)).astype(np.float16)
        v = rng.standard_normal((dpt + 1, HK, HD)).astype(np.float16)
        ses.kv_write(1, s_, 0, k.view(np.uint16), v.view(np.uint16))
        kf, vf = k.astype(np.float32), v.astype(np.float32)
        if okv[kv_types[0]] is not None:
            kf = oracle.kv_round(okv[kv_types[0]], kf)
        if okv[kv_types[1]] is not None:
            vf = oracle.kv_round(okv[kv_types[1]], vf)
        kc[s_, :, :dpt + 1] = kf.transpose(1, 0, 2)
        vc[s_, :, :dpt + 1] = vf.transpose(1, 0, 2)
    q = rng.standard_normal((3, H, HD)).astype(np.float32)
    qd = torch.from_numpy(q).cuda()
    out = torch.zeros((3, H, HD), dtype=torch.float32, device="cuda")
    ses.attn_dev(1, qd.data_ptr(), np.array(depth, np.int32), out.data_ptr(), seq=np.arange(3, dtype=np.int32), matrix_cores=matrix_cores)
    ses.synchronize()
    got = out.cpu().numpy()
    scale = 1.0 / np.sqrt(HD)
    for s_, dpt in enumerate(depth):
        want = oracle.attn_token(q[s_], kc[s_], vc[s_], dpt, scale)
        rel = np.linalg.norm(got[s_] - want) / np.linalg.norm(want)
        # all-f32 kernel: accumulation order only; matrix-core kernel: q and the probabilities pass through f16
        assert rel < (2e-3 if matrix_cores else 2e-5), (s_, dpt, rel)
    ses.close()
    st.close()
