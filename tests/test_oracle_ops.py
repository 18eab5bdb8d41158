"""Pins the oracle's operators against library routines and closed forms that do not share its code:
numpy float64 matmul, torch float64 rms_norm / scaled_dot_product_attention / silu, complex rotation."""
import numpy as np
import pytest
import torch

import oracle

RNG = lambda s: np.random.Generator(np.random.PCG64(s))


@pytest.mark.parametrize("type_", [oracle.Q4_K, oracle.Q6_K, oracle.Q5_0, oracle.Q8_0, oracle.F16, oracle.F32])
def test_mul_mat_is_dequant_times_x(type_):
    rng = RNG(type_)
    M, K, T = 24, 512, 3
    rb = oracle.row_bytes(type_, K)
    W = rng.integers(0, 256, M * rb, dtype=np.uint8)
    if type_ in (oracle.F16, oracle.F32):  # keep random bit patterns finite
        W = rng.standard_normal(M * K).astype(np.float16 if type_ == oracle.F16 else np.float32).view(np.uint8)
    else:
        # random bytes make wild fp16 scales; overwrite every block's scale fields with tame ones
        be, bb = {oracle.Q4_K: (256, 144), oracle.Q6_K: (256, 210), oracle.Q5_0: (32, 22), oracle.Q8_0: (32, 34)}[type_]
        Wb = W.reshape(-1, bb)
        d = rng.uniform(1e-3, 2e-2, Wb.shape[0]).astype(np.float16).view(np.uint8).reshape(-1, 2)
        if type_ == oracle.Q4_K:
            Wb[:, 0:2] = d
            Wb[:, 2:4] = d
        elif type_ == oracle.Q6_K:
            Wb[:, 208:210] = d
        else:
            Wb[:, 0:2] = d
    x = rng.standard_normal((T, K)).astype(np.float32)
    bias = rng.standard_normal(M).astype(np.float32)
    Wd = np.stack([oracle.dequantize(type_, W[m * rb:(m + 1) * rb], K) for m in range(M)]).astype(np.float64)
    ref = x.astype(np.float64) @ Wd.T + bias
    got = oracle.mul_mat(type_, W, M, K, x, bias)
    assert np.allclose(got, ref.astype(np.float32), rtol=1e-6, atol=1e-6)
    got_nb = oracle.mul_mat(type_, W, M, K, x)
    assert np.allclose(got_nb, (ref - bias).astype(np.float32), rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("eps", [1e-5, 1e-6])
def test_rms_norm_vs_torch(eps):
    rng = RNG(11)
    x = (rng.standard_normal((5, 896)) * 3).astype(np.float32)
    w = (1 + 0.02 * rng.standard_normal(896)).astype(np.float32)
    ref = torch.nn.functional.rms_norm(torch.from_numpy(x).double(), (896,), torch.from_numpy(w).double(), eps)
    got = oracle.rms_norm(x, w, eps)
    assert np.allclose(got, ref.numpy(), rtol=2e-6, atol=1e-7)


@pytest.mark.parametrize("mode", [oracle.ROPE_NORM, oracle.ROPE_NEOX])
@pytest.mark.parametrize("base,hd", [(500000.0, 128), (1000000.0, 64)])
def test_rope_vs_complex_rotation(mode, base, hd):
    rng = RNG(hd)
    T, H = 6, 3
    x = rng.standard_normal((T, H, hd)).astype(np.float32)
    pos = np.array([0, 1, 7, 100, 4095, 8191], dtype=np.int32)
    got = oracle.rope(x, pos, hd, base, mode)
    i = np.arange(hd // 2)
    ang = pos[:, None].astype(np.float64) * base ** (-2.0 * i / hd)        # [T, hd/2]
    rot = np.exp(1j * ang)[:, None, :]
    xd = x.astype(np.float64)
    if mode == oracle.ROPE_NORM:
        z = (xd[..., 0::2] + 1j * xd[..., 1::2]) * rot
        ref = np.empty_like(xd)
        ref[..., 0::2], ref[..., 1::2] = z.real, z.imag
    else:
        z = (xd[..., :hd // 2] + 1j * xd[..., hd // 2:]) * rot
        ref = np.concatenate([z.real, z.imag], axis=-1)
    # the f32 theta recurrence drifts ~1e-7 relative per step; at pos 8191 that is a few 1e-3 rad
    assert np.allclose(got, ref, atol=2e-2)
    assert np.allclose(got[:4], ref[:4], atol=2e-4)
    # norm preservation is exact up to rounding
    assert np.allclose(np.linalg.norm(got, axis=-1), np.linalg.norm(x, axis=-1), rtol=1e-5)
    # position 0 is the identity
    assert np.array_equal(got[0], x[0])


def test_rope_partial_rotation_leaves_tail():
    rng = RNG(1)
    x = rng.standard_normal((2, 2, 64)).astype(np.float32)
    got = oracle.rope(x, np.array([3, 9], np.int32), 32, 10000.0, oracle.ROPE_NEOX)
    assert np.array_equal(got[..., 32:], x[..., 32:])
    assert not np.array_equal(got[..., :32], x[..., :32])


@pytest.mark.parametrize("n_head,n_kv,hd", [(8, 2, 64), (4, 4, 128), (14, 2, 64)])
def test_attn_vs_torch_sdpa(n_head, n_kv, hd):
    rng = RNG(n_head)
    ctx, n_past = 40, 29
    q = rng.standard_normal((n_head, hd)).astype(np.float32)
    k = (rng.standard_normal((n_kv, ctx, hd))).astype(np.float16)
    v = (rng.standard_normal((n_kv, ctx, hd))).astype(np.float16)
    scale = 1.0 / np.sqrt(hd)
    got = oracle.attn_token(q, k.view(np.uint16), v.view(np.uint16), n_past, scale)
    tq = torch.from_numpy(q).double()[None, :, None, :]                       # [1, H, 1, hd]
    tk = torch.from_numpy(k.astype(np.float64))[None, :, :n_past + 1]         # [1, Hkv, n, hd]
    tv = torch.from_numpy(v.astype(np.float64))[None, :, :n_past + 1]
    ref = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, scale=scale, enable_gqa=True)[0, :, 0]
    assert np.allclose(got, ref.numpy(), rtol=1e-5, atol=1e-6)


def test_swiglu_vs_torch():
    rng = RNG(2)
    g = (rng.standard_normal(1000) * 4).astype(np.float32)
    u = rng.standard_normal(1000).astype(np.float32)
    ref = torch.nn.functional.silu(torch.from_numpy(g).double()) * torch.from_numpy(u).double()
    assert np.allclose(oracle.swiglu(g, u), ref.numpy(), rtol=1e-5, atol=1e-7)


def test_moe_route_vs_numpy():
    rng = RNG(8)
    for trial in range(20):
        logits = rng.standard_normal(128).astype(np.float32)
        mask = np.zeros(128, np.float32)
        if trial % 2:
            mask[rng.choice(128, 64, replace=False)] = -np.inf
        ids, w = oracle.moe_route(logits, mask, 8, True)
        z = logits.astype(np.float64)
        p = np.exp(z - z.max())
        p /= p.sum()                                   # softmax over ALL experts; the mask only steers selection
        order = np.argsort(-(p + mask), kind="stable")[:8]
        assert list(ids) == list(order)
        assert np.allclose(w, p[order] / p[order].sum(), rtol=1e-6)
        assert np.all(mask[ids] == 0)
        ids2, w2 = oracle.moe_route(logits, mask, 8, False)
        assert list(ids2) == list(order) and np.allclose(w2, p[order], rtol=1e-6)


def test_moe_shard_equals_masked_full_model():
    # a shard file holds the router rows of its experts only: with normalised weights, routing over the shard's
    # logits equals routing over all logits with the other experts masked
    rng = RNG(9)
    logits = rng.standard_normal(128).astype(np.float32)
    keep = np.sort(rng.choice(128, 64, replace=False))
    mask = np.full(128, -np.inf, np.float32)
    mask[keep] = 0
    ids_full, w_full = oracle.moe_route(logits, mask, 8, True)
    ids_shard, w_shard = oracle.moe_route(logits[keep], None, 8, True)
    assert list(keep[ids_shard]) == list(ids_full)
    assert np.allclose(w_shard, w_full, rtol=1e-5)
