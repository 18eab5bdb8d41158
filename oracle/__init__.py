"""ctypes front end of the CPU oracle (oracle/mesh_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the cpu_baseline leg of
bench.py as the checker -- never by the product path.  Parity against ggml itself is unpinned (its
source is not reachable offline); tests/test_oracle_*.py pin each routine by independent means.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmesh_oracle.so")

F32, F16, Q4_0, Q5_0, Q8_0, Q4_K, Q6_K = 0, 1, 2, 6, 8, 12, 14
ROPE_NORM, ROPE_NEOX = 0, 2

_lib = None


def build(force=False):
    """Compile the oracle with gcc (seconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libmesh_oracle.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        c = ctypes
        vp, i64, i32, f32 = c.c_void_p, c.c_int64, c.c_int32, c.c_float
        L.mo_fp32_to_fp16.restype = c.c_uint16
        L.mo_fp32_to_fp16.argtypes = [f32]
        L.mo_fp16_to_fp32.restype = f32
        L.mo_fp16_to_fp32.argtypes = [c.c_uint16]
        L.mo_fp32_to_fp16_row.argtypes = [vp, vp, i64]
        L.mo_fp16_to_fp32_row.argtypes = [vp, vp, i64]
        for fn in (L.mo_block_elems, L.mo_block_bytes):
            fn.restype = i64
            fn.argtypes = [i32]
        L.mo_row_bytes.restype = i64
        L.mo_row_bytes.argtypes = [i32, i64]
        L.mo_quantize_row_q8_0.argtypes = [vp, vp, i64]
        L.mo_dequantize_row.restype = i32
        L.mo_dequantize_row.argtypes = [i32, vp, vp, i64]
        L.mo_mul_mat.restype = i32
        L.mo_mul_mat.argtypes = [i32, vp, i64, i64, vp, i64, vp, vp]
        L.mo_rms_norm.argtypes = [vp, vp, f32, i64, i64, vp]
        L.mo_rope.argtypes = [vp, i64, i32, i32, i32, vp, f32, i32]
        L.mo_swiglu.argtypes = [vp, vp, vp, i64]
        L.mo_attn_token.argtypes = [vp, vp, vp, i32, i32, i32, i64, i64, f32, vp]
        L.mo_attn_token_f32.argtypes = [vp, vp, vp, i32, i32, i32, i64, i64, f32, vp]
        L.mo_quantize_row_q4_0.argtypes = [vp, vp, i64]
        L.mo_moe_route.argtypes = [vp, vp, i32, i32, i32, vp, vp]
        L.mo_set_threads.argtypes = [i32]
        L.mo_get_threads.restype = i32
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def set_threads(n):
    lib().mo_set_threads(int(n))


def get_threads():
    return int(lib().mo_get_threads())


def row_bytes(type_, k):
    return int(lib().mo_row_bytes(type_, k))


def fp32_to_fp16(x):
    """f32 array -> uint16 array of binary16 bit patterns."""
    x = _f32(x)
    y = np.empty(x.shape, dtype=np.uint16)
    lib().mo_fp32_to_fp16_row(_p(x), _p(y), x.size)
    return y


def fp16_to_fp32(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    y = np.empty(h.shape, dtype=np.float32)
    lib().mo_fp16_to_fp32_row(_p(h), _p(y), h.size)
    return y


def quantize_q8_0(x):
    """f32 array (size % 32 == 0) -> uint8 array of 34-byte blocks."""
    x = _f32(x)
    assert x.size % 32 == 0
    y = np.empty(x.size // 32 * 34, dtype=np.uint8)
    lib().mo_quantize_row_q8_0(_p(x), _p(y), x.size)
    return y


def quantize_q4_0(x):
    """f32 array (size % 32 == 0) -> uint8 array of 18-byte blocks."""
    x = _f32(x)
    assert x.size % 32 == 0
    y = np.empty(x.size // 32 * 18, dtype=np.uint8)
    lib().mo_quantize_row_q4_0(_p(x), _p(y), x.size)
    return y


def kv_round(type_, x):
    """The values a KV cache of `type_` (F16, Q8_0 or Q4_0) holds for the f32 rows x [..., head_dim], as f32."""
    x = _f32(x)
    if type_ == F16:
        return fp16_to_fp32(fp32_to_fp16(x)).reshape(x.shape)
    packed = quantize_q8_0(x) if type_ == Q8_0 else quantize_q4_0(x)
    return dequantize(type_, packed, x.size).reshape(x.shape)


def dequantize(type_, data, k):
    """k elements of `type_` blocks held in the uint8 array `data` -> f32[k]."""
    data = np.ascontiguousarray(data, dtype=np.uint8)
    nb = row_bytes(type_, k)
    assert nb >= 0 and data.size >= nb, (type_, k, data.size)
    y = np.empty(k, dtype=np.float32)
    rc = lib().mo_dequantize_row(type_, _p(data), _p(y), k)
    assert rc == 0
    return y


def mul_mat(type_, W, M, K, x, bias=None):
    """x: [T, K] f32 -> [T, M] f32; W: M rows of `type_` blocks (uint8 array)."""
    W = np.ascontiguousarray(W, dtype=np.uint8)
    x = _f32(x).reshape(-1, K)
    T = x.shape[0]
    assert W.size == M * row_bytes(type_, K), (W.size, M, K, type_)
    y = np.empty((T, M), dtype=np.float32)
    b = _f32(bias) if bias is not None else None
    rc = lib().mo_mul_mat(type_, _p(W), M, K, _p(x), T, _p(b) if b is not None else None, _p(y))
    assert rc == 0
    return y


def rms_norm(x, w, eps):
    x = _f32(x)
    n = x.shape[-1]
    w = _f32(w)
    y = np.empty_like(x)
    lib().mo_rms_norm(_p(x), _p(w), eps, n, x.size // n, _p(y))
    return y


def rope(x, pos, n_rot, freq_base, mode):
    """x: [T, n_head, head_dim] -> rotated copy."""
    x = _f32(x).copy()
    T, n_head, hd = x.shape
    pos = np.ascontiguousarray(pos, dtype=np.int32)
    assert pos.size == T
    lib().mo_rope(_p(x), T, n_head, hd, n_rot, _p(pos), freq_base, mode)
    return x


def swiglu(gate, up):
    gate, up = _f32(gate), _f32(up)
    out = np.empty_like(gate)
    lib().mo_swiglu(_p(gate), _p(up), _p(out), gate.size)
    return out


def attn_token(q, kcache, vcache, n_past, scale):
    """q: [n_head, hd] f32; kcache/vcache: [n_kv, ctx, hd], both uint16 (f16 bits) or both float32 (the values a
    quantised cache holds); attends to [0, n_past]."""
    q = _f32(q)
    n_head, hd = q.shape
    as_f32 = kcache.dtype == np.float32
    assert vcache.dtype == kcache.dtype and kcache.dtype in (np.float32, np.uint16)
    kcache = np.ascontiguousarray(kcache)
    vcache = np.ascontiguousarray(vcache)
    n_kv, ctx, hd2 = kcache.shape
    assert hd2 == hd and vcache.shape == kcache.shape and n_past < ctx
    out = np.empty_like(q)
    fn = lib().mo_attn_token_f32 if as_f32 else lib().mo_attn_token
    fn(_p(q), _p(kcache), _p(vcache), n_head, n_kv, hd, ctx, n_past, scale, _p(out))
    return out


def moe_route(logits, mask, top_k, norm_w=True):
    logits = _f32(logits)
    n = logits.size
    m = _f32(mask) if mask is not None else None
    ids = np.empty(top_k, dtype=np.int32)
    w = np.empty(top_k, dtype=np.float32)
    lib().mo_moe_route(_p(logits), _p(m) if m is not None else None, n, top_k, int(norm_w), _p(ids), _p(w))
    return ids, w
