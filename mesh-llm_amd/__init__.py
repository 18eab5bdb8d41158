"""Host-side binding of libmeshstage.so (the MI355X pipeline-stage executor) over its C ABI.

This is the ctypes twin of the stub a Rust `*-ffi` crate would carry: it declares exactly the entry
points of include/mesh_stage.h and turns negative status codes into MeshError.  There is no CPU
fallback: without the built HIP library, importing a symbol raises.

The directory name is not a Python identifier; load it with __graft_entry__.load_package() (module
name `mesh_llm_amd`).
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmeshstage.so")

# ggml type ids (include/mesh_stage.h: mesh_dtype)
F32, F16, Q4_0, Q5_0, Q8_0, Q4_K, Q6_K = 0, 1, 2, 6, 8, 12, 14

OK, ERR_INVALID, ERR_DEVICE, ERR_NOMEM, ERR_IO, ERR_FORMAT, ERR_UNSUPPORTED = 0, -1, -2, -3, -4, -5, -6


class MeshError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("mesh status %d: %s" % (code, message))
        self.code = code
        self.message = message


_vp, _i64, _i32, _sz, _cp = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_size_t, ctypes.c_char_p

# name -> (restype, argtypes); must list every symbol of include/mesh_stage.h
SIGNATURES = {
    "mesh_last_error": (_cp, []),
    "mesh_device_count": (_i32, []),
    "mesh_device_select": (_i32, [_cp]),
    "mesh_hbm_read_probe": (_i32, [_sz, _i32, _i32, _vp]),
    "mesh_hbm_mix_probe_dev": (_i32, [_vp, _vp, _sz, _i32, _i32, _vp]),
    "mesh_mfma_f16_probe": (_i32, [_i32, _i32, _i32, _vp]),
    "mesh_act_packed_size": (_sz, [_i32, _i64, _i64]),
    "mesh_act_pack": (_i32, [_i32, _vp, _vp, _i64]),
    "mesh_act_unpack": (_i32, [_i32, _vp, _vp, _i64]),
    "mesh_act_pack_noalloc": (_i32, [_i32, _vp, _vp, _i64]),
    "mesh_act_pack_dev": (_i32, [_i32, _vp, _vp, _i64, _vp]),
    "mesh_act_unpack_dev": (_i32, [_i32, _vp, _vp, _i64, _vp]),
    "mesh_dequantize_dev": (_i32, [_i32, _vp, _vp, _i64, _vp]),
}



class ModelInfo(ctypes.Structure):
    """mesh_model_info"""
    _fields_ = [("arch", ctypes.c_char * 32)] + [(n, ctypes.c_uint32) for n in (
        "n_layer", "n_embd", "n_head", "n_head_kv", "head_dim", "n_ff", "n_vocab", "n_rot", "rope_mode",
        "n_expert", "n_expert_used", "n_ff_exp")] + [("rms_eps", ctypes.c_float), ("rope_freq_base", ctypes.c_float),
        ("gguf_version", ctypes.c_uint32), ("alignment", ctypes.c_uint32),
        ("n_tensors", ctypes.c_uint64), ("data_offset", ctypes.c_uint64), ("file_size", ctypes.c_uint64)]


class TensorInfo(ctypes.Structure):
    """mesh_tensor_info"""
    _fields_ = [("type", ctypes.c_uint32), ("n_dims", ctypes.c_uint32), ("ne", ctypes.c_uint64 * 4),
                ("file_offset", ctypes.c_uint64), ("nbytes", ctypes.c_uint64)]


class StageOpts(ctypes.Structure):
    """mesh_stage_opts"""
    _fields_ = [("device", ctypes.c_char_p), ("n_ctx", ctypes.c_int32), ("n_seq_max", ctypes.c_int32),
                ("n_batch_max", ctypes.c_int32), ("kv_type", ctypes.c_int32), ("kv_type_v", ctypes.c_int32),
                ("tuning", ctypes.c_char_p)]


class Batch(ctypes.Structure):
    """mesh_batch"""
    _fields_ = [("n_tokens", ctypes.c_int32), ("pos", ctypes.POINTER(ctypes.c_int32)),
                ("seq_id", ctypes.POINTER(ctypes.c_int32))]


class Profile(ctypes.Structure):
    """mesh_profile"""
    _fields_ = [("ms", ctypes.c_double * 5), ("launches", ctypes.c_uint64 * 5)]


PROF_GEMV, PROF_ROPE, PROF_ATTN, PROF_CODEC, PROF_PREP = 0, 1, 2, 3, 4
TOKENS, LOGITS = 100, 101
_pp = ctypes.POINTER(ctypes.c_void_p)
_psz = ctypes.POINTER(ctypes.c_size_t)

SIGNATURES.update({
    "mesh_weight_upload": (_i32, [_i32, _vp, _i64, _i64, _pp]),
    "mesh_weight_free": (None, [_vp]),
    "mesh_weight_nbytes": (_sz, [_vp]),
    "mesh_mul_mat_dev": (_i32, [_vp, _vp, _i64, _vp, _vp]),
    "mesh_weight_download": (_i32, [_vp, _vp]),
    "mesh_gguf_probe": (_i32, [_cp, ctypes.POINTER(ModelInfo)]),
    "mesh_gguf_tensor": (_i32, [_cp, _cp, ctypes.POINTER(TensorInfo)]),
    "mesh_stage_open": (_i32, [_cp, _i32, _i32, ctypes.POINTER(StageOpts), _pp]),
    "mesh_stage_close": (None, [_vp]),
    "mesh_stage_info": (_i32, [_vp, ctypes.POINTER(ModelInfo)]),
    "mesh_stage_weight_bytes": (_sz, [_vp]),
    "mesh_stage_session_new": (_i32, [_vp, _pp]),
    "mesh_stage_session_free": (None, [_vp]),
    "mesh_stage_decode": (_i32, [_vp, ctypes.POINTER(Batch), _vp, _i32, _vp, _i32, _sz, _psz]),
    "mesh_stage_decode_dev": (_i32, [_vp, ctypes.POINTER(Batch), _vp, _i32, _vp, _i32, _sz, _psz]),
    "mesh_session_stream": (_vp, [_vp]),
    "mesh_session_synchronize": (_i32, [_vp]),
    "mesh_session_graph_replays": (_i64, [_vp]),
    "mesh_session_profile": (_i32, [_vp, _i32]),
    "mesh_session_profile_read": (_i32, [_vp, ctypes.POINTER(Profile)]),
    "mesh_session_set_expert_mask": (_i32, [_vp, _vp, _i32]),
    "mesh_session_moe_last_ids": (_i32, [_vp, _vp, _i32]),
    "mesh_session_f16_saturations": (_i32, [_vp, ctypes.POINTER(ctypes.c_uint64)]),
    "mesh_session_set_option": (_i32, [_vp, ctypes.c_char_p, _i32]),
    "mesh_session_get_option": (_i32, [_vp, ctypes.c_char_p, ctypes.POINTER(_i32)]),
    "mesh_session_kv_write": (_i32, [_vp, _i32, _i32, _i32, _i32, _vp, _vp]),
    "mesh_session_kv_read": (_i32, [_vp, _i32, _i32, _i32, _i32, _vp, _vp]),
    "mesh_op_q16_bytes": (_sz, [_i64, _i64]),
    "mesh_op_rms_norm_q16_dev": (_i32, [_vp, _vp, ctypes.c_float, _i64, _i64, _vp, _vp]),
    "mesh_op_rms_norm_f16k8_dev": (_i32, [_vp, _vp, ctypes.c_float, _i64, _i64, _vp, _vp]),
    "mesh_op_swiglu_f16k8_dev": (_i32, [_vp, _vp, _i64, _i64, _vp, _vp]),
    "mesh_session_attn_dev": (_i32, [_vp, _i32, _vp, ctypes.POINTER(Batch), _vp, _i32]),
})

_lib = None


def lib():
    """The loaded C library; raises if it has not been built (no fallback path exists)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("%s is missing: run `python -c 'import __graft_entry__ as g; g.build()'`" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def last_error():
    return lib().mesh_last_error().decode("utf-8", "replace")


def check(rc):
    if rc != 0:
        raise MeshError(rc, last_error())
    return rc


def device_count():
    return int(lib().mesh_device_count())


def device_select(name):
    check(lib().mesh_device_select(str(name).encode()))


def hbm_read_probe(nbytes=512 << 20, warmup=3, runs=20):
    """GB/s of `runs` streaming-read passes over a buffer of nbytes (mesh_hbm_read_probe), ascending."""
    out = (ctypes.c_double * runs)()
    check(lib().mesh_hbm_read_probe(nbytes, warmup, runs, out))
    return sorted(out)


def mfma_f16_probe(iters=4000, warmup=3, runs=20):
    """TFLOP/s of `runs` launches of the register-only f16 matrix-core kernel (mesh_mfma_f16_probe), ascending."""
    out = (ctypes.c_double * runs)()
    check(lib().mesh_mfma_f16_probe(iters, warmup, runs, out))
    return sorted(out)


def hbm_mix_probe_dev(src_ptr, dst_ptr, big_bytes, ratio, big_is_read, stream=0):
    """Queue one plain streaming kernel that moves big_bytes on its larger side and big_bytes / ratio on the other
    (mesh_hbm_mix_probe_dev); device pointers, not waited for."""
    check(lib().mesh_hbm_mix_probe_dev(src_ptr, dst_ptr, big_bytes, ratio, int(bool(big_is_read)), stream))


def op_q16_bytes(n_tokens, n):
    return int(lib().mesh_op_q16_bytes(n_tokens, n))


def op_rms_norm_q16_dev(x_ptr, w_ptr, eps, n_tokens, n, out_ptr, stream=0):
    check(lib().mesh_op_rms_norm_q16_dev(x_ptr, w_ptr, eps, n_tokens, n, out_ptr, stream))


def op_rms_norm_f16k8_dev(x_ptr, w_ptr, eps, n_tokens, n, out_ptr, stream=0):
    check(lib().mesh_op_rms_norm_f16k8_dev(x_ptr, w_ptr, eps, n_tokens, n, out_ptr, stream))


def op_swiglu_f16k8_dev(gate_ptr, up_ptr, n_tokens, n, out_ptr, stream=0):
    check(lib().mesh_op_swiglu_f16k8_dev(gate_ptr, up_ptr, n_tokens, n, out_ptr, stream))


def act_packed_size(fmt, n_tokens, n_embd):
    return int(lib().mesh_act_packed_size(fmt, n_tokens, n_embd))


def _np_ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def act_pack(fmt, x):
    """Host form: numpy f32 array -> numpy uint8 array of packed bytes."""
    import numpy as np
    x = np.ascontiguousarray(x, dtype=np.float32)
    per = {F32: (1, 4), F16: (1, 2), Q8_0: (32, 34)}.get(fmt)
    if per is None or x.size % per[0]:
        # let the library produce the error text
        out = np.empty(max(x.size * 4, 1), dtype=np.uint8)
    else:
        out = np.empty(x.size // per[0] * per[1], dtype=np.uint8)
    check(lib().mesh_act_pack(fmt, _np_ptr(x), _np_ptr(out), x.size))
    return out


def act_pack_noalloc(fmt, x):
    """act_pack through the entry point that allocates no GPU memory (at most 1 Mi elements)."""
    import numpy as np
    x = np.ascontiguousarray(x, dtype=np.float32)
    per = {F32: (1, 4), F16: (1, 2), Q8_0: (32, 34)}.get(fmt)
    out = np.empty(max(x.size * 4, 1) if per is None or x.size % per[0] else x.size // per[0] * per[1], dtype=np.uint8)
    check(lib().mesh_act_pack_noalloc(fmt, _np_ptr(x), _np_ptr(out), x.size))
    return out


def act_unpack(fmt, packed, n):
    """Host form: packed bytes (numpy uint8) -> numpy f32[n]."""
    import numpy as np
    packed = np.ascontiguousarray(packed).view(np.uint8)
    out = np.empty(max(n, 0), dtype=np.float32)
    check(lib().mesh_act_unpack(fmt, _np_ptr(packed), _np_ptr(out), n))
    return out


def act_pack_dev(fmt, d_src, d_dst, n, stream=0):
    check(lib().mesh_act_pack_dev(fmt, d_src, d_dst, n, stream))


def act_unpack_dev(fmt, d_src, d_dst, n, stream=0):
    check(lib().mesh_act_unpack_dev(fmt, d_src, d_dst, n, stream))


def dequantize_dev(type_, d_src, d_dst, n, stream=0):
    check(lib().mesh_dequantize_dev(type_, d_src, d_dst, n, stream))


# ---------------------------------------------------------------------------------------------- weights
class Weight:
    """One matrix resident in HBM (mesh_weight)."""

    def __init__(self, type_, data, n_rows, row_len):
        import numpy as np
        data = np.ascontiguousarray(data).view(np.uint8)
        self._h = ctypes.c_void_p()
        check(lib().mesh_weight_upload(type_, _np_ptr(data), n_rows, row_len, ctypes.byref(self._h)))
        self.type, self.n_rows, self.row_len = type_, n_rows, row_len

    @property
    def nbytes(self):
        return int(lib().mesh_weight_nbytes(self._h))

    def mul_mat_dev(self, d_x, n_tokens, d_y, stream=0):
        check(lib().mesh_mul_mat_dev(self._h, d_x, n_tokens, d_y, stream))

    def download(self):
        import numpy as np
        out = np.empty(self.nbytes, dtype=np.uint8)
        check(lib().mesh_weight_download(self._h, _np_ptr(out)))
        return out

    def close(self):
        if self._h:
            lib().mesh_weight_free(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


# ---------------------------------------------------------------------------------------------- gguf
def gguf_probe(path):
    info = ModelInfo()
    check(lib().mesh_gguf_probe(os.fsencode(path), ctypes.byref(info)))
    return info


def gguf_tensor(path, name):
    info = TensorInfo()
    check(lib().mesh_gguf_tensor(os.fsencode(path), name.encode(), ctypes.byref(info)))
    return info


# ---------------------------------------------------------------------------------------------- stage
class Stage:
    """Layers [layer_begin, layer_end) of a GGUF model resident on the GPU (mesh_stage)."""

    def __init__(self, gguf_path, layer_begin, layer_end=-1, n_ctx=0, n_seq_max=0, n_batch_max=0, device=None, kv_types=None, tuning=None):
        """kv_types: (K, V) cache row types, one of (F16, F16), (Q8_0, Q4_0), (Q4_0, Q4_0); None = f16 / f16.
        tuning: kernel-selection switches, {"name": value} or "name=value,..." (mesh_stage_opts.tuning)."""
        kt, vt = kv_types if kv_types else (0, 0)
        if isinstance(tuning, dict):
            tuning = ",".join("%s=%d" % (k, int(v)) for k, v in tuning.items())
        opts = StageOpts(device.encode() if device else None, n_ctx, n_seq_max, n_batch_max, kt, vt, tuning.encode() if tuning else None)
        self._h = ctypes.c_void_p()
        check(lib().mesh_stage_open(os.fsencode(gguf_path), layer_begin, layer_end, ctypes.byref(opts), ctypes.byref(self._h)))
        self.info = ModelInfo()
        check(lib().mesh_stage_info(self._h, ctypes.byref(self.info)))

    @property
    def weight_bytes(self):
        return int(lib().mesh_stage_weight_bytes(self._h))

    def session(self, **options):
        """options: session-level kernel-selection switches (mesh_session_set_option), e.g. session(skinny_f16=0)."""
        ses = Session(self)
        for name, value in options.items():
            ses.set_option(name, value)
        return ses

    def close(self):
        if self._h:
            lib().mesh_stage_close(self._h)
            self._h = ctypes.c_void_p()


class Session:
    """KV cache + activation buffers of one set of sequences (mesh_session).  Single-threaded."""

    def __init__(self, stage):
        self.stage = stage
        self._h = ctypes.c_void_p()
        check(lib().mesh_stage_session_new(stage._h, ctypes.byref(self._h)))

    @staticmethod
    def _batch(pos, seq):
        import numpy as np
        pos = np.ascontiguousarray(pos, dtype=np.int32)
        seq = np.zeros_like(pos) if seq is None else np.ascontiguousarray(seq, dtype=np.int32)
        b = Batch(pos.size, pos.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)), seq.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)))
        return b, (pos, seq)

    def decode(self, inp, pos, seq=None, in_fmt=F32, out_fmt=F32):
        """Host form.  inp: numpy array holding the packed input (f32 rows, f16 bits, q8_0 bytes or int32 ids)."""
        import numpy as np
        b, keep = self._batch(pos, seq)
        inp = np.ascontiguousarray(inp)
        T = b.n_tokens
        if out_fmt == LOGITS:
            cap = T * max(self.stage.info.n_vocab, 1) * 4 + 16
            cap = max(cap, 1 << 20)
        else:
            cap = T * self.stage.info.n_embd * 4
        out = np.empty(cap, dtype=np.uint8)
        n = ctypes.c_size_t(0)
        rc = lib().mesh_stage_decode(self._h, ctypes.byref(b), _np_ptr(inp), in_fmt, _np_ptr(out), out_fmt, cap, ctypes.byref(n))
        if rc == ERR_INVALID and out_fmt == LOGITS and n.value > cap:
            cap = n.value
            out = np.empty(cap, dtype=np.uint8)
            rc = lib().mesh_stage_decode(self._h, ctypes.byref(b), _np_ptr(inp), in_fmt, _np_ptr(out), out_fmt, cap, ctypes.byref(n))
        check(rc)
        return out[:n.value]

    def decode_dev(self, d_in, pos, d_out, out_cap, seq=None, in_fmt=F32, out_fmt=F32):
        b, keep = self._batch(pos, seq)
        n = ctypes.c_size_t(0)
        check(lib().mesh_stage_decode_dev(self._h, ctypes.byref(b), d_in, in_fmt, d_out, out_fmt, out_cap, ctypes.byref(n)))
        return n.value

    @property
    def stream(self):
        return lib().mesh_session_stream(self._h) or 0

    def synchronize(self):
        check(lib().mesh_session_synchronize(self._h))

    def attn_dev(self, layer, d_q, pos, d_out, seq=None, matrix_cores=True):
        """Decode attention of one layer over this session's KV cache (mesh_session_attn_dev); device pointers."""
        b, keep = self._batch(pos, seq)
        check(lib().mesh_session_attn_dev(self._h, layer, d_q, ctypes.byref(b), d_out, 1 if matrix_cores else 0))

    @property
    def graph_replays(self):
        """Decode steps so far whose layer launches were replayed from a captured graph."""
        return int(lib().mesh_session_graph_replays(self._h))

    def profile(self, enable):
        check(lib().mesh_session_profile(self._h, 1 if enable else 0))

    def profile_read(self):
        p = Profile()
        check(lib().mesh_session_profile_read(self._h, ctypes.byref(p)))
        names = ("gemv", "rope", "attn", "codec", "prep")
        return {n: {"ms": p.ms[i], "launches": int(p.launches[i])} for i, n in enumerate(names)}

    def set_expert_mask(self, allowed):
        """allowed: bool array over the file's experts, or None to clear."""
        import numpy as np
        if allowed is None:
            check(lib().mesh_session_set_expert_mask(self._h, None, 0))
            return
        a = np.ascontiguousarray(allowed, dtype=np.uint8)
        check(lib().mesh_session_set_expert_mask(self._h, _np_ptr(a), a.size))

    def moe_last_ids(self, n_tokens):
        import numpy as np
        out = np.empty((n_tokens, self.stage.info.n_expert_used), dtype=np.int32)
        check(lib().mesh_session_moe_last_ids(self._h, _np_ptr(out), n_tokens))
        return out

    def set_option(self, name, value):
        check(lib().mesh_session_set_option(self._h, name.encode(), int(value)))

    def get_option(self, name):
        v = ctypes.c_int32(0)
        check(lib().mesh_session_get_option(self._h, name.encode(), ctypes.byref(v)))
        return int(v.value)

    def f16_saturations(self):
        """Values clamped to the f16 range by the batched paths since the session was created."""
        n = ctypes.c_uint64(0)
        check(lib().mesh_session_f16_saturations(self._h, ctypes.byref(n)))
        return int(n.value)

    def kv_write(self, layer, seq_id, pos0, k, v):
        """k, v: uint16 arrays [n_pos, n_head_kv, head_dim] of f16 bits."""
        import numpy as np
        k = np.ascontiguousarray(k, dtype=np.uint16)
        v = np.ascontiguousarray(v, dtype=np.uint16)
        check(lib().mesh_session_kv_write(self._h, layer, seq_id, pos0, k.shape[0], _np_ptr(k), _np_ptr(v)))

    def kv_read(self, layer, seq_id, pos0, n_pos):
        import numpy as np
        i = self.stage.info
        k = np.empty((n_pos, i.n_head_kv, i.head_dim), dtype=np.uint16)
        v = np.empty_like(k)
        check(lib().mesh_session_kv_read(self._h, layer, seq_id, pos0, n_pos, _np_ptr(k), _np_ptr(v)))
        return k, v

    def close(self):
        if self._h:
            lib().mesh_stage_session_free(self._h)
            self._h = ctypes.c_void_p()
