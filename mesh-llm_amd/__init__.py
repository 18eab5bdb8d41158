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
F32, F16, Q5_0, Q8_0, Q4_K, Q6_K = 0, 1, 6, 8, 12, 14

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
    "mesh_act_packed_size": (_sz, [_i32, _i64, _i64]),
    "mesh_act_pack": (_i32, [_i32, _vp, _vp, _i64]),
    "mesh_act_unpack": (_i32, [_i32, _vp, _vp, _i64]),
    "mesh_act_pack_dev": (_i32, [_i32, _vp, _vp, _i64, _vp]),
    "mesh_act_unpack_dev": (_i32, [_i32, _vp, _vp, _i64, _vp]),
    "mesh_dequantize_dev": (_i32, [_i32, _vp, _vp, _i64, _vp]),
}

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
