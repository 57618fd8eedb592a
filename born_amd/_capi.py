"""ctypes binding of the C ABI declared in include/born_rocm.h (born_amd/lib/libborn_rocm.so).

There is no CPU fallback: if the HIP library is missing or fails to load, importing a
symbol from here raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# the library built in-tree, unless BORN_ROCM_LIB names another build of it
LIB_PATH = os.environ.get("BORN_ROCM_LIB") or os.path.join(_HERE, "lib", "libborn_rocm.so")

OK, ERR_ARGUMENT, ERR_HIP, ERR_UNSUPPORTED, ERR_DATA = 0, 1, 2, 3, 4


class SamplerConfigC(C.Structure):
    _fields_ = [("temperature", C.c_float), ("top_k", C.c_int32), ("top_p", C.c_float),
                ("repetition_penalty", C.c_float), ("seed", C.c_int64), ("min_p", C.c_float),
                ("frequency_penalty", C.c_float), ("presence_penalty", C.c_float)]


class RowConfigsC(C.Structure):
    _fields_ = [("temperature", C.c_void_p), ("top_k", C.c_void_p), ("top_p", C.c_void_p), ("repetition_penalty", C.c_void_p),
                ("min_p", C.c_void_p), ("frequency_penalty", C.c_void_p), ("presence_penalty", C.c_void_p),
                ("row_kinds", C.c_uint32)]


ROWS_SMALL_TOP_K, ROWS_NO_TOP_K, ROWS_OTHER = 1, 2, 4


# every symbol include/born_rocm.h declares: name -> (restype, argtypes)
_vp, _i64, _i32p, _f32p = C.c_void_p, C.c_int64, C.POINTER(C.c_int32), C.POINTER(C.c_float)
SYMBOLS = {
    "born_rocm_last_error": (C.c_char_p, []),
    "born_rocm_device_count": (C.c_int, [_i32p]),
    "born_rocm_device_name": (C.c_int, [C.c_int32, C.c_char_p, _i64]),
    "born_rocm_alloc": (C.c_int, [_i64, C.POINTER(_vp)]),
    "born_rocm_free": (C.c_int, [_vp]),
    "born_rocm_h2d": (C.c_int, [_vp, _vp, _i64, _vp]),
    "born_rocm_d2h": (C.c_int, [_vp, _vp, _i64, _vp]),
    "born_rocm_stream_sync": (C.c_int, [_vp]),
    "born_rocm_sampler_create": (C.c_int, [C.POINTER(SamplerConfigC), _i64, _i64, C.POINTER(_vp)]),
    "born_rocm_sampler_destroy": (C.c_int, [_vp]),
    "born_rocm_sampler_get_config": (C.c_int, [_vp, C.POINTER(SamplerConfigC)]),
    "born_rocm_sampler_set_config": (C.c_int, [_vp, C.POINTER(SamplerConfigC)]),
    "born_rocm_sampler_set_path": (C.c_int, [_vp, C.c_int32]),
    "born_rocm_sampler_get_step": (C.c_int, [_vp, C.POINTER(_i64)]),
    "born_rocm_sampler_set_step": (C.c_int, [_vp, _i64]),
    "born_rocm_sampler_status": (C.c_int, [_vp, _vp]),
    "born_rocm_sampler_counters": (C.c_int, [_vp, _vp, C.POINTER(_i64), C.POINTER(_i64), C.POINTER(_i64)]),
    "born_rocm_argmax": (C.c_int, [_vp, _vp, _i64, _i64, _i64, _vp, _vp]),
    "born_rocm_softmax": (C.c_int, [_vp, _vp, _i64, _i64, _i64, _vp, _vp]),
    "born_rocm_log_softmax": (C.c_int, [_vp, _vp, _i64, _i64, _i64, _vp, _vp]),
    "born_rocm_sample": (C.c_int, [_vp, _vp, _i64, _i64, _i64, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _vp]),
    "born_rocm_sample_static": (C.c_int, [C.POINTER(SamplerConfigC), _vp, _i64, _i64, _i64, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp]),
    "born_rocm_sample_rows": (C.c_int, [_vp, _vp, _i64, _i64, _i64, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp]),
    "born_rocm_token_logprobs": (C.c_int, [_vp, _vp, _i64, _i64, _i64, _vp, _vp, _i64, _vp, _vp, _vp]),
    "born_rocm_history_append": (C.c_int, [_vp, _vp, _vp, _i64, _vp, _i64, _i64, _vp]),
    "born_rocm_gather_rows": (C.c_int, [_vp, _vp, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp]),
    "born_rocm_spec_verify": (C.c_int, [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp]),
    "born_rocm_spec_verify_bonus": (C.c_int, [_vp, _vp, _i64, _vp, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp]),
    "born_rocm_exp": (C.c_int, [_vp, _vp, _i64, _vp]),
    "born_rocm_expneg": (C.c_int, [_vp, _vp, _i64, _vp]),
    "born_rocm_uniforms": (C.c_int, [_i64, _i64, _vp, _i64, _vp]),
    "born_rocm_linear": (C.c_int, [_vp, _i64, _i64, _i64, _vp, _i64, _i64, _vp, _vp, _i64, _vp]),
    "born_rocm_matmul": (C.c_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _vp]),
    "born_rocm_linear_argmax": (C.c_int, [_vp, _vp, _i64, _i64, _i64, _vp, _i64, _i64, _vp, _vp, _vp]),
    "born_rocm_linear_sample": (C.c_int, [_vp, _vp, _i64, _i64, _i64, _vp, _i64, _i64, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _vp]),
    "born_rocm_broadcast_shape": (C.c_int, [_vp, C.c_int32, _vp, C.c_int32, _vp]),
    "born_rocm_add": (C.c_int, [_vp, _vp, C.c_int32, _vp, _vp, C.c_int32, _vp, _vp]),
    "born_rocm_sub": (C.c_int, [_vp, _vp, C.c_int32, _vp, _vp, C.c_int32, _vp, _vp]),
    "born_rocm_mul": (C.c_int, [_vp, _vp, C.c_int32, _vp, _vp, C.c_int32, _vp, _vp]),
    "born_rocm_div": (C.c_int, [_vp, _vp, C.c_int32, _vp, _vp, C.c_int32, _vp, _vp]),
    "born_rocm_transpose": (C.c_int, [_vp, _vp, C.c_int32, _vp, _vp, _vp]),
    "born_rocm_conv2d": (C.c_int, [_vp, _vp, _vp, _vp, C.c_int32, C.c_int32, _vp, _vp, _vp]),
    "born_rocm_maxpool2d": (C.c_int, [_vp, _vp, C.c_int32, C.c_int32, _vp, _vp, _vp]),
    "born_rocm_reshape": (C.c_int, [_vp, _vp, C.c_int32, _vp, C.c_int32, _vp, _vp]),
}

_lib = None


def lib():
    """Loads the HIP library; raises if it has not been built (python -m born_amd.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"born_amd: {LIB_PATH} is missing; build it with `python -m born_amd.build` "
                               "(there is no CPU fallback)")
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(L, name)          # AttributeError if the library does not export it
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


class BornRocmError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(msg)
        self.code = code


def check(rc):
    if rc != OK:
        msg = lib().born_rocm_last_error().decode("utf-8", "replace")
        raise BornRocmError(rc, msg or f"born_rocm error {rc}")
