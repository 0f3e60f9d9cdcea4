"""ctypes binding of libq8_hip.so (the C ABI declared in include/q8_hip.h).

The library is loaded on first use. There is no fallback: if it is missing the call raises.
"""
import ctypes
import os
import threading

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libq8_hip.so")

# element types / flags, mirrored from include/q8_hip.h
Q8_I8, Q8_E4M3, Q8_BF16, Q8_F16, Q8_F32 = 0, 1, 2, 3, 4
Q8_QUANT_RNE, Q8_QUANT_SCALE_DIV = 1, 2
Q8_V_DS, Q8_V_SD = 0, 1
Q8_ATTN_SUM_ROUNDED_P, Q8_ATTN_P_UNIT_RANGE, Q8_ATTN_O_TOKEN_MAJOR, Q8_ATTN_LAZY_MAX = 1, 2, 4, 8
Q8_PREP_FHT, Q8_PREP_PAIR_TABLES, Q8_PREP_SHARED_TABLES = 1, 2, 4
# values of q8_gemm_last_kernel (tests)
Q8_GEMM_KERNEL_PIPE256, Q8_GEMM_KERNEL_TILE128, Q8_GEMM_KERNEL_TILE64 = 1, 2, 3
Q8_GEMM_KERNEL_PERSIST256, Q8_GEMM_KERNEL_PERSIST192, Q8_GEMM_KERNEL_RESIDUAL = 4, 5, 16

_c = ctypes
_vp, _i, _i64, _f = _c.c_void_p, _c.c_int, _c.c_int64, _c.c_float

# name -> (restype, argtypes): every symbol include/q8_hip.h declares
SIGNATURES = {
    "q8_strerror": (_c.c_char_p, [_i]),
    "q8_last_error": (_c.c_char_p, []),
    "q8_device_info": (_i, [_c.POINTER(_i), _c.POINTER(_i), _c.POINTER(_i64), _c.c_char_p]),
    "q8_quant_rows": (_i, [_vp, _i, _vp, _i, _vp, _i64, _i, _i64, _i, _vp]),
    "q8_fht": (_i, [_vp, _i, _vp, _i, _i64, _i, _f, _vp]),
    "q8_rmsnorm": (_i, [_vp, _i, _vp, _vp, _i, _vp, _i64, _i, _f, _vp]),
    "q8_rope": (_i, [_vp, _i, _vp, _vp, _vp, _i, _i64, _i, _vp]),
    "q8_fma": (_i, [_vp, _i, _vp, _i, _vp, _i, _vp, _i, _i64, _i, _i64, _i64, _f, _vp]),
    "q8_adaln_rows": (_i, [_vp, _vp, _vp, _i, _i64, _i, _vp]),
    "q8_gelu": (_i, [_vp, _i, _vp, _i, _i64, _vp]),
    "q8_gelu_backward": (_i, [_vp, _i, _vp, _i, _vp, _i, _i64, _vp]),
    "q8_rope_backward": (_i, [_vp, _i, _vp, _vp, _vp, _i, _i64, _i, _vp]),
    "q8_rmsnorm_backward": (_i, [_vp, _i, _vp, _vp, _i, _vp, _vp, _i, _i64, _i, _vp]),
    "q8_fht_quant_rows": (_i, [_vp, _i, _vp, _i, _vp, _i64, _i, _f, _i, _i, _vp]),
    "q8_rmsnorm_quant_rows": (_i, [_vp, _i, _vp, _vp, _i, _vp, _vp, _i64, _i, _f, _i, _i, _vp]),
    "q8_norm_mod_fht_quant_rows": (_i, [_vp, _vp, _i, _vp, _vp, _i, _i64, _f, _i, _f, _vp, _i, _vp, _i64, _i, _i, _vp]),
    "q8_attn_prep_qk": (_i, [_vp, _i64, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _i, _vp]),
    "q8_attn_prep_qk_pair": (_i, [_vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _i, _vp]),
    "q8_attn_prep_qkv": (_i, [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i,
                              _f, _i, _vp]),
    "q8_attn_prep_kv": (_i, [_vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _i, _vp]),
    "q8_attn_prep_v": (_i, [_vp, _i64, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "q8_gemm": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "q8_gemm_residual": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "q8_gemm_gated_residual": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _vp, _i, _i, _i, _i, _i, _vp]),
    "q8_gemm_qkv": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _i, _vp]),
    "q8_gemm_i32": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "q8_gemm_set_config": (_i, [_i]),
    "q8_attn_set_config": (_i, [_i]),
    "q8_gemm_last_kernel": (_i, []),
    "q8_attn_fwd": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i64, _f, _i, _i, _vp]),
}

_lock = threading.Lock()
_lib = None


class Q8Error(RuntimeError):
    """Raised when a libq8_hip entry point returns a negative status."""

    def __init__(self, status, message):
        super().__init__("libq8_hip: %s (status %d)" % (message, status))
        self.status = status


def lib():
    """The loaded shared library with argtypes set; raises if it has not been built."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                if not os.path.exists(LIB_PATH):
                    raise RuntimeError(
                        "libq8_hip.so not found at %s: build it with `python -m q8_kernels_amd.build` "
                        "(there is no fallback path)" % LIB_PATH)
                handle = ctypes.CDLL(LIB_PATH)
                for name, (res, args) in SIGNATURES.items():
                    fn = getattr(handle, name)
                    fn.restype = res
                    fn.argtypes = args
                _lib = handle
    return _lib


def check(status):
    if status != 0:
        l = lib()
        msg = l.q8_last_error().decode() or l.q8_strerror(status).decode()
        raise Q8Error(status, msg)


def device_info():
    cu, mhz, mem = _i(0), _i(0), _i64(0)
    name = ctypes.create_string_buffer(64)
    check(lib().q8_device_info(ctypes.byref(cu), ctypes.byref(mhz), ctypes.byref(mem), name))
    return {"cu_count": cu.value, "clock_mhz": mhz.value, "hbm_bytes": mem.value, "arch": name.value.decode()}
