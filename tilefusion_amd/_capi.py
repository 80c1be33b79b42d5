"""ctypes view of the C ABI in include/tilefusion_c.h (libtilefusion_hip.so).

The library is built in-tree by `make -C tilefusion_amd/csrc` (or __graft_entry__.build()).
There is no CPU fallback: loading fails loudly when the library is missing.
"""

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtilefusion_hip.so")

TF_OK, TF_ERR_INVALID_ARG, TF_ERR_UNSUPPORTED, TF_ERR_LDS, TF_ERR_HIP = range(5)
TF_DTYPE_F32, TF_DTYPE_F16, TF_DTYPE_BF16 = range(3)

_vp, _i, _i64, _d, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_double, ctypes.c_size_t

# name -> (restype, argtypes); every symbol include/tilefusion_c.h declares
SIGNATURES = {
    "tf_gemm_f16": (_i, [_vp, _vp, _vp, _i, _i64, _i64, _i64, _i, _i, _i, _i, _i, _vp]),
    "tf_fused_two_gemms_f16": (_i, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i, _i, _i, _i, _vp]),
    "tf_flash_attention_fwd_f16": (_i, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i, _i, _i, _i, _i, _d, _i, _vp]),
    "tf_gemm": (_i, [_vp, _vp, _vp, _i, _i, _i64, _i64, _i64, _i, _i, _i, _i, _i, _vp]),
    "tf_fused_two_gemms": (_i, [_vp, _vp, _vp, _vp, _i, _i64, _i64, _i64, _i64, _i64, _i, _i, _i, _i, _vp]),
    "tf_fused_two_gemms_workspace_bytes": (_sz, [_i, _i64, _i64, _i64, _i64, _i64]),
    "tf_fused_two_gemms_ws": (_i, [_vp, _vp, _vp, _vp, _i, _i64, _i64, _i64, _i64, _i64, _i, _i, _i, _i, _vp, _sz, _vp]),
    "tf_flash_attention_fwd": (_i, [_vp, _vp, _vp, _vp, _i, _i64, _i64, _i64, _i64, _i64, _i, _i, _i, _i, _i, _d, _i, _vp]),
    "tf_flash_decode_workspace_bytes": (_sz, [_i64, _i64, _i]),
    "tf_flash_decode_f16": (_i, [_vp, _vp, _vp, _vp, _vp, _sz, _i64, _i64, _i64, _i, _d, _vp]),
    "tf_flash_decode": (_i, [_vp, _vp, _vp, _vp, _i, _vp, _sz, _i64, _i64, _i64, _i, _d, _vp]),
    "tf_flash_decode_static_max_partials": (_sz, []),
    "tf_flash_decode_static_prepare": (_i, []),
    "tf_flash_decode_static_f16": (_i, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i, _d, _vp]),
    "tf_scatter_nd": (_i, [_vp, _vp, _vp, ctypes.POINTER(_i64), _i, _i64, _i, _i, _vp]),
    "tf_jit_compile": (_i, [ctypes.c_char_p, ctypes.c_char_p, ctypes.POINTER(ctypes.c_char_p), _i,
                            ctypes.POINTER(ctypes.c_char_p), _i, ctypes.POINTER(_vp)]),
    "tf_jit_launch": (_i, [_vp] + [ctypes.c_uint] * 7 + [_vp, ctypes.POINTER(_vp)]),
    "tf_jit_clear_cache": (_i, []),
    "tf_jit_cache_dir": (ctypes.c_char_p, []),
    "tf_last_error": (ctypes.c_char_p, []),
    "tf_version": (ctypes.c_char_p, []),
}

_lib = None


def load():
    """Load libtilefusion_hip.so once and attach the argument types."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C tilefusion_amd/csrc` "
                "(there is no CPU fallback)")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def check(status, what):
    """Turn a non-zero status of the C ABI into a RuntimeError carrying tf_last_error()."""
    if status != TF_OK:
        msg = load().tf_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what} failed (status {status}): {msg}")
