"""ctypes binding of the kernel C-ABI (include/mhip.h).

There is no fallback: if ``libmetalhlo_hip.so`` is missing or a symbol cannot be
resolved, importing callers get an ImportError naming the build command.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libmetalhlo_hip.so")

_i64, _i32, _f32, _vp = C.c_int64, C.c_int, C.c_float, C.c_void_p

# name -> (restype, argtypes); mirrors include/mhip.h one to one.
SIGNATURES = {
    "mhip_version": (C.c_char_p, []),
    "mhip_last_error": (C.c_char_p, []),
    "mhip_device_count": (_i32, []),
    "mhip_device_info": (_i32, [_i32, C.POINTER(_i32), C.POINTER(_i32), C.c_char_p, C.c_size_t]),
    "mhip_softmax": (_i32, [_vp, _vp, _vp, _i64, _i64, _i32]),
    "mhip_softmax_strided": (_i32, [_vp, _vp, _vp, _i64, _i64, _i64, _i32]),
    "mhip_layer_norm": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _f32, _i32]),
    "mhip_rms_norm": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _f32, _i32]),
    "mhip_bias_gelu": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i32]),
    "mhip_bias_gelu_erf": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i32]),
    "mhip_gemm": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64,
                         _i32, _i32, _i32, _i32]),
    "mhip_gemm_residual": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64,
                                  _i32, _i32, _i32, _i32]),
    "mhip_flash_attention": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64,
                                    _f32, _i32, _i64, _i64, _i32]),
    "mhip_flash_attention_strided": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64,
                                            _f32, _i32, _i64, _i64, _i32, _vp]),
    "mhip_copy": (_i32, [_vp, _vp, _vp, _i64]),
    "mhip_gather_rows": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _i32]),
    "mhip_embed_tokens": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i32, _i32]),
    "mhip_add": (_i32, [_vp, _vp, _vp, _vp, _i64, _i32]),
    "mhip_convert": (_i32, [_vp, _vp, _vp, _i64, _i32, _i32]),
    "mhip_convert_batch": (_i32, [_vp, _i32, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_i64), _i32, _i32]),
    "mhip_transpose_0213": (_i32, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i32]),
    "mhip_split_qkv_heads": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i32]),
    "mhip_rope": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _i32]),
    "mhip_batch_norm": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _f32, _i32]),
    "mhip_depth_attention": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _f32, _i32]),
    "mhip_elementwise_chain": (_i32, [_vp, _i32, C.POINTER(_vp), C.POINTER(_i64), _i32, C.POINTER(_i32), _vp, _i64, _i32]),
    "mhip_iota": (_i32, [_vp, _vp, _i64, _i64, _i64, _i32]),
    "mhip_unary": (_i32, [_vp, _i32, _vp, _vp, _i64, _i32]),
    "mhip_binary": (_i32, [_vp, _i32, _vp, _vp, _vp, _i64, _i32]),
    "mhip_compare": (_i32, [_vp, _i32, _vp, _vp, _vp, _i64, _i32]),
    "mhip_select": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i32, _i32]),
    "mhip_strided_copy": (_i32, [_vp, _vp, _vp, _i32, C.POINTER(_i64), C.POINTER(_i64), _i64, _i32]),
    "mhip_gather": (_i32, [_vp, _vp, _vp, _vp, _i32, C.POINTER(_i64), C.POINTER(_i64), C.POINTER(_i64), _i32, _i64,
                           C.POINTER(_i64), C.POINTER(_i64), _i32, _i32]),
    "mhip_reduce": (_i32, [_vp, _i32, _vp, _vp, _i64, _i64, _i64, C.c_double, _i32]),
    "mhip_fill": (_i32, [_vp, _vp, _i64, C.c_uint64, _i32]),
    "mhip_argmax": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i32, _i32]),
    "mhip_gemm_autotune_in_model": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _i32, _i32,
                                           _i32, _i32, _vp, _i64, C.POINTER(C.c_int), C.POINTER(C.c_float)]),
    "mhip_tuning_set_gemm": (_i32, [_i64, _i64, _i64, _i64, _i32, _i32, _i32, _i32, C.c_float]),
    "mhip_gemm_last_variant": (_i32, []),
    "mhip_gemm_autotune": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _i32, _i32,
                                  _i32, _i32, C.POINTER(C.c_int), C.POINTER(C.c_float)]),
    "mhip_row_autotune": (_i32, [_vp, _i32, _vp, _vp, _vp, _vp, _i64, _i64, C.c_float, _i32, _i32, C.POINTER(C.c_int),
                                 C.POINTER(C.c_float)]),
    "mhip_attention_autotune": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, C.c_float, _i32, _i32, _i32,
                                       C.POINTER(C.c_int), C.POINTER(C.c_float)]),
    "mhip_tuning_save": (_i32, [C.c_char_p]),
    "mhip_tuning_load": (_i32, [C.c_char_p]),
    "mhip_tuning_clear": (None, []),
    "mhip_tuning_count": (_i32, []),
    "mhip_tuning_device": (C.c_char_p, []),
}

_lib = None


def load() -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is not built; run `python -m metalhlo_amd.build` "
            "(hipcc cross-compiles gfx950 without a GPU)")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as e:
            raise ImportError(f"{LIB_PATH} does not export {name}; rebuild it") from e
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


class MhipError(RuntimeError):
    def __init__(self, code: int, msg: str):
        super().__init__(f"mhip status {code}: {msg}")
        self.code = code


def check(code: int) -> None:
    if code != 0:
        raise MhipError(code, load().mhip_last_error().decode("utf-8", "replace"))
