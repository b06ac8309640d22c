"""ctypes view of libCMetalHLO.so (include/metalhlo.h) for tests and examples."""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libCMetalHLO.so")

ELEMENT_TYPE = {"f16": 0, "f32": 1, "f64": 2, "bf16": 3, "i1": 4, "i8": 5, "i16": 6, "i32": 7, "i64": 8,
                "ui8": 9, "ui16": 10, "ui32": 11, "ui64": 12}
NUMPY_OF = {1: np.float32, 2: np.float64, 0: np.float16, 3: np.uint16, 4: np.uint8, 5: np.int8, 6: np.int16,
            7: np.int32, 8: np.int64, 9: np.uint8, 10: np.uint16, 11: np.uint32, 12: np.uint64}


class CompileConfig(C.Structure):
    _fields_ = [("optimization_level", C.c_int), ("enable_caching", C.c_bool), ("enable_debug_info", C.c_bool),
                ("device_policy", C.c_int)]


class ExecutionStats(C.Structure):
    _fields_ = [("execution_count", C.c_int64), ("total_execution_time_ms", C.c_double),
                ("last_execution_time_ms", C.c_double), ("average_execution_time_ms", C.c_double)]


class ExecutionProfile(C.Structure):
    _fields_ = [("partition_count", C.c_int32), ("gpu_partition_count", C.c_int32), ("ane_partition_count", C.c_int32),
                ("gpu_time_ms", C.c_double), ("ane_time_ms", C.c_double), ("transfer_time_ms", C.c_double),
                ("total_time_ms", C.c_double), ("used_ane", C.c_bool)]


_vp, _i32, _i64p = C.c_void_p, C.c_int32, C.POINTER(C.c_int64)
SIGNATURES = {
    "mhlo_version": (C.c_char_p, []),
    "mhlo_get_last_error": (C.c_char_p, []),
    "mhlo_clear_error": (None, []),
    "mhlo_element_type_size": (C.c_size_t, [C.c_int]),
    "mhlo_client_create": (C.c_int, [C.POINTER(_vp)]),
    "mhlo_client_destroy": (None, [_vp]),
    "mhlo_client_device_name": (_vp, [_vp]),
    "mhlo_compile_config_init": (None, [C.POINTER(CompileConfig)]),
    "mhlo_ane_available": (C.c_bool, []),
    "mhlo_compile": (C.c_int, [_vp, C.c_char_p, C.POINTER(_vp)]),
    "mhlo_compile_n": (C.c_int, [_vp, C.c_char_p, C.c_size_t, C.POINTER(_vp)]),
    "mhlo_compile_with_config": (C.c_int, [_vp, C.c_char_p, C.POINTER(CompileConfig), C.POINTER(_vp)]),
    "mhlo_executable_destroy": (None, [_vp]),
    "mhlo_executable_input_count": (_i32, [_vp]),
    "mhlo_executable_output_count": (_i32, [_vp]),
    "mhlo_executable_input_type": (C.c_int, [_vp, _i32, _i64p, C.POINTER(_i32), C.POINTER(C.c_int)]),
    "mhlo_executable_output_type": (C.c_int, [_vp, _i32, _i64p, C.POINTER(_i32), C.POINTER(C.c_int)]),
    "mhlo_executable_get_stats": (C.c_int, [_vp, C.POINTER(ExecutionStats)]),
    "mhlo_executable_reset_stats": (None, [_vp]),
    "mhlo_buffer_create": (C.c_int, [_vp, _vp, C.c_size_t, _i64p, _i32, C.c_int, C.POINTER(_vp)]),
    "mhlo_buffer_create_uninitialized": (C.c_int, [_vp, _i64p, _i32, C.c_int, C.POINTER(_vp)]),
    "mhlo_buffer_destroy": (None, [_vp]),
    "mhlo_buffer_shape": (None, [_vp, _i64p, C.POINTER(_i32)]),
    "mhlo_buffer_rank": (_i32, [_vp]),
    "mhlo_buffer_element_type": (C.c_int, [_vp]),
    "mhlo_buffer_byte_count": (C.c_size_t, [_vp]),
    "mhlo_buffer_to_host": (C.c_int, [_vp, _vp, C.c_size_t]),
    "mhlo_execute": (C.c_int, [_vp, C.POINTER(_vp), _i32, C.POINTER(_vp), C.POINTER(_i32)]),
    "mhlo_execute_with_timing": (C.c_int, [_vp, C.POINTER(_vp), _i32, C.POINTER(_vp), C.POINTER(_i32),
                                           C.POINTER(C.c_double), C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "mhlo_execute_with_profile": (C.c_int, [_vp, C.POINTER(_vp), _i32, C.POINTER(_vp), C.POINTER(_i32),
                                            C.POINTER(ExecutionProfile)]),
    "mhlo_free_string": (None, [_vp]),
    "mhlo_ext_executable_ops": (_vp, [_vp]),     # extension: op list after pattern recognition
    "mhlo_ext_executable_plan": (_vp, [_vp]),    # extension: memory plan and launch statistics
    "mhlo_ext_executable_profile": (_vp, [_vp]), # extension: per-operation device time of the last profiled execution
}

_lib = None


def load() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is not built; run `python -m metalhlo_amd.build`")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


class MHLOError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"mhlo status {code}: {msg}")
        self.code = code


def _check(code):
    if code != 0:
        msg = load().mhlo_get_last_error()
        raise MHLOError(code, msg.decode() if msg else "")


class Session:
    """Small convenience wrapper: compile text, run numpy arrays through it."""

    def __init__(self):
        self.lib = load()
        self.client = _vp()
        _check(self.lib.mhlo_client_create(C.byref(self.client)))

    def close(self):
        if self.client:
            self.lib.mhlo_client_destroy(self.client)
            self.client = _vp()

    def compile(self, mlir: str, opt_level: int = None):
        exe = _vp()
        if opt_level is None:
            _check(self.lib.mhlo_compile(self.client, mlir.encode(), C.byref(exe)))
        else:
            cfg = CompileConfig()
            self.lib.mhlo_compile_config_init(C.byref(cfg))
            cfg.optimization_level = opt_level
            _check(self.lib.mhlo_compile_with_config(self.client, mlir.encode(), C.byref(cfg), C.byref(exe)))
        return exe

    def ops(self, exe):
        """Names of the operations the executable runs (custom calls by target)."""
        p = self.lib.mhlo_ext_executable_ops(exe)
        try:
            return C.string_at(p).decode().split(",") if p else []
        finally:
            self.lib.mhlo_free_string(p)

    def plan(self, exe) -> dict:
        """Memory plan and launch statistics of an executable (integers by name)."""
        p = self.lib.mhlo_ext_executable_plan(exe)
        try:
            return {k: int(v) for k, v in (kv.split("=") for kv in C.string_at(p).decode().split(","))} if p else {}
        finally:
            self.lib.mhlo_free_string(p)

    def profile(self, exe) -> list:
        """(operation, result shape, microseconds) of the last profiled execution."""
        p = self.lib.mhlo_ext_executable_profile(exe)
        try:
            lines = C.string_at(p).decode().splitlines() if p else []
        finally:
            self.lib.mhlo_free_string(p)
        out = []
        for ln in lines:
            name, shape, us = ln.rsplit(" ", 2)
            out.append((name, shape, float(us)))
        return out

    def buffer(self, array: np.ndarray, element_type: str):
        a = np.asarray(array)
        if not a.flags.c_contiguous:
            a = np.ascontiguousarray(a)
        shape = (C.c_int64 * max(a.ndim, 1))(*a.shape)      # (a rank-0 array stays rank 0)
        buf = _vp()
        _check(self.lib.mhlo_buffer_create(self.client, a.ctypes.data_as(_vp), a.nbytes, shape, a.ndim,
                                           ELEMENT_TYPE[element_type], C.byref(buf)))
        return buf

    def to_numpy(self, buf) -> np.ndarray:
        rank = self.lib.mhlo_buffer_rank(buf)
        shape = (C.c_int64 * max(rank, 1))()
        r = _i32()
        self.lib.mhlo_buffer_shape(buf, shape, C.byref(r))
        et = self.lib.mhlo_buffer_element_type(buf)
        out = np.empty([shape[i] for i in range(rank)], dtype=NUMPY_OF[et])
        _check(self.lib.mhlo_buffer_to_host(buf, out.ctypes.data_as(_vp), out.nbytes))
        return out

    def run(self, exe, inputs):
        """inputs: list of (numpy array, element type name). Returns numpy arrays
        (bf16 comes back as its uint16 bit pattern)."""
        bufs = [self.buffer(a, t) for a, t in inputs]
        n_out = self.lib.mhlo_executable_output_count(exe)
        outs = (_vp * max(n_out, 1))()
        got = _i32()
        arr = (_vp * max(len(bufs), 1))(*bufs)
        try:
            _check(self.lib.mhlo_execute(exe, arr, len(bufs), outs, C.byref(got)))
            res = [self.to_numpy(outs[i]) for i in range(got.value)]
            for i in range(got.value):
                self.lib.mhlo_buffer_destroy(outs[i])
            return res
        finally:
            for b in bufs:
                self.lib.mhlo_buffer_destroy(b)
