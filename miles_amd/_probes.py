"""ctypes binding of libmq_probes.so (declared in include/miles_quant_probes.h): device self-tests of the gfx950
instructions the kernels rely on, a plain copy and the streaming probes.  Loaded by the GPU tests and by bench.py only;
nothing on the product path imports this module."""

from __future__ import annotations

import ctypes
import os

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libmq_probes.so")

_c = ctypes
_vp, _i64, _i32 = _c.c_void_p, _c.c_int64, _c.c_int

SIGNATURES = {
    "mqp_selftest_convert": [_vp, _vp],
    "mqp_selftest_reciprocal": [_vp, _vp],
    "mqp_copy_bytes": [_vp, _vp, _i64, _vp],
    "mqp_stream_probe": [_i32, _vp, _vp, _i64, _i64, _vp],
}
FLAT_2_1, FLAT_1_2, LOOP_2_1, TILE_2_1, TILE_READ, TILE_WRITE = range(6)      # MQP_* shapes of mqp_stream_probe

_lib = None


def lib_path() -> str:
    return _LIB_PATH


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(f"{_LIB_PATH} is missing: build it with `python -m miles_amd.build`")
        lib = ctypes.CDLL(_LIB_PATH)
        lib.mqp_last_error.restype = _c.c_char_p
        lib.mqp_last_error.argtypes = []
        for name, argtypes in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = _i32
            fn.argtypes = argtypes
        _lib = lib
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        raise RuntimeError(load().mqp_last_error().decode() or f"libmq_probes error {rc}")
