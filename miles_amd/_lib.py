"""ctypes binding of libmiles_quant.so (the C-ABI HIP library declared in include/miles_quant.h).

The library is built in-tree by `python -m miles_amd.build` (or __graft_entry__.build()).  There is no
fallback: if the shared object is missing or does not load, every quantizer raises.
"""

from __future__ import annotations

import ctypes
import os

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libmiles_quant.so")

MQ_BF16, MQ_F16, MQ_F32 = 0, 1, 2
DTYPE_CODE = {torch.bfloat16: MQ_BF16, torch.float16: MQ_F16, torch.float32: MQ_F32}

_c = ctypes
_vp, _i64, _i32, _f32, _u32 = _c.c_void_p, _c.c_int64, _c.c_int, _c.c_float, _c.c_uint32

# symbol -> argtypes; every function returns int except the two noted below
SIGNATURES = {
    "mq_fp8_block_quant": [_vp, _i32, _i64, _vp, _vp, _i64, _i64, _i32, _i32, _vp],
    "mq_fp8_block_quant_pow2": [_vp, _i32, _i64, _vp, _vp, _i64, _i64, _vp],
    "mq_fp8_blockwise_cast": [_vp, _i32, _i64, _i64, _vp, _vp, _i64, _i64, _i32, _i32, _vp],
    "mq_fp8_scaled_quant": [_vp, _i32, _i64, _vp, _vp, _vp, _i64, _i64, _i32, _f32, _vp],
    "mq_fp8_scaled_quant_static": [_vp, _i32, _i64, _vp, _vp, _i64, _i64, _i32, _f32, _vp],
    "mq_ue8m0_pack_scales": [_vp, _vp, _i64, _i64, _i64, _i64, _i32, _vp],
    "mq_fp8_block_dequant": [_vp, _vp, _vp, _i64, _i64, _i32, _vp],
    "mq_mxfp8_quant": [_vp, _i32, _vp, _vp, _i64, _i64, _vp],
    "mq_e8m0_bytes_to_f32": [_vp, _vp, _i64, _vp],
    "mq_fp8_scales_pow2_flag": [_vp, _i64, _i64, _i64, _vp, _vp],
    "mq_e8m0_expand_tile_scales": [_vp, _i32, _i64, _vp, _i64, _i64, _vp],
    "mq_fp8_block_to_mxfp8": [_vp, _vp, _i64, _vp, _vp, _i64, _i64, _vp],
    "mq_int4_fake_quant": [_vp, _i32, _vp, _vp, _vp, _i64, _i64, _i32, _i32, _i32, _vp],
    "mq_int4_unpack_dequant": [_vp, _vp, _i32, _vp, _i64, _i64, _i32, _vp],
    "mq_mxfp4_to_fp8_block": [_vp, _vp, _vp, _vp, _i64, _i64, _vp],
    "mq_fake_quant": [_vp, _i32, _vp, _i64, _i32, _vp],
    "mq_fp8_act_quant": [_vp, _i32, _vp, _vp, _i64, _i32, _i32, _vp],
    "mq_mxfp4_quant": [_vp, _i32, _vp, _vp, _i64, _i32, _vp],
    "mq_mxfp4_dequant": [_vp, _vp, _vp, _i64, _i32, _vp],
    "mq_int4_group_quant_pack": [_vp, _i32, _vp, _vp, _i64, _i64, _i32, _vp],
    "mq_int4_group_quant_pack_asym": [_vp, _i32, _vp, _vp, _vp, _vp, _i64, _i64, _i32, _vp],
    "mq_fill_u32": [_vp, _u32, _i64, _vp],
    "mq_nvfp4_amax": [_vp, _i32, _i64, _vp, _i32, _vp],
    "mq_nvfp4_quant": [_vp, _i32, _vp, _i32, _vp, _vp, _vp, _i64, _i64, _i32, _i32, _vp],
    "mq_nvfp4_fold": [_vp, _i32, _i32, _vp],
    "mq_nvfp4_qdq": [_vp, _i32, _vp, _vp, _i64, _i32, _i32, _vp],
    "mq_run_jobs": [_vp, _i64, _vp],
    "mq_tune_tile_launch_tiles": [_i64, _vp],
    "mq_job_table_fill": [_vp, _i64, _vp],
    "mq_run_jobs_tabled": [_vp, _i64, _vp, _vp],
    "mq_run_jobs_feedback": [_vp, _i64, _vp, _vp, _vp, _vp],
}

MAX_GROUP = 64                                            # MQ_MAX_GROUP: tensors per fused launch of mq_run_jobs
TABLE_ENTRY_BYTES, TABLE_GROUP = 56, 8192                 # MQ_JOB_TABLE_ENTRY_BYTES, MQ_TABLE_GROUP (mq_run_jobs_tabled)
NVFP4_4OVER6, NVFP4_ERR_MSE, NVFP4_ERR_FP16 = 1, 2, 4     # flags of mq_nvfp4_quant / mq_nvfp4_qdq
NVFP4_CARRY_AMAX = 8                                      # MQ_NVFP4_CARRY_AMAX: NVFP4 jobs of a re-submitted list only
# words of an amax record behind its four sections of 256 partial maxima (MQ_NVFP4_RECORD_*_WORD)
RECORD_AMAX_WORD, RECORD_REDO_WORD, RECORD_VOLATILE_WORD = 1024, 1028, 1029

(JOB_FP8_BLOCK, JOB_FP8_BLOCKWISE_CAST, JOB_FP8_DEQUANT, JOB_MXFP8, JOB_INT4_PACK, JOB_NVFP4, JOB_MXFP4,
 JOB_COPY, JOB_FP8_BLOCK_POW2, JOB_UE8M0_PACK, JOB_FP8_TENSOR, JOB_INT4_PACK_ASYM, JOB_MXFP4_TO_FP8,
 JOB_FP8_TO_MXFP8, JOB_E8M0_EXPAND, JOB_INT4_UNPACK, JOB_MXFP4_DEQUANT) = range(17)


class Job(_c.Structure):
    """struct mq_job of include/miles_quant.h"""

    _fields_ = [("kind", _c.c_int32), ("dtype", _c.c_int32), ("inp", _vp), ("out", _vp), ("scale", _vp),
                ("aux", _vp), ("aux2", _vp), ("rows", _i64), ("cols", _i64), ("ld", _i64), ("p0", _c.c_int32),
                ("p1", _c.c_int32), ("rows_per_block", _i64), ("block_stride", _i64)]


_lib = None


class MilesQuantError(RuntimeError):
    pass


def lib_path() -> str:
    return _LIB_PATH


def load() -> ctypes.CDLL:
    """Load the HIP library or raise; never falls back to another implementation."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise MilesQuantError(
            f"{_LIB_PATH} is missing: build it with `python -m miles_amd.build` (hipcc, gfx950). "
            "miles_amd has no CPU or PyTorch fallback for its quantizers."
        )
    lib = ctypes.CDLL(_LIB_PATH)
    lib.mq_version.restype = _i32
    lib.mq_version.argtypes = []
    lib.mq_last_error.restype = _c.c_char_p
    lib.mq_last_error.argtypes = []
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = _i32
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(rc: int, exc=MilesQuantError) -> None:
    if rc != 0:
        raise exc(load().mq_last_error().decode() or f"libmiles_quant error {rc}")


def stream_ptr(device: torch.device | None = None) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def require_gpu(t: torch.Tensor, what: str) -> None:
    if t.device.type != "cuda":
        raise MilesQuantError(f"{what}: expected a tensor on the GPU, got device {t.device}; "
                              "miles_amd runs its quantizers on the HIP library only")


def dtype_code(t: torch.Tensor, what: str) -> int:
    try:
        return DTYPE_CODE[t.dtype]
    except KeyError:
        raise MilesQuantError(f"{what}: unsupported dtype {t.dtype}") from None
