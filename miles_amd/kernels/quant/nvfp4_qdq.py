"""Fused NVFP4 quantize-dequantize ("fake quantization") for quantization-aware training.

Mirror of the public surface of the reference's `miles/kernels/quant/nvfp4_qdq.py` (`__all__`, :1259-1266):
`NVFP4QDQConfig` / `NVFP4QDQErrorMode` (:48-74), `current_nvfp4_qdq_config` (:93-117), `compute_nvfp4_amax`
(:1213-1217), `fused_nvfp4_qdq` (:1220-1229) and `fake_nvfp4_quantization_ste` (:1248-1256).  The reference builds a
CuTe-DSL kernel for Blackwell; here the contract is one gfx950 kernel and the amax is
the two-kernel reduction of the NVFP4 quantizer.  Four Over Six (MAE / MSE, fp32 / fp16 candidate error) is a
second instantiation of the same kernel.
"""

from __future__ import annotations

import os
from dataclasses import dataclass
from enum import IntEnum

import torch

from miles_amd import _lib, launch

_FP4_BLOCK_SIZE = 16

_RECORD_WORDS = 1280     # MQ_NVFP4_RECORD_WORDS; the folded amax sits in word 1024


class NVFP4QDQErrorMode(IntEnum):
    """Four Over Six candidate error metric."""

    MAE = 0
    MSE = 1


@dataclass(frozen=True)
class NVFP4QDQConfig:
    """Numerical contract of the fused kernel (field names and checks of the reference's dataclass)."""

    use_4over6: bool = False
    e4m3_max: int = 448
    error_mode: NVFP4QDQErrorMode = NVFP4QDQErrorMode.MAE
    error_use_fast_math: bool = False

    def __post_init__(self) -> None:
        if self.e4m3_max not in (256, 448):
            raise ValueError(f"NVFP4 E4M3 max must be 256 or 448, got {self.e4m3_max}.")
        if not self.use_4over6 and self.e4m3_max != 448:
            raise ValueError("E4M3 max 256 is only supported by Four Over Six.")
        if not self.use_4over6 and self.error_use_fast_math:
            raise ValueError("The FP16 error contract only applies to Four Over Six.")


def _flag(name: str, default: str = "0") -> bool:
    value = os.getenv(name, default).strip()
    if value in ("0", "", "1"):
        return value == "1"
    raise ValueError(f"{name} must be 0 or 1, got {value!r}.")


def _covers_weights(name: str, default: str) -> bool:
    value = os.getenv(name, default).strip().lower()
    if value not in ("none", "weights", "activations", "all"):
        raise ValueError(f"{name} must be one of none, weights, activations, or all; got {value!r}.")
    return value in ("weights", "all")


def current_nvfp4_qdq_config() -> NVFP4QDQConfig:
    """The weight QDQ contract selected by Transformer Engine's environment variables."""
    if _flag("NVTE_USE_FAST_MATH"):
        raise ValueError("Fused NVFP4 QDQ requires NVTE_USE_FAST_MATH=0; ordinary quant fast math "
                         "is outside its numerical contract.")
    use_4over6 = _covers_weights("NVTE_NVFP4_4OVER6", "none")
    use_256 = _covers_weights("NVTE_NVFP4_4OVER6_E4M3_USE_256", "all")
    mode_name = os.getenv("NVTE_NVFP4_4OVER6_ERR_MODE", "MAE").strip().upper()
    if mode_name not in NVFP4QDQErrorMode.__members__:
        raise ValueError(f"NVTE_NVFP4_4OVER6_ERR_MODE must be MAE or MSE, got {mode_name!r}.")
    fp16_error = _flag("NVTE_NVFP4_4OVER6_ERR_USE_FAST_MATH")
    return NVFP4QDQConfig(use_4over6=use_4over6, e4m3_max=256 if use_4over6 and use_256 else 448,
                          error_mode=NVFP4QDQErrorMode[mode_name], error_use_fast_math=use_4over6 and fp16_error)


def compute_nvfp4_amax(x: torch.Tensor) -> torch.Tensor:
    """FP32 0-dim tensor max|x| (the reference uses torch.linalg.vector_norm(x, inf)); stays on the device."""
    if x.numel() == 0:
        raise ValueError("Cannot compute NVFP4 amax for an empty tensor.")
    _lib.require_gpu(x, "compute_nvfp4_amax")
    xc = x.detach().contiguous()
    record = torch.empty(_RECORD_WORDS, dtype=torch.int32, device=xc.device)
    lib, stream = _lib.load(), _lib.stream_ptr(xc.device)
    launch.note_direct_call()
    _lib.check(lib.mq_nvfp4_amax(xc.data_ptr(), _lib.dtype_code(xc, "compute_nvfp4_amax"), xc.numel(), record.data_ptr(), 0, stream))
    _lib.check(lib.mq_nvfp4_fold(record.data_ptr(), 1, 448, stream))
    return record[1024:1025].view(torch.float32).reshape(())


def _validate_input(x: torch.Tensor, amax: torch.Tensor) -> None:
    """Checks and error types of the reference (:1128-1156), minus its SM10x and int32-size limits."""
    if not x.is_cuda:
        raise ValueError("Fused NVFP4 QDQ requires a CUDA tensor.")
    if x.dtype not in (torch.bfloat16, torch.float16):
        raise TypeError(f"Fused NVFP4 QDQ supports BF16 and FP16, got {x.dtype}.")
    if x.ndim != 2:
        raise ValueError(f"Fused NVFP4 QDQ requires a rank-2 tensor, got shape {tuple(x.shape)}.")
    if not x.is_contiguous():
        raise ValueError("Fused NVFP4 QDQ requires a contiguous tensor.")
    if x.data_ptr() % 16 != 0:
        raise ValueError("Fused NVFP4 QDQ requires a 16-byte-aligned input tensor.")
    if x.shape[1] % _FP4_BLOCK_SIZE != 0:
        raise ValueError(f"Fused NVFP4 QDQ requires K divisible by {_FP4_BLOCK_SIZE}, got {x.shape[1]}.")
    if x.numel() == 0:
        raise ValueError("Fused NVFP4 QDQ does not support empty tensors.")
    if not amax.is_cuda or amax.device != x.device:
        raise ValueError("The FP32 per-tensor amax must be on the input tensor's CUDA device.")
    if amax.dtype != torch.float32 or amax.numel() != 1:
        raise TypeError("The per-tensor amax must contain exactly one FP32 value.")


def fused_nvfp4_qdq(x: torch.Tensor, amax: torch.Tensor, config: NVFP4QDQConfig | None = None) -> torch.Tensor:
    """Quantize to NVFP4 and dequantize again in registers; returns a detached tensor in the dtype of x."""
    if config is None:
        config = current_nvfp4_qdq_config()
    _validate_input(x, amax)
    flags = 0
    if config.use_4over6:
        flags = _lib.NVFP4_4OVER6 | (_lib.NVFP4_ERR_MSE if config.error_mode == NVFP4QDQErrorMode.MSE else 0) \
            | (_lib.NVFP4_ERR_FP16 if config.error_use_fast_math else 0)
    out = torch.empty_like(x)
    launch.note_direct_call()
    rc = _lib.load().mq_nvfp4_qdq(x.detach().data_ptr(), _lib.dtype_code(x, "fused_nvfp4_qdq"), amax.detach().data_ptr(),
                                  out.data_ptr(), x.numel(), config.e4m3_max, flags, _lib.stream_ptr(x.device))
    _lib.check(rc)
    return out


class _QDQStraightThrough(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, amax, config):
        return fused_nvfp4_qdq(x, amax, config)

    @staticmethod
    def backward(ctx, grad_output):
        return grad_output, None, None


def fake_nvfp4_quantization_ste(x: torch.Tensor, config: NVFP4QDQConfig | None = None) -> torch.Tensor:
    """NVFP4 QDQ forward, identity backward; a Megatron `main_grad` attribute follows the output."""
    if config is None:
        config = current_nvfp4_qdq_config()
    output = _QDQStraightThrough.apply(x, compute_nvfp4_amax(x), config)
    if hasattr(x, "main_grad"):
        output.main_grad = x.main_grad
    return output


__all__ = ["NVFP4QDQConfig", "NVFP4QDQErrorMode", "compute_nvfp4_amax", "current_nvfp4_qdq_config",
           "fake_nvfp4_quantization_ste", "fused_nvfp4_qdq"]
