"""Block-wise FP8 quantization of activations (1 x block groups of the last dimension), DeepSeek-V4 style.

Mirror of the reference's `miles/kernels/quant/fp8_act_quant.py`: `act_quant` (:110-137) with the same arguments
and return values, and of the quantize / cast-back simulation built on it in
`miles_plugins/models/deepseek_v4/ops/qat.py` (`fp8_simulate` :8-23, `fp8_simulate_qat` :26-36).  The reference's
TileLang kernel (:49-107) is one gfx950 kernel here; with `inplace=True` (and in `fp8_simulate`) quantization and the
cast back happen in the same pass.
"""

from __future__ import annotations

import torch

from miles_amd import _lib, launch

ACT_ROUND_SCALE, ACT_SCALE_E8M0, ACT_INPLACE = 1, 2, 4     # flags of mq_fp8_act_quant


def _run(z: torch.Tensor, y: torch.Tensor, s: torch.Tensor, block_size: int, flags: int) -> None:
    launch.note_direct_call()
    rc = _lib.load().mq_fp8_act_quant(z.data_ptr(), _lib.dtype_code(z, "act_quant"), y.data_ptr(), s.data_ptr(),
                                      z.numel(), int(block_size), flags, _lib.stream_ptr(z.device))
    _lib.check(rc)


def act_quant(x: torch.Tensor, block_size: int = 128, scale_fmt: str | None = None,
              scale_dtype: torch.dtype = torch.float32, inplace: bool = False):
    """Returns `(y, s)`: float8_e4m3fn codes shaped like x and one scale per group, `[..., N / block_size]` in
    `scale_dtype` (float32 or float8_e8m0fnu).  When `scale_fmt` is set the scales are rounded up to powers of two.
    `inplace=True` overwrites x with the quantize-dequantize result and returns x."""
    n = x.size(-1)
    assert n % block_size == 0
    _lib.require_gpu(x, "act_quant")
    e8m0 = scale_dtype == torch.float8_e8m0fnu
    if scale_dtype not in (torch.float32, torch.float8_e8m0fnu):
        raise ValueError(f"act_quant scales are float32 or float8_e8m0fnu, got {scale_dtype}")
    if e8m0 and scale_fmt is None:
        raise ValueError("float8_e8m0fnu scales need scale_fmt (power-of-two scales)")
    flags = (ACT_ROUND_SCALE if scale_fmt is not None else 0) | (ACT_SCALE_E8M0 if e8m0 else 0)
    z = x.contiguous()
    s = z.new_empty(*z.size()[:-1], n // block_size, dtype=scale_dtype)
    if inplace:
        _run(z, z, s, block_size, flags | ACT_INPLACE)
        if z is not x:
            x.copy_(z)
        return x
    y = torch.empty_like(z, dtype=torch.float8_e4m3fn)
    _run(z, y, s, block_size, flags)
    return y, s


def fp8_simulate(x: torch.Tensor, block_size: int) -> torch.Tensor:
    """Per-token FP8 (e4m3) cast and cast back with power-of-two (UE8M0) scales; x is left untouched."""
    _lib.require_gpu(x, "fp8_simulate")
    assert x.size(-1) % block_size == 0
    z = x.contiguous()
    out = torch.empty_like(z)
    s = z.new_empty(*z.size()[:-1], z.size(-1) // block_size, dtype=torch.float32)
    _run(z, out, s, block_size, ACT_ROUND_SCALE | ACT_INPLACE)
    return out


class DeepSeekV4LinearQATFunc(torch.autograd.Function):
    """`fp8_simulate` forward, identity backward."""

    @staticmethod
    def forward(ctx, kv, block_size=128):
        return fp8_simulate(kv, block_size)

    @staticmethod
    def backward(ctx, grad_kv):
        return grad_kv, None


fp8_simulate_qat = DeepSeekV4LinearQATFunc.apply
