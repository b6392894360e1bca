"""Block fake quantization for quantization-aware training: values are rounded to the low-precision grid and
returned in the input dtype; the backward pass is the identity (straight-through).

Mirror of the reference's `miles/kernels/quant/fake_quant.py`: `fake_quant_fp8_forward` / `fake_quant_fp4_forward`
/ `fake_quant_compressed_kv_forward` (:90-99) and the autograd wrappers `fake_quant_fp8` / `fake_quant_fp4` /
`fake_quant_compressed_kv` (:102-124).  The reference's Triton kernel (:25-63) is one gfx950 kernel here.
"""

from __future__ import annotations

import torch

from miles_amd import _lib, launch

FP8_MAX = 448.0
FP4_MAX = 6.0
BLOCK_SIZE = 32
COMPRESSED_KV_BLOCK_SIZE = 16
FP8_AMAX_FLOOR = 1e-4
FP4_AMAX_FLOOR = 6 * 2.0**-126
COMPRESSED_KV_SCALE_MIN = 2.0**-9

_MODE_FP8, _MODE_FP4, _MODE_COMPRESSED_KV = 0, 1, 2


def _fake_quant(x: torch.Tensor, fp4: bool, compressed_kv: bool = False) -> torch.Tensor:
    block = COMPRESSED_KV_BLOCK_SIZE if compressed_kv else BLOCK_SIZE
    assert x.shape[-1] % block == 0
    _lib.require_gpu(x, "fake_quant")
    xc = x.contiguous()
    out = torch.empty_like(xc)
    mode = _MODE_COMPRESSED_KV if compressed_kv else (_MODE_FP4 if fp4 else _MODE_FP8)
    launch.note_direct_call()
    rc = _lib.load().mq_fake_quant(xc.data_ptr(), _lib.dtype_code(xc, "fake_quant"), out.data_ptr(), xc.numel(), mode,
                                   _lib.stream_ptr(xc.device))
    _lib.check(rc)
    return out


def _forward(fp4: bool, compressed_kv: bool = False):
    def forward(x: torch.Tensor) -> torch.Tensor:
        return _fake_quant(x, fp4, compressed_kv=compressed_kv)

    return forward


fake_quant_fp8_forward = _forward(False)
fake_quant_fp4_forward = _forward(True)
fake_quant_compressed_kv_forward = _forward(True, compressed_kv=True)


class _IdentityGradient(torch.autograd.Function):
    """Straight-through estimator: the rounded values go forward, the incoming gradient goes back untouched."""

    @staticmethod
    def forward(ctx, x, quantizer):
        return quantizer(x)

    @staticmethod
    def backward(ctx, grad_output):
        return grad_output, None


def _straight_through(quantizer):
    def apply(x: torch.Tensor) -> torch.Tensor:
        return _IdentityGradient.apply(x, quantizer)

    return apply


fake_quant_fp8 = _straight_through(fake_quant_fp8_forward)
fake_quant_fp4 = _straight_through(fake_quant_fp4_forward)
fake_quant_compressed_kv = _straight_through(fake_quant_compressed_kv_forward)
