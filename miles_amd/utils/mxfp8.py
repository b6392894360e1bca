"""MXFP8 (e4m3 + 1x32 E8M0) weight quantization.

Mirror of the reference's `miles/utils/mxfp8.py` (constants :4-25, `should_use_mxfp8` :27-48,
`mxfp8_quantize` :51-78).  The reference pads rows to a multiple of 32 for Transformer Engine and crops
the swizzle-padded scale buffer afterwards; groups are row-local, so the gfx950 kernel writes the compact
[..., K/32] scale tensor directly and needs neither.
"""

from __future__ import annotations

import torch

from miles_amd import _lib, launch

MXFP8_GROUP_SIZE = 32

# name fragments of tensors that stay in high precision whatever their shape
MXFP8_SKIP_WEIGHT_SUBSTRINGS = tuple(
    "layernorm embed router mlp.gate. norm lm_head eh_proj weights_proj head. wo_a ffn.gate. compressor.".split())

MXFP8_SOURCE_FP8_DTYPES = tuple(getattr(torch, n) for n in ("float8_e4m3fn", "float8_e4m3fnuz") if hasattr(torch, n))

_HIGH_PRECISION_DTYPES = (torch.float16, torch.bfloat16, torch.float32)


def should_use_mxfp8(name: str, shape: tuple[int, ...], dtype: torch.dtype, *,
                     skip_substrings: tuple[str, ...] = MXFP8_SKIP_WEIGHT_SUBSTRINGS,
                     allow_source_fp8: bool = False, packed_mxfp4_experts: bool = False) -> bool:
    """Whether a checkpoint tensor is stored as MXFP8 in the rollout layout: a `.weight` matrix outside the skip list
    whose last dimension splits into 1x32 groups (for packed MXFP4 experts the stored byte holds two weights, and the
    dtype is not looked at); FP8 sources only count when the caller re-scales them."""
    is_matrix_weight = name.endswith(".weight") and len(shape) >= 2
    if not is_matrix_weight or any(fragment in name for fragment in skip_substrings):
        return False
    width = shape[-1] * (2 if packed_mxfp4_experts else 1)
    if width % MXFP8_GROUP_SIZE:
        return False
    if packed_mxfp4_experts:
        return True
    return dtype in _HIGH_PRECISION_DTYPES or (allow_source_fp8 and dtype in MXFP8_SOURCE_FP8_DTYPES)


def mxfp8_quantize(weight: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """weight [..., K] -> (float8_e4m3fn, same shape; uint8 E8M0 scales [..., K/32], compact, unswizzled)."""
    k = weight.shape[-1]
    if k % MXFP8_GROUP_SIZE != 0:
        raise ValueError(f"Last dim {k} must be divisible by {MXFP8_GROUP_SIZE} for MXFP8.")
    _lib.require_gpu(weight, "mxfp8_quantize")
    w = weight.contiguous()
    rows = w.numel() // k if k else 0
    q = torch.empty(w.shape, dtype=torch.float8_e4m3fn, device=w.device)
    scale = torch.empty((*w.shape[:-1], k // MXFP8_GROUP_SIZE), dtype=torch.uint8, device=w.device)
    _lib.dtype_code(w, "mxfp8_quantize")
    launch.submit(_lib.JOB_MXFP8, w, q, scale, None, None, rows, k, k)
    return q, scale
