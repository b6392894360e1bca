"""MXFP4 (E2M1 elements + E8M0 block scales) pack / unpack.

Mirror of the reference's `miles/utils/mxfp4.py` (`quantize_mxfp4` :11-31, `dequantize_mxfp4` :34-59): same
arguments, results, dtypes, shapes and assertion behaviour.  The reference writes both as chains of torch
ops; here each is one gfx950 kernel.
"""

from __future__ import annotations

import torch

from miles_amd import _lib, launch

_E2M1_VALUES = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)


def quantize_mxfp4(weight: torch.Tensor, group_size: int):
    """weight [..., K] -> (uint8 [..., K/2], two codes per byte, even element low; uint8 E8M0 [..., K/group_size])."""
    assert weight.shape[-1] % group_size == 0
    assert weight.shape[-1] % 2 == 0
    _lib.require_gpu(weight, "quantize_mxfp4")
    w = weight.contiguous()
    k = w.shape[-1]
    rows = w.numel() // k if k else 0
    packed = torch.empty((*w.shape[:-1], k // 2), dtype=torch.uint8, device=w.device)
    scale = torch.empty((*w.shape[:-1], k // group_size), dtype=torch.uint8, device=w.device)
    _lib.dtype_code(w, "quantize_mxfp4")
    launch.submit(_lib.JOB_MXFP4, w, packed, scale, None, None, rows, k, k, int(group_size), 0)
    return packed, scale


def dequantize_mxfp4(weight_packed: torch.Tensor, weight_scale: torch.Tensor, group_size: int) -> torch.Tensor:
    """(uint8 [..., K/2], uint8 E8M0 scales, group_size) -> bfloat16 [..., K]."""
    assert weight_packed.dtype == torch.uint8
    assert weight_scale.dtype == torch.uint8
    assert group_size > 0
    _lib.require_gpu(weight_packed, "dequantize_mxfp4")
    if weight_scale.device != weight_packed.device:
        raise _lib.MilesQuantError("dequantize_mxfp4: scales and codes must be on the same device")
    packed = weight_packed.contiguous()
    scale = weight_scale.contiguous()
    numel = packed.numel() * 2
    assert numel % group_size == 0
    assert scale.numel() == numel // group_size
    out = torch.empty((*packed.shape[:-1], packed.shape[-1] * 2), dtype=torch.bfloat16, device=packed.device)
    # a job of the batched driver: inside `launch.deferred()` the tensors of a whole shard share grouped launches
    if numel:
        launch.submit(_lib.JOB_MXFP4_DEQUANT, packed, out, None, scale, None, 1, numel, numel, int(group_size))
    return out
