"""FP8 block-scale -> BF16 dequantizer of the offline converter.

Mirror of the reference's tools/fp8_cast_bf16.py `weight_dequant` (:30-40; Triton kernel :15-27).
"""

from __future__ import annotations

import torch

from miles_amd import _lib, launch


def weight_dequant(x: torch.Tensor, s: torch.Tensor, block_size: int = 128) -> torch.Tensor:
    """x e4m3 [M, N], s float32 [ceil(M/B), ceil(N/B)] -> bfloat16 [M, N] = bf16(float(x) * s[i//B, j//B]).

    The reference allocates the output in the default dtype, which its tool sets to bfloat16 before the
    first call (tools/fp8_cast_bf16.py:44); this function always writes bfloat16.
    """
    assert x.is_contiguous() and s.is_contiguous()
    assert x.dim() == 2 and s.dim() == 2
    _lib.require_gpu(x, "weight_dequant")
    if s.dtype != torch.float32:
        raise _lib.MilesQuantError(f"weight_dequant expects float32 scales, got {s.dtype}")
    M, N = x.size()
    y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    launch.submit(_lib.JOB_FP8_DEQUANT, x, y, None, s, None, M, N, N, int(block_size), 0)
    return y
