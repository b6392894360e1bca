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


# ---- FP8 128x128 block-scaled sources (tools/convert_hf_to_mxfp8.py:56-102,180-195) ---------------------------------
SOURCE_FP8_TILE = 128


def _grids(weight: torch.Tensor, scale: torch.Tensor):
    """(codes [B, N, K], tile-scale grid [B, >= ceil(N/128), >= ceil(K/128)] with unit column stride) of a source weight
    [..., N, K] and its scale tensor; the grid may be larger than the weight needs (the reference crops it)."""
    _lib.require_gpu(weight, "FP8 source weight")
    _lib.require_gpu(scale, "FP8 source scale")
    if weight.dim() < 2 or scale.dim() != weight.dim() or weight.element_size() != 1:
        raise ValueError(f"expected FP8 codes [..., N, K] and a scale grid of the same rank, got {tuple(weight.shape)} "
                         f"{weight.dtype} and {tuple(scale.shape)}")
    n, k = weight.shape[-2:]
    nt, kt = -(-n // SOURCE_FP8_TILE), -(-k // SOURCE_FP8_TILE)
    if scale.shape[-2] < nt or scale.shape[-1] < kt or scale.shape[:-2] != weight.shape[:-2]:
        raise ValueError(f"scale grid {tuple(scale.shape)} does not cover a weight of shape {tuple(weight.shape)}")
    if scale.stride(-1) != 1 and scale.shape[-1] > 1:
        scale = scale.contiguous()
    batch = 1
    for d in weight.shape[:-2]:
        batch *= d
    w3 = weight.contiguous().view(batch, n, k)
    s3 = scale.reshape(batch, *scale.shape[-2:]) if scale.dim() > 2 else scale.unsqueeze(0)
    return w3, s3, nt, kt


def fp8_tile_scales_pow2(sources) -> list[bool]:
    """For every (weight, fp32 tile scales) of `sources`: whether each scale the weight uses has a zero mantissa and a
    clear sign bit -- the reference's test for a source that is relabelled instead of re-quantized
    (`_load_source_scale_u8`, :81-86).  One small kernel per grid, one read of all the flags."""
    sources = list(sources)
    if not sources:
        return []
    lib = _lib.load()
    device = sources[0][0].device
    grids, counts = [], []
    for weight, scale in sources:
        if scale.dtype != torch.float32:
            raise ValueError(f"expected fp32 tile scales, got {scale.dtype}")
        _w3, s3, nt, kt = _grids(weight, scale)
        grids.extend((s3[b], nt, kt) for b in range(s3.shape[0]))
        counts.append(s3.shape[0])
    flags = torch.empty(max(len(grids), 1), dtype=torch.int32, device=device)
    launch.note_direct_call()
    stream = _lib.stream_ptr(device)
    for i, (grid, nt, kt) in enumerate(grids):
        _lib.check(lib.mq_fp8_scales_pow2_flag(grid.data_ptr(), nt, kt, grid.stride(0) if nt > 1 else max(kt, 1),
                                               flags.data_ptr() + 4 * i, stream))
    host = flags.cpu().tolist()
    out, at = [], 0
    for count in counts:
        out.append(all(host[at:at + count]))
        at += count
    return out


def expand_tile_scales_e8m0(weight: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """One exponent byte per 128x128 tile -> one per 1x32 group, uint8 [..., N, K/32] (`_source_fp8_to_mxfp8_scale_u8`,
    :98-102).  `scale` holds the bytes (uint8) or fp32 powers of two, whose byte is bits 23..30 (:85)."""
    if scale.dtype not in (torch.uint8, torch.float32):
        raise ValueError(f"expected uint8 or fp32 tile scales, got {scale.dtype}")
    w3, s3, nt, kt = _grids(weight, scale)
    n, k = w3.shape[-2:]
    groups = k // MXFP8_GROUP_SIZE
    out = torch.empty((*weight.shape[:-1], groups), dtype=torch.uint8, device=weight.device)
    o3 = out.view(w3.shape[0], n, groups)
    for b in range(w3.shape[0] if n and groups else 0):
        launch.submit(_lib.JOB_E8M0_EXPAND, s3[b], o3[b], None, None, None, n, groups,
                      s3[b].stride(0) if nt > 1 else max(s3.shape[-1], 1))
    return out


def requantize_fp8_block_to_mxfp8(weight: torch.Tensor, scale: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """FP8 codes [..., N, K] with fp32 128x128 tile scales -> (float8_e4m3fn [..., N, K], uint8 [..., N, K/32]): the
    result of `mxfp8_quantize(block_quant_dequant(weight, scale, [128, 128], torch.float32))` (:187-190) without the fp32
    tensor ever reaching memory."""
    k = weight.shape[-1]
    if k % MXFP8_GROUP_SIZE != 0:
        raise ValueError(f"Last dim {k} must be divisible by {MXFP8_GROUP_SIZE} for MXFP8.")
    if weight.dtype != torch.float8_e4m3fn and weight.dtype != torch.uint8:
        raise ValueError(f"the FP8 to MXFP8 re-quantizer reads float8_e4m3fn codes, got {weight.dtype}")
    if scale.dtype != torch.float32:
        raise ValueError(f"expected fp32 tile scales, got {scale.dtype}")
    w3, s3, nt, _kt = _grids(weight, scale)
    n = w3.shape[-2]
    q = torch.empty(weight.shape, dtype=torch.float8_e4m3fn, device=weight.device)
    out_scale = torch.empty((*weight.shape[:-1], k // MXFP8_GROUP_SIZE), dtype=torch.uint8, device=weight.device)
    q3, o3 = q.view(w3.shape[0], n, k), out_scale.view(w3.shape[0], n, k // MXFP8_GROUP_SIZE)
    for b in range(w3.shape[0] if n and k else 0):
        launch.submit(_lib.JOB_FP8_TO_MXFP8, w3[b], q3[b], o3[b], s3[b], None, n, k,
                      s3[b].stride(0) if nt > 1 else max(s3.shape[-1], 1))
    return q, out_scale


def exponent_bytes_to_fp32(scale: torch.Tensor) -> torch.Tensor:
    """E8M0 exponent bytes -> the fp32 powers of two they stand for (`(u8.to(int32) << 23).view(float32)`, :93)."""
    _lib.require_gpu(scale, "E8M0 scale bytes")
    if scale.dtype != torch.uint8:
        raise ValueError(f"expected uint8 exponent bytes, got {scale.dtype}")
    src = scale.contiguous()
    out = torch.empty(src.shape, dtype=torch.float32, device=src.device)
    launch.note_direct_call()
    _lib.check(_lib.load().mq_e8m0_bytes_to_f32(src.data_ptr(), out.data_ptr(), src.numel(), _lib.stream_ptr(src.device)))
    return out


def dequantize_fp8_source(weight: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """FP8 codes [..., N, K] with fp32 128x128 tile scales -> bf16: `block_quant_dequant(weight, scale, [128, 128],
    torch.bfloat16)` (:203-215), one fp32 multiply and one rounding per element, through the FP8 block dequantizer."""
    from miles_amd.tools.fp8_cast_bf16 import weight_dequant

    w3, s3, nt, kt = _grids(weight, scale)
    n, k = w3.shape[-2:]
    if w3.shape[0] == 1:
        return weight_dequant(w3[0], s3[0][:nt, :kt].contiguous()).view(weight.shape)
    out = torch.empty(weight.shape, dtype=torch.bfloat16, device=weight.device)
    o3 = out.view(w3.shape[0], n, k)
    for b in range(w3.shape[0]):
        o3[b].copy_(weight_dequant(w3[b], s3[b][:nt, :kt].contiguous()))
    return out
