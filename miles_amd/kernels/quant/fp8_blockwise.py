"""FP8 e4m3 block-scale cast used on the weight-sync path.

Same call as the reference's `miles.kernels.quant.fp8_blockwise.fp8_blockwise_cast`
(miles/kernels/quant/fp8_blockwise.py:61-79); the Triton kernel there (:24-58) is replaced by the
gfx950 kernel behind `mq_fp8_blockwise_cast`.
"""

from __future__ import annotations

import torch

from miles_amd import _lib, launch

fp8_dtype = torch.float8_e4m3fn
fp8_max = torch.finfo(fp8_dtype).max
fp8_min = -fp8_max


def ceil_div(x: int, y: int) -> int:
    return -(-x // y)


def fp8_blockwise_cast(x: torch.Tensor, block_size=None) -> tuple[torch.Tensor, torch.Tensor]:
    """x [M, N] (any strides) -> (float8_e4m3fn [M, N] contiguous, float32 [ceil(M/bm), ceil(N/bn)]).

    Per tile: absmax = max(max|x|, 1e-10); scale = absmax / 448; y = e4m3(clamp(x * (1 / scale), +-448)).

    Extension used by the sync driver: x may also be a 3-D view [B, R, N] whose rows are contiguous
    (strides (s, N, 1)) with R a multiple of 128 -- B blocks of R rows, e.g. the q rows of a fused per-group
    QKV weight.  It is quantized in place as the [B*R, N] matrix it stands for, without a regrouping copy.
    """
    bm, bn = (128, 128) if not block_size else (int(block_size[0]), int(block_size[1]))
    _lib.require_gpu(x, "fp8_blockwise_cast")
    _lib.dtype_code(x, "fp8_blockwise_cast")
    if x.dim() == 3:
        B, R, N = x.shape
        if not (x.stride(2) == 1 and x.stride(1) == N and R % 128 == 0 and (bm, bn) == (128, 128)
                and x.dtype in (torch.bfloat16, torch.float16)):
            return fp8_blockwise_cast(x.reshape(B * R, N), block_size)
        M = B * R
        y = torch.empty(M, N, device=x.device, dtype=fp8_dtype)
        s = torch.empty(ceil_div(M, bm), ceil_div(N, bn), dtype=torch.float32, device=x.device)
        launch.submit(_lib.JOB_FP8_BLOCKWISE_CAST, x, y, s, None, None, M, N, N, bm, bn, R, x.stride(0))
        return y, s
    M, N = x.shape
    y = torch.empty(M, N, device=x.device, dtype=fp8_dtype)
    s = torch.empty(ceil_div(M, bm), ceil_div(N, bn), dtype=torch.float32, device=x.device)
    if x.stride(1) == 1 or N <= 1:
        launch.submit(_lib.JOB_FP8_BLOCKWISE_CAST, x, y, s, None, None, M, N, x.stride(0), bm, bn)
    else:  # general column stride: direct entry point, not batchable
        launch.note_direct_call()
        rc = _lib.load().mq_fp8_blockwise_cast(x.data_ptr(), _lib.dtype_code(x, "fp8_blockwise_cast"), x.stride(0),
                                               x.stride(1), y.data_ptr(), s.data_ptr(), M, N, bm, bn,
                                               _lib.stream_ptr(x.device))
        _lib.check(rc)
    return y, s


def per_block_cast_to_fp8(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """x [M, N] -> (float8_e4m3fn [M, N], float32 [ceil(M/128), ceil(N/128)]) with power-of-two scales.

    Stands in for SGLang's `per_block_cast_to_fp8` (sglang.srt.layers.quantization.fp8_utils; imported at
    miles/backends/megatron_utils/sglang.py:9-12 and called at .../processors/quantizer_fp8.py:139-147 when
    NVTE_FP8_BLOCK_SCALING_FP32_SCALES=0).  Its source is not part of the reference tree; the published algorithm is
    restated: per 128x128 tile amax = max(max|x|, 1e-4), sf = 2^ceil(log2(amax / 448)), y = e4m3(x * (1 / sf)).
    Also accepts the row-blocked 3-D views of `fp8_blockwise_cast`.
    """
    _lib.require_gpu(x, "per_block_cast_to_fp8")
    _lib.dtype_code(x, "per_block_cast_to_fp8")
    rpb, bstride = 0, 0
    if x.dim() == 3:
        B, R, N = x.shape
        if x.stride(2) == 1 and x.stride(1) == N and R % 128 == 0 and x.dtype in (torch.bfloat16, torch.float16):
            rpb, bstride, M, ld = R, x.stride(0), B * R, N
        else:
            x = x.reshape(B * R, N)
    if x.dim() != 3:
        assert x.dim() == 2
        if x.stride(1) != 1 and x.shape[1] > 1:
            x = x.contiguous()
        (M, N), ld = x.shape, x.stride(0)
    y = torch.empty(M, N, device=x.device, dtype=fp8_dtype)
    s = torch.empty(ceil_div(M, 128), ceil_div(N, 128), dtype=torch.float32, device=x.device)
    launch.submit(_lib.JOB_FP8_BLOCK_POW2, x, y, s, None, None, M, N, ld, 128, 128, rpb, bstride)
    return y, s


def quant_weight_ue8m0(weight_dequant: torch.Tensor, weight_block_size) -> tuple[torch.Tensor, torch.Tensor]:
    """bf16 [..., n, k] -> (float8_e4m3fn [..., n, k], float32 [..., ceil(n/128), ceil(k/128)] power-of-two scales).

    Stands in for SGLang's `quant_weight_ue8m0` (imported at miles/backends/megatron_utils/sglang.py:13-20, called
    at .../processors/quantizer_fp8.py:141): `per_block_cast_to_fp8` over the weight flattened to [-1, k].  SGLang's
    source is not part of the reference tree; the published algorithm is restated.
    """
    assert list(weight_block_size) == [128, 128]
    assert weight_dequant.dtype == torch.bfloat16
    *batch_dims, n, k = weight_dequant.shape
    out_w, out_s = per_block_cast_to_fp8(weight_dequant.view((-1, k)))
    return out_w.view((*batch_dims, n, k)), out_s.view((*batch_dims, ceil_div(n, 128), ceil_div(k, 128)))


def transform_scale_ue8m0(sf: torch.Tensor, mn: int) -> torch.Tensor:
    """float32 [(b,) ceil(mn/128), kb] tile scales -> int32 [(b,) mn, ceil(kb/4)] with strides (1, align(mn, 4)).

    Stands in for SGLang's `transform_scale_ue8m0` (.../processors/quantizer_fp8.py:142): every weight row gets the
    scales of its tile row (`index_select(-2, arange(mn) // 128)`), then DeepGEMM's
    `get_mn_major_tma_aligned_packed_ue8m0_tensor`: the exponent byte of each scale, four neighbours along k in one
    int32 (lowest byte first, zero padded), rows contiguous in memory and padded to a multiple of 4.  Restated from
    the published algorithm; neither library is part of the reference tree.
    """
    _lib.require_gpu(sf, "transform_scale_ue8m0")
    assert sf.dtype == torch.float32 and sf.dim() in (2, 3)
    squeeze = sf.dim() == 2
    if squeeze:
        sf = sf.unsqueeze(0)
    b, tile_rows, kb = sf.shape
    if ceil_div(mn, 128) > tile_rows:
        raise IndexError(f"index out of range: {mn} rows need {ceil_div(mn, 128)} tile rows of scales, got {tile_rows}")
    sf = sf.contiguous()            # no copy for the scales a quantizer just produced (they may not be computed yet)
    storage = torch.empty((b, ceil_div(kb, 4), ceil_div(mn, 4) * 4), dtype=torch.int32, device=sf.device)
    launch.submit(_lib.JOB_UE8M0_PACK, sf, storage, None, None, None, mn, kb, 0, b, tile_rows)
    packed = storage.mT[:, :mn, :]
    return packed.squeeze(0) if squeeze else packed
