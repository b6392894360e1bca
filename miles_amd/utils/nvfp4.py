"""NVFP4 (e2m1 + 1x16 e4m3 block scales + fp32 global scale) weight quantization.

Mirror of the reference's `miles/utils/nvfp4.py`: `nvfp4_weight_e4m3_max` (:11-16), the global scale closed
forms (:19-39), `nvfp4_quantize_1d` (:54-82) and `nvfp4_quantize_1d_pair` (:85-114).  Transformer Engine's
quantizer is replaced by the two gfx950 passes `mq_nvfp4_amax` / `mq_nvfp4_quant`; the global amax never
leaves the device, and a gate/up pair shares it by reducing both tensors into the same word instead of
concatenating them.
"""

from __future__ import annotations

import os

import torch

from miles_amd import _lib, launch

FP4_E2M1_MAX = 6.0
FP8_E4M3_MAX = 448.0
NVFP4_GROUP_SIZE = 16
AMAX_RECORD_WORDS = 1280   # MQ_NVFP4_RECORD_WORDS: per-workgroup partial maxima of a tensor (or pair) on the device


def nvfp4_weight_e4m3_max() -> int:
    four_over_six = os.getenv("NVTE_NVFP4_4OVER6", "").strip().lower() in ("weights", "all")
    use_256 = os.getenv("NVTE_NVFP4_4OVER6_E4M3_USE_256", "all").strip().lower() in ("weights", "all")
    return 256 if four_over_six and use_256 else int(FP8_E4M3_MAX)


def _nvfp4_4over6_enabled() -> bool:
    return os.getenv("NVTE_NVFP4_4OVER6", "").strip().lower() in ("weights", "all")


def nvfp4_global_encode_scale_te(global_amax: torch.Tensor, nvfp4_e4m3_max: int = int(FP8_E4M3_MAX)) -> torch.Tensor:
    """min(e4m3_max * 6 / amax, FLT_MAX), with an exact zero repaired to 1; no host read of the amax."""
    enc = torch.div(float(nvfp4_e4m3_max) * FP4_E2M1_MAX, global_amax.to(torch.float32))
    enc = enc.clamp_max(torch.finfo(torch.float32).max)
    return torch.where(enc == 0.0, 1.0, enc)


def nvfp4_global_decode_scale_te(global_amax: torch.Tensor, nvfp4_e4m3_max: int = int(FP8_E4M3_MAX)) -> torch.Tensor:
    return torch.div(1.0, nvfp4_global_encode_scale_te(global_amax, nvfp4_e4m3_max))


def _quantizer_options() -> tuple[int, int]:
    """(e4m3_max, flags) of the weight quantizer from Transformer Engine's environment variables: Four Over Six on or
    off (NVTE_NVFP4_4OVER6), its error metric (NVTE_NVFP4_4OVER6_ERR_MODE, passed to NVFP4Quantizer at
    miles/utils/nvfp4.py:72) and the fp16 candidate-error form (NVTE_NVFP4_4OVER6_ERR_USE_FAST_MATH)."""
    flags = 0
    if _nvfp4_4over6_enabled():
        flags |= _lib.NVFP4_4OVER6
        mode = os.getenv("NVTE_NVFP4_4OVER6_ERR_MODE", "MAE").strip().upper()
        if mode not in ("MAE", "MSE"):
            raise ValueError(f"NVTE_NVFP4_4OVER6_ERR_MODE must be MAE or MSE, got {mode!r}.")
        if mode == "MSE":
            flags |= _lib.NVFP4_ERR_MSE
        if os.getenv("NVTE_NVFP4_4OVER6_ERR_USE_FAST_MATH", "0").strip() == "1":
            flags |= _lib.NVFP4_ERR_FP16
    return nvfp4_weight_e4m3_max(), flags


def _alloc_outputs(w: torch.Tensor):
    """The three outputs of one tensor: packed codes, block scales, global scale."""
    rows, cols = w.shape
    _lib.dtype_code(w, "nvfp4")
    q = torch.empty((rows, cols // 2), dtype=torch.uint8, device=w.device)
    block_scale = torch.empty((rows, cols // NVFP4_GROUP_SIZE), dtype=torch.float8_e4m3fn, device=w.device)
    global_scale = torch.empty((), dtype=torch.float32, device=w.device)
    return q, block_scale, global_scale


def nvfp4_quantize_1d(weight: torch.Tensor, *, out=None) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """weight [M, K] -> (uint8 [M, K/2], float8_e4m3fn [M, K/16], float32 [] = weight_scale_2).
    `out` (not in the reference): three contiguous tensors of those shapes to write into, e.g. one matrix's slices
    of stacked outputs, so that a caller inside a deferred batch never has to read results before the batch runs."""
    _lib.require_gpu(weight, "nvfp4_quantize_1d")
    e4m3_max, flags = _quantizer_options()
    w = weight.contiguous()
    if w.shape[1] % NVFP4_GROUP_SIZE != 0:
        raise ValueError(f"NVFP4 requires K divisible by {NVFP4_GROUP_SIZE}, got {w.shape[1]}.")
    word = torch.empty(AMAX_RECORD_WORDS, dtype=torch.int32, device=w.device)   # written by the amax pass of the job driver
    if out is None:
        out = _alloc_outputs(w)
    else:
        _lib.dtype_code(w, "nvfp4")
        want = ((w.shape[0], w.shape[1] // 2), (w.shape[0], w.shape[1] // NVFP4_GROUP_SIZE), ())
        if any(tuple(t.shape) != shape or not t.is_contiguous() for t, shape in zip(out, want)):
            raise ValueError("nvfp4_quantize_1d: `out` tensors must be contiguous and shaped like the results")
    launch.submit(_lib.JOB_NVFP4, w, out[0], out[1], word, out[2], w.shape[0], w.shape[1], w.shape[1], e4m3_max, flags)
    return out


def nvfp4_quantize_1d_pair(first: torch.Tensor, second: torch.Tensor):
    """Quantize a gate/up pair with ONE global amax taken over both tensors."""
    if first.dim() != 2 or second.dim() != 2:
        raise ValueError("nvfp4_quantize_1d_pair expects two 2D tensors.")
    if first.shape[1] != second.shape[1]:
        raise ValueError(
            f"NVFP4 paired quantization requires matching K dimensions, got {first.shape[1]} and {second.shape[1]}."
        )
    _lib.require_gpu(first, "nvfp4_quantize_1d_pair")
    _lib.require_gpu(second, "nvfp4_quantize_1d_pair")
    e4m3_max, flags = _quantizer_options()
    a, b = first.contiguous(), second.contiguous()
    if a.shape[1] % NVFP4_GROUP_SIZE != 0:
        raise ValueError(f"NVFP4 requires K divisible by {NVFP4_GROUP_SIZE}, got {a.shape[1]}.")
    word = torch.empty(AMAX_RECORD_WORDS, dtype=torch.int32, device=a.device)
    outs = (_alloc_outputs(a), _alloc_outputs(b))
    # two adjacent jobs on one amax word: the driver reduces both tensors before it quantizes either
    with _pair_scope() as submit:
        for w, out in zip((a, b), outs):
            submit(_lib.JOB_NVFP4, w, out[0], out[1], word, out[2], w.shape[0], w.shape[1], w.shape[1], e4m3_max, flags)
    return outs


class _pair_scope:
    """Submits the two jobs of a pair together even when no deferred() block is active."""

    def __enter__(self):
        self._own = launch.active_batch() is None
        if self._own:
            self._ctx = launch.deferred()
            self._ctx.__enter__()
        return launch.submit

    def __exit__(self, *exc):
        if self._own:
            return self._ctx.__exit__(*exc)
        return False
