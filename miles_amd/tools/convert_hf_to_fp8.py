"""FP8 e4m3 weight quantizers of the offline converter.

Mirror of the reference's tools/convert_hf_to_fp8.py quantizer functions: `block_fp8` (:39-70),
`channel_fp8` (:73-78), `tensor_fp8` (:81-86), `quant_fp8` (:89-95).  The chain of ~8 full-tensor
PyTorch kernels there is one gfx950 kernel here (`mq_fp8_block_quant` / `mq_fp8_scaled_quant`).
"""

from __future__ import annotations

import torch

from miles_amd import _lib, launch

FP8_INFO = torch.finfo(torch.float8_e4m3fn)
FP8_MAX, FP8_MIN = FP8_INFO.max, FP8_INFO.min


def ceildiv(a, b):
    return -(-a // b)


def block_fp8(weight: torch.Tensor, block_size):
    """weight [N, K] -> (float8_e4m3fn [N, K], float32 [ceil(N/bn), ceil(K/bk)]).

    Per (zero-padded) tile: scale = amax / 448 with a true division, q = e4m3(clamp(w / scale, +-448)).
    An all-zero tile keeps the reference's CPU result: scale 0 and every byte 0xFF.
    """
    _lib.require_gpu(weight, "block_fp8")
    bn, bk = int(block_size[0]), int(block_size[1])
    n, k = weight.shape
    w = weight if weight.stride(1) == 1 else weight.contiguous()
    q = torch.empty((n, k), dtype=torch.float8_e4m3fn, device=w.device)
    scale = torch.empty((ceildiv(n, bn), ceildiv(k, bk)), dtype=torch.float32, device=w.device)
    _lib.dtype_code(w, "block_fp8")
    launch.submit(_lib.JOB_FP8_BLOCK, w, q, scale, None, None, n, k, w.stride(0), bn, bk)
    return q, scale


def _scaled_fp8(weight: torch.Tensor, per_channel: bool):
    _lib.require_gpu(weight, "channel_fp8" if per_channel else "tensor_fp8")
    n, k = weight.shape
    w = weight if weight.stride(1) == 1 else weight.contiguous()
    q = torch.empty((n, k), dtype=torch.float8_e4m3fn, device=w.device)
    scale = torch.empty((n, 1) if per_channel else (1,), dtype=torch.float32, device=w.device)
    ws = torch.empty(max(n, 1), dtype=torch.int32, device=w.device)
    launch.note_direct_call()
    floor = float(torch.tensor(1e-12, dtype=w.dtype).float())  # clamp(min=1e-12) acts in the weight dtype
    rc = _lib.load().mq_fp8_scaled_quant(w.data_ptr(), _lib.dtype_code(w, "fp8"), w.stride(0), q.data_ptr(),
                                         scale.data_ptr(), ws.data_ptr(), n, k, int(per_channel), floor,
                                         _lib.stream_ptr(w.device))
    _lib.check(rc)
    return q, scale


def channel_fp8(weight: torch.Tensor):
    """One scale per output channel: (float8_e4m3fn [N, K], float32 [N, 1])."""
    return _scaled_fp8(weight, True)


def tensor_fp8(weight: torch.Tensor):
    """One scale per tensor: (float8_e4m3fn [N, K], float32 [1])."""
    return _scaled_fp8(weight, False)


def quant_fp8(weight, strategy, block_size=None):
    if strategy == "tensor":
        return tensor_fp8(weight)
    if strategy == "channel":
        return channel_fp8(weight)
    return block_fp8(weight, block_size)
