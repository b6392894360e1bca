"""INT4 fake quantization (values, scale, zero point in the input dtype).

Stands in for the reference's pybind11 CUDA module `fake_int4_quant_cuda`
(miles/kernels/quant/int4_fake/fake_int4_quant_cuda.cu:319-364): same arguments, same three outputs,
same argument checks (raised as RuntimeError like TORCH_CHECK).
"""

from __future__ import annotations

import torch

from miles_amd import _lib, launch


def fake_int4_quant_cuda(x: torch.Tensor, block_size, sym: bool):
    """x [M, N] on the GPU, block_size (block_m, block_n) -> (out [M, N], scale, zero), all in x.dtype."""
    if x.dim() != 2:
        raise RuntimeError("Input must be 2D")
    if x.device.type != "cuda":
        raise RuntimeError("Input must be on CUDA")
    block_m, block_n = int(block_size[0]), int(block_size[1])
    if block_m <= 0 or block_n <= 0:
        raise RuntimeError(f"Block sizes must be positive, got block_m={block_m}, block_n={block_n}")
    if (block_m * block_n) % 32 != 0:
        raise RuntimeError(f"block_m * block_n ({block_m * block_n}) must be divisible by 32. "
                           f"But got a {block_m}x{block_n} block.")
    M, N = x.shape
    xc = x.contiguous()
    out = torch.empty_like(xc)
    scale = torch.empty((-(-M // block_m), -(-N // block_n)), dtype=x.dtype, device=x.device)
    zero = torch.empty_like(scale)  # left unwritten in symmetric mode, as in the reference
    launch.note_direct_call()
    rc = _lib.load().mq_int4_fake_quant(xc.data_ptr(), _lib.dtype_code(x, "fake_int4_quant_cuda"), out.data_ptr(),
                                        scale.data_ptr(), zero.data_ptr(), M, N, block_m, block_n, int(bool(sym)),
                                        _lib.stream_ptr(x.device))
    _lib.check(rc, RuntimeError)
    return out, scale, zero


def pack_layer(weight: torch.Tensor, group_size: int, sym: bool = True):
    """weight [M, K] -> (int32 [M, K/8], weight.dtype [M, K/group_size], packed zero points or None).

    Fused form of the reference's `pack_layer`
    (miles/backends/megatron_utils/megatron_to_hf/processors/quantizer_compressed_tensors.py:235-265,
    identical to tools/convert_hf_to_int4_direct.py:121-151): the fake-quant kernel, the dequantize/requantize
    round trip in the weight's dtype and pack_to_int32 collapse into one pass that writes the packed words
    and the scales directly.  With sym=False the third result is the AWQ-ordered int32 [K/group_size, M/8]
    zero-point tensor; with sym=True it is None.
    """
    _lib.require_gpu(weight, "pack_layer")
    if weight.dim() != 2:
        raise RuntimeError("Input must be 2D")
    M, K = weight.shape
    if not sym:
        return _pack_layer_asym(weight, int(group_size))
    if K % group_size != 0 or K % 8 != 0:
        raise RuntimeError(f"shape {tuple(weight.shape)} is not divisible into groups of {group_size} and words of 8")
    w = weight.contiguous()
    packed = torch.empty((M, K // 8), dtype=torch.int32, device=w.device)
    scale = torch.empty((M, K // group_size), dtype=w.dtype, device=w.device)
    _lib.dtype_code(w, "pack_layer")
    launch.submit(_lib.JOB_INT4_PACK, w, packed, scale, None, None, M, K, K, int(group_size), 0)
    return packed, scale, None


def _pack_layer_asym(weight: torch.Tensor, group_size: int):
    M, K = weight.shape
    if K % group_size != 0 or group_size % 8 != 0 or M % 8 != 0:
        raise RuntimeError(f"shape {tuple(weight.shape)} is not divisible into groups of {group_size}, "
                           f"words of 8 and zero-point words of 8 rows")
    w = weight.contiguous()
    groups = K // group_size
    packed = torch.empty((M, K // 8), dtype=torch.int32, device=w.device)
    scale = torch.empty((M, groups), dtype=w.dtype, device=w.device)
    zero = torch.empty((M, groups), dtype=torch.uint8, device=w.device)
    packed_zp = torch.empty((groups, M // 8), dtype=torch.int32, device=w.device)
    _lib.dtype_code(w, "pack_layer")
    launch.submit(_lib.JOB_INT4_PACK_ASYM, w, packed, scale, zero, packed_zp, M, K, K, int(group_size), 0)
    return packed, scale, packed_zp
