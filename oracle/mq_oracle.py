"""ctypes front end of the CPU oracle (oracle/mq_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg as the checker / reported baseline.  The product
package (miles_amd) never imports this module.

All functions take and return CPU torch tensors; bf16 / fp16 / fp32 inputs.
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libmq_oracle.so")

_DTYPE = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}


def build(force: bool = False) -> str:
    """Compile oracle/mq_oracle.c with gcc (see oracle/Makefile)."""
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(
        os.path.join(_HERE, "mq_oracle.c")
    ):
        subprocess.check_call(["make", "-C", _HERE, "-B"], stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        c = ctypes
        vp, i64, i32, f32 = c.c_void_p, c.c_int64, c.c_int, c.c_float
        L.mqo_f32_to_e4m3fn.restype = c.c_uint8
        L.mqo_f32_to_e4m3fn.argtypes = [f32]
        L.mqo_f32_to_e4m3fn_sat.restype = c.c_uint8
        L.mqo_f32_to_e4m3fn_sat.argtypes = [f32]
        L.mqo_e4m3fn_to_f32.restype = f32
        L.mqo_e4m3fn_to_f32.argtypes = [c.c_uint8]
        L.mqo_f32_to_e2m1.restype = c.c_uint8
        L.mqo_f32_to_e2m1.argtypes = [f32]
        L.mqo_e2m1_to_f32.restype = f32
        L.mqo_e2m1_to_f32.argtypes = [c.c_uint8]
        L.mqo_f32_to_e8m0_ceil.restype = c.c_uint8
        L.mqo_f32_to_e8m0_ceil.argtypes = [f32]
        L.mqo_block_fp8.restype = None
        L.mqo_block_fp8.argtypes = [vp, i32, i64, i64, i64, i32, i32, vp, vp]
        L.mqo_fp8_per_tensor_or_channel.restype = None
        L.mqo_fp8_per_tensor_or_channel.argtypes = [vp, i32, i64, i64, i64, i32, f32, vp, vp]
        L.mqo_fp8_blockwise_cast.restype = None
        L.mqo_fp8_blockwise_cast.argtypes = [vp, i32, i64, i64, i64, i64, i32, i32, vp, vp]
        L.mqo_ue8m0_pack_scales.restype = None
        L.mqo_ue8m0_pack_scales.argtypes = [vp, i64, i64, i64, vp]
        L.mqo_fp8_block_pow2.restype = None
        L.mqo_fp8_block_pow2.argtypes = [vp, i32, i64, i64, i64, vp, vp]
        L.mqo_fp8_block_dequant.restype = None
        L.mqo_fp8_block_dequant.argtypes = [vp, vp, i64, i64, i32, vp]
        L.mqo_mxfp8.restype = None
        L.mqo_mxfp8.argtypes = [vp, i32, i64, i64, vp, vp]
        L.mqo_fp8_block_to_mxfp8.restype = None
        L.mqo_fp8_block_to_mxfp8.argtypes = [vp, vp, i64, i64, i64, vp, vp]
        L.mqo_fp8_scales_pow2.restype = i32
        L.mqo_fp8_scales_pow2.argtypes = [vp, i64, i64, i64]
        L.mqo_e8m0_expand_tile_scales.restype = None
        L.mqo_e8m0_expand_tile_scales.argtypes = [vp, i32, i64, i64, i64, vp]
        L.mqo_int4_fake_quant.restype = None
        L.mqo_int4_fake_quant.argtypes = [vp, i32, i64, i64, i32, i32, vp, vp, vp]
        L.mqo_int4_fake_quant_block.restype = None
        L.mqo_int4_fake_quant_block.argtypes = [vp, i32, i64, i64, i32, i32, i32, vp, vp, vp]
        L.mqo_int4_unpack_dequant.restype = None
        L.mqo_int4_unpack_dequant.argtypes = [vp, vp, i32, i64, i64, i32, vp]
        L.mqo_mxfp4_to_fp8_block.restype = None
        L.mqo_mxfp4_to_fp8_block.argtypes = [vp, vp, i64, i64, vp, vp]
        L.mqo_nvfp4_qdq.restype = None
        L.mqo_nvfp4_qdq.argtypes = [vp, i32, i64, f32, i32, i32, vp]
        L.mqo_nvfp4_quant_ex.restype = None
        L.mqo_nvfp4_quant_ex.argtypes = [vp, i32, i64, i64, f32, i32, i32, vp, vp]
        L.mqo_fake_quant.restype = None
        L.mqo_fake_quant.argtypes = [vp, i32, i64, i32, vp]
        L.mqo_fp8_act_quant.restype = None
        L.mqo_fp8_act_quant.argtypes = [vp, i32, i64, i32, i32, vp, vp]
        L.mqo_mxfp4_quant.restype = None
        L.mqo_mxfp4_quant.argtypes = [vp, i32, i64, i32, vp, vp]
        L.mqo_mxfp4_dequant.restype = None
        L.mqo_mxfp4_dequant.argtypes = [vp, vp, i64, i32, vp]
        L.mqo_int4_pack_layer.restype = None
        L.mqo_int4_pack_layer.argtypes = [vp, i32, i64, i64, i32, vp, vp]
        L.mqo_int4_pack_layer_asym.restype = None
        L.mqo_int4_pack_layer_asym.argtypes = [vp, i32, i64, i64, i32, vp, vp, vp]
        L.mqo_nvfp4_amax.restype = f32
        L.mqo_nvfp4_amax.argtypes = [vp, i32, i64]
        L.mqo_nvfp4_global_encode_scale.restype = f32
        L.mqo_nvfp4_global_encode_scale.argtypes = [f32, i32]
        L.mqo_nvfp4_global_decode_scale.restype = f32
        L.mqo_nvfp4_global_decode_scale.argtypes = [f32, i32]
        L.mqo_nvfp4_quant.restype = None
        L.mqo_nvfp4_quant.argtypes = [vp, i32, i64, i64, f32, i32, vp, vp]
        L.mqo_f32_to_e4m3fn_vec.restype = None
        L.mqo_f32_to_e4m3fn_vec.argtypes = [vp, i64, vp, i32]
        L.mqo_f32_to_e2m1_vec.restype = None
        L.mqo_f32_to_e2m1_vec.argtypes = [vp, i64, vp]
        L.mqo_f32_to_bf16_vec.restype = None
        L.mqo_f32_to_bf16_vec.argtypes = [vp, i64, vp]
        L.mqo_f32_to_e8m0_vec.restype = None
        L.mqo_f32_to_e8m0_vec.argtypes = [vp, i64, vp]
        L.mqo_fnv1a64.restype = c.c_uint64
        L.mqo_fnv1a64.argtypes = [vp, i64]
        _lib = L
    return _lib


def _check_cpu(t: torch.Tensor) -> None:
    assert t.device.type == "cpu", "the oracle runs on CPU tensors"
    assert t.dtype in _DTYPE, f"unsupported dtype {t.dtype}"


def ceil_div(a: int, b: int) -> int:
    return -(-a // b)


# --------------------------------------------------------------------------
# FP8 128x128
# --------------------------------------------------------------------------
def block_fp8(weight: torch.Tensor, block_size=(128, 128)):
    """tools/convert_hf_to_fp8.py:39-70 -> (float8_e4m3fn [M,K], float32 [nt,kt])."""
    _check_cpu(weight)
    assert weight.dim() == 2 and weight.stride(1) == 1
    M, K = weight.shape
    bm, bk = int(block_size[0]), int(block_size[1])
    q = torch.empty((M, K), dtype=torch.uint8)
    s = torch.empty((ceil_div(M, bm), ceil_div(K, bk)), dtype=torch.float32)
    lib().mqo_block_fp8(weight.data_ptr(), _DTYPE[weight.dtype], M, K, weight.stride(0), bm, bk,
                        q.data_ptr(), s.data_ptr())
    return q.view(torch.float8_e4m3fn), s


def tensor_fp8(weight: torch.Tensor):
    """tools/convert_hf_to_fp8.py:81-86 -> (e4m3fn [M,K], float32 [1])."""
    return _per_tensor_or_channel(weight, False)


def channel_fp8(weight: torch.Tensor):
    """tools/convert_hf_to_fp8.py:73-78 -> (e4m3fn [M,K], float32 [M,1])."""
    return _per_tensor_or_channel(weight, True)


def _per_tensor_or_channel(weight, per_channel):
    _check_cpu(weight)
    assert weight.dim() == 2 and weight.stride(1) == 1
    M, K = weight.shape
    floor = float(torch.tensor(1e-12, dtype=weight.dtype).float())
    q = torch.empty((M, K), dtype=torch.uint8)
    s = torch.empty((M, 1) if per_channel else (1,), dtype=torch.float32)
    lib().mqo_fp8_per_tensor_or_channel(weight.data_ptr(), _DTYPE[weight.dtype], M, K, weight.stride(0),
                                        int(per_channel), floor, q.data_ptr(), s.data_ptr())
    return q.view(torch.float8_e4m3fn), s


def fp8_blockwise_cast(x: torch.Tensor, block_size=None):
    """miles/kernels/quant/fp8_blockwise.py:61-79 (any strides)."""
    _check_cpu(x)
    assert x.dim() == 2
    bm, bn = (128, 128) if not block_size else (int(block_size[0]), int(block_size[1]))
    M, N = x.shape
    y = torch.empty((M, N), dtype=torch.uint8)
    s = torch.empty((ceil_div(M, bm), ceil_div(N, bn)), dtype=torch.float32)
    lib().mqo_fp8_blockwise_cast(x.data_ptr(), _DTYPE[x.dtype], M, N, x.stride(0), x.stride(1), bm, bn,
                                 y.data_ptr(), s.data_ptr())
    return y.view(torch.float8_e4m3fn), s


def per_block_cast_to_fp8(x: torch.Tensor):
    """SGLang's per_block_cast_to_fp8 (power-of-two scales), restated: parity unpinned."""
    _check_cpu(x)
    assert x.dim() == 2 and (x.stride(1) == 1 or x.shape[1] <= 1)
    M, N = x.shape
    y = torch.empty((M, N), dtype=torch.uint8)
    s = torch.empty((ceil_div(M, 128), ceil_div(N, 128)), dtype=torch.float32)
    lib().mqo_fp8_block_pow2(x.data_ptr(), _DTYPE[x.dtype], M, N, x.stride(0), y.data_ptr(), s.data_ptr())
    return y.view(torch.float8_e4m3fn), s


def transform_scale_ue8m0(sf: torch.Tensor, mn: int) -> torch.Tensor:
    """SGLang's transform_scale_ue8m0 (DeepGEMM packed UE8M0 layout), restated: parity unpinned.
    float32 [(b,) ceil(mn/128), kb] -> int32 [(b,) mn, ceil(kb/4)] with strides (1, align(mn, 4))."""
    _check_cpu(sf)
    assert sf.dtype == torch.float32 and sf.dim() in (2, 3)
    squeeze = sf.dim() == 2
    sf3 = (sf.unsqueeze(0) if squeeze else sf)[:, : ceil_div(mn, 128)].contiguous()
    b, _, kb = sf3.shape
    storage = torch.empty((b, ceil_div(kb, 4), ceil_div(mn, 4) * 4), dtype=torch.int32)
    lib().mqo_ue8m0_pack_scales(sf3.data_ptr(), b, mn, kb, storage.data_ptr())
    packed = storage.mT[:, :mn, :]
    return packed.squeeze(0) if squeeze else packed


def weight_dequant(x: torch.Tensor, s: torch.Tensor, block_size: int = 128) -> torch.Tensor:
    """tools/fp8_cast_bf16.py:30-40 -> bf16 [M,N]."""
    assert x.is_contiguous() and s.is_contiguous() and x.dim() == 2 and s.dim() == 2
    assert x.element_size() == 1 and s.dtype == torch.float32
    M, N = x.shape
    y = torch.empty((M, N), dtype=torch.bfloat16)
    lib().mqo_fp8_block_dequant(x.data_ptr(), s.data_ptr(), M, N, int(block_size), y.data_ptr())
    return y


# --------------------------------------------------------------------------
# MXFP8
# --------------------------------------------------------------------------
def mxfp8_quantize(weight: torch.Tensor):
    """miles/utils/mxfp8.py:51-78 -> (e4m3fn like weight, uint8 [..., K/32])."""
    _check_cpu(weight)
    weight = weight.contiguous()
    k = weight.shape[-1]
    if k % 32 != 0:
        raise ValueError(f"Last dim {k} must be divisible by 32 for MXFP8.")
    rows = weight.numel() // k
    q = torch.empty(weight.shape, dtype=torch.uint8)
    s = torch.empty((*weight.shape[:-1], k // 32), dtype=torch.uint8)
    lib().mqo_mxfp8(weight.data_ptr(), _DTYPE[weight.dtype], rows, k, q.data_ptr(), s.data_ptr())
    return q.view(torch.float8_e4m3fn), s


def _tile_grid(weight: torch.Tensor, scale: torch.Tensor):
    """The [ceil(M/128), ceil(K/128)] corner of a 2-D tile-scale grid and its row stride in elements."""
    assert weight.dim() == 2 and scale.dim() == 2 and scale.stride(1) == 1
    m, k = weight.shape
    nt, kt = ceil_div(m, 128), ceil_div(k, 128)
    assert scale.shape[0] >= nt and scale.shape[1] >= kt
    return nt, kt, scale.stride(0)


def fp8_block_to_mxfp8(weight: torch.Tensor, scale: torch.Tensor):
    """tools/convert_hf_to_mxfp8.py:187-190: block_quant_dequant(w, s, [128,128], float32) -> mxfp8_quantize.
    weight e4m3fn (or uint8 codes) [M,K], scale fp32 grid -> (e4m3fn [M,K], uint8 [M,K/32])."""
    assert weight.device.type == "cpu" and weight.element_size() == 1 and scale.dtype == torch.float32
    weight = weight.contiguous()
    m, k = weight.shape
    if k % 32 != 0:
        raise ValueError(f"Last dim {k} must be divisible by 32 for MXFP8.")
    _nt, _kt, lds = _tile_grid(weight, scale)
    q = torch.empty((m, k), dtype=torch.uint8)
    s = torch.empty((m, k // 32), dtype=torch.uint8)
    lib().mqo_fp8_block_to_mxfp8(weight.data_ptr(), scale.data_ptr(), lds, m, k, q.data_ptr(), s.data_ptr())
    return q.view(torch.float8_e4m3fn), s


def fp8_scales_are_pow2(weight: torch.Tensor, scale: torch.Tensor) -> bool:
    """tools/convert_hf_to_mxfp8.py:81-86 on the cropped grid of an fp32 scale tensor."""
    assert scale.dtype == torch.float32
    nt, kt, lds = _tile_grid(weight, scale)
    return bool(lib().mqo_fp8_scales_pow2(scale.data_ptr(), nt, kt, lds))


def expand_tile_scales_e8m0(weight: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """tools/convert_hf_to_mxfp8.py:85,98-102: exponent bytes of a tile-scale grid (uint8, or fp32 powers of two)
    repeated to one byte per 1x32 group -> uint8 [M, K/32]."""
    assert scale.dtype in (torch.uint8, torch.float32)
    _nt, _kt, lds = _tile_grid(weight, scale)
    m, k = weight.shape
    out = torch.empty((m, k // 32), dtype=torch.uint8)
    lib().mqo_e8m0_expand_tile_scales(scale.data_ptr(), int(scale.dtype == torch.float32), lds, m, k // 32, out.data_ptr())
    return out


# --------------------------------------------------------------------------
# INT4
# --------------------------------------------------------------------------
def fake_int4_quant(x: torch.Tensor, block_size, sym: bool):
    """fake_int4_quant_cuda.cu:319-364 for block (BM, BN) -> (out, scale, zero) in x.dtype."""
    _check_cpu(x)
    assert x.dim() == 2
    x = x.contiguous()
    BM, BN = int(block_size[0]), int(block_size[1])
    M, N = x.shape
    out = torch.empty_like(x)
    scale = torch.empty((ceil_div(M, BM), ceil_div(N, BN)), dtype=x.dtype)
    zero = torch.zeros_like(scale)
    lib().mqo_int4_fake_quant_block(x.data_ptr(), _DTYPE[x.dtype], M, N, BM, BN, int(sym), out.data_ptr(),
                                    scale.data_ptr(), zero.data_ptr())
    return out, scale, zero


def pack_layer(weight: torch.Tensor, group_size: int, sym: bool = True):
    """quantizer_compressed_tensors.py:235-265 -> (int32 [M,K/8], dtype [M,K/G], None | int32 [K/G,M/8])."""
    _check_cpu(weight)
    weight = weight.contiguous()
    M, K = weight.shape
    assert K % group_size == 0 and K % 8 == 0
    packed = torch.empty((M, K // 8), dtype=torch.int32)
    scale = torch.empty((M, K // group_size), dtype=weight.dtype)
    if not sym:
        assert group_size % 8 == 0 and M % 8 == 0
        packed_zp = torch.empty((K // group_size, M // 8), dtype=torch.int32)
        lib().mqo_int4_pack_layer_asym(weight.data_ptr(), _DTYPE[weight.dtype], M, K, int(group_size),
                                       packed.data_ptr(), scale.data_ptr(), packed_zp.data_ptr())
        return packed, scale, packed_zp
    lib().mqo_int4_pack_layer(weight.data_ptr(), _DTYPE[weight.dtype], M, K, int(group_size),
                              packed.data_ptr(), scale.data_ptr())
    return packed, scale, None


def int4_unpack_dequant(weight_packed: torch.Tensor, weight_scale: torch.Tensor, weight_shape, group_size: int):
    """tools/convert_kimi_int4_to_bf16.py:57-86 -> bfloat16 [M, K]."""
    assert weight_packed.device.type == "cpu" and weight_packed.dtype == torch.int32
    _check_cpu(weight_scale)
    M, K = (int(v) for v in (weight_shape.view(-1).tolist() if isinstance(weight_shape, torch.Tensor) else weight_shape))
    if group_size <= 0:                 # :75-76, one scale per element
        weight_scale, group_size = weight_scale.reshape(M, K), 1
    p, s = weight_packed.contiguous(), weight_scale.contiguous()
    assert p.shape == (M, -(-K // 8)) and K % group_size == 0 and s.numel() == M * (K // group_size)
    out = torch.empty((M, K), dtype=torch.bfloat16)
    lib().mqo_int4_unpack_dequant(p.data_ptr(), s.data_ptr(), _DTYPE[s.dtype], M, K, int(group_size), out.data_ptr())
    return out


# --------------------------------------------------------------------------
# block fake quantization
# --------------------------------------------------------------------------
def fake_quant(x: torch.Tensor, kind: str) -> torch.Tensor:
    """miles/kernels/quant/fake_quant.py:66-99; kind in {"fp8", "fp4", "compressed_kv"}."""
    _check_cpu(x)
    mode = {"fp8": 0, "fp4": 1, "compressed_kv": 2}[kind]
    assert x.shape[-1] % (16 if mode == 2 else 32) == 0
    xc = x.contiguous()
    out = torch.empty_like(xc)
    lib().mqo_fake_quant(xc.data_ptr(), _DTYPE[xc.dtype], xc.numel(), mode, out.data_ptr())
    return out


def act_quant(x: torch.Tensor, block_size: int = 128, scale_fmt: str | None = None,
              scale_dtype: torch.dtype = torch.float32, inplace: bool = False):
    """miles/kernels/quant/fp8_act_quant.py:110-137 -> (float8_e4m3fn codes, scales), or with `inplace` the
    quantize-dequantize result in x's dtype (returned, x is left alone)."""
    _check_cpu(x)
    n = x.shape[-1]
    assert n % block_size == 0
    e8m0 = scale_dtype == torch.float8_e8m0fnu
    assert scale_fmt is not None or not e8m0, "E8M0 storage needs power-of-two scales"
    z = x.contiguous()
    y = torch.empty_like(z) if inplace else torch.empty(z.shape, dtype=torch.uint8)
    s = torch.empty((*z.shape[:-1], n // block_size), dtype=torch.uint8 if e8m0 else torch.float32)
    flags = (1 if scale_fmt is not None else 0) | (2 if e8m0 else 0) | (4 if inplace else 0)
    lib().mqo_fp8_act_quant(z.data_ptr(), _DTYPE[z.dtype], z.numel(), int(block_size), flags, y.data_ptr(), s.data_ptr())
    if e8m0:
        s = s.view(torch.float8_e8m0fnu)
    return y if inplace else (y.view(torch.float8_e4m3fn), s)


def fp8_simulate(x: torch.Tensor, block_size: int) -> torch.Tensor:
    """miles_plugins/models/deepseek_v4/ops/qat.py:8-23."""
    return act_quant(x, block_size, "ue8m0", inplace=True)


# --------------------------------------------------------------------------
# MXFP4
# --------------------------------------------------------------------------
def quantize_mxfp4(weight: torch.Tensor, group_size: int):
    """miles/utils/mxfp4.py:11-31 -> (uint8 [..., K/2], uint8 [..., K/group_size])."""
    _check_cpu(weight)
    assert weight.shape[-1] % group_size == 0
    assert weight.shape[-1] % 2 == 0
    w = weight.contiguous()
    k = w.shape[-1]
    packed = torch.empty((*w.shape[:-1], k // 2), dtype=torch.uint8)
    scale = torch.empty((*w.shape[:-1], k // group_size), dtype=torch.uint8)
    lib().mqo_mxfp4_quant(w.data_ptr(), _DTYPE[w.dtype], w.numel(), int(group_size), packed.data_ptr(),
                          scale.data_ptr())
    return packed, scale


def dequantize_mxfp4(weight_packed: torch.Tensor, weight_scale: torch.Tensor, group_size: int) -> torch.Tensor:
    """miles/utils/mxfp4.py:34-59 -> bfloat16 [..., K]."""
    assert weight_packed.device.type == "cpu" and weight_scale.device.type == "cpu", "the oracle runs on CPU tensors"
    assert weight_packed.dtype == torch.uint8 and weight_scale.dtype == torch.uint8 and group_size > 0
    p, s = weight_packed.contiguous(), weight_scale.contiguous()
    assert (2 * p.numel()) % group_size == 0 and s.numel() == 2 * p.numel() // group_size
    out = torch.empty((*p.shape[:-1], p.shape[-1] * 2), dtype=torch.bfloat16)
    lib().mqo_mxfp4_dequant(p.data_ptr(), s.data_ptr(), p.numel(), int(group_size), out.data_ptr())
    return out


def cast_e2m1fn_to_e4m3fn(x: torch.Tensor, scale: torch.Tensor):
    """tools/convert_mxfp4_to_fp8.py:30-49: int8 [out, in/2] e2m1 pairs + E8M0 [out, in/32] -> (e4m3fn [out, in], fp32 tiles)."""
    assert x.device.type == "cpu" and x.dtype == torch.int8 and x.ndim == 2
    out_dim, in_dim = x.size(0), x.size(1) * 2
    assert out_dim % 128 == 0 and in_dim % 128 == 0 and tuple(scale.shape) == (out_dim, in_dim // 32)
    p, s = x.contiguous().view(torch.uint8), scale.contiguous().view(torch.uint8)
    y = torch.empty((out_dim, in_dim), dtype=torch.float8_e4m3fn)
    ts = torch.empty((out_dim // 128, in_dim // 128), dtype=torch.float32)
    lib().mqo_mxfp4_to_fp8_block(p.data_ptr(), s.data_ptr(), out_dim, in_dim, y.data_ptr(), ts.data_ptr())
    return y, ts


# --------------------------------------------------------------------------
# NVFP4
# --------------------------------------------------------------------------
def nvfp4_amax(weight: torch.Tensor) -> float:
    _check_cpu(weight)
    w = weight.contiguous()
    return float(lib().mqo_nvfp4_amax(w.data_ptr(), _DTYPE[w.dtype], w.numel()))


def nvfp4_global_encode_scale(amax: float, e4m3_max: int = 448) -> float:
    return float(lib().mqo_nvfp4_global_encode_scale(amax, e4m3_max))


def nvfp4_global_decode_scale(amax: float, e4m3_max: int = 448) -> float:
    return float(lib().mqo_nvfp4_global_decode_scale(amax, e4m3_max))


NVFP4_4OVER6, NVFP4_ERR_MSE, NVFP4_ERR_FP16 = 1, 2, 4


def nvfp4_quantize_1d(weight: torch.Tensor, amax: float | None = None, e4m3_max: int = 448, flags: int = 0):
    """miles/utils/nvfp4.py:54-82 -> (uint8 [M,K/2], e4m3fn [M,K/16], float32 []).  `flags`: Four Over Six options."""
    _check_cpu(weight)
    assert weight.dim() == 2
    w = weight.contiguous()
    M, K = w.shape
    assert K % 16 == 0
    if amax is None:
        amax = nvfp4_amax(w)
    q = torch.empty((M, K // 2), dtype=torch.uint8)
    s = torch.empty((M, K // 16), dtype=torch.uint8)
    lib().mqo_nvfp4_quant_ex(w.data_ptr(), _DTYPE[w.dtype], M, K, amax, e4m3_max, flags, q.data_ptr(), s.data_ptr())
    g = torch.tensor(nvfp4_global_decode_scale(amax, e4m3_max), dtype=torch.float32)
    return q, s.view(torch.float8_e4m3fn), g


def nvfp4_quantize_1d_pair(first: torch.Tensor, second: torch.Tensor, e4m3_max: int = 448, flags: int = 0):
    """miles/utils/nvfp4.py:85-114: one amax over both tensors."""
    amax = max(nvfp4_amax(first), nvfp4_amax(second))
    return nvfp4_quantize_1d(first, amax, e4m3_max, flags), nvfp4_quantize_1d(second, amax, e4m3_max, flags)


# --------------------------------------------------------------------------
# scalar / vector conversion helpers
# --------------------------------------------------------------------------
def f32_to_e4m3fn(x: torch.Tensor, sat: bool = False) -> torch.Tensor:
    x = x.contiguous().float()
    out = torch.empty(x.shape, dtype=torch.uint8)
    lib().mqo_f32_to_e4m3fn_vec(x.data_ptr(), x.numel(), out.data_ptr(), int(sat))
    return out


def f32_to_e2m1(x: torch.Tensor) -> torch.Tensor:
    x = x.contiguous().float()
    out = torch.empty(x.shape, dtype=torch.uint8)
    lib().mqo_f32_to_e2m1_vec(x.data_ptr(), x.numel(), out.data_ptr())
    return out


def f32_to_bf16_bits(x: torch.Tensor) -> torch.Tensor:
    x = x.contiguous().float()
    out = torch.empty(x.shape, dtype=torch.int16)
    lib().mqo_f32_to_bf16_vec(x.data_ptr(), x.numel(), out.data_ptr())
    return out


def f32_to_e8m0(x: torch.Tensor) -> torch.Tensor:
    x = x.contiguous().float()
    out = torch.empty(x.shape, dtype=torch.uint8)
    lib().mqo_f32_to_e8m0_vec(x.data_ptr(), x.numel(), out.data_ptr())
    return out


def fnv1a64(t: torch.Tensor) -> int:
    t = t.contiguous()
    return int(lib().mqo_fnv1a64(t.data_ptr(), t.numel() * t.element_size()))


def fused_nvfp4_qdq(x: torch.Tensor, amax=None, e4m3_max: int = 448, flags: int = 0) -> torch.Tensor:
    """miles/kernels/quant/nvfp4_qdq.py:1220-1229 -> tensor in the dtype of x."""
    _check_cpu(x)
    assert x.dtype in (torch.bfloat16, torch.float16) and x.numel() % 16 == 0
    xc = x.contiguous()
    a = float(nvfp4_amax(xc)) if amax is None else float(amax)
    out = torch.empty_like(xc)
    lib().mqo_nvfp4_qdq(xc.data_ptr(), _DTYPE[xc.dtype], xc.numel(), a, e4m3_max, flags, out.data_ptr())
    return out
