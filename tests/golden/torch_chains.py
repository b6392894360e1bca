"""The reference's tensor-op chains for every quantizer on the path, written with plain torch ops in the
reference's own order so that PyTorch's CPU kernels (float8 / bfloat16 casts, IEEE division, clamp, round-half-even)
produce the expected bytes.  Used by tests/test_oracle_pins.py to pin the C oracle and by make_fixtures.py to
write the golden files in this directory.  Nothing here calls the oracle or the HIP library.

MXFP8 and the NVFP4 block arithmetic restate Transformer Engine's published algorithm (its source is not in the
reference tree); fp8_blockwise_cast restates the Triton expressions with IEEE division.
"""

import torch

F8 = torch.float8_e4m3fn
FP8_MAX = 448.0


def torch_block_fp8(weight, block_size):
    bn, bk = block_size
    n, k = weight.shape
    nt, kt = -(-n // bn), -(-k // bk)
    padded = torch.nn.functional.pad(weight, (0, kt * bk - k, 0, nt * bn - n), mode="constant", value=0.0)
    tiles = padded.reshape(nt, bn, kt, bk)
    amax = tiles.abs().max(dim=1, keepdim=True)[0].max(dim=3, keepdim=True)[0]
    scale = amax.to(torch.float32) / FP8_MAX
    q = (tiles / scale).clamp(min=-FP8_MAX, max=FP8_MAX).reshape(nt * bn, kt * bk).to(F8)
    return q[:n, :k].clone(), scale.reshape(nt, kt)


def torch_fp8_blockwise_cast(x, bm=128, bn=128):
    m, n = x.shape
    mt, nt = -(-m // bm), -(-n // bn)
    xf = torch.zeros((mt * bm, nt * bn), dtype=torch.float32)
    xf[:m, :n] = x.float()
    tiles = xf.reshape(mt, bm, nt, bn)
    absmax = torch.maximum(tiles.abs().amax(dim=(1, 3), keepdim=True), torch.tensor(1e-10, dtype=torch.float32))
    x_s = absmax / torch.tensor(FP8_MAX, dtype=torch.float32)
    s_inv = torch.tensor(1.0, dtype=torch.float32) / x_s
    y = (tiles * s_inv).clamp(-FP8_MAX, FP8_MAX).reshape(mt * bm, nt * bn)[:m, :n].to(F8)
    return y, x_s.reshape(mt, nt)


def torch_dequant_fp8_block(weight, scale_inv):
    rows, cols = weight.shape
    scale = scale_inv.float().repeat_interleave(128, dim=0)[:rows].repeat_interleave(128, dim=1)
    return (weight.float() * scale[:, :cols]).to(torch.bfloat16)


def torch_mxfp8(w):
    k = w.shape[-1]
    x = w.float().reshape(-1, k // 32, 32)
    amax = x.abs().amax(dim=-1, keepdim=True)
    v = amax * torch.tensor(0x3B124925, dtype=torch.int32).view(torch.float32)  # f32(1/448)
    mant, expo = torch.frexp(v)
    e_unb = torch.where(mant == 0.5, expo - 1, expo)            # ceil(log2 v)
    e = torch.where(v == 0, torch.zeros_like(e_unb), (e_unb + 127).clamp(0, 254))
    # v below 2^-127 has no representable ceil power in E8M0: code 0 up to 2^-127, code 1 above
    e = torch.where((v > 0) & (v <= 2.0**-127), torch.zeros_like(e), e)
    e = torch.where((v > 2.0**-127) & (v <= 2.0**-126), torch.ones_like(e), e)
    inv = torch.where(e == 0, torch.ones_like(v), torch.ldexp(torch.ones_like(v), 127 - e))
    q = (x * inv).clamp(-FP8_MAX, FP8_MAX).to(F8)
    return q.reshape(w.shape), e.to(torch.uint8).reshape(*w.shape[:-1], k // 32)


def torch_block_quant_dequant_f32(codes, scale):
    """SGLang's block_quant_dequant(x_q, x_s, [128, 128], torch.float32) as the reference calls it
    (tools/convert_hf_to_mxfp8.py:187-189): the tile scales repeated over their tiles, cropped, one fp32 multiply."""
    n, k = codes.shape[-2:]
    wide = scale.repeat_interleave(128, dim=-2).repeat_interleave(128, dim=-1)[..., :n, :k]
    return codes.to(torch.float32) * wide


def torch_fp8_block_to_mxfp8(codes, scale):
    """tools/convert_hf_to_mxfp8.py:187-190: dequantize to fp32, quantize again as MXFP8."""
    nt, kt = -(-codes.shape[-2] // 128), -(-codes.shape[-1] // 128)
    return torch_mxfp8(torch_block_quant_dequant_f32(codes, scale[..., :nt, :kt].contiguous()).contiguous())


def torch_scales_pow2(scale_fp32):
    """tools/convert_hf_to_mxfp8.py:81-84."""
    bits = scale_fp32.contiguous().view(torch.int32)
    return (not torch.any((bits & 0x007FFFFF) != 0).item()) and (not torch.any(bits < 0).item())


def torch_source_scale_bytes(scale):
    """tools/convert_hf_to_mxfp8.py:85 (fp32 powers of two) / :74-75 (stored bytes)."""
    if scale.dtype == torch.uint8:
        return scale
    return ((scale.contiguous().view(torch.int32) >> 23) & 0xFF).to(torch.uint8)


def torch_source_fp8_to_mxfp8_scale_u8(weight_shape, scale_u8):
    """tools/convert_hf_to_mxfp8.py:98-102."""
    n, k = weight_shape[-2:]
    wide = scale_u8.repeat_interleave(128, dim=-2).repeat_interleave(4, dim=-1)
    return wide[..., :n, : k // 32].contiguous()


def torch_quantize_mxfp4(weight, group_size):
    """miles/utils/mxfp4.py:11-31."""
    blocks = weight.reshape(-1, group_size)
    amax = blocks.abs().amax(dim=-1, keepdim=True).float()
    scale_exp = torch.ceil(torch.log2(amax / 6.0)).clamp_(-127, 127)
    normalized = blocks.float() * torch.exp2(-scale_exp)
    magnitude = torch.zeros_like(normalized, dtype=torch.uint8)
    for bound in (0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0):
        magnitude.add_(normalized.abs() > bound)
    encoded = magnitude | (torch.signbit(normalized).to(torch.uint8) << 3)
    packed = encoded[:, 0::2] | (encoded[:, 1::2] << 4)
    packed = packed.reshape(*weight.shape[:-1], weight.shape[-1] // 2).contiguous()
    scale = (scale_exp + 127).to(torch.uint8)
    return packed, scale.reshape(*weight.shape[:-1], weight.shape[-1] // group_size).contiguous()


def torch_dequantize_mxfp4(weight_packed, weight_scale, group_size):
    """miles/utils/mxfp4.py:34-59."""
    unpacked = torch.empty(*weight_packed.shape[:-1], weight_packed.shape[-1] * 2, dtype=torch.uint8)
    unpacked[..., 0::2] = weight_packed & 0x0F
    unpacked[..., 1::2] = (weight_packed >> 4) & 0x0F
    signs = 1.0 - 2.0 * ((unpacked & 0b1000) >> 3).float()
    values = torch.tensor((0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0), dtype=torch.float32)
    dequantized = (signs * values[(unpacked & 0b0111).long()]).reshape(-1, group_size)
    scales = torch.exp2(weight_scale.float().reshape(-1, 1) - 127.0)
    return (dequantized * scales).reshape(unpacked.shape).to(torch.bfloat16).contiguous()


def torch_fake_int4_sym(x, G):
    """fake_int4_quant_cuda.cu:216-252 as fp32 tensor ops on the CPU (true division)."""
    m, n = x.shape
    xf = x.float().reshape(m, n // G, G)
    amax = xf.abs().amax(dim=-1, keepdim=True)
    scale = torch.maximum(amax * torch.tensor(1.0 / 7.0, dtype=torch.float32), torch.tensor(1e-5, dtype=torch.float32))
    out = torch.round(xf / scale)
    return out.reshape(m, n).to(x.dtype), scale.reshape(m, n // G).to(x.dtype)


def torch_pack_layer_python_half(w, scale, G):
    """quantizer_compressed_tensors.py:237-264 given the kernel's (w, scale) in the input dtype."""
    m, k = w.shape
    w4 = w.view(m, 1, k // G, G)
    s4 = scale.view(m, 1, k // G, 1)
    deq = (w4 * s4).view(m, k)
    scale2 = s4.view(m, -1).contiguous()
    x = deq.unflatten(-1, (k // G, G))
    scaled = x / scale2.unsqueeze(-1)
    q = torch.round(torch.clamp(scaled, -128, 127)).to(torch.int8).flatten(start_dim=-2)
    value = (q + 8).to(torch.uint8)
    reshaped = value.view(m, k // 8, 8).to(torch.int32)
    shifts = torch.arange(8, dtype=torch.int32) * 4
    return (reshaped << shifts).sum(dim=2, dtype=torch.int32), scale2


def torch_fake_int4_asym(x, G):
    """fake_int4_quant_cuda.cu:216-254, asymmetric branch, as fp32 tensor ops on the CPU."""
    m, n = x.shape
    xf = x.float().reshape(m, n // G, G)
    mx, mn = xf.amax(dim=-1, keepdim=True), xf.amin(dim=-1, keepdim=True)
    scale = torch.maximum((mx - mn) * torch.tensor(1.0 / 15.0, dtype=torch.float32),
                          torch.tensor(1e-5, dtype=torch.float32))
    zero = torch.clamp(-torch.round(mn / scale), 0.0, 15.0) + 0.0   # device max(-0, +0) = +0
    out = torch.round(xf / scale) + zero
    return out.reshape(m, n).to(x.dtype), scale.reshape(m, n // G).to(x.dtype), zero.reshape(m, n // G).to(x.dtype)


def torch_pack_layer_asym_python_half(w, scale, zp, G):
    """quantizer_compressed_tensors.py:237-264 with sym=False, the reference's tensor ops in their order."""
    m, k = w.shape
    w4 = w.view(m, 1, k // G, G)
    s4 = scale.view(m, 1, k // G, 1)
    z4 = zp.view(m, 1, k // G, 1)
    deq = ((w4 - z4) * s4).view(m, k)
    scale2 = s4.view(m, -1).contiguous()
    zp2 = z4.view(m, -1)
    zeros = zp2.t().contiguous().to(torch.float32).to(torch.int32)
    zeros = zeros.reshape(-1, zeros.shape[1] // 8, 8)
    zeros = zeros << (torch.tensor([0, 4, 1, 5, 2, 6, 3, 7]) * 4)
    packed_zp = torch.sum(zeros, dim=-1).to(torch.int32)
    x = deq.unflatten(-1, (k // G, G))
    scaled = x / scale2.unsqueeze(-1)
    scaled += zp2.unsqueeze(-1).to(x.dtype)
    q = torch.round(torch.clamp(scaled, 0, 255)).to(torch.uint8).flatten(start_dim=-2)
    reshaped = q.view(m, k // 8, 8).to(torch.int32)
    shifts = torch.arange(8, dtype=torch.int32) * 4
    return (reshaped << shifts).sum(dim=2, dtype=torch.int32), scale2, packed_zp


def torch_nvfp4(w, amax=None):
    """Block arithmetic of miles/kernels/quant/nvfp4_qdq.py:716-743,859-889 in fp32 tensor ops."""
    f32 = torch.float32
    m, k = w.shape
    x = w.float().reshape(m, k // 16, 16)
    if amax is None:
        amax = x.abs().max()
    amax = torch.as_tensor(amax, dtype=f32)
    flt_max = torch.tensor(torch.finfo(f32).max)
    s_enc = torch.min(torch.tensor(2688.0, dtype=f32) / amax, flt_max)
    if amax == 0 or s_enc == 0:
        s_enc = torch.tensor(1.0, dtype=f32)
    s_dec = torch.tensor(1.0, dtype=f32) / s_enc
    sixth = torch.tensor(0x3E2AAAAB, dtype=torch.int32).view(f32)
    bmax = x.abs().amax(dim=-1, keepdim=True)
    s_hp = torch.where(bmax == 0, torch.zeros_like(bmax), bmax * (s_enc * sixth))
    s8 = s_hp.clamp(max=FP8_MAX).to(F8)
    inv = torch.min(torch.tensor(1.0, dtype=f32) / (s8.float() * s_dec), flt_max)
    y = x * inv
    mag = y.abs().clamp(max=6.0)
    step = torch.where(mag < 2.0, 0.5, torch.where(mag < 4.0, 1.0, 2.0))
    val = torch.round(mag / step) * step
    code = torch.bucketize(val, torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])).to(torch.uint8)
    code = code | (torch.signbit(y).to(torch.uint8) << 3)
    code = code.reshape(m, k)
    return code[:, 0::2] | (code[:, 1::2] << 4), s8.reshape(m, k // 16)


def torch_fake_quant_reference(x, kind):
    """The torch statement the reference's own test checks its kernels against, exactly
    (tests/fast-gpu/kernels/quant/test_fake_quant.py:24-49): fp8 / fp4 with power-of-two scales over 32-wide blocks,
    fp4 with e4m3 scales over 16-wide blocks ("compressed_kv")."""
    def ceil_pow2(value):
        mantissa, exponent = torch.frexp(value)
        return torch.ldexp(torch.ones_like(value), torch.where(mantissa == 0.5, exponent - 1, exponent))

    def round_to_fp4_grid(scaled):
        magnitude = scaled.abs()
        step = torch.where(magnitude < 2.0, 0.5, torch.where(magnitude < 4.0, 1.0, 2.0))
        return torch.round(magnitude / step) * step * torch.sign(scaled)

    block = 16 if kind == "compressed_kv" else 32
    blocks = x.float().reshape(-1, block)
    amax = blocks.abs().amax(dim=1, keepdim=True)
    if kind == "compressed_kv":
        scale = (amax / 6.0).clamp(2.0**-9, FP8_MAX).to(F8).float()
        quantized = round_to_fp4_grid((blocks / scale).clamp(-6.0, 6.0))
    elif kind == "fp4":
        scale = ceil_pow2(amax.clamp(min=6 * 2.0**-126) / 6.0)
        quantized = round_to_fp4_grid((blocks / scale).clamp(-6.0, 6.0))
    else:
        scale = ceil_pow2(amax.clamp(min=1e-4) / FP8_MAX)
        quantized = (blocks / scale).clamp(-FP8_MAX, FP8_MAX).to(F8).float()
    return (quantized * scale).reshape(x.shape).to(x.dtype)


def torch_cast_e2m1fn_to_e4m3fn(x, scale):
    """tools/convert_mxfp4_to_fp8.py:30-49, the reference's tensor ops in their order (scale: float8_e8m0fnu)."""
    table = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0])
    out_dim, in_dim = x.size(0), x.size(1) * 2
    x = x.view(torch.uint8)
    x = torch.stack([table[(x & 0x0F).long()], table[(x >> 4).long()]], dim=-1).reshape(out_dim, in_dim)
    b_out, b_in = out_dim // 128, in_dim // 128
    x = x.view(b_out, 128, b_in, 128).transpose(1, 2)
    scale = scale.float().view(b_out, 128, b_in, -1).transpose(1, 2).flatten(2)
    tile_scale = scale.amax(dim=-1, keepdim=True) / 2**6
    offset = (scale / tile_scale).unflatten(-1, (128, -1)).repeat_interleave(32, dim=-1)
    x = (x * offset).transpose(1, 2).reshape(out_dim, in_dim)
    return x.to(F8), tile_scale.squeeze(-1).float()


def torch_nvfp4_qdq(x, amax=None):
    """Standard fused QDQ of miles/kernels/quant/nvfp4_qdq.py: torch_nvfp4 codes and block scales, then
    value * RN(RN(f32(s8) * amax) * f32(1/2688)) cast to the input dtype (:993-1029)."""
    m, k = x.shape
    if amax is None:
        amax = x.float().abs().max()
    amax = torch.as_tensor(amax, dtype=torch.float32)
    packed, s8 = torch_nvfp4(x, amax)
    codes = torch.stack([packed & 0xF, packed >> 4], dim=-1).reshape(m, k)
    table = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0])
    final = (s8.float() * amax) * torch.tensor(1.0 / 2688.0, dtype=torch.float32)
    return (table[codes.long()].reshape(m, k // 16, 16) * final.unsqueeze(-1)).reshape(m, k).to(x.dtype)


def torch_nvfp4_4over6(w, amax=None, e4m3_max=448, mse=False, fp16_error=False):
    """Four Over Six block scaling (miles/kernels/quant/nvfp4_qdq.py:893-990) with fp32 tensor ops: both candidates are
    quantized for every block, errors are accumulated element by element in fp32, map-to-4 wins on a strictly smaller
    error.  Returns (packed codes, e4m3 block scales)."""
    f32 = torch.float32
    m, k = w.shape
    x = w.float().reshape(m, k // 16, 16)
    if amax is None:
        amax = x.abs().max()
    amax = torch.as_tensor(amax, dtype=f32)
    flt_max = torch.tensor(torch.finfo(f32).max)
    numer = torch.tensor(float(e4m3_max * 6), dtype=f32)
    s_enc = torch.min(numer / amax, flt_max)
    if amax == 0 or s_enc == 0:
        s_enc = torch.tensor(1.0, dtype=f32)
    s_dec = torch.tensor(1.0, dtype=f32) / s_enc
    bmax = x.abs().amax(dim=-1, keepdim=True)
    s6_hp = (bmax / torch.tensor(6.0, dtype=f32)) * s_enc
    s4_hp = s6_hp * torch.tensor(1.5, dtype=f32)
    table = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])

    def candidate(s_hp):
        s8 = s_hp.clamp(max=FP8_MAX).to(F8)
        inv = torch.min(torch.tensor(1.0, dtype=f32) / (s8.float() * s_dec), flt_max)
        y = x * inv
        mag = y.abs().clamp(max=6.0)
        step = torch.where(mag < 2.0, 0.5, torch.where(mag < 4.0, 1.0, 2.0))
        val = torch.round(mag / step) * step
        code = torch.bucketize(val, table).to(torch.uint8) | (torch.signbit(y).to(torch.uint8) << 3)
        cand = torch.where(torch.signbit(y), -val, val)
        if fp16_error:
            diff = (cand.half() * s8.float().half()).float() - x * s_enc
        else:
            diff = ((cand * s8.float()) * amax) / torch.tensor(float(6 * e4m3_max), dtype=f32) - x
        term = diff * diff if mse else diff.abs()
        err = torch.zeros(m, k // 16, dtype=f32)
        for i in range(16):
            err = err + term[..., i]
        return code, s8, err

    c4, s4, e4 = candidate(s4_hp)
    c6, s6, e6 = candidate(s6_hp)
    pick4 = e4 < e6
    code = torch.where(pick4.unsqueeze(-1), c4, c6).reshape(m, k)
    s8 = torch.where(pick4.unsqueeze(-1), s4.view(torch.uint8), s6.view(torch.uint8)).view(F8)
    return code[:, 0::2] | (code[:, 1::2] << 4), s8.reshape(m, k // 16)


def torch_fake_int4_block(x, bm, bn, sym):
    """fake_int4_quant_cuda.cu for a general (bm, bn) block (:95-150 for (32,1), :159-259): tiles of the zero-padded
    matrix, fp32 arithmetic, outputs in the dtype of x."""
    m, n = x.shape
    gm, gn = -(-m // bm), -(-n // bn)
    xf = torch.zeros((gm * bm, gn * bn), dtype=torch.float32)
    xf[:m, :n] = x.float()
    t = xf.reshape(gm, bm, gn, bn)
    if sym:
        amax = t.abs().amax(dim=(1, 3), keepdim=True)
        scale = torch.maximum(amax * torch.tensor(1.0 / 7.0, dtype=torch.float32), torch.tensor(1e-5, dtype=torch.float32))
        zero = torch.zeros_like(scale)
        out = torch.round(t / scale)
    else:
        mx, mn = t.amax(dim=(1, 3), keepdim=True), t.amin(dim=(1, 3), keepdim=True)
        scale = torch.maximum((mx - mn) * torch.tensor(1.0 / 15.0, dtype=torch.float32), torch.tensor(1e-5, dtype=torch.float32))
        zero = torch.clamp(-torch.round(mn / scale), 0.0, 15.0) + 0.0
        out = torch.round(t / scale) + zero
    out = out.reshape(gm * bm, gn * bn)[:m, :n]
    return out.to(x.dtype), scale.reshape(gm, gn).to(x.dtype), zero.reshape(gm, gn).to(x.dtype)


def torch_per_block_cast_to_fp8(x):
    """SGLang's per_block_cast_to_fp8 as published (third party; its source is not in the reference tree):
    zero-padded 128x128 tiles, amax clamped at 1e-4, sf = 2^ceil(log2(amax / 448)), x * (1 / sf) cast to e4m3."""
    m, n = x.shape
    pm, pn = -(-m // 128) * 128, -(-n // 128) * 128
    x_padded = torch.zeros((pm, pn), dtype=x.dtype)
    x_padded[:m, :n] = x
    x_view = x_padded.view(-1, 128, pn // 128, 128)
    x_amax = x_view.abs().float().amax(dim=(1, 3), keepdim=True).clamp(1e-4)
    sf = torch.pow(2.0, torch.ceil(torch.log2((x_amax / 448.0).abs())))
    x_scaled = (x_view * (1.0 / sf)).to(F8)
    return x_scaled.view_as(x_padded)[:m, :n].contiguous(), sf.view(x_view.size(0), x_view.size(2))


def torch_act_quant(x, block_size, round_scale, inplace):
    """act_quant (miles/kernels/quant/fp8_act_quant.py:49-137) as torch CPU ops: 1 x block groups of the last
    dimension, amax floored at 1e-4, scale = amax * f32(1/448) (round_scale: rounded up to a power of two through
    frexp), fp32 division, clamp, e4m3 cast; `inplace` returns dtype(f32(code) * scale).  Returns (y, fp32 scales)."""
    n = x.shape[-1]
    xf = x.float().reshape(-1, n // block_size, block_size)
    amax = xf.abs().amax(dim=-1, keepdim=True).clamp(min=1e-4)
    s = amax * torch.tensor(1.0 / 448.0, dtype=torch.float32)
    if round_scale:
        mant, exp = torch.frexp(s)                      # s = mant * 2^exp, mant in [0.5, 1)
        s = torch.ldexp(torch.ones_like(s), torch.where(mant == 0.5, exp - 1, exp))
    code = (xf / s).clamp(-448.0, 448.0).to(F8)
    scales = s.reshape(*x.shape[:-1], n // block_size)
    if inplace:
        return (code.float() * s).to(x.dtype).reshape(x.shape), scales
    return code.reshape(x.shape), scales
