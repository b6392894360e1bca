"""Pins the CPU oracle (oracle/mq_oracle.c) BEFORE it is trusted as the parity checker.

Each oracle function is compared with evidence that does not come from the oracle:
  * PyTorch's own CPU routines (float8_e4m3fn / bfloat16 casts, true fp32 division, clamp,
    round-half-even, bf16 elementwise ops) chained exactly as the reference chains them;
  * the golden vectors and known-answer tests the reference's own tests hold for this path;
  * closed forms / invariants (decode tables, per-tile max == 448, ceil-to-power-of-two,
    constant rows, all 256 fp8 codes).
MXFP8 and the NVFP4 block arithmetic restate Transformer Engine (third party, source not in the
reference repository): the checks here fix them against the published closed form and an
independent torch restatement only -- "parity unpinned" against TE itself.
"""

import math

import numpy as np
import pytest
import torch

from miles_amd import workloads as W
from tests.golden.torch_chains import (torch_act_quant, torch_per_block_cast_to_fp8, torch_fake_int4_block, torch_nvfp4_4over6, torch_nvfp4_qdq, torch_cast_e2m1fn_to_e4m3fn, torch_fake_quant_reference, torch_block_fp8, torch_dequant_fp8_block, torch_dequantize_mxfp4,
                                       torch_fake_int4_asym, torch_fake_int4_sym, torch_fp8_blockwise_cast,
                                       torch_mxfp8, torch_nvfp4, torch_pack_layer_asym_python_half,
                                       torch_pack_layer_python_half, torch_quantize_mxfp4)

F8 = torch.float8_e4m3fn
FP8_MAX = 448.0


# ----------------------------------------------------------------------------------------------
# conversions
# ----------------------------------------------------------------------------------------------
def _interesting_floats() -> torch.Tensor:
    """Every (sign, exponent, top-3-mantissa) prefix with the low 20 bits at each rounding-decisive
    pattern, plus 2^22 random bit patterns."""
    hi = torch.arange(0, 1 << 12, dtype=torch.int64) << 20
    lows = torch.tensor([0x0, 0x1, 0x7FFFF, 0x80000, 0x80001, 0xFFFFF, 0x40000, 0xC0000], dtype=torch.int64)
    grid = (hi[:, None] | lows[None, :]).reshape(-1)
    g = torch.Generator().manual_seed(7)
    rnd = torch.randint(0, 1 << 32, (1 << 22,), generator=g, dtype=torch.int64)
    bits = torch.cat([grid, rnd])
    bits = torch.where(bits >= (1 << 31), bits - (1 << 32), bits).to(torch.int32)
    return bits.view(torch.float32)


def test_e4m3fn_cast_matches_torch(oracle):
    x = _interesting_floats()
    want = x.to(F8).view(torch.uint8)
    got = oracle.f32_to_e4m3fn(x)
    nan = torch.isnan(x)
    assert torch.equal(got[~nan], want[~nan])
    # NaN: magnitude 0x7F; torch keeps the sign bit
    assert torch.equal(got[nan] & 0x7F, torch.full_like(got[nan], 0x7F))
    assert torch.equal(got[nan], want[nan])


def test_e4m3fn_cast_known_answers(oracle):
    # PyTorch float8_e4m3fn semantics: RNE, subnormal step 2^-9, 464 ties to 448, >464 -> NaN code
    x = torch.tensor([2.0**-10, 1.5 * 2.0**-10, 17, 18, 19, 21, 448, 464, 465, float("nan"), -0.0])
    assert oracle.f32_to_e4m3fn(x).tolist() == [0, 1, 88, 89, 90, 90, 126, 126, 127, 127, 128]
    # saturating form: >=448 and inf clamp to 0x7E, NaN -> 0x7F
    y = torch.tensor([448.0, 464.0, 465.0, 1e30, float("inf"), -float("inf"), -500.0, float("nan")])
    assert oracle.f32_to_e4m3fn(y, sat=True).tolist() == [126, 126, 126, 126, 126, 254, 254, 127]


def test_e4m3fn_sat_equals_clamp_then_torch_cast(oracle):
    x = _interesting_floats()
    x = x[~torch.isnan(x)]
    want = x.clamp(-FP8_MAX, FP8_MAX).to(F8).view(torch.uint8)
    assert torch.equal(oracle.f32_to_e4m3fn(x, sat=True), want)


def test_e4m3fn_decode_table(oracle):
    codes = torch.arange(256, dtype=torch.uint8)
    want = codes.view(F8).float()
    got = torch.tensor([oracle.lib().mqo_e4m3fn_to_f32(int(c)) for c in codes])
    nan = torch.isnan(want)
    assert nan.sum() == 2 and torch.equal(torch.isnan(got), nan)
    assert torch.equal(got[~nan].view(torch.int32), want[~nan].view(torch.int32))


def test_bf16_rounding_matches_torch(oracle):
    x = _interesting_floats()
    hi = torch.arange(0, 1 << 16, dtype=torch.int64) << 16
    lows = torch.tensor([0x0, 0x1, 0x7FFF, 0x8000, 0x8001, 0xFFFF], dtype=torch.int64)
    grid = (hi[:, None] | lows[None, :]).reshape(-1)
    grid = torch.where(grid >= (1 << 31), grid - (1 << 32), grid).to(torch.int32).view(torch.float32)
    x = torch.cat([x, grid])
    x = x[~torch.isnan(x)]
    assert torch.equal(oracle.f32_to_bf16_bits(x), x.to(torch.bfloat16).view(torch.int16))


def test_e2m1_grid_ties_and_saturation(oracle):
    # closed form: grid {0,.5,1,1.5,2,3,4,6}; ties go to the even code; satfinite; NaN -> +6 code
    x = torch.tensor([0.0, 0.25, 0.2500001, 0.5, 0.75, 1.0, 1.25, 1.2500001, 1.5, 1.75, 2.0, 2.5, 2.5000002, 3.0,
                      3.5, 4.0, 5.0, 5.0000005, 6.0, 7.0, 1e30, float("inf"), float("nan"), -0.0, -0.25, -0.75,
                      -6.5, -float("inf")])
    want = [0, 0, 1, 1, 2, 2, 2, 3, 3, 4, 4, 4, 5, 5, 6, 6, 6, 7, 7, 7, 7, 7, 7, 8, 8, 10, 15, 15]
    assert oracle.f32_to_e2m1(x).tolist() == want


def test_e2m1_matches_round_to_fp4_grid(oracle):
    # independent statement of RNE on the e2m1 grid: tests/fast-gpu/kernels/quant/test_fake_quant.py:29-32
    g = torch.Generator().manual_seed(3)
    x = torch.cat([8 * torch.rand(1 << 18, generator=g) - 4, torch.linspace(-7, 7, 2241)])
    mag = x.abs().clamp(max=6.0)
    step = torch.where(mag < 2.0, 0.5, torch.where(mag < 4.0, 1.0, 2.0))
    want = torch.round(mag / step) * step
    codes = oracle.f32_to_e2m1(x)
    table = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])
    assert torch.equal(table[(codes & 7).long()], want)
    assert torch.equal((codes >> 3).bool(), torch.signbit(x))


def test_e8m0_is_ceil_pow2(oracle):
    # ceil-to-power-of-two, corroborated by miles/kernels/quant/fake_quant.py:15-21 and the frexp form
    # of tests/fast-gpu/kernels/quant/test_fake_quant.py:24-26
    g = torch.Generator().manual_seed(5)
    v = torch.cat([torch.rand(1 << 16, generator=g) * 10 ** (torch.rand(1 << 16, generator=g) * 60 - 30),
                   2.0 ** torch.arange(-120, 120, dtype=torch.float32)])
    mant, expo = torch.frexp(v)
    p2 = torch.ldexp(torch.ones_like(v), torch.where(mant == 0.5, expo - 1, expo))
    want = (torch.log2(p2).round() + 127).to(torch.uint8)
    assert torch.equal(oracle.f32_to_e8m0(v), want)
    special = torch.tensor([0.0, float("inf"), float("nan"), 2.0**-127, 1.5 * 2.0**-127, 2.0**-126, 3e38])
    assert oracle.f32_to_e8m0(special).tolist() == [0, 254, 255, 0, 1, 1, 254]


# ----------------------------------------------------------------------------------------------
# A-1a block_fp8 : tools/convert_hf_to_fp8.py:39-70 chained through torch's CPU kernels
# ----------------------------------------------------------------------------------------------


def _same_fp8(a, b):
    return torch.equal(a.view(torch.uint8), b.view(torch.uint8))


@pytest.mark.parametrize("shape", W.SMALL_REFERENCE_SHAPES + [(130, 257), (1, 1), (127, 129)])
@pytest.mark.parametrize("kind", W.PATTERNS)
def test_block_fp8_matches_torch_chain(oracle, shape, kind):
    w = W.reference_pattern(kind, shape, spread=512.0, amplitude=16.0)
    q, s = oracle.block_fp8(w, (128, 128))
    q_t, s_t = torch_block_fp8(w, (128, 128))
    assert torch.equal(s.view(torch.int32), s_t.view(torch.int32))
    assert _same_fp8(q, q_t)


def test_block_fp8_c1_slice_with_zero_tile(oracle):
    w = W.gaussian_outliers((384, 512), std=0.02, p_outlier=0.001, gain=20.0, seed=1001)
    w[128:256, 128:256] = 0
    w[300, 7] = -0.0
    q, s = oracle.block_fp8(w, (128, 128))
    q_t, s_t = torch_block_fp8(w, (128, 128))
    assert torch.equal(s.view(torch.int32), s_t.view(torch.int32)) and _same_fp8(q, q_t)
    # scale 0 and 0/0: every byte of the zero tile is the negative NaN code
    assert s[1, 1].item() == 0.0
    assert torch.all(q.view(torch.uint8)[128:256, 128:256] == 0xFF)
    # invariant: a tile with amax > 0 reaches +-448 somewhere
    dec = q.float()
    for ti in range(3):
        for tj in range(4):
            if (ti, tj) != (1, 1):
                assert dec[ti * 128:(ti + 1) * 128, tj * 128:(tj + 1) * 128].abs().max().item() == FP8_MAX


def test_block_fp8_other_block_sizes_and_dtypes(oracle):
    g = torch.Generator().manual_seed(11)
    for dtype in (torch.bfloat16, torch.float16, torch.float32):
        w = (0.05 * torch.randn((96, 160), generator=g)).to(dtype)
        for bs in ((32, 32), (64, 128), (128, 64)):
            q, s = oracle.block_fp8(w, bs)
            q_t, s_t = torch_block_fp8(w, bs)
            assert torch.equal(s, s_t) and _same_fp8(q, q_t), (dtype, bs)


def test_tensor_and_channel_fp8_match_torch_chain(oracle):
    # tools/convert_hf_to_fp8.py:73-86
    g = torch.Generator().manual_seed(12)
    for dtype in (torch.bfloat16, torch.float32):
        w = (0.02 * torch.randn((64, 96), generator=g)).to(dtype)
        w[3] = 0
        s_t = w.abs().max().clamp(min=1e-12).to(torch.float32) / FP8_MAX
        q_t = (w / s_t).clamp(min=-FP8_MAX, max=FP8_MAX).to(F8)
        q, s = oracle.tensor_fp8(w)
        assert torch.equal(s, s_t.view(1)) and _same_fp8(q, q_t)
        s_c = w.abs().max(dim=-1, keepdim=True)[0].clamp(min=1e-12).to(torch.float32) / FP8_MAX
        q_c = (w / s_c).clamp(min=-FP8_MAX, max=FP8_MAX).to(F8)
        q, s = oracle.channel_fp8(w)
        assert torch.equal(s, s_c) and _same_fp8(q, q_c)


# ----------------------------------------------------------------------------------------------
# A-1b fp8_blockwise_cast : miles/kernels/quant/fp8_blockwise.py:51-58 with IEEE division
# ----------------------------------------------------------------------------------------------


@pytest.mark.parametrize("shape", W.SMALL_REFERENCE_SHAPES + [(130, 257)])
@pytest.mark.parametrize("kind", W.PATTERNS)
def test_fp8_blockwise_cast_matches_torch_chain(oracle, shape, kind):
    x = W.reference_pattern(kind, shape, spread=512.0, amplitude=16.0)
    y, s = oracle.fp8_blockwise_cast(x)
    y_t, s_t = torch_fp8_blockwise_cast(x)
    assert torch.equal(s.view(torch.int32), s_t.view(torch.int32)) and _same_fp8(y, y_t)
    if kind == "zeros":  # epsilon floor: scale 1e-10/448, codes 0
        assert torch.all(y.view(torch.uint8) == 0) and s[0, 0].item() == pytest.approx(1e-10 / 448, rel=1e-6)


def test_fp8_blockwise_cast_strided_input(oracle):
    base = W.gaussian_outliers((256, 300), std=0.02, p_outlier=0.001, gain=20.0, seed=5)
    for view in (base[:, :256], base.t(), base[::2, 1::2]):
        y, s = oracle.fp8_blockwise_cast(view)
        y_t, s_t = torch_fp8_blockwise_cast(view.contiguous())
        assert torch.equal(s, s_t) and _same_fp8(y, y_t)


# ----------------------------------------------------------------------------------------------
# A-5 dequant : tools/fp8_cast_bf16.py:15-40 == tools/convert_mimo_v2_to_bf16.py:44-47
# ----------------------------------------------------------------------------------------------


def test_dequant_all_codes_random_scales(oracle):
    g = torch.Generator().manual_seed(21)
    codes = torch.arange(256, dtype=torch.uint8).repeat(300, 2)[:, :400].contiguous()  # [300,400]
    s = torch.exp(torch.randn((3, 4), generator=g) * 4).float()
    y = oracle.weight_dequant(codes.view(F8), s)
    y_t = torch_dequant_fp8_block(codes.view(F8), s)
    nan = torch.isnan(y_t)
    assert torch.equal(torch.isnan(y), nan)
    assert torch.equal(y.view(torch.int16)[~nan], y_t.view(torch.int16)[~nan])


def test_quant_dequant_round_trip_as_reference_test(oracle):
    # tests/fast/tools/test_convert_mimo_v2_to_bf16.py:17-54: quantise with clamp(1e-12), dequantise, compare
    # exactly with float(q) * scale -> bf16 and loosely with the source.
    g = torch.Generator().manual_seed(22)
    weight = torch.randn((448, 256), generator=g)
    padded = torch.zeros(512, 256)
    padded[:448] = weight
    blocks = padded.view(4, 128, 2, 128)
    scale = blocks.abs().amax(dim=(1, 3)).clamp(min=1e-12) / FP8_MAX
    quant = (blocks / scale[:, None, :, None]).view_as(padded)[:448].to(F8)
    out = oracle.weight_dequant(quant.contiguous(), scale.contiguous())
    expected = (quant.float() * scale.repeat_interleave(128, 0)[:448].repeat_interleave(128, 1)).to(torch.bfloat16)
    assert torch.equal(out, expected)
    assert (out.float() - weight).abs().max() < 0.07 * weight.abs().max()
    # and the oracle's own block quantiser agrees with that formula when no tile is all-zero
    q2, s2 = oracle.block_fp8(weight, (128, 128))
    assert torch.equal(s2, scale) and _same_fp8(q2, quant)


# ----------------------------------------------------------------------------------------------
# A-2 MXFP8 (closed form; Transformer Engine itself is not available -> parity unpinned vs TE)
# ----------------------------------------------------------------------------------------------


@pytest.mark.parametrize("shape", W.SMALL_REFERENCE_SHAPES)
@pytest.mark.parametrize("kind", W.PATTERNS)
def test_mxfp8_matches_closed_form(oracle, shape, kind):
    w = W.reference_pattern(kind, shape, spread=512.0, amplitude=16.0)
    q, s = oracle.mxfp8_quantize(w)
    q_t, s_t = torch_mxfp8(w)
    assert q.shape == w.shape and q.dtype == F8 and s.dtype == torch.uint8
    assert s.shape == (*w.shape[:-1], w.shape[-1] // 32)  # tests/fast-gpu/test_mxfp8_quantizer.py:165-168
    assert torch.equal(s, s_t) and _same_fp8(q, q_t)


def test_mxfp8_student_t_rows_and_invariants(oracle):
    w = W.student_t_rows((96, 2048), std=0.02, seed=3001)
    q, s = oracle.mxfp8_quantize(w)
    q_t, s_t = torch_mxfp8(w)
    assert torch.equal(s, s_t) and _same_fp8(q, q_t)
    # scale is the smallest power of two with amax/scale <= 448: decoded magnitudes lie in (224, 448]
    dec = q.float().reshape(96, 64, 32).abs().amax(dim=-1)
    nz = w.float().reshape(96, 64, 32).abs().amax(dim=-1) > 0
    assert torch.all(dec[nz] <= 448) and torch.all(dec[nz] >= 224)
    with pytest.raises(ValueError, match="must be divisible by 32"):
        oracle.mxfp8_quantize(torch.zeros(4, 48, dtype=torch.bfloat16))


# ----------------------------------------------------------------------------------------------
# MXFP4 (miles/utils/mxfp4.py) -- the reference is plain torch ops, restated here op for op
# ----------------------------------------------------------------------------------------------


def test_mxfp4_dequantize_reference_golden(oracle):
    # tests/fast/backends/megatron_utils/test_quantizer_mxfp4.py:6-16: nibble order, sign bit, E8M0 bias
    packed = torch.tensor([[0x10, 0x32, 0x54, 0x76]], dtype=torch.uint8)
    scales = torch.tensor([127, 128], dtype=torch.uint8)
    expected = torch.tensor([[0.0, 0.5, 1.0, 1.5, 4.0, 6.0, 8.0, 12.0]], dtype=torch.bfloat16)
    assert torch.equal(oracle.dequantize_mxfp4(packed, scales, 4), expected)


def test_mxfp4_dequantize_all_codes_all_scales(oracle):
    packed = torch.arange(256, dtype=torch.uint8).repeat(255, 1)            # [255, 256] -> 512 values per row
    scales = torch.arange(255, dtype=torch.uint8).repeat_interleave(16)     # group 32: 16 groups per row
    got = oracle.dequantize_mxfp4(packed, scales, 32)
    want = torch_dequantize_mxfp4(packed, scales, 32)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape,G", [((16, 64), 32), ((3, 128), 32), ((64, 64), 32), ((8, 2048), 32), ((4, 64), 16),
                                     ((5, 24), 4), ((2, 3, 64), 32)])
def test_mxfp4_quantize_matches_torch_chain(oracle, shape, G, dtype):
    w = W.student_t_rows((int(np.prod(shape[:-1])), shape[-1]), std=0.02, seed=6001).reshape(shape).to(dtype)
    flat = w.reshape(-1, shape[-1])
    flat[0, :G] = 0
    flat[1, :G] = torch.tensor([6.0, -6.0, 3.0, 0.25] * (G // 4)).to(dtype)          # amax/6 an exact power of two
    flat[2, :4] = torch.tensor([0.75, 1.75, 3.5, -0.0]).to(dtype); flat[2, 4] = 6.0    # ties round down; -0 keeps its sign
    packed, scale = oracle.quantize_mxfp4(w, G)
    packed_t, scale_t = torch_quantize_mxfp4(w, G)
    assert packed.shape == packed_t.shape and scale.shape == scale_t.shape
    assert torch.equal(scale, scale_t) and torch.equal(packed, packed_t)


def test_mxfp4_ties_and_signed_zero_known_answer(oracle):
    w = torch.tensor([[0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0, -0.0, -0.25, -0.75, 0.76, 0.26, 5.25, -6.0, 0.0]],
                     dtype=torch.bfloat16)
    packed, scale = oracle.quantize_mxfp4(w, 16)
    codes = torch.stack([packed & 0xF, packed >> 4], dim=-1).reshape(-1).tolist()
    assert scale.item() == 127
    assert codes == [0, 1, 2, 3, 4, 5, 6, 7, 8, 8, 9, 2, 1, 7, 15, 0]


def test_mxfp4_requantizing_a_checkpoint_is_the_identity(oracle):
    # tests/fast-gpu/test_quantizer_ci.py:41-60: any value an MXFP4 checkpoint can hold re-encodes to the same bits
    g = torch.Generator().manual_seed(11)
    packed = torch.randint(0, 256, (16, 64), dtype=torch.uint8, generator=g)
    scale = torch.randint(96, 144, (16, 4), dtype=torch.uint8, generator=g)
    weight = oracle.dequantize_mxfp4(packed, scale, 32)
    p2, s2 = oracle.quantize_mxfp4(weight, 32)
    assert torch.equal(oracle.dequantize_mxfp4(p2, s2, 32).view(torch.int16), weight.view(torch.int16))


def test_mxfp4_scale_exponent_from_bits_equals_float_log2_for_16_bit_inputs():
    # the gfx950 kernel reads ceil(log2(amax/6)) off the bits of the quotient; for every bf16 and fp16 amax this
    # equals ceil(log2f(.)) as the reference computes it
    for dt in (torch.bfloat16, torch.float16):
        bits = torch.arange(0, 0x7C00 if dt == torch.float16 else 0x7F80, dtype=torch.int32).to(torch.int16)
        amax = bits.view(dt).float()
        q = amax / 6.0
        want = torch.ceil(torch.log2(q)).clamp_(-127, 127) + 127
        u = q.view(torch.int32)
        e, m = u >> 23, u & 0x7FFFFF
        got = torch.where(e == 0, (m > 0x400000).to(torch.int32), torch.clamp(e + (m != 0).to(torch.int32), max=254))
        assert torch.equal(got, want.to(torch.int32))
    # bf16 fast path: the same byte read straight off the amax pattern, byte = E - 2 + (mantissa > 1.5), no division
    bits = torch.arange(0, 0x7F81, dtype=torch.int32)           # every finite bf16 magnitude and +inf
    q = bits.to(torch.int16).view(torch.bfloat16).float() / 6.0
    want = torch.ceil(torch.log2(q)).clamp_(-127, 127) + 127
    e, gt = bits >> 7, ((bits & 0x7F) > 0x40).to(torch.int32)
    got = torch.where(e == 255, torch.full_like(e, 254), torch.clamp(e - 2 + gt, min=0))
    assert torch.equal(got, want.to(torch.int32))


# ----------------------------------------------------------------------------------------------
# block fake quantization (miles/kernels/quant/fake_quant.py)
# ----------------------------------------------------------------------------------------------
def _fake_quant_input(dtype, seed=0):
    # the reference test's input (tests/fast-gpu/kernels/quant/test_fake_quant.py:55-60): six decades of magnitudes
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(3, 37, 512, generator=g) * torch.logspace(-3, 3, 512)).to(dtype)
    x[0, 0, :32] = 0
    return x


@pytest.mark.parametrize("kind", ["fp8", "fp4", "compressed_kv"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_fake_quant_matches_the_reference_tests_torch_statement(oracle, kind, dtype):
    for seed in (0, 1):
        x = _fake_quant_input(dtype, seed)
        x[1, 0, :64] = torch.tensor([-0.0, 0.0] * 32).to(dtype)
        x[1, 1, :8] = torch.tensor([448.0, -448.0, 6.0, -6.0, 3.5, 2.5, 0.75, -1e-30]).to(dtype)
        got = oracle.fake_quant(x, kind)
        want = torch_fake_quant_reference(x, kind)
        bits = torch.int32 if dtype == torch.float32 else torch.int16
        # the reference statement multiplies by torch.sign (0 for an exact zero); compare values, then zero signs apart
        assert torch.equal(got.float(), want.float())
        nz = want != 0
        assert torch.equal(got.view(bits)[nz], want.view(bits)[nz])


def test_fake_quant_known_answers(oracle):
    # one 32-block with amax 448: scale 1, the e4m3 grid itself
    x = torch.tensor([448.0, 17.0, 18.0, 19.0, 21.0, 0.3, -0.3, 1e-3] + [0.0] * 24, dtype=torch.float32)
    got = oracle.fake_quant(x, "fp8").tolist()
    assert got[:8] == [448.0, 16.0, 18.0, 20.0, 20.0, 0.3125, -0.3125, 0.001953125]
    # fp4: amax 6 -> scale 1; ties go to even codes, and an exact zero comes back as +0 whatever its sign
    x = torch.tensor([6.0, 0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, -0.0, -0.2] + [0.0] * 22, dtype=torch.float32)
    got = oracle.fake_quant(x, "fp4")
    assert got[:8].tolist() == [6.0, 0.0, 1.0, 1.0, 2.0, 2.0, 4.0, 4.0]
    assert got[8].item() == 0.0 and not torch.signbit(got[8]) and torch.signbit(got[9]) and got[9].item() == 0.0
    # compressed kv: a 16-block with amax 3 -> scale e4m3(0.5) = 0.5: values land on multiples of the fp4 grid * 0.5
    x = torch.tensor([3.0, 0.3, -1.1, 2.2] + [0.0] * 12, dtype=torch.float32)
    assert oracle.fake_quant(x, "compressed_kv")[:4].tolist() == [3.0, 0.25, -1.0, 2.0]



def _mxfp4_checkpoint_tensor(out_dim, in_dim, seed, lo=100, hi=140):
    g = torch.Generator().manual_seed(seed)
    packed = torch.randint(0, 256, (out_dim, in_dim // 2), dtype=torch.uint8, generator=g).view(torch.int8)
    scale = torch.randint(lo, hi, (out_dim, in_dim // 32), dtype=torch.uint8, generator=g).view(torch.float8_e8m0fnu)
    return packed, scale


@pytest.mark.parametrize("shape,lo,hi", [((128, 128), 100, 140), ((256, 384), 120, 128), ((128, 256), 0, 30), ((128, 128), 225, 255)])
def test_mxfp4_to_fp8_recode_matches_torch_chain(oracle, shape, lo, hi):
    packed, scale = _mxfp4_checkpoint_tensor(*shape, seed=41, lo=lo, hi=hi)
    y, ts = oracle.cast_e2m1fn_to_e4m3fn(packed, scale)
    y_t, ts_t = torch_cast_e2m1fn_to_e4m3fn(packed, scale)
    assert torch.equal(ts.view(torch.int32), ts_t.view(torch.int32)) and _same_fp8(y, y_t)
    # lossless whenever the scales of a tile span at most 2^3 (fp4 values need e4m3's 2^-6 .. 2^8 normal range):
    if hi - lo <= 8:
        deq = y.float().view(shape[0] // 128, 128, shape[1] // 128, 128) * ts[:, None, :, None]
        assert torch.equal(deq.reshape(shape).to(torch.bfloat16), oracle.dequantize_mxfp4(packed.view(torch.uint8), scale.view(torch.uint8), 32))



# ----------------------------------------------------------------------------------------------
# A-3 INT4
# ----------------------------------------------------------------------------------------------


@pytest.mark.parametrize("shape,G", [((4, 128), 128), ((16, 256), 128), ((64, 1024), 128), ((8, 7168), 128),
                                     ((16, 256), 32), ((5, 96), 32)])
def test_int4_matches_torch_chain(oracle, shape, G):
    w = W.gaussian_outliers(shape, std=0.015, p_outlier=0.0005, gain=30.0, seed=4001)
    w[0] = 0            # amax < 7e-5 -> scale floor 1e-5
    w[1, :G] = 3e-6
    out, scale, _ = oracle.fake_int4_quant(w, (1, G), True)
    out_t, scale_t = torch_fake_int4_sym(w, G)
    assert torch.equal(out.view(torch.int16), out_t.view(torch.int16))
    assert torch.equal(scale.view(torch.int16), scale_t.view(torch.int16))
    packed, pscale, zp = oracle.pack_layer(w, G)
    packed_t, pscale_t = torch_pack_layer_python_half(out_t, scale_t, G)
    assert zp is None and torch.equal(packed, packed_t) and torch.equal(pscale.view(torch.int16), pscale_t.view(torch.int16))
    # codes are rint(x/scale_f32)+8 in [1,15]: the bf16 round trip of pack_layer never moves a code
    nib = torch.stack([(packed >> (4 * i)) & 0xF for i in range(8)], dim=-1).reshape(shape)
    assert nib.min() >= 1 and nib.max() <= 15
    assert torch.equal(nib.to(torch.float32) - 8, out.float())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape,G", [((8, 128), 128), ((16, 256), 128), ((64, 1024), 128), ((8, 7168), 128),
                                     ((16, 256), 32), ((24, 192), 64)])
def test_int4_asym_matches_torch_chain(oracle, shape, G, dtype):
    w = W.gaussian_outliers(shape, std=0.015, p_outlier=0.0005, gain=30.0, seed=4101).to(dtype)
    w[0] = 0                      # range 0 -> scale floor
    w[1] = w[1].abs() + 0.25      # minimum far above zero: zero point clamps to 0 and codes run past 15
    w[2] = -w[2].abs() - 0.25     # maximum far below zero: zero point clamps to 15, codes clamp at 0
    w[3, :G] = 3e-6
    out, scale, zero = oracle.fake_int4_quant(w, (1, G), False)
    out_t, scale_t, zero_t = torch_fake_int4_asym(w, G)
    bits = torch.int32 if dtype == torch.float32 else torch.int16
    assert torch.equal(out.view(bits), out_t.view(bits))
    assert torch.equal(scale.view(bits), scale_t.view(bits))
    assert torch.equal(zero.view(bits), zero_t.view(bits))
    packed, pscale, pzp = oracle.pack_layer(w, G, sym=False)
    packed_t, pscale_t, pzp_t = torch_pack_layer_asym_python_half(out_t, scale_t, zero_t, G)
    assert torch.equal(packed, packed_t)
    assert torch.equal(pscale.view(bits), pscale_t.view(bits))
    assert pzp.shape == (shape[1] // G, shape[0] // 8) and torch.equal(pzp, pzp_t)


@pytest.mark.parametrize("G", [32, 128])
def test_int4_fp16_overflow_corners_match_torch_chain(oracle, G):
    # fp16 weights whose round trip in pack_layer leaves the finite range: a group maximum of 65504 (7 x scale rounds to
    # infinity in the symmetric chain) and ranges whose scale reaches 4096 (16 x scale in the asymmetric chain).  The
    # oracle against the torch op chains on exactly those groups, next to ordinary ones.
    w = W.gaussian_outliers((16, 4 * G), std=0.015, p_outlier=0.0, gain=1.0, seed=4501, dtype=torch.float16)
    w[1, :G] = torch.linspace(-65504, 65504, G).to(torch.float16)
    w[2, 5] = 65504.0
    w[3, :G] = 65504.0
    for i, top in enumerate((61000.0, 61400.0, 61440.0, 61500.0, 65504.0)):
        w[4 + i, :G] = torch.linspace(0.0, top, G).to(torch.float16)
        w[9 + i, G:2 * G] = torch.linspace(-top / 2, top / 2, G).to(torch.float16)
    out_t, scale_t = torch_fake_int4_sym(w, G)
    packed, pscale, _ = oracle.pack_layer(w, G)
    packed_t, pscale_t = torch_pack_layer_python_half(out_t, scale_t, G)
    assert torch.equal(packed, packed_t) and torch.equal(pscale.view(torch.int16), pscale_t.view(torch.int16))
    out_t, scale_t, zero_t = torch_fake_int4_asym(w, G)
    packed, pscale, pzp = oracle.pack_layer(w, G, sym=False)
    packed_t, pscale_t, pzp_t = torch_pack_layer_asym_python_half(out_t, scale_t, zero_t, G)
    assert torch.equal(packed, packed_t) and torch.equal(pscale.view(torch.int16), pscale_t.view(torch.int16))
    assert torch.equal(pzp, pzp_t)


def test_int4_asym_known_answers(oracle):
    # a group spanning [0, 15] exactly: scale 1, zero 0, codes are the values themselves
    row = torch.arange(16, dtype=torch.float32).repeat(8)
    w = row.to(torch.bfloat16).repeat(8, 1)
    w[1] = w[1] - 15          # [-15, 0]: zero point 15, same codes
    w[2] = w[2] - 7           # [-7, 8]: zero point 7
    packed, scale, pzp = oracle.pack_layer(w, 128, sym=False)
    want = sum(i << (4 * i) for i in range(8))
    want2 = sum((8 + i) << (4 * i) for i in range(8))
    for r in range(3):
        assert scale[r, 0].item() == 1.0
        assert (packed[r, 0].item() & 0xFFFFFFFF) == want and (packed[r, 1].item() & 0xFFFFFFFF) == want2
    # rows 0..7 carry zero points 0,15,7,0,0,0,0,0 in nibbles 0,4,1,5,2,6,3,7
    assert (pzp[0, 0].item() & 0xFFFFFFFF) == (0 << 0) | (15 << 16) | (7 << 4)

def torch_int4_dequantize_tensor(weight_packed, weight_scale, shape, group_size):
    """tools/convert_kimi_int4_to_bf16.py:57-86 with compressed-tensors' unpack_from_int32 written out
    (published algorithm: nibble i of word j -> element 8j+i, crop to the original width, subtract 8)."""
    m, k = shape
    unpacked = torch.zeros((weight_packed.shape[0], weight_packed.shape[1] * 8), dtype=torch.int32)
    for i in range(8):
        unpacked[:, i::8] = (weight_packed >> (4 * i)) & 0xF
    weight = (unpacked[:, :k] - 8).to(torch.int8)
    if group_size > 0:
        scales = torch.repeat_interleave(weight_scale.to(torch.float32), repeats=group_size, dim=1)
    else:
        scales = weight_scale.to(torch.float32).reshape_as(weight)
    return (weight.to(torch.float32) * scales).to(torch.bfloat16).contiguous()


@pytest.mark.parametrize("sdt", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape,G", [((4, 128), 128), ((16, 256), 32), ((3, 100), 20), ((64, 1024), 128)])
def test_int4_unpack_dequant_matches_torch_chain(oracle, shape, G, sdt):
    g = torch.Generator().manual_seed(31)
    m, k = shape
    packed = torch.randint(-2**31, 2**31 - 1, (m, -(-k // 8)), dtype=torch.int64, generator=g).to(torch.int32)
    scale = torch.exp(torch.randn((m, k // G), generator=g) * 3).to(sdt)
    got = oracle.int4_unpack_dequant(packed, scale, shape, G)
    want = torch_int4_dequantize_tensor(packed, scale, shape, G)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("flat", [False, True])
def test_int4_unpack_dequant_per_element_scales(oracle, flat):
    # group_size <= 0: the scale tensor has one entry per weight, in the weight's shape or flattened (:75-82)
    g = torch.Generator().manual_seed(32)
    m, k = 5, 44
    packed = torch.randint(-2**31, 2**31 - 1, (m, -(-k // 8)), dtype=torch.int64, generator=g).to(torch.int32)
    scale = torch.exp(torch.randn((m, k), generator=g) * 3).to(torch.bfloat16)
    if flat:
        scale = scale.reshape(-1)
    got = oracle.int4_unpack_dequant(packed, scale, (m, k), 0)
    want = torch_int4_dequantize_tensor(packed, scale, (m, k), 0)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_int4_unpack_inverts_pack_layer(oracle):
    # pack_layer followed by the unpacker gives q * scale in bf16 for every element (symmetric codes 1..15)
    w = W.gaussian_outliers((16, 512), std=0.015, p_outlier=0.0005, gain=30.0, seed=4001)
    packed, scale, _ = oracle.pack_layer(w, 128)
    out, fscale, _ = oracle.fake_int4_quant(w, (1, 128), True)
    deq = oracle.int4_unpack_dequant(packed, scale, w.shape, 128)
    want = (out.float().reshape(16, 4, 128) * scale.float().unsqueeze(-1)).reshape(16, 512).to(torch.bfloat16)
    assert torch.equal(deq.view(torch.int16), (want + 0.0).view(torch.int16))   # -0 * s: the unpacker has no -0 codes


def test_int4_asym_round_trip_is_identity_for_unclamped_codes():
    # The bf16 fast path of the asymmetric packer emits rint(x/s) + z directly when the zero point was not clamped
    # (codes in [0, 16]) and the bf16 scale is at most 1e37.  Exhaustive over every such scale, code and zero point:
    # the reference's chain  bf16((w1 - z) * s) / s + z -> clamp -> round  returns w1.
    bits = torch.arange(1, 0x7F80, dtype=torch.int32).to(torch.int16)
    sb = bits.view(torch.bfloat16)
    sb = sb[(sb.float() >= 9.9e-6) & (sb.float() <= 1e37)]
    for z in range(16):
        zt = torch.tensor(float(z), dtype=torch.bfloat16)
        for w1 in range(17):
            w = torch.tensor(float(w1), dtype=torch.bfloat16)
            r = ((w - zt) * sb) / sb + zt
            code = torch.round(torch.clamp(r, 0, 255)).to(torch.uint8)
            assert torch.all(code == w1), (z, w1)


def test_int4_asym_round_trip_in_fp16_is_identity_for_scales_below_4096():
    # The fp16 instance of the asymmetric packer emits rint(x/s) + z directly when the zero point was not clamped (codes
    # in [0, 16]) and the scale is below 4094 (so that fp16(s) < 4096).  Exhaustive over every fp16 scale from the floor,
    # every code and zero point: the reference's chain in fp16 returns the code for every scale below 4096 and fails
    # from 4096 on, where 16 x scale is no longer finite.
    sb = torch.arange(1, 0x7C00, dtype=torch.int32).to(torch.int16).view(torch.float16)
    sb = sb[sb >= torch.tensor(1e-5, dtype=torch.float16)]
    bad = torch.zeros(sb.shape, dtype=torch.bool)
    for z in range(16):
        zt = torch.tensor(float(z), dtype=torch.float16)
        for w1 in range(17):
            w = torch.tensor(float(w1), dtype=torch.float16)
            r = ((w - zt) * sb) / sb + zt
            bad |= torch.round(torch.clamp(r, 0, 255)).to(torch.int16) != w1
    assert bad.any() and sb[bad].min().item() == 4096.0 and not bad[sb.float() < 4096.0].any()


def test_int4_sym_round_trip_in_fp16_is_identity_below_the_overflow():
    # The fp16 instance of the symmetric packer emits rint(x/s) + 8 directly.  Exhaustive over every fp16 scale from the
    # floor fp16(1e-5) (a subnormal) upwards and the fifteen codes: the reference's chain in fp16
    # fp16(q * s) / s -> clamp -> round returns q unless 7 * s overflows, and the only group maximum whose scale
    # fp16(max * f32(1/7)) reaches that is 65504, which the kernel sends through the written-out chain.
    sb = torch.arange(1, 0x7C00, dtype=torch.int32).to(torch.int16).view(torch.float16)
    sb = sb[sb >= torch.tensor(1e-5, dtype=torch.float16)]
    assert sb.numel() == 31576 and sb[0].view(torch.int16).item() == 0xA8
    safe = sb[sb.float() < 9360.0]
    for q in range(-7, 8):
        qt = torch.tensor(float(q), dtype=torch.float16)
        r = (qt * safe) / safe
        code = torch.round(torch.clamp(r, -128, 127)).to(torch.int8)
        assert torch.all(code == q), q
    amax = torch.arange(1, 0x7C00, dtype=torch.int32).to(torch.int16).view(torch.float16).float()
    s = torch.maximum(amax * torch.tensor(1.0 / 7.0, dtype=torch.float32), torch.tensor(1e-5, dtype=torch.float32)).to(torch.float16)
    overflowing = amax[(s.float() >= 9360.0)]
    assert overflowing.tolist() == [65504.0]


def test_int4_constant_rows_known_answer(oracle):
    for c in (0.5, 0.013, 3.0):
        w = torch.full((2, 128), c, dtype=torch.bfloat16)
        w[1] = -w[1]
        packed, scale, _ = oracle.pack_layer(w, 128)
        assert torch.all(packed[0] == torch.tensor(0xFFFFFFFF - (1 << 32), dtype=torch.int64).to(torch.int32))  # code 15
        assert torch.all(packed[1] == 0x11111111)  # code 1
        want = (w[0, :1].float() * torch.tensor(1.0 / 7.0, dtype=torch.float32)).to(torch.bfloat16)
        assert torch.all(scale == want)


def test_pack_to_int32_nibble_order(oracle):
    # nibble i of each int32 is element 8j+i (sequential order): quantizer_compressed_tensors.py:171-175
    row = torch.tensor([[-7, -5, -3, -1, 1, 3, 5, 7] * 16], dtype=torch.float32)
    w = (row * (7.0 / 7.0)).to(torch.bfloat16)
    packed, scale, _ = oracle.pack_layer(w, 128)
    want = sum((int(v) + 8) << (4 * i) for i, v in enumerate([-7, -5, -3, -1, 1, 3, 5, 7]))
    assert scale[0, 0].item() == 1.0
    assert (packed[0, 0].item() & 0xFFFFFFFF) == want


# ----------------------------------------------------------------------------------------------
# A-4 NVFP4
# ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("e4m3_max", [256, 448])
def test_nvfp4_global_scale_vectors(oracle, e4m3_max):
    # tests/fast-gpu/test_nvfp4_quantizer.py:108-143: overflow clamp, underflow repair, NaN propagation
    values = torch.tensor([0.0, 1.0, 3.5, torch.finfo(torch.float32).tiny, torch.finfo(torch.float32).max,
                           float("inf"), -float("inf"), float("nan")], dtype=torch.float32)
    numerator = torch.tensor(float(e4m3_max), dtype=torch.float32) * torch.tensor(6.0, dtype=torch.float32)
    expected = torch.div(numerator, values)
    expected = torch.min(expected, torch.tensor(torch.finfo(torch.float32).max))
    expected = torch.where(expected == 0.0, torch.ones_like(expected), expected)
    for v, enc in zip(values.tolist(), expected.tolist()):
        got = oracle.nvfp4_global_encode_scale(v, e4m3_max)
        dec = oracle.nvfp4_global_decode_scale(v, e4m3_max)
        if math.isnan(enc):
            assert math.isnan(got) and math.isnan(dec)
        else:
            assert got == enc
            assert dec == torch.div(1.0, torch.tensor(enc, dtype=torch.float32)).item()
    # zero tensor: decode scale is 1/FLT_MAX, not 1
    assert oracle.nvfp4_global_decode_scale(0.0) == torch.div(1.0, torch.tensor(torch.finfo(torch.float32).max)).item()


@pytest.mark.parametrize("shape", W.SMALL_REFERENCE_SHAPES + [(1, 16), (3, 48), (31, 128)])
@pytest.mark.parametrize("kind", ["random", "boundary", "zeros", "signed_zeros", "maxes"])
def test_nvfp4_matches_torch_chain(oracle, shape, kind):
    w = W.reference_pattern(kind, shape, spread=12.0)
    if kind == "random" and shape[0] > 1:
        w[0].zero_()
    q, s, g = oracle.nvfp4_quantize_1d(w)
    q_t, s_t = torch_nvfp4(w)
    assert q.shape == (shape[0], shape[1] // 2) and s.shape == (shape[0], shape[1] // 16) and g.shape == ()
    assert _same_fp8(s, s_t) and torch.equal(q, q_t)
    amax = w.float().abs().max()
    enc = torch.div(2688.0, amax).clamp_max(torch.finfo(torch.float32).max)
    enc = torch.where(enc == 0.0, 1.0, enc)
    assert g.item() == torch.div(1.0, enc).item()   # miles/utils/nvfp4.py:19-39
    if kind == "signed_zeros":   # zero-amax blocks keep the sign bit: nibbles 0x8 / 0x0
        assert torch.all(q == 0x08) and torch.all(s.view(torch.uint8) == 0)


def test_nvfp4_nibble_order_golden(oracle):
    # tests/fast/backends/megatron_utils/test_quantizer_mxfp4.py:6-16 pins the e2m1 code table and that
    # element 2i sits in the low nibble: bytes 0x10 0x32 0x54 0x76 decode to codes 0..7 in order.
    row = torch.tensor([[0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0]])
    q, s, g = oracle.nvfp4_quantize_1d(row.to(torch.bfloat16))
    assert q[0].tolist() == [0x10, 0x32, 0x54, 0x76, 0x98, 0xBA, 0xDC, 0xFE]
    assert s.view(torch.uint8).item() == 0x7E      # block scale 448 = amax * (2688/amax) / 6
    assert g.item() == pytest.approx(6.0 / 2688.0, rel=1e-6)
    table = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    for c in range(16):
        assert oracle.lib().mqo_e2m1_to_f32(c) == (-table[c & 7] if c & 8 else table[c & 7])


def test_nvfp4_pair_shares_one_amax(oracle):
    gate = W.reference_pattern("random", (16, 64), spread=12.0, seed=1)
    up = 3 * W.reference_pattern("random", (24, 64), spread=12.0, seed=2)
    (gq, gs, gg), (uq, us, ug) = oracle.nvfp4_quantize_1d_pair(gate, up)
    cq, cs, cg = oracle.nvfp4_quantize_1d(torch.cat((gate, up), dim=0))
    assert torch.equal(torch.cat((gq, uq)), cq) and _same_fp8(torch.cat((gs, us)), cs)
    assert gg.item() == ug.item() == cg.item()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(1, 16), (3, 48), (16, 64), (64, 128), (128, 1024)])
@pytest.mark.parametrize("kind", ["random", "boundary", "zeros", "signed_zeros", "maxes"])
def test_nvfp4_qdq_matches_torch_chain(oracle, shape, kind, dtype):
    x = W.reference_pattern(kind, shape, dtype=dtype, spread=12.0)
    got = oracle.fused_nvfp4_qdq(x)
    want = torch_nvfp4_qdq(x)
    assert got.dtype == dtype and torch.equal(got.view(torch.int16), want.view(torch.int16))
    if kind == "random":      # dequantized values stay within half a grid step of the input, in units of the block scale
        assert (got.float() - x.float()).abs().max() <= x.float().abs().max() / 6.0 * 1.1


@pytest.mark.parametrize("e4m3_max,mse,fp16", [(448, False, False), (256, False, False), (256, True, False), (256, False, True),
                                               (448, True, True)])
@pytest.mark.parametrize("shape", [(1, 16), (3, 48), (16, 64), (64, 128), (128, 1024)])
@pytest.mark.parametrize("kind", ["random", "boundary", "zeros", "signed_zeros", "maxes"])
def test_nvfp4_four_over_six_matches_torch_chain(oracle, shape, kind, e4m3_max, mse, fp16):
    w = W.reference_pattern(kind, shape, spread=12.0)
    if kind == "random" and shape[0] > 1:
        w[0].zero_()
    flags = oracle.NVFP4_4OVER6 | (oracle.NVFP4_ERR_MSE if mse else 0) | (oracle.NVFP4_ERR_FP16 if fp16 else 0)
    q, s, g = oracle.nvfp4_quantize_1d(w, e4m3_max=e4m3_max, flags=flags)
    q_t, s_t = torch_nvfp4_4over6(w, e4m3_max=e4m3_max, mse=mse, fp16_error=fp16)
    assert _same_fp8(s, s_t) and torch.equal(q, q_t)
    if kind == "random" and shape[0] >= 16:
        # both candidates are really in play, and the chosen one never has the larger error
        q6, s6, _ = oracle.nvfp4_quantize_1d(w, e4m3_max=e4m3_max)
        assert 0 < (s.view(torch.uint8) != s6.view(torch.uint8)).sum() < s.numel()


@pytest.mark.parametrize("sym", [True, False])
@pytest.mark.parametrize("shape,block", [((64, 96), (32, 1)), ((70, 33), (32, 1)), ((16, 64), (4, 8)), ((18, 40), (2, 16)),
                                          ((8, 96), (1, 32)), ((40, 64), (8, 32)), ((5, 200), (1, 64))])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_int4_fake_quant_general_blocks_match_torch_chain(oracle, shape, block, sym, dtype):
    w = W.gaussian_outliers(shape, std=0.015, p_outlier=0.001, gain=30.0, seed=4003, dtype=dtype)
    w[0] = 0
    out, scale, zero = oracle.fake_int4_quant(w, block, sym)
    out_t, scale_t, zero_t = torch_fake_int4_block(w, block[0], block[1], sym)
    bits = torch.int32 if dtype == torch.float32 else torch.int16
    assert scale.shape == (-(-shape[0] // block[0]), -(-shape[1] // block[1]))
    assert torch.equal(out.view(bits), out_t.view(bits)) and torch.equal(scale.view(bits), scale_t.view(bits))
    if not sym:
        assert torch.equal(zero.view(bits), zero_t.view(bits))


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_fp16_inputs_match_the_torch_chains(oracle, seed):
    # the oracle's reading of fp16 tensors (what the fp16 instances of the GPU kernels are compared with): every block its
    # own magnitude, subnormals, the format's extremes and zero blocks, against the same torch op chains
    g = torch.Generator().manual_seed(9000 + seed)
    rows, cols = 130, 512
    ex = torch.randint(-20, 12, (rows, cols // 16, 1), generator=g).float()
    w = (torch.randn(rows, cols // 16, 16, generator=g) * torch.exp2(ex)).reshape(rows, cols).clamp(-65504, 65504).to(torch.float16)
    w[0] = 0
    w[1, :32] = torch.arange(1, 33, dtype=torch.int16).view(torch.float16)
    w[2, :4] = torch.tensor([65504.0, -65504.0, 0.0, -0.0], dtype=torch.float16)
    y, s = oracle.fp8_blockwise_cast(w)
    y_t, s_t = torch_fp8_blockwise_cast(w)
    assert torch.equal(s.view(torch.int32), s_t.view(torch.int32)) and _same_fp8(y, y_t)
    y, s = oracle.per_block_cast_to_fp8(w)
    y_t, s_t = torch_per_block_cast_to_fp8(w)
    assert torch.equal(s.view(torch.int32), s_t.view(torch.int32)) and _same_fp8(y, y_t)
    q, s = oracle.block_fp8(w, (128, 128))
    q_t, s_t = torch_block_fp8(w, (128, 128))
    assert torch.equal(s.view(torch.int32), s_t.view(torch.int32)) and _same_fp8(q, q_t)
    q, s = oracle.mxfp8_quantize(w)
    q_t, s_t = torch_mxfp8(w)
    assert torch.equal(s, s_t) and _same_fp8(q, q_t)
    small = (w.float() * 2.0 ** -4).to(torch.float16)         # keeps 2688 / amax and the block scales in range
    q, s, _ = oracle.nvfp4_quantize_1d(small)
    q_t, s_t = torch_nvfp4(small)
    assert _same_fp8(s, s_t) and torch.equal(q, q_t)


@pytest.mark.parametrize("shape", W.SMALL_REFERENCE_SHAPES + [(130, 257), (256, 384)])
@pytest.mark.parametrize("kind", W.PATTERNS)
def test_fp8_power_of_two_scales_match_torch_chain(oracle, shape, kind):
    # parity with SGLang itself is unpinned (its source is not in the tree); this fixes the restated algorithm
    x = W.reference_pattern(kind, shape, spread=512.0, amplitude=16.0)
    y, s = oracle.per_block_cast_to_fp8(x)
    y_t, s_t = torch_per_block_cast_to_fp8(x)
    assert torch.equal(s.view(torch.int32), s_t.view(torch.int32)) and _same_fp8(y, y_t)
    mant = s.view(torch.int32) & 0x7FFFFF
    assert torch.all(mant == 0)                                   # every scale is a power of two
    if kind == "zeros":
        assert torch.all(s == 2.0 ** -22)                         # 2^ceil(log2(1e-4 / 448))
    if kind == "maxes":
        assert torch.all(y.float().abs().amax() <= 448)


# ---------------------------------------------------------------------------------------------------
# act_quant / fp8_simulate (miles/kernels/quant/fp8_act_quant.py, miles_plugins/models/deepseek_v4/ops/qat.py)
def _act_input(dtype, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(24, 1024, generator=g) * torch.logspace(-6, 4, 1024)).to(dtype)
    x[0, :128] = 0
    x[1, :4] = torch.tensor([448.0, -448.0, -0.0, 1e-6]).to(dtype)
    x[2, :128] = -0.0
    x[3, :128] = 2.0 ** -20          # below the 1e-4 amax floor
    return x


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("block", [16, 32, 64, 128, 256])
@pytest.mark.parametrize("round_scale", [False, True])
def test_act_quant_matches_torch_chain(oracle, dtype, block, round_scale):
    x = _act_input(dtype)
    fmt = "ue8m0" if round_scale else None
    bits = torch.int32 if dtype == torch.float32 else torch.int16
    y, s = oracle.act_quant(x, block, fmt)
    y_t, s_t = torch_act_quant(x, block, round_scale, False)
    assert y.dtype == torch.float8_e4m3fn and s.shape == (24, 1024 // block)
    assert torch.equal(y.view(torch.uint8), y_t.view(torch.uint8)) and torch.equal(s.view(torch.int32), s_t.view(torch.int32))
    qdq = oracle.act_quant(x, block, fmt, inplace=True)
    qdq_t, _ = torch_act_quant(x, block, round_scale, True)
    assert torch.equal(qdq.view(bits), qdq_t.view(bits))          # signs of zeros included
    if round_scale:
        y8, s8 = oracle.act_quant(x, block, fmt, scale_dtype=torch.float8_e8m0fnu)
        assert torch.equal(s8.float(), s_t) and torch.equal(y8.view(torch.uint8), y.view(torch.uint8))
        assert torch.equal(oracle.fp8_simulate(x, block).view(bits), qdq_t.view(bits))


def test_act_quant_known_answers(oracle):
    # one group of 128 with amax 448: scale 448 * f32(1/448) = 1 - 2^-24 rounds to 1.0f?  f32(1/448) is just above 1/448,
    # so the product is 1.0000001 -> 1.0 after rounding; codes are then the values themselves
    x = torch.zeros(1, 128)
    x[0, :6] = torch.tensor([448.0, -1.0, 0.5, 1.0625, 2.0 ** -9, 2.0 ** -11])
    y, s = oracle.act_quant(x, 128)
    assert s.item() == pytest.approx(1.0, rel=1e-6)
    assert y.float()[0, :6].tolist() == [448.0, -1.0, 0.5, 1.0, 2.0 ** -9, 0.0]      # 1.0625 is a tie -> even; 2^-11 -> 0
    y, s = oracle.act_quant(x, 128, "ue8m0")
    assert s.item() in (1.0, 2.0) and (s.view(torch.int32) & 0x7FFFFF).item() == 0
    # all-zero group: the 1e-4 floor sets the scale, codes are +0
    y, s = oracle.act_quant(torch.zeros(1, 64), 64, "ue8m0")
    assert s.item() == 2.0 ** -22 and torch.all(y.view(torch.uint8) == 0)
    assert oracle.act_quant(torch.zeros(1, 64), 64)[1].item() == pytest.approx(1e-4 / 448, rel=1e-6)


def torch_transform_scale_ue8m0(sf, mn):
    """SGLang's transform_scale_ue8m0 as published: broadcast tile rows to weight rows, then DeepGEMM's torch form of
    get_mn_major_tma_aligned_packed_ue8m0_tensor (exponent bytes, pad, reinterpret 4 bytes as int32, transpose)."""
    sf = sf.index_select(-2, torch.arange(mn) // 128)
    exps = (sf.view(torch.int32) >> 23).to(torch.uint8)
    squeeze = sf.dim() == 2
    if squeeze:
        exps = exps.unsqueeze(0)
    b, _, k = exps.shape
    amn, ak = -(-mn // 4) * 4, -(-k // 4) * 4
    padded = torch.zeros((b, amn, ak), dtype=torch.uint8)
    padded[:, :mn, :k] = exps
    words = padded.view(-1).view(torch.int32).view(b, amn, ak // 4)
    transposed = torch.zeros((b, ak // 4, amn), dtype=torch.int32).mT
    transposed[:, :, :] = words
    out = transposed[:, :mn, :]
    return out.squeeze(0) if squeeze else out


@pytest.mark.parametrize("shape,mn", [((1, 1), 1), ((2, 5), 200), ((3, 4), 384), ((3, 2, 7), 130), ((1, 3, 8), 128),
                                      ((2, 4), 250)])
def test_transform_scale_ue8m0_matches_torch_chain(oracle, shape, mn):
    g = torch.Generator().manual_seed(41)
    sf = torch.exp2(torch.randint(-40, 20, shape, generator=g).float())
    got, want = oracle.transform_scale_ue8m0(sf, mn), torch_transform_scale_ue8m0(sf, mn)
    assert got.shape == want.shape and got.stride() == want.stride() and got.dtype == torch.int32
    assert torch.equal(got, want)


def test_transform_scale_ue8m0_known_answer(oracle):
    # 2^e has exponent byte e + 127; five scales along k fill one word and the lowest byte of the next
    sf = torch.tensor([[1.0, 2.0, 0.5, 4.0, 2.0 ** -126]])
    out = oracle.transform_scale_ue8m0(sf, 3)
    assert out.shape == (3, 2) and out.stride() == (1, 4)
    assert [v & 0xFFFFFFFF for v in out[:, 0].tolist()] == [127 | 128 << 8 | 126 << 16 | 129 << 24] * 3
    assert out[:, 1].tolist() == [1] * 3
