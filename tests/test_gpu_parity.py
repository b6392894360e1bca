"""GPU parity: every entry point of libmiles_quant.so, called through the reference-shaped Python wrappers
(ctypes -> C ABI), against the CPU oracle on the same seeded inputs.  Bit-exact everywhere: codes, scales,
packed words; dequant 0 ULP in bf16.
"""

import pytest
import torch

from miles_amd import workloads as W

pytestmark = pytest.mark.gpu
F8 = torch.float8_e4m3fn
DEV = "cuda:0"


def _u8(t):
    return t.detach().cpu().contiguous().view(torch.uint8)


def _bits(t):
    t = t.detach().cpu().contiguous()
    return t.view({1: torch.uint8, 2: torch.int16, 4: torch.int32}[t.element_size()])


def _assert_same(got, want, what):
    g, w = _bits(got), _bits(want)
    assert g.shape == w.shape, f"{what}: shape {tuple(g.shape)} vs {tuple(w.shape)}"
    if not torch.equal(g, w):
        bad = (g != w).nonzero()
        i = tuple(bad[0].tolist())
        raise AssertionError(f"{what}: {bad.shape[0]} of {g.numel()} differ; first at {i}: got {g[i].item()} want {w[i].item()}")


@pytest.fixture(scope="module")
def lib():
    from miles_amd import _lib

    return _lib.load()


# ---------------------------------------------------------------------------------------------------
@pytest.fixture(scope="module")
def probes():
    """libmq_probes.so: the device self-tests (not part of the product library)."""
    from miles_amd import _probes

    return _probes.load()


def test_hardware_converts_agree_with_software_rne(probes):
    counts = torch.zeros(16, dtype=torch.int64, device=DEV)
    assert probes.mqp_selftest_convert(counts.data_ptr(), None) == 0
    torch.cuda.synchronize()
    c = counts.cpu().tolist()
    print("selftest counts", c[:8])
    assert c[0] == 0, "v_cvt_pk_fp8_f32 differs from RNE e4m3fn inside +-448"
    assert c[2] == 0, "v_cvt_scalef32_pk_fp4_f32 differs from RNE satfinite e2m1"
    assert c[3] == 0, "f32->bf16 convert differs from RNE"
    assert c[4] == 0, "v_cvt_pk_f32_fp8 decode table differs"
    assert c[7] == 0, "packed e2m1 convert nibble order"


def test_refined_hardware_reciprocal_is_the_ieee_quotient(probes):
    count = torch.ones(2, dtype=torch.int64, device=DEV)[:1]
    assert probes.mqp_selftest_reciprocal(count.data_ptr(), None) == 0
    torch.cuda.synchronize()
    assert count.item() == 0, "v_rcp_f32 + one Newton step differs from 1.0f / s inside the shared-divisor range"


# ---------------------------------------------------------------------------------------------------
FP8_SHAPES = W.SMALL_REFERENCE_SHAPES + [(130, 264), (1, 8), (127, 136), (200, 1000), (5, 3)]


@pytest.mark.parametrize("shape", FP8_SHAPES)
@pytest.mark.parametrize("kind", W.PATTERNS)
def test_block_fp8(oracle, shape, kind):
    from miles_amd.tools.convert_hf_to_fp8 import block_fp8

    w = W.reference_pattern(kind, shape, spread=512.0, amplitude=16.0)
    q, s = block_fp8(w.to(DEV), [128, 128])
    q_o, s_o = oracle.block_fp8(w, (128, 128))
    assert q.dtype == F8 and s.dtype == torch.float32 and q.is_contiguous()
    _assert_same(s, s_o, "scale")
    _assert_same(q, q_o, "codes")


def test_block_fp8_zero_tile_negative_zero_and_row_stride(oracle):
    from miles_amd.tools.convert_hf_to_fp8 import block_fp8

    w = W.gaussian_outliers((384, 640), std=0.02, p_outlier=0.001, gain=20.0, seed=1001)
    w[128:256, 128:256] = 0
    w[300, 7] = -0.0
    w[5, 5] = 1e-30   # |w/scale| far below the e4m3 subnormal step
    w[6, 6] = -1e-38
    q, s = block_fp8(w.to(DEV), [128, 128])
    q_o, s_o = oracle.block_fp8(w, (128, 128))
    _assert_same(s, s_o, "scale")
    _assert_same(q, q_o, "codes")
    assert torch.all(_u8(q)[128:256, 128:256] == 0xFF) and s[1, 1].item() == 0.0
    view = w.to(DEV)[:, :512]          # row stride 640, unit column stride
    q, s = block_fp8(view, [128, 128])
    q_o, s_o = oracle.block_fp8(w[:, :512].contiguous(), (128, 128))
    _assert_same(s, s_o, "scale (strided)")
    _assert_same(q, q_o, "codes (strided)")


def test_block_fp8_extreme_scales(oracle):
    from miles_amd.tools.convert_hf_to_fp8 import block_fp8

    g = torch.Generator().manual_seed(9)
    base = torch.randn((128, 512), generator=g)
    w = torch.cat([base[:, :128] * 1e-36, base[:, 128:256] * 1e30, base[:, 256:384] * 3e-39, base[:, 384:] * 1e37],
                  dim=1).to(torch.bfloat16)
    q, s = block_fp8(w.to(DEV), [128, 128])
    q_o, s_o = oracle.block_fp8(w, (128, 128))
    _assert_same(s, s_o, "scale")
    _assert_same(q, q_o, "codes")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("bs", [(32, 32), (64, 128), (128, 64), (128, 128)])
def test_block_fp8_generic_blocks_and_dtypes(oracle, dtype, bs):
    from miles_amd.tools.convert_hf_to_fp8 import block_fp8, quant_fp8

    g = torch.Generator().manual_seed(11)
    w = (0.05 * torch.randn((200, 330), generator=g)).to(dtype)
    w[0:32, 0:32] = 0
    q, s = quant_fp8(w.to(DEV), "block", list(bs))
    q_o, s_o = oracle.block_fp8(w, bs)
    _assert_same(s, s_o, "scale")
    _assert_same(q, q_o, "codes")
    assert block_fp8 is not None


def _fp16_tile_case(shape, seed, *, specials):
    g = torch.Generator().manual_seed(seed)
    w = (0.05 * torch.randn(shape, generator=g)).to(torch.float16)
    m, n = shape
    if m >= 8 and n >= 64:
        w[0, :32] = torch.arange(1, 33, dtype=torch.int16).view(torch.float16)               # subnormals
        w[1, :32] = (torch.arange(0x3E0, 0x400, dtype=torch.int16) - 0x8000).to(torch.int16).view(torch.float16)
        w[2, :4] = torch.tensor([-0.0, 0.0, 65504.0, -65504.0], dtype=torch.float16)
        w[3, 8:16] = torch.tensor([6.1e-5, -6.1e-5, 6.0e-8, 1.2e-7, 448.0, 464.0, 0.0009765625, 3.0], dtype=torch.float16)
    if m > 128 and n > 256:
        w[128:256, 128:256] = 0                           # a tile of zeros
        w[m - 1, 130] = -0.0
        w[:128, 256:384] *= 1e-3                          # a tile whose values are mostly fp16 subnormals
    if specials and m > 5 and n > 140:
        w[5, 3] = float("inf")
        w[4, 130] = float("nan")
        w[m - 1, n - 1] = float("-inf")
    return w


@pytest.mark.parametrize("shape", [(384, 640), (130, 264), (127, 136), (1, 8), (8, 64), (1024, 2048)])
def test_fp8_tile_kernels_read_fp16(oracle, shape):
    """fp16 tensors take the same tuned 128x128 kernels as bf16 ones (their own instances): the three scale rules against
    the oracle, with fp16 subnormals, the format's extremes, signed zeros, a zero tile and, where the rule defines it
    (the two casts with reciprocal scales), infinities and NaNs; then bf16 and fp16 tensors alternating in one recorded
    job list, which has to split its launches by dtype."""
    from miles_amd import launch
    from miles_amd.kernels.quant.fp8_blockwise import fp8_blockwise_cast, per_block_cast_to_fp8
    from miles_amd.tools.convert_hf_to_fp8 import block_fp8

    w = _fp16_tile_case(shape, 31 + shape[1], specials=False)
    q, s = block_fp8(w.to(DEV), [128, 128])
    q_o, s_o = oracle.block_fp8(w, (128, 128))
    _assert_same(s, s_o, "block_fp8 scale")
    _assert_same(q, q_o, "block_fp8 codes")
    for specials in (False, True):
        x = _fp16_tile_case(shape, 77 + shape[0], specials=specials)
        for name, fn, ref in (("fp8_blockwise_cast", fp8_blockwise_cast, oracle.fp8_blockwise_cast),
                              ("per_block_cast_to_fp8", per_block_cast_to_fp8, oracle.per_block_cast_to_fp8)):
            y, s = fn(x.to(DEV))
            y_o, s_o = ref(x)
            _assert_same(s, s_o, f"{name} scale (specials={specials})")
            _assert_same(y, y_o, f"{name} codes (specials={specials})")
    if shape[0] > 1000:
        return
    tensors = []
    for i in range(10):
        t = _fp16_tile_case(shape, 500 + i, specials=False)
        tensors.append(t if i % 3 else t.float().to(torch.bfloat16))
    dev = [t.to(DEV) for t in tensors]
    with launch.recording() as batch:
        outs = [fp8_blockwise_cast(t) for t in dev] + [block_fp8(t, [128, 128]) for t in dev]
    for rep in range(2):
        batch.run()
        torch.cuda.synchronize()
        for i, t in enumerate(tensors):
            for (got, want, what) in zip(outs[i] + outs[10 + i], oracle.fp8_blockwise_cast(t) + oracle.block_fp8(t, (128, 128)),
                                         ("cast codes", "cast scale", "block codes", "block scale")):
                _assert_same(got, want, f"tensor {i} ({t.dtype}) {what}, run {rep}")
        for o in outs:
            for t in o:
                t.view(torch.uint8).fill_(0x5A)
        if rep == 0:
            batch.freeze()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_tensor_and_channel_fp8(oracle, dtype):
    from miles_amd.tools.convert_hf_to_fp8 import quant_fp8

    g = torch.Generator().manual_seed(12)
    w = (0.02 * torch.randn((96, 200), generator=g)).to(dtype)
    w[3] = 0
    q, s = quant_fp8(w.to(DEV), "tensor")
    q_o, s_o = oracle.tensor_fp8(w)
    assert s.shape == (1,)
    _assert_same(s, s_o, "tensor scale")
    _assert_same(q, q_o, "tensor codes")
    q, s = quant_fp8(w.to(DEV), "channel")
    q_o, s_o = oracle.channel_fp8(w)
    assert s.shape == (96, 1)
    _assert_same(s, s_o, "channel scale")
    _assert_same(q, q_o, "channel codes")


@pytest.mark.parametrize("shape", [(64, 2048), (37, 7168), (5, 16384), (3, 16392), (130, 264), (2048, 7168)])
def test_tensor_and_channel_fp8_bf16_row_kernels(oracle, shape):
    # the bf16 kernels: rows held by one wavefront (K <= 2048), by a workgroup (K <= 16384), longer rows on the plain
    # kernels; an all-zero row, a row of signed zeros, a row below the 1e-12 floor, format-sized magnitudes
    from miles_amd.tools.convert_hf_to_fp8 import quant_fp8

    w = W.gaussian_outliers(shape, std=0.02, p_outlier=0.001, gain=25.0, seed=1300 + shape[1], dtype=torch.bfloat16)
    w[0] = 0
    w[1, :64] = torch.tensor([-0.0, 0.0] * 32, dtype=torch.bfloat16)
    w[2] = 1e-20
    w[2, 5] = -3e-20
    for strategy, ref in (("tensor", oracle.tensor_fp8), ("channel", oracle.channel_fp8)):
        q, s = quant_fp8(w.to(DEV), strategy)
        q_o, s_o = ref(w)
        _assert_same(s, s_o, f"{strategy} scale")
        _assert_same(q, q_o, f"{strategy} codes")
    big = w.clone()
    big[1, 7] = 3e38                               # one huge value: every other quotient underflows, signs must survive
    q, s = quant_fp8(big.to(DEV), "tensor")
    q_o, s_o = oracle.tensor_fp8(big)
    _assert_same(s, s_o, "tensor scale, huge amax")
    _assert_same(q, q_o, "tensor codes, huge amax")
    # rows taken from a wider matrix (row stride != K): per channel reads them in place
    wide = W.gaussian_outliers((shape[0], shape[1] + 64), std=0.02, p_outlier=0.001, gain=25.0, seed=77, dtype=torch.bfloat16)
    view = wide.to(DEV)[:, : shape[1]]
    for strategy, ref in (("tensor", oracle.tensor_fp8), ("channel", oracle.channel_fp8)):
        q, s = quant_fp8(view, strategy)
        q_o, s_o = ref(wide[:, : shape[1]].contiguous())
        _assert_same(s, s_o, f"{strategy} scale, strided rows")
        _assert_same(q, q_o, f"{strategy} codes, strided rows")


def _same_fp8_codes(got, want, what):
    """Byte equality with the two e4m3 NaN codes 0x7F / 0xFF counted as one (the sign of a 0 / 0 is the host FPU's choice)."""
    g, w = _u8(got).clone(), _u8(want).clone()
    g[(g & 0x7F) == 0x7F] = 0x7F
    w[(w & 0x7F) == 0x7F] = 0x7F
    assert g.shape == w.shape and torch.equal(g, w), f"{what}: {(g != w).sum().item()} of {g.numel()} differ"


@pytest.mark.parametrize("shape", [(64, 2048), (37, 7168), (5, 16384), (130, 264), (2048, 7168)])
def test_tensor_and_channel_fp8_fp16(oracle, shape):
    """fp16 weights on the per-channel row kernels and on the per-tensor job form: fp16 has no 1e-12 floor (it rounds to
    zero), so a row / tensor of zeros divides 0 by 0 and every code is NaN; subnormals, the format's extremes, strided
    rows; per tensor also as a recorded list that mixes bf16 and fp16 tensors and then carries the amax over."""
    from miles_amd import launch
    from miles_amd.tools.convert_hf_to_fp8 import quant_fp8

    w = W.gaussian_outliers(shape, std=0.02, p_outlier=0.001, gain=25.0, seed=1400 + shape[1], dtype=torch.float16)
    w[0] = 0
    w[1, :64] = torch.tensor([-0.0, 0.0] * 32, dtype=torch.float16)
    w[2] = 6e-8
    w[2, 5] = -1.2e-7
    w[3, :4] = torch.tensor([65504.0, -65504.0, 3.0, -1e-4], dtype=torch.float16)
    for strategy, ref in (("tensor", oracle.tensor_fp8), ("channel", oracle.channel_fp8)):
        q, s = quant_fp8(w.to(DEV), strategy)
        q_o, s_o = ref(w)
        _assert_same(s, s_o, f"{strategy} scale")
        _same_fp8_codes(q, q_o, f"{strategy} codes")
    z = torch.zeros(16, 256, dtype=torch.float16)
    q, s = quant_fp8(z.to(DEV), "tensor")
    q_o, s_o = oracle.tensor_fp8(z)
    _assert_same(s, s_o, "zero tensor scale")
    _same_fp8_codes(q, q_o, "zero tensor codes")
    wide = W.gaussian_outliers((shape[0], shape[1] + 64), std=0.02, p_outlier=0.001, gain=25.0, seed=78, dtype=torch.float16)
    q, s = quant_fp8(wide.to(DEV)[:, : shape[1]], "channel")
    q_o, s_o = oracle.channel_fp8(wide[:, : shape[1]].contiguous())
    _assert_same(s, s_o, "channel scale, strided rows")
    _same_fp8_codes(q, q_o, "channel codes, strided rows")
    if shape[0] > 1000:
        return
    tensors = [W.gaussian_outliers((24 + i, 512), std=0.02, p_outlier=0.001, gain=20.0, seed=1500 + i,
                                   dtype=torch.float16 if i % 3 else torch.bfloat16) for i in range(9)]
    dev = [t.to(DEV) for t in tensors]
    with launch.recording() as batch:
        outs = [quant_fp8(t, "tensor") for t in dev]
    assert len(batch) == len(tensors) and batch.direct_calls == 0
    batch.device = torch.device(DEV)

    def check(what):
        batch.run()
        torch.cuda.synchronize()
        for i, (t, (q, sc)) in enumerate(zip(dev, outs)):
            q_o, s_o = oracle.tensor_fp8(t.cpu())
            _assert_same(sc, s_o, f"{what}: tensor {i} ({t.dtype}) scale")
            _same_fp8_codes(q, q_o, f"{what}: tensor {i} ({t.dtype}) codes")

    check("first run")
    assert batch.carry_amax() == len(tensors)
    check("carried")
    dev[1].mul_(2.0)
    dev[5].mul_(0.25)
    check("two fp16 amax moved")
    check("settled")


# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("shape", FP8_SHAPES)
@pytest.mark.parametrize("kind", W.PATTERNS)
def test_fp8_blockwise_cast(oracle, shape, kind):
    from miles_amd.kernels.quant.fp8_blockwise import fp8_blockwise_cast

    x = W.reference_pattern(kind, shape, spread=512.0, amplitude=16.0)
    y, s = fp8_blockwise_cast(x.to(DEV))
    y_o, s_o = oracle.fp8_blockwise_cast(x)
    assert y.dtype == F8 and y.is_contiguous() and s.dtype == torch.float32
    _assert_same(s, s_o, "scale")
    _assert_same(y, y_o, "codes")


def test_fp8_blockwise_cast_strided_and_block_size(oracle):
    from miles_amd.kernels.quant.fp8_blockwise import fp8_blockwise_cast

    base = W.gaussian_outliers((256, 304), std=0.02, p_outlier=0.001, gain=20.0, seed=5)
    dev = base.to(DEV)
    for view_fn in (lambda t: t[:, :256], lambda t: t.t(), lambda t: t[::2, 1::2], lambda t: t.chunk(2, dim=0)[1]):
        y, s = fp8_blockwise_cast(view_fn(dev))
        y_o, s_o = oracle.fp8_blockwise_cast(view_fn(base))
        _assert_same(s, s_o, "scale")
        _assert_same(y, y_o, "codes")
    y, s = fp8_blockwise_cast(dev, [64, 32])
    y_o, s_o = oracle.fp8_blockwise_cast(base, [64, 32])
    _assert_same(s, s_o, "scale 64x32")
    _assert_same(y, y_o, "codes 64x32")


# ---------------------------------------------------------------------------------------------------
def test_weight_dequant_all_codes(oracle):
    from miles_amd.tools.fp8_cast_bf16 import weight_dequant

    g = torch.Generator().manual_seed(21)
    for shape in [(300, 400), (128, 1024), (257, 144), (5, 7)]:
        codes = torch.randint(0, 256, shape, generator=g, dtype=torch.int32).to(torch.uint8)
        codes[0, : min(256, shape[1])] = torch.arange(min(256, shape[1]), dtype=torch.uint8)
        s = torch.exp(torch.randn((-(-shape[0] // 128), -(-shape[1] // 128)), generator=g) * 4).float()
        y = weight_dequant(codes.view(F8).to(DEV), s.to(DEV))
        y_o = oracle.weight_dequant(codes.view(F8), s)
        assert y.dtype == torch.bfloat16
        _assert_same(y, y_o, f"dequant {shape}")   # NaN codes give 0x7FC0 on both sides


def test_quant_dequant_round_trip(oracle):
    from miles_amd.tools.convert_hf_to_fp8 import block_fp8
    from miles_amd.tools.fp8_cast_bf16 import weight_dequant

    w = W.gaussian_outliers((512, 896), std=0.02, p_outlier=0.0, gain=1.0, seed=5001)
    q, s = block_fp8(w.to(DEV), [128, 128])
    y = weight_dequant(q, s)
    y_o = oracle.weight_dequant(*oracle.block_fp8(w, (128, 128)))
    _assert_same(y, y_o, "round trip")
    err = (y.float().cpu() - w.float()).abs()
    # half an e4m3 step at 448 times the scale, plus the bf16 rounding of the product
    bound = s.cpu().repeat_interleave(128, 0).repeat_interleave(128, 1) * 16.0 + y.float().cpu().abs() * 2.0**-8
    assert torch.all(err <= bound * 1.001 + 1e-12)
    with pytest.raises(AssertionError):
        weight_dequant(q.t(), s)


# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("shape", W.SMALL_REFERENCE_SHAPES + [(7, 96), (1024, 2048)])
@pytest.mark.parametrize("kind", W.PATTERNS)
def test_mxfp8(oracle, shape, kind):
    from miles_amd.utils.mxfp8 import mxfp8_quantize

    w = W.reference_pattern(kind, shape, spread=512.0, amplitude=16.0)
    q, s = mxfp8_quantize(w.to(DEV))
    q_o, s_o = oracle.mxfp8_quantize(w)
    assert q.shape == w.shape and q.dtype == F8 and s.dtype == torch.uint8
    assert s.shape == (*w.shape[:-1], w.shape[-1] // 32)
    _assert_same(s, s_o, "scales")
    _assert_same(q, q_o, "codes")


def test_mxfp8_heavy_tails_3d_dtypes_and_errors(oracle):
    from miles_amd.utils.mxfp8 import mxfp8_quantize

    w = W.student_t_rows((768, 2048), std=0.02, seed=3001)
    w[3, :64] = 0
    w[4, :32] = 1e-38
    w[5, 32:64] = float("inf")
    q, s = mxfp8_quantize(w.to(DEV))
    q_o, s_o = oracle.mxfp8_quantize(w)
    _assert_same(s, s_o, "scales")
    _assert_same(q, q_o, "codes")
    w3 = W.student_t_rows((6 * 16, 64), std=1.0, seed=1).reshape(6, 16, 64)
    for dtype in (torch.bfloat16, torch.float16, torch.float32):
        q, s = mxfp8_quantize(w3.to(dtype).to(DEV))
        q_o, s_o = oracle.mxfp8_quantize(w3.to(dtype))
        assert s.shape == (6, 16, 2)
        _assert_same(s, s_o, f"scales {dtype}")
        _assert_same(q, q_o, f"codes {dtype}")
    q, s = mxfp8_quantize(w.to(DEV).t()[:2048:2].t())    # non-contiguous input is made contiguous
    q_o, s_o = oracle.mxfp8_quantize(w.t()[:2048:2].t())
    _assert_same(q, q_o, "codes (strided)")
    with pytest.raises(ValueError, match="Last dim 48 must be divisible by 32 for MXFP8."):
        mxfp8_quantize(torch.zeros(4, 48, dtype=torch.bfloat16, device=DEV))


@pytest.mark.parametrize("shape", [(384, 640), (8, 64), (5, 32), (1024, 2048)])
def test_mxfp8_reads_fp16(oracle, shape):
    """fp16 tensors take the tuned MXFP8 kernel's fp16 instance: subnormals, the format's extremes, signed zeros, groups
    of zeros, infinities and NaNs against the oracle; then bf16 and fp16 tensors alternating in one recorded job list."""
    from miles_amd import launch
    from miles_amd.utils.mxfp8 import mxfp8_quantize

    for specials in (False, True):
        w = _fp16_tile_case(shape, 900 + shape[1], specials=specials)
        if shape[0] > 4:
            w[4, :32] = 0
        q, s = mxfp8_quantize(w.to(DEV))
        q_o, s_o = oracle.mxfp8_quantize(w)
        _assert_same(s, s_o, f"scales (specials={specials})")
        _assert_same(q, q_o, f"codes (specials={specials})")
    if shape[0] > 1000:
        return
    tensors = []
    for i in range(9):
        t = _fp16_tile_case(shape, 950 + i, specials=False)
        tensors.append(t if i % 3 else t.float().to(torch.bfloat16))
    dev = [t.to(DEV) for t in tensors]
    with launch.recording() as batch:
        outs = [mxfp8_quantize(t) for t in dev]
    for rep in range(2):
        batch.run()
        torch.cuda.synchronize()
        for i, t in enumerate(tensors):
            for got, want, what in zip(outs[i], oracle.mxfp8_quantize(t), ("codes", "scales")):
                _assert_same(got, want, f"tensor {i} ({t.dtype}) {what}, run {rep}")
        for o in outs:
            for t in o:
                t.view(torch.uint8).fill_(0x5A)
        if rep == 0:
            batch.freeze()


# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("shape,G", [((4, 128), 128), ((16, 256), 128), ((64, 1024), 128), ((24, 7168), 128),
                                     ((16, 256), 32), ((5, 96), 32), ((9, 192), 64), ((3, 160), 160)])
def test_int4_pack_layer(oracle, shape, G):
    from miles_amd.kernels.quant.int4_fake import pack_layer

    w = W.gaussian_outliers(shape, std=0.015, p_outlier=0.0005, gain=30.0, seed=4001)
    w[0] = 0
    w[1, :G] = 3e-6
    w[2, :G] = torch.linspace(-1, 1, G)     # exact ties of x/scale are likely here
    packed, scale, zp = pack_layer(w.to(DEV), G)
    packed_o, scale_o, _ = oracle.pack_layer(w, G)
    assert zp is None and packed.dtype == torch.int32 and scale.dtype == torch.bfloat16
    _assert_same(scale, scale_o, "scales")
    _assert_same(packed, packed_o, "packed")


@pytest.mark.parametrize("shape,G", [((4, 128), 128), ((16, 256), 128), ((64, 1024), 128), ((24, 7168), 128),
                                     ((16, 256), 32), ((9, 192), 64), ((2048, 7168), 128)])
def test_int4_pack_layer_fp16(oracle, shape, G):
    """fp16 weights take the fused packer's fp16 instance (groups of 32 / 64 / 128): scales in fp16, the scale floor
    (a subnormal fp16), subnormal inputs, ties, and groups whose maximum is 65504, where 7 x scale overflows in the
    reference's fp16 round trip and the kernel has to follow the written-out chain; then bf16 and fp16 tensors
    alternating in one recorded job list."""
    from miles_amd import launch
    from miles_amd.kernels.quant.int4_fake import pack_layer

    def case(seed):
        w = W.gaussian_outliers(shape, std=0.015, p_outlier=0.0005, gain=30.0, seed=seed, dtype=torch.float16)
        w[0] = 0
        w[1, :G] = 3e-6
        w[2, :G] = torch.linspace(-1, 1, G).to(torch.float16)
        w[3, :32] = torch.arange(1, 33, dtype=torch.int16).view(torch.float16)       # subnormals only: floor scale
        if shape[0] > 8:
            w[4, :G] = torch.linspace(-65504, 65504, G).to(torch.float16)
            w[5, 7] = 65504.0
            w[6, G - 1] = -65504.0
            w[7, :G] = 65504.0
            w[8, :G] = torch.linspace(-60000, 65472, G).to(torch.float16)              # just below the overflow
        return w

    w = case(4001)
    packed, scale, zp = pack_layer(w.to(DEV), G)
    packed_o, scale_o, _ = oracle.pack_layer(w, G)
    assert zp is None and packed.dtype == torch.int32 and scale.dtype == torch.float16
    _assert_same(scale, scale_o, "scales")
    _assert_same(packed, packed_o, "packed")
    if shape[0] > 1000:
        return
    tensors = [case(4100 + i) if i % 3 else case(4100 + i).float().clamp(-3e4, 3e4).to(torch.bfloat16) for i in range(9)]
    dev = [t.to(DEV) for t in tensors]
    with launch.recording() as batch:
        outs = [pack_layer(t, G)[:2] for t in dev]
    for rep in range(2):
        batch.run()
        torch.cuda.synchronize()
        for i, t in enumerate(tensors):
            for got, want, what in zip(outs[i], oracle.pack_layer(t, G)[:2], ("packed", "scales")):
                _assert_same(got, want, f"tensor {i} ({t.dtype}) {what}, run {rep}")
        for o in outs:
            for t in o:
                t.view(torch.uint8).fill_(0x5A)
        if rep == 0:
            batch.freeze()


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_int4_pack_layer_other_dtypes(oracle, dtype):
    from miles_amd.kernels.quant.int4_fake import pack_layer

    w = W.gaussian_outliers((8, 256), std=0.015, p_outlier=0.0, gain=1.0, seed=7, dtype=dtype)
    packed, scale, _ = pack_layer(w.to(DEV), 128)
    packed_o, scale_o, _ = oracle.pack_layer(w, 128)
    _assert_same(scale, scale_o, "scales")
    _assert_same(packed, packed_o, "packed")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape,G", [((8, 128), 128), ((16, 256), 128), ((64, 1024), 128), ((24, 7168), 128),
                                     ((16, 256), 32), ((24, 192), 64), ((8, 2048), 1024), ((2048, 7168), 128)])
def test_int4_pack_layer_asymmetric(oracle, shape, G, dtype):
    from miles_amd.kernels.quant.int4_fake import pack_layer

    if shape[0] > 1000 and dtype != torch.bfloat16:
        pytest.skip("the full-size tensor is checked in bf16 only")
    w = W.gaussian_outliers(shape, std=0.015, p_outlier=0.0005, gain=30.0, seed=4101, dtype=dtype)
    w[0] = 0                      # zero range: scale floor, zero point +0
    w[1] = w[1].abs() + 0.25      # minimum far above zero: codes run past 15 and carry into the next nibble
    w[2] = -w[2].abs() - 0.25     # maximum far below zero: zero point clamps to 15, codes clamp at 0
    w[3, :G] = 3e-6
    w[4, :G] = torch.linspace(-1, 1, G).to(dtype)
    packed, scale, zp = pack_layer(w.to(DEV), G, sym=False)
    packed_o, scale_o, zp_o = oracle.pack_layer(w, G, sym=False)
    assert packed.dtype == torch.int32 and scale.dtype == dtype and zp.dtype == torch.int32
    assert zp.shape == (shape[1] // G, shape[0] // 8)
    _assert_same(scale, scale_o, "scales")
    _assert_same(zp, zp_o, "packed zero points")
    _assert_same(packed, packed_o, "packed")


@pytest.mark.parametrize("G", [32, 64, 128])
def test_int4_pack_layer_asymmetric_shifted_groups(oracle, G):
    """Groups shifted so that rint(min / scale) sweeps from below -15 to above 0: the fused form of the packed kernel
    ends exactly at an unclamped zero point, and both neighbours (zero point clamped at 15 or at 0) take the written-out
    chain; huge and tiny scales and an infinite extremum sit next to ordinary groups of the same wavefront."""
    from miles_amd.kernels.quant.int4_fake import pack_layer

    rows, cols = 64, 2048
    gen = torch.Generator().manual_seed(4201)
    w = torch.randn(rows, cols, generator=gen) * 0.02
    groups = w.view(rows, cols // G, G)
    span = groups.amax(-1, keepdim=True) - groups.amin(-1, keepdim=True)
    # group minimum at -(k / 15) * span for k from -4 to 20 in steps of 0.25, plus half-way cases
    k = (torch.arange(rows * (cols // G), dtype=torch.float32).view(rows, cols // G, 1) % 97) * 0.25 - 4.0
    groups += -groups.amin(-1, keepdim=True) - k / 15.0 * span
    w = groups.reshape(rows, cols).to(torch.bfloat16)
    w[5, :G] *= 2.0 ** 100          # scale beyond the range of the shared-divisor sequence
    w[6, :G] *= 2.0 ** -100
    w[7, 3] = float("inf")
    w[8, 5] = float("-inf")
    w[9, 7] = float("nan")
    w[10, G:2 * G] = 3.3e38         # bf16(scale) above 1e37 with an all-equal group next to it
    w[11, :G] = torch.linspace(-3.3e38, 3.3e38, G).to(torch.bfloat16)
    w[12, :G] = float("inf")        # equal infinities: the range is NaN and the scale falls to its floor
    w[13, G:2 * G] = float("-inf")
    w[14, :G] = float("nan")
    packed, scale, zp = pack_layer(w.to(DEV), G, sym=False)
    packed_o, scale_o, zp_o = oracle.pack_layer(w, G, sym=False)
    _assert_same(scale, scale_o, "scales")
    _assert_same(zp, zp_o, "packed zero points")
    _assert_same(packed, packed_o, "packed")


@pytest.mark.parametrize("G", [32, 64, 128])
def test_int4_pack_layer_asymmetric_fp16(oracle, G):
    """The asymmetric packer's fp16 instance: zero points from clamped-at-15 to clamped-at-0 (the fused form ends exactly
    at an unclamped zero point), scales around 4096 where 16 x scale leaves fp16 (those groups take the written-out
    chain), the format's extremes, groups of subnormals, infinities and NaN next to ordinary groups; then bf16 and fp16
    tensors alternating in one recorded job list."""
    from miles_amd import launch
    from miles_amd.kernels.quant.int4_fake import pack_layer

    rows, cols = 64, 2048
    gen = torch.Generator().manual_seed(4301)
    w = torch.randn(rows, cols, generator=gen) * 0.02
    groups = w.view(rows, cols // G, G)
    span = groups.amax(-1, keepdim=True) - groups.amin(-1, keepdim=True)
    k = (torch.arange(rows * (cols // G), dtype=torch.float32).view(rows, cols // G, 1) % 97) * 0.25 - 4.0
    groups += -groups.amin(-1, keepdim=True) - k / 15.0 * span
    w = groups.reshape(rows, cols).to(torch.float16)
    for i, top in enumerate((61000.0, 61400.0, 61440.0, 61500.0, 65504.0, 30000.0)):     # scales 4066 ... 4367 and 2000
        w[16 + i, :G] = torch.linspace(0.0, top, G).to(torch.float16)
        w[24 + i, G:2 * G] = torch.linspace(-top / 2, top / 2, G).to(torch.float16)
    w[32, :G] = torch.linspace(-65504, 65504, G).to(torch.float16)
    w[33, :32] = torch.arange(1, 33, dtype=torch.int16).view(torch.float16)              # subnormals: the scale floor
    w[34, :G] = 65504.0
    w[35, 3] = float("inf")
    w[36, 5] = float("-inf")
    w[37, 7] = float("nan")
    w[38, :G] = float("inf")
    w[39, :G] = float("nan")
    packed, scale, zp = pack_layer(w.to(DEV), G, sym=False)
    packed_o, scale_o, zp_o = oracle.pack_layer(w, G, sym=False)
    assert scale.dtype == torch.float16
    _assert_same(scale, scale_o, "scales")
    _assert_same(zp, zp_o, "packed zero points")
    _assert_same(packed, packed_o, "packed")
    tensors = []
    for i in range(9):
        t = W.gaussian_outliers((32, 1024), std=0.015, p_outlier=0.0005, gain=30.0, seed=4400 + i, dtype=torch.float16)
        t[1] = t[1].abs() + 0.25
        t[2] = -t[2].abs() - 0.25
        tensors.append(t if i % 3 else t.float().to(torch.bfloat16))
    dev = [t.to(DEV) for t in tensors]
    with launch.recording() as batch:
        outs = [pack_layer(t, G, sym=False) for t in dev]
    batch.freeze()
    for rep in range(2):
        for o in outs:
            for t in o:
                t.view(torch.uint8).fill_(0x5A)
        batch.run()
        torch.cuda.synchronize()
        for i, t in enumerate(tensors):
            for got, want, what in zip(outs[i], oracle.pack_layer(t, G, sym=False), ("packed", "scales", "zero points")):
                _assert_same(got, want, f"tensor {i} ({t.dtype}) {what}, run {rep}")


def test_int4_pack_layer_asymmetric_argument_checks():
    from miles_amd.kernels.quant.int4_fake import pack_layer

    with pytest.raises(RuntimeError, match="not divisible"):
        pack_layer(torch.zeros(4, 128, dtype=torch.bfloat16, device=DEV), 128, sym=False)   # rows % 8
    with pytest.raises(RuntimeError, match="not divisible"):
        pack_layer(torch.zeros(8, 96, dtype=torch.bfloat16, device=DEV), 128, sym=False)


@pytest.mark.parametrize("sdt", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape,G", [((4, 128), 128), ((16, 256), 32), ((3, 100), 20), ((64, 1024), 128),
                                     ((2048, 7168), 128)])
def test_int4_unpack_dequant(oracle, shape, G, sdt):
    from miles_amd.tools.convert_kimi_int4_to_bf16 import _dequantize_tensor

    if shape[0] > 1000 and sdt != torch.bfloat16:
        pytest.skip("the full-size tensor is checked with bf16 scales only")
    g = torch.Generator().manual_seed(31)
    m, k = shape
    packed = torch.randint(-2**31, 2**31 - 1, (m, -(-k // 8)), dtype=torch.int64, generator=g).to(torch.int32)
    scale = torch.exp(torch.randn((m, k // G), generator=g) * 3).to(sdt)
    # non-finite scales: the reference's rounding to bf16 writes the one quiet NaN 0x7FC0 for any NaN (and for 0 x inf)
    flat = scale.view(-1)
    if flat.numel() >= 4:
        flat[0], flat[1], flat[2] = float("nan"), float("inf"), float("-inf")
        if sdt == torch.bfloat16:
            flat.view(torch.int16)[3] = -42        # a NaN with a sign and a payload
    if flat.numel() >= 16:
        # zero, negative and tiny scales (the sign of a zero product is the product's), and the largest finite ones
        big = {torch.bfloat16: 3.0e38, torch.float16: 65504.0, torch.float32: 3.0e38}[sdt]
        tiny = {torch.bfloat16: 1e-40, torch.float16: 6e-8, torch.float32: 1e-44}[sdt]
        for at, v in enumerate((0.0, -0.0, -1.5, tiny, -tiny, big, -big, big / 4, big / 16, big / 32), start=4):
            flat[at] = v
    got = _dequantize_tensor(packed.to(DEV), scale.to(DEV), torch.tensor(shape, dtype=torch.int32), G)
    want = oracle.int4_unpack_dequant(packed, scale, shape, G)
    assert got.dtype == torch.bfloat16
    _assert_same(got, want, "dequantized values")


@pytest.mark.parametrize("flat", [False, True])
@pytest.mark.parametrize("shape", [(5, 44), (64, 1024)])
def test_int4_unpack_dequant_per_element_scales(oracle, shape, flat):
    # group_size <= 0 means one scale per weight, given in the weight's shape or flattened
    from miles_amd.tools.convert_kimi_int4_to_bf16 import _dequantize_tensor

    g = torch.Generator().manual_seed(33)
    m, k = shape
    packed = torch.randint(-2**31, 2**31 - 1, (m, -(-k // 8)), dtype=torch.int64, generator=g).to(torch.int32)
    scale = torch.exp(torch.randn((m, k), generator=g) * 3).to(torch.bfloat16)
    if flat:
        scale = scale.reshape(-1)
    got = _dequantize_tensor(packed.to(DEV), scale.to(DEV), shape, 0)
    _assert_same(got, oracle.int4_unpack_dequant(packed, scale, shape, 0), "per-element scales")
    with pytest.raises(ValueError, match="incompatible"):
        _dequantize_tensor(packed.to(DEV), scale.to(DEV)[..., :-1], shape, -1)


def test_int4_pack_then_unpack_round_trip(oracle):
    from miles_amd.kernels.quant.int4_fake import pack_layer
    from miles_amd.tools.convert_kimi_int4_to_bf16 import _dequantize_tensor

    w = W.gaussian_outliers((256, 7168), std=0.015, p_outlier=0.0005, gain=30.0, seed=4001)
    packed, scale, _ = pack_layer(w.to(DEV), 128)
    deq = _dequantize_tensor(packed, scale, w.shape, 128)
    # |w - dequantized| <= scale/2 plus the bf16 roundings of the scale and of the product (each <= 7*scale*2^-9, measured against the rounded scale)
    err = (deq.float().cpu() - w.float()).abs().reshape(256, 56, 128).amax(dim=-1)
    assert torch.all(err <= scale.float().cpu() * 0.55 + 1e-12)
    _assert_same(deq, oracle.int4_unpack_dequant(packed.cpu(), scale.cpu(), w.shape, 128), "round trip")


@pytest.mark.parametrize("sym", [True, False])
@pytest.mark.parametrize("shape,G", [((16, 256), 128), ((8, 200), 32), ((4, 128), 32), ((3, 7168), 128)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_fake_int4_quant(oracle, sym, shape, G, dtype):
    from miles_amd.kernels.quant.int4_fake import fake_int4_quant_cuda

    w = W.gaussian_outliers(shape, std=0.015, p_outlier=0.001, gain=30.0, seed=4002, dtype=dtype)
    w[0] = 0
    out, scale, zero = fake_int4_quant_cuda(w.to(DEV), (1, G), sym)
    out_o, scale_o, zero_o = oracle.fake_int4_quant(w, (1, G), sym)
    assert out.dtype == dtype and scale.shape == (shape[0], -(-shape[1] // G))
    _assert_same(out, out_o, "values")          # includes the -0.0 produced by rint of small negatives
    _assert_same(scale, scale_o, "scales")
    if not sym:
        _assert_same(zero, zero_o, "zero points")


def test_fake_int4_quant_argument_checks():
    from miles_amd.kernels.quant.int4_fake import fake_int4_quant_cuda

    x = torch.zeros(4, 64, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="must be divisible by 32"):
        fake_int4_quant_cuda(x, (1, 48), True)
    with pytest.raises(RuntimeError, match="Input must be 2D"):
        fake_int4_quant_cuda(x.reshape(2, 2, 64), (1, 32), True)
    with pytest.raises(RuntimeError, match="Input must be on CUDA"):
        fake_int4_quant_cuda(x.cpu(), (1, 32), True)


# ---------------------------------------------------------------------------------------------------
# MXFP4 (miles/utils/mxfp4.py)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape,G", [((16, 64), 32), ((3, 128), 32), ((64, 64), 32), ((8, 2048), 32), ((4, 64), 16),
                                     ((5, 24), 4), ((2, 3, 64), 32), ((513, 7168), 32)])
def test_mxfp4_quantize(oracle, shape, G, dtype):
    from miles_amd.utils.mxfp4 import quantize_mxfp4

    rows = 1
    for d in shape[:-1]:
        rows *= d
    w = W.student_t_rows((rows, shape[-1]), std=0.02, seed=6001).reshape(shape).to(dtype)
    flat = w.reshape(-1, shape[-1])
    flat[0, :G] = 0
    flat[1, :G] = torch.tensor([6.0, -6.0, 3.0, 0.25] * (G // 4)).to(dtype)
    flat[2, :4] = torch.tensor([0.75, 1.75, 3.5, -0.0]).to(dtype)
    flat[2, 4] = 6.0
    packed, scale = quantize_mxfp4(w.to(DEV), G)
    packed_o, scale_o = oracle.quantize_mxfp4(w, G)
    assert packed.dtype == torch.uint8 and scale.dtype == torch.uint8
    assert packed.shape == packed_o.shape and scale.shape == scale_o.shape
    _assert_same(scale, scale_o, "E8M0 scales")
    _assert_same(packed, packed_o, "packed codes")


def test_mxfp4_quantize_extreme_magnitudes(oracle):
    from miles_amd.utils.mxfp4 import quantize_mxfp4

    # groups of denormals (scale exponent clamps at -127), of the largest finite bf16 values, and ties at every bound
    tiny = torch.tensor([1, 2, 3, 0x40, 0x7F, 0x80, 0x81, 0x100] * 4, dtype=torch.int16).view(torch.bfloat16)
    huge = torch.tensor([0x7F7F, 0x7F00, 0x7E80, -0x7F7F + 0x10000 - 0x10000] * 8, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    ties = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0] * 4, dtype=torch.bfloat16)
    w = torch.stack([tiny, -tiny, huge, ties, ties * 2 ** -20, -ties * 2 ** 40])
    packed, scale = quantize_mxfp4(w.to(DEV), 32)
    packed_o, scale_o = oracle.quantize_mxfp4(w, 32)
    _assert_same(scale, scale_o, "E8M0 scales")
    _assert_same(packed, packed_o, "packed codes")


def test_mxfp4_dequantize_reference_golden_and_all_codes(oracle):
    from miles_amd.utils.mxfp4 import dequantize_mxfp4

    packed = torch.tensor([[0x10, 0x32, 0x54, 0x76]], dtype=torch.uint8)
    scales = torch.tensor([127, 128], dtype=torch.uint8)
    expected = torch.tensor([[0.0, 0.5, 1.0, 1.5, 4.0, 6.0, 8.0, 12.0]], dtype=torch.bfloat16)
    got = dequantize_mxfp4(packed.to(DEV), scales.to(DEV), 4)      # tests/fast/.../test_quantizer_mxfp4.py:6-16
    assert got.dtype == torch.bfloat16 and torch.equal(got.cpu(), expected)
    # every byte under every scale byte (0 = 2^-127 ... 254 = 2^127, 255 = 2^128 = inf), packed and generic paths
    packed = torch.arange(256, dtype=torch.uint8).repeat(256, 1)
    scales = torch.arange(256, dtype=torch.int32).to(torch.uint8).repeat_interleave(16)
    for G, sc in ((32, scales), (512, torch.arange(256, dtype=torch.int32).to(torch.uint8)), (2, None)):
        if sc is None:
            sc = torch.arange(256, dtype=torch.int32).to(torch.uint8).repeat_interleave(256)
        got = dequantize_mxfp4(packed.to(DEV), sc.to(DEV), G)
        want = oracle.dequantize_mxfp4(packed, sc, G)
        _assert_same(got, want, f"dequantized values, group {G}")


def test_mxfp4_requantizing_a_checkpoint_is_the_identity():
    from miles_amd.megatron_to_hf.processors.quantizer_compressed_tensors import quantize_params_compressed_tensors
    from miles_amd.utils.mxfp4 import dequantize_mxfp4, quantize_mxfp4

    # tests/fast-gpu/test_quantizer_ci.py:41-91
    g = torch.Generator().manual_seed(11)
    packed = torch.randint(0, 256, (16, 64), dtype=torch.uint8, generator=g).to(DEV)
    scale = torch.randint(96, 144, (16, 4), dtype=torch.uint8, generator=g).to(DEV)
    weight = dequantize_mxfp4(packed, scale, 32)
    p2, s2 = quantize_mxfp4(weight, 32)
    assert torch.equal(dequantize_mxfp4(p2, s2, 32).view(torch.int16), weight.view(torch.int16))
    config = {"format": "mxfp4-pack-quantized",
              "config_groups": {"group_0": {"weights": {"group_size": 32, "symmetric": True, "type": "float",
                                                        "num_bits": 4, "scale_dtype": "torch.uint8"}}}}
    results = quantize_params_compressed_tensors(
        [("model.layers.0.experts.0.w1.weight", torch.randn(64, 64, device=DEV))], config,
        {"model.layers.0.experts.0.w1"})
    assert [(n, t.dtype, tuple(t.shape)) for n, t in results] == [
        ("model.layers.0.experts.0.w1.weight_packed", torch.uint8, (64, 32)),
        ("model.layers.0.experts.0.w1.weight_scale", torch.uint8, (64, 2))]


def test_mxfp4_quantize_fp16(oracle):
    """The MXFP4 quantizer's fp16 instance: every fp16 pattern as a group maximum (the scale byte is read off the fp32
    pattern of the amax; subnormals, 65504, infinity and NaN included), ties at every bound in several binades, all
    fp16 patterns as elements, and a recorded list mixing bf16 and fp16 tensors."""
    from miles_amd import launch
    from miles_amd.utils.mxfp4 import quantize_mxfp4

    pats = torch.arange(0, 0x8000, dtype=torch.int32).to(torch.int16).view(torch.float16)          # 0 ... NaN patterns
    amax_rows = torch.zeros(0x8000, 32, dtype=torch.float16)
    amax_rows[:, 3] = pats                                      # one group per pattern: that value and small company
    amax_rows[:, 7] = (pats.float() * -0.6).to(torch.float16)
    amax_rows[:, 11] = (pats.float() * 0.31).to(torch.float16)
    ties = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0] * 4, dtype=torch.float16)
    tie_rows = torch.stack([ties, -ties, ties * 2 ** -10, ties * 2 ** 8, (ties.float() * 2 ** -14).to(torch.float16)])
    everything = torch.arange(-0x8000, 0x8000, dtype=torch.int32).to(torch.int16).view(torch.float16).reshape(2048, 32)
    for name, w in (("every amax", amax_rows), ("ties", tie_rows), ("every pattern", everything)):
        packed, scale = quantize_mxfp4(w.to(DEV), 32)
        packed_o, scale_o = oracle.quantize_mxfp4(w, 32)
        bad = torch.isnan(w.float()).any(dim=1)                  # a NaN in the group: the reference's result is undefined
        _assert_same(scale[~bad], scale_o[~bad], f"E8M0 scales ({name})")
        _assert_same(packed[~bad], packed_o[~bad], f"packed codes ({name})")
    tensors = []
    for i in range(9):
        t = W.student_t_rows((64 + 8 * i, 512), std=0.02, seed=6200 + i)
        tensors.append(t.to(torch.float16) if i % 3 else t)
    dev = [t.to(DEV) for t in tensors]
    with launch.recording() as batch:
        outs = [quantize_mxfp4(t, 32) for t in dev]
    batch.freeze()
    for rep in range(2):
        batch.run()
        torch.cuda.synchronize()
        for i, t in enumerate(tensors):
            for got, want, what in zip(outs[i], oracle.quantize_mxfp4(t, 32), ("packed", "scales")):
                _assert_same(got, want, f"tensor {i} ({t.dtype}) {what}, run {rep}")
        for o in outs:
            for t in o:
                t.view(torch.uint8).fill_(0x5A)


def test_mxfp4_grouped_jobs(oracle):
    from miles_amd import launch
    from miles_amd.utils.mxfp4 import quantize_mxfp4

    ws = [W.student_t_rows((96 + 32 * i, 256), std=0.02, seed=6100 + i) for i in range(5)]
    with launch.deferred():
        outs = [quantize_mxfp4(w.to(DEV), 32) for w in ws]
    for w, (p, s) in zip(ws, outs):
        p_o, s_o = oracle.quantize_mxfp4(w, 32)
        _assert_same(s, s_o, "E8M0 scales (grouped)")
        _assert_same(p, p_o, "packed codes (grouped)")


@pytest.mark.parametrize("shape,lo,hi", [((128, 128), 100, 140), ((256, 384), 120, 128), ((128, 256), 0, 30),
                                         ((128, 128), 225, 255), ((2048, 7168), 110, 135),
                                         ((256, 512), 250, 256), ((256, 256), 0, 256)])      # with the NaN byte 255
def test_mxfp4_to_fp8_recode(oracle, shape, lo, hi):
    from miles_amd.tools.convert_mxfp4_to_fp8 import cast_e2m1fn_to_e4m3fn

    g = torch.Generator().manual_seed(41)
    packed = torch.randint(0, 256, (shape[0], shape[1] // 2), dtype=torch.uint8, generator=g).view(torch.int8)
    scale = torch.randint(lo, hi, (shape[0], shape[1] // 32), dtype=torch.uint8, generator=g).view(torch.float8_e8m0fnu)
    y, ts = cast_e2m1fn_to_e4m3fn(packed.to(DEV), scale.to(DEV))
    y_o, ts_o = oracle.cast_e2m1fn_to_e4m3fn(packed, scale)
    assert y.dtype == torch.float8_e4m3fn and ts.dtype == torch.float32 and ts.shape == (shape[0] // 128, shape[1] // 128)
    _assert_same(ts, ts_o, "tile scales")
    _assert_same(y, y_o, "e4m3 codes")
    with pytest.raises(AssertionError):
        cast_e2m1fn_to_e4m3fn(packed[:100].to(DEV), scale[:100].to(DEV))


def test_mxfp4_to_fp8_recode_grouped(oracle):
    """A shard's experts re-coded inside `launch.deferred()`: tensors of different shapes share grouped launches
    (the larger ones set the grid, a single-pair tensor rides along), bytes as from single calls."""
    from miles_amd import launch
    from miles_amd.tools.convert_mxfp4_to_fp8 import cast_e2m1fn_to_e4m3fn

    g = torch.Generator().manual_seed(43)
    shapes = [(256, 512), (256, 384), (128, 128), (384, 256), (256, 512), (2048, 7168), (7168, 2048), (128, 256)]
    ins = []
    for shape in shapes:
        packed = torch.randint(0, 256, (shape[0], shape[1] // 2), dtype=torch.uint8, generator=g).view(torch.int8)
        scale = torch.randint(100, 140, (shape[0], shape[1] // 32), dtype=torch.uint8, generator=g).view(torch.float8_e8m0fnu)
        ins.append((packed, scale))
    dev = [(p.to(DEV), s.to(DEV)) for p, s in ins]
    with launch.deferred() as batch:
        outs = [cast_e2m1fn_to_e4m3fn(p, s) for p, s in dev]
    assert len(batch) == len(shapes) and batch.direct_calls == 0
    for (p, s), (y, ts) in zip(ins, outs):
        y_o, ts_o = oracle.cast_e2m1fn_to_e4m3fn(p, s)
        _assert_same(ts, ts_o, "tile scales (grouped)")
        _assert_same(y, y_o, "e4m3 codes (grouped)")
    # scale bytes off a 4-byte boundary: the group falls back to the one-launch tile form
    odd = []
    for p, s in ins[:3]:
        flat = torch.zeros(s.numel() + 1, dtype=torch.uint8, device=DEV)
        flat[1:] = s.view(torch.uint8).reshape(-1).to(DEV)
        odd.append((p.to(DEV), flat[1:].view(s.shape).view(torch.float8_e8m0fnu)))
    assert all(s.data_ptr() % 4 == 1 for _, s in odd)
    with launch.deferred():
        outs = [cast_e2m1fn_to_e4m3fn(p, s) for p, s in odd]
    for (p, s), (y, ts) in zip(ins[:3], outs):
        y_o, ts_o = oracle.cast_e2m1fn_to_e4m3fn(p, s)
        _assert_same(ts, ts_o, "tile scales (grouped, unaligned scales)")
        _assert_same(y, y_o, "e4m3 codes (grouped, unaligned scales)")


def test_unpacking_jobs_grouped(oracle):
    """A shard's INT4 experts unpacked, and its MXFP4 tensors dequantized, inside `launch.deferred()`: tensors of
    different sizes share grouped launches (the largest sets the grid, a one-row tensor rides along); a tensor the flat
    kernel does not take (a group that is no power-of-two number of words, scales of another dtype) goes out on its
    own; values as from single calls, which are checked against the oracle."""
    from miles_amd import launch
    from miles_amd.tools.convert_kimi_int4_to_bf16 import _dequantize_tensor
    from miles_amd.utils.mxfp4 import dequantize_mxfp4

    g = torch.Generator().manual_seed(47)
    cases = [((256, 512), 128, torch.bfloat16), ((1, 128), 128, torch.bfloat16), ((2048, 7168), 128, torch.bfloat16),
             ((7168, 2048), 128, torch.bfloat16), ((3, 100), 20, torch.bfloat16), ((64, 256), 128, torch.float32),
             ((64, 256), 32, torch.bfloat16), ((512, 1024), 128, torch.bfloat16)]
    ins = []
    for (m, k), G, sdt in cases:
        packed = torch.randint(-2**31, 2**31 - 1, (m, -(-k // 8)), dtype=torch.int64, generator=g).to(torch.int32)
        ins.append((packed, torch.exp(torch.randn((m, k // G), generator=g) * 3).to(sdt), (m, k), G))
    dev = [(p.to(DEV), s.to(DEV), shape, G) for p, s, shape, G in ins]
    with launch.deferred() as batch:
        outs = [_dequantize_tensor(*args) for args in dev]
    assert len(batch) == len(cases) and batch.direct_calls == 0
    for (p, s, shape, G), got in zip(ins, outs):
        _assert_same(got, oracle.int4_unpack_dequant(p, s, shape, G), f"INT4 unpack (grouped) {shape} group {G}")

    m4 = []
    for shape, G in (((256, 512), 32), ((1, 32), 32), ((2048, 7168), 32), ((7168, 2048), 32), ((16, 48), 16),
                     ((8, 64), 2), ((512, 1024), 32)):
        packed = torch.randint(0, 256, (shape[0], shape[1] // 2), dtype=torch.uint8, generator=g)
        scale = torch.randint(0, 256, (shape[0] * shape[1] // G,), dtype=torch.int32, generator=g).to(torch.uint8)
        m4.append((packed, scale, G))
    with launch.deferred() as batch:
        outs = [dequantize_mxfp4(p.to(DEV), s.to(DEV), G) for p, s, G in m4]
    assert len(batch) == len(m4) and batch.direct_calls == 0
    for (p, s, G), got in zip(m4, outs):
        _assert_same(got, oracle.dequantize_mxfp4(p, s, G), f"MXFP4 dequantize (grouped) {tuple(p.shape)} group {G}")


def test_unpacking_job_argument_checks(lib):
    from miles_amd import _lib

    buf = torch.zeros(1 << 16, dtype=torch.uint8, device=DEV)
    def job(kind, rows, cols, group, dtype=0, aux=True):
        return (_lib.Job * 1)(_lib.Job(kind, dtype, buf.data_ptr(), buf.data_ptr() + 32768, None,
                                       buf.data_ptr() + 16384 if aux else None, None, rows, cols, cols, group, 0, 0, 0))
    for kind in (_lib.JOB_INT4_UNPACK, _lib.JOB_MXFP4_DEQUANT):
        assert lib.mq_run_jobs(job(kind, 8, 128, 32), 1, None) == 0
        assert lib.mq_run_jobs(job(kind, 0, 128, 32, aux=False), 1, None) == 0     # an empty tensor has no address
        assert lib.mq_run_jobs(job(kind, 8, 128, 0), 1, None) != 0                 # no group size
        assert lib.mq_run_jobs(job(kind, 8, 128, 32, aux=False), 1, None) != 0     # no scales
        assert b"unpacking job" in lib.mq_last_error()
    assert lib.mq_run_jobs(job(_lib.JOB_INT4_UNPACK, 8, 100, 32), 1, None) != 0    # K not a multiple of the group
    assert lib.mq_run_jobs(job(_lib.JOB_INT4_UNPACK, 8, 128, 32, dtype=3), 1, None) != 0
    assert lib.mq_run_jobs(job(_lib.JOB_MXFP4_DEQUANT, 3, 11, 32), 1, None) != 0   # 33 elements
    torch.cuda.synchronize()


def test_mxfp4_to_fp8_job_argument_checks(lib):
    from miles_amd import _lib

    buf = torch.zeros(1 << 16, dtype=torch.uint8, device=DEV)
    def job(rows, cols, offset=0):
        return (_lib.Job * 1)(_lib.Job(_lib.JOB_MXFP4_TO_FP8, 0, buf.data_ptr() + offset, buf.data_ptr(), buf.data_ptr(),
                                       buf.data_ptr(), None, rows, cols, cols, 0, 0, 0, 0))
    assert lib.mq_run_jobs(job(128, 128), 1, None) == 0
    assert lib.mq_run_jobs(job(100, 128), 1, None) != 0          # rows not a multiple of 128
    assert lib.mq_run_jobs(job(128, 128, offset=8), 1, None) != 0  # packed codes off a 16-byte boundary
    torch.cuda.synchronize()


# ---------------------------------------------------------------------------------------------------
# block fake quantization (miles/kernels/quant/fake_quant.py)
@pytest.mark.parametrize("kind", ["fp8", "fp4", "compressed_kv"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_fake_quant_forward(oracle, kind, dtype):
    from miles_amd.kernels.quant import fake_quant as fq

    fn = {"fp8": fq.fake_quant_fp8_forward, "fp4": fq.fake_quant_fp4_forward,
          "compressed_kv": fq.fake_quant_compressed_kv_forward}[kind]
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(3, 37, 512, generator=g) * torch.logspace(-3, 3, 512)).to(dtype)   # the reference test's input
    x[0, 0, :32] = 0
    x[1, 0, :64] = torch.tensor([-0.0, 0.0] * 32).to(dtype)
    x[1, 1, :8] = torch.tensor([448.0, -448.0, 6.0, -6.0, 3.5, 2.5, 0.75, -1e-30]).to(dtype)
    x[1, 2, :32] = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0] * 4).to(dtype)     # every fp4 tie, scale 1
    x[2, 0, :32] = torch.finfo(dtype).max if dtype != torch.float32 else 1e38
    got = fn(x.to(DEV))
    assert got.dtype == dtype and got.shape == x.shape
    _assert_same(got, oracle.fake_quant(x, kind), f"fake_quant {kind}")


def test_fake_quant_backward_is_straight_through_and_checks_shape():
    from miles_amd.kernels.quant import fake_quant as fq

    for fn in (fq.fake_quant_fp8, fq.fake_quant_fp4, fq.fake_quant_compressed_kv):   # test_fake_quant.py:63-70
        x = torch.randn(64, 256, device=DEV, dtype=torch.bfloat16, requires_grad=True)
        grad = torch.randn_like(x)
        fn(x).backward(grad)
        assert torch.equal(x.grad, grad)
    with pytest.raises(AssertionError):
        fq.fake_quant_fp8_forward(torch.zeros(4, 48, device=DEV, dtype=torch.bfloat16))
    # 16-wide blocks: 48 columns are fine here; 1 -> scale e4m3(1/6) = 0.171875, 1/scale = 5.8 -> 6 -> 1.03125
    assert torch.equal(fq.fake_quant_compressed_kv_forward(torch.ones(4, 48, device=DEV)).cpu(), torch.full((4, 48), 1.03125))


# ---------------------------------------------------------------------------------------------------
NV_SHAPES = W.SMALL_REFERENCE_SHAPES + [(1, 16), (1, 32), (3, 48), (31, 128), (256, 256), (1024, 2048)]


@pytest.mark.parametrize("shape", NV_SHAPES)
@pytest.mark.parametrize("kind", ["random", "boundary", "zeros", "signed_zeros", "maxes"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_nvfp4_quantize_1d(oracle, shape, kind, dtype):
    from miles_amd.utils.nvfp4 import nvfp4_quantize_1d

    if dtype == torch.float32 and shape[0] * shape[1] > 300000:
        pytest.skip("generic-dtype path is covered by the smaller shapes")
    w = W.reference_pattern(kind, shape, dtype=dtype, spread=12.0)
    if kind == "random" and shape[0] > 1:
        w[0].zero_()
    q, s, g = nvfp4_quantize_1d(w.to(DEV))
    q_o, s_o, g_o = oracle.nvfp4_quantize_1d(w)
    assert q.dtype == torch.uint8 and s.dtype == F8 and g.dtype == torch.float32 and g.shape == ()
    _assert_same(g, g_o, "global scale")
    _assert_same(s, s_o, "block scales")
    _assert_same(q, q_o, "codes")


def test_nvfp4_pair_and_global_scale_helpers(oracle):
    from miles_amd.utils import nvfp4 as N

    base = W.reference_pattern("random", (64, 256), spread=12.0, seed=3)
    base[40:] *= 5
    dev = base.to(DEV)
    gate, up = dev.chunk(2, dim=0)
    (gq, gs, gg), (uq, us, ug) = N.nvfp4_quantize_1d_pair(gate, up)
    (gq_o, gs_o, gg_o), (uq_o, us_o, ug_o) = oracle.nvfp4_quantize_1d_pair(base[:32], base[32:])
    for got, want, what in [(gq, gq_o, "gate codes"), (gs, gs_o, "gate scales"), (gg, gg_o, "gate global"),
                            (uq, uq_o, "up codes"), (us, us_o, "up scales"), (ug, ug_o, "up global")]:
        _assert_same(got, want, what)
    assert gg.data_ptr() != ug.data_ptr() and gg.item() == ug.item()
    with pytest.raises(ValueError, match="expects two 2D tensors"):
        N.nvfp4_quantize_1d_pair(gate[0], up)
    with pytest.raises(ValueError, match="matching K dimensions"):
        N.nvfp4_quantize_1d_pair(gate, up[:, :128])
    # closed forms on the device without a host read (tests/fast-gpu/test_nvfp4_quantizer.py:108-143)
    values = torch.tensor([0.0, 1.0, 3.5, torch.finfo(torch.float32).tiny, torch.finfo(torch.float32).max,
                           float("inf"), -float("inf"), float("nan")], dtype=torch.float32)
    for e4m3_max in (256, 448):
        expected = torch.div(torch.tensor(float(e4m3_max)) * torch.tensor(6.0), values)
        expected = torch.min(expected, torch.tensor(torch.finfo(torch.float32).max))
        expected = torch.where(expected == 0.0, torch.ones_like(expected), expected)
        enc = N.nvfp4_global_encode_scale_te(values.to(DEV), e4m3_max).cpu()
        dec = N.nvfp4_global_decode_scale_te(values.to(DEV), e4m3_max).cpu()
        torch.testing.assert_close(enc, expected, rtol=0, atol=0, equal_nan=True)
        torch.testing.assert_close(dec, torch.div(1.0, expected), rtol=0, atol=0, equal_nan=True)


# ---------------------------------------------------------------------------------------------------
# benchmark-sized tensors: full byte comparison against the oracle
# ---------------------------------------------------------------------------------------------------
def test_c1_full_size_block_fp8(oracle):
    from miles_amd.tools.convert_hf_to_fp8 import block_fp8

    for name, w in W.c1_mlp().items():
        q, s = block_fp8(w.to(DEV), [128, 128])
        q_o, s_o = oracle.block_fp8(w, (128, 128))
        _assert_same(s, s_o, f"C1 {name} scale")
        _assert_same(q, q_o, f"C1 {name} codes")


def test_c2_layer_full_size_blockwise_cast(oracle):
    from miles_amd.kernels.quant.fp8_blockwise import fp8_blockwise_cast

    for idx, (name, shape) in enumerate(W.c2_layer_shapes()):
        w = W.c2_tensor(17, idx, shape)
        y, s = fp8_blockwise_cast(w.to(DEV))
        y_o, s_o = oracle.fp8_blockwise_cast(w)
        _assert_same(s, s_o, f"C2 {name} scale")
        _assert_same(y, y_o, f"C2 {name} codes")


def test_c3_c4_c5_full_size_experts(oracle):
    from miles_amd.kernels.quant.int4_fake import pack_layer
    from miles_amd.tools.convert_hf_to_fp8 import block_fp8
    from miles_amd.tools.fp8_cast_bf16 import weight_dequant
    from miles_amd.utils.mxfp8 import mxfp8_quantize
    from miles_amd.utils.nvfp4 import nvfp4_quantize_1d, nvfp4_quantize_1d_pair

    for which in (0, 2):
        w = W.c3_expert(5, 77, which)
        q, s = mxfp8_quantize(w.to(DEV))
        q_o, s_o = oracle.mxfp8_quantize(w)
        _assert_same(s, s_o, "C3 scales")
        _assert_same(q, q_o, "C3 codes")
    for which in (1, 2):
        w = W.c4_expert(3, which)
        p, s, _ = pack_layer(w.to(DEV), 128)
        p_o, s_o, _ = oracle.pack_layer(w, 128)
        _assert_same(s, s_o, "C4 scales")
        _assert_same(p, p_o, "C4 packed")
    gate, up, down = (W.c5_expert(9, i) for i in range(3))
    both = torch.cat((gate, up), dim=0).to(DEV)
    (gq, gs, gg), (uq, us, ug) = nvfp4_quantize_1d_pair(*both.chunk(2, dim=0))
    (gq_o, gs_o, gg_o), (uq_o, us_o, ug_o) = oracle.nvfp4_quantize_1d_pair(gate, up)
    for got, want, what in [(gq, gq_o, "C5 gate codes"), (gs, gs_o, "C5 gate scales"), (gg, gg_o, "C5 gate global"),
                            (uq, uq_o, "C5 up codes"), (us, us_o, "C5 up scales"), (ug, ug_o, "C5 up global")]:
        _assert_same(got, want, what)
    dq, ds, dg = nvfp4_quantize_1d(down.to(DEV))
    dq_o, ds_o, dg_o = oracle.nvfp4_quantize_1d(down)
    _assert_same(dq, dq_o, "C5 down codes")
    _assert_same(ds, ds_o, "C5 down scales")
    _assert_same(dg, dg_o, "C5 down global")
    q, s = block_fp8(down.to(DEV), [128, 128])
    y = weight_dequant(q, s)
    _assert_same(y, oracle.weight_dequant(*oracle.block_fp8(down, (128, 128))), "C5b round trip")


# ---------------------------------------------------------------------------------------------------
# batched submission and the raw C ABI
# ---------------------------------------------------------------------------------------------------
def test_deferred_batch_equals_immediate_calls(oracle):
    from miles_amd import launch
    from miles_amd.kernels.quant.fp8_blockwise import fp8_blockwise_cast
    from miles_amd.kernels.quant.int4_fake import pack_layer
    from miles_amd.tools.convert_hf_to_fp8 import block_fp8
    from miles_amd.tools.fp8_cast_bf16 import weight_dequant
    from miles_amd.utils.mxfp8 import mxfp8_quantize
    from miles_amd.utils.nvfp4 import nvfp4_quantize_1d, nvfp4_quantize_1d_pair

    shapes = [(256, 384), (128, 128), (130, 384), (1024, 512), (64, 7168)] * 15     # 75 tensors: more than one group
    ws = [W.gaussian_outliers(s, std=0.02, p_outlier=0.001, gain=20.0, seed=100 + i) for i, s in enumerate(shapes)]
    odd = W.gaussian_outliers((96, 100), std=0.02, p_outlier=0.0, gain=1.0, seed=7)      # not 8-aligned: generic kernel
    dev = [w.to(DEV) for w in ws]
    q_in, s_in = oracle.block_fp8(ws[0], (128, 128))
    with launch.deferred() as batch:
        cast = [fp8_blockwise_cast(w) for w in dev]
        cast_odd = fp8_blockwise_cast(odd.to(DEV))
        blk = [block_fp8(w, [128, 128]) for w in dev[:5]]
        mx = [mxfp8_quantize(w) for w in dev]
        i4 = [pack_layer(w, 128) for w in dev[:5]]
        nv = [nvfp4_quantize_1d(w) for w in dev[:5]]
        nv_pair = nvfp4_quantize_1d_pair(dev[0], dev[5])
        deq = weight_dequant(q_in.to(DEV), s_in.to(DEV))
        assert len(batch) == 75 + 1 + 5 + 75 + 5 + 5 + 2 + 1
    for w, (y, s) in zip(ws, cast):
        y_o, s_o = oracle.fp8_blockwise_cast(w)
        _assert_same(s, s_o, "cast scale")
        _assert_same(y, y_o, "cast codes")
    _assert_same(cast_odd[0], oracle.fp8_blockwise_cast(odd)[0], "cast codes (generic in batch)")
    for w, (y, s) in zip(ws, blk):
        y_o, s_o = oracle.block_fp8(w, (128, 128))
        _assert_same(s, s_o, "block scale")
        _assert_same(y, y_o, "block codes")
    for w, (y, s) in zip(ws, mx):
        y_o, s_o = oracle.mxfp8_quantize(w)
        _assert_same(s, s_o, "mx scale")
        _assert_same(y, y_o, "mx codes")
    for w, (p, s, _) in zip(ws, i4):
        p_o, s_o, _ = oracle.pack_layer(w, 128)
        _assert_same(s, s_o, "int4 scale")
        _assert_same(p, p_o, "int4 packed")
    for w, (q, s, g) in zip(ws, nv):
        q_o, s_o, g_o = oracle.nvfp4_quantize_1d(w)
        _assert_same(g, g_o, "nv global")
        _assert_same(s, s_o, "nv scale")
        _assert_same(q, q_o, "nv codes")
    (aq, a_s, ag), (bq, b_s, bg) = nv_pair
    (aq_o, as_o, ag_o), (bq_o, bs_o, bg_o) = oracle.nvfp4_quantize_1d_pair(ws[0], ws[5])
    for got, want, what in [(aq, aq_o, "pair a codes"), (a_s, as_o, "pair a scales"), (ag, ag_o, "pair a global"),
                            (bq, bq_o, "pair b codes"), (b_s, bs_o, "pair b scales"), (bg, bg_o, "pair b global")]:
        _assert_same(got, want, what)
    _assert_same(deq, oracle.weight_dequant(q_in, s_in), "dequant in batch")


def test_c_abi_single_tensor_entry_points(oracle, lib):
    """Each extern "C" quantizer called directly with raw pointers, as a non-Python host would."""
    w = W.gaussian_outliers((256, 512), std=0.02, p_outlier=0.001, gain=20.0, seed=77)
    d = w.to(DEV)
    M, K = w.shape
    q = torch.empty((M, K), dtype=torch.uint8, device=DEV)
    s = torch.empty((2, 4), dtype=torch.float32, device=DEV)
    assert lib.mq_fp8_block_quant(d.data_ptr(), 0, K, q.data_ptr(), s.data_ptr(), M, K, 128, 128, None) == 0
    q_o, s_o = oracle.block_fp8(w, (128, 128))
    _assert_same(q, q_o, "mq_fp8_block_quant codes")
    _assert_same(s, s_o, "mq_fp8_block_quant scale")
    assert lib.mq_fp8_blockwise_cast(d.data_ptr(), 0, K, 1, q.data_ptr(), s.data_ptr(), M, K, 128, 128, None) == 0
    q_o, s_o = oracle.fp8_blockwise_cast(w)
    _assert_same(q, q_o, "mq_fp8_blockwise_cast codes")
    y = torch.empty((M, K), dtype=torch.bfloat16, device=DEV)
    assert lib.mq_fp8_block_dequant(q.data_ptr(), s.data_ptr(), y.data_ptr(), M, K, 128, None) == 0
    _assert_same(y, oracle.weight_dequant(q_o, s_o), "mq_fp8_block_dequant")
    sc = torch.empty((M, K // 32), dtype=torch.uint8, device=DEV)
    assert lib.mq_mxfp8_quant(d.data_ptr(), 0, q.data_ptr(), sc.data_ptr(), M, K, None) == 0
    q_o, sc_o = oracle.mxfp8_quantize(w)
    _assert_same(q, q_o, "mq_mxfp8_quant codes")
    _assert_same(sc, sc_o, "mq_mxfp8_quant scales")
    packed = torch.empty((M, K // 8), dtype=torch.int32, device=DEV)
    s16 = torch.empty((M, K // 128), dtype=torch.bfloat16, device=DEV)
    assert lib.mq_int4_group_quant_pack(d.data_ptr(), 0, packed.data_ptr(), s16.data_ptr(), M, K, 128, None) == 0
    p_o, s_o, _ = oracle.pack_layer(w, 128)
    _assert_same(packed, p_o, "mq_int4_group_quant_pack words")
    _assert_same(s16, s_o, "mq_int4_group_quant_pack scales")
    word = torch.empty(1280, dtype=torch.int32, device=DEV)
    q4 = torch.empty((M, K // 2), dtype=torch.uint8, device=DEV)
    s8 = torch.empty((M, K // 16), dtype=torch.uint8, device=DEV)
    g = torch.empty((), dtype=torch.float32, device=DEV)
    assert lib.mq_fill_u32(word.data_ptr(), 0x7F800000, 1280, None) == 0   # stale contents must not matter
    assert lib.mq_nvfp4_amax(d.data_ptr(), 0, M * K, word.data_ptr(), 0, None) == 0
    assert lib.mq_nvfp4_quant(d.data_ptr(), 0, word.data_ptr(), 1, q4.data_ptr(), s8.data_ptr(), g.data_ptr(), M, K, 448, 0,
                              None) == 0
    q_o, s_o, g_o = oracle.nvfp4_quantize_1d(w)
    _assert_same(q4, q_o, "mq_nvfp4_quant codes")
    _assert_same(s8, s_o, "mq_nvfp4_quant scales")
    _assert_same(g, g_o, "mq_nvfp4_quant global")
    assert word[:256].view(torch.float32).max().item() == w.float().abs().max().item()
    # argument errors come back as codes with a message, never as a fault
    from miles_amd import _lib as L

    assert lib.mq_mxfp8_quant(d.data_ptr(), 0, q.data_ptr(), sc.data_ptr(), M, 48, None) == -1
    assert b"divisible by 32" in lib.mq_last_error()
    assert lib.mq_fp8_block_quant(None, 0, K, q.data_ptr(), s.data_ptr(), M, K, 128, 128, None) == -1
    assert L.load() is lib


# ---------------------------------------------------------------------------------------------------
# fused NVFP4 quantize-dequantize (miles/kernels/quant/nvfp4_qdq.py)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(1, 16), (3, 48), (16, 64), (64, 128), (128, 1024), (2048, 7168)])
@pytest.mark.parametrize("kind", ["random", "boundary", "zeros", "signed_zeros", "maxes"])
def test_nvfp4_qdq(oracle, shape, kind, dtype):
    from miles_amd.kernels.quant.nvfp4_qdq import NVFP4QDQConfig, compute_nvfp4_amax, fused_nvfp4_qdq

    if shape[0] > 1000 and (kind != "random" or dtype != torch.bfloat16):
        pytest.skip("the full-size tensor is checked once")
    x = W.reference_pattern(kind, shape, dtype=dtype, spread=12.0)
    xd = x.to(DEV)
    amax = compute_nvfp4_amax(xd)
    assert amax.dtype == torch.float32 and amax.dim() == 0 and amax.item() == x.float().abs().max().item()
    got = fused_nvfp4_qdq(xd, amax, NVFP4QDQConfig())
    assert got.dtype == dtype and got.shape == x.shape
    _assert_same(got, oracle.fused_nvfp4_qdq(x), "dequantized values")


def test_nvfp4_qdq_ste_and_argument_checks(monkeypatch):
    from miles_amd.kernels.quant import nvfp4_qdq as m

    for name in ("NVTE_USE_FAST_MATH", "NVTE_NVFP4_4OVER6", "NVTE_NVFP4_4OVER6_E4M3_USE_256"):
        monkeypatch.delenv(name, raising=False)
    x = torch.randn(64, 256, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    x.main_grad = torch.zeros_like(x)
    y = m.fake_nvfp4_quantization_ste(x)
    grad = torch.randn_like(x)
    y.backward(grad)
    assert torch.equal(x.grad, grad) and y.main_grad is x.main_grad
    amax = m.compute_nvfp4_amax(x)
    with pytest.raises(TypeError, match="BF16 and FP16"):
        m.fused_nvfp4_qdq(x.detach().float(), amax)
    with pytest.raises(ValueError, match="K divisible by 16"):
        m.fused_nvfp4_qdq(torch.zeros(4, 24, device=DEV, dtype=torch.bfloat16), amax)
    with pytest.raises(ValueError, match="rank-2"):
        m.fused_nvfp4_qdq(torch.zeros(64, device=DEV, dtype=torch.bfloat16), amax)
    with pytest.raises(TypeError, match="exactly one FP32"):
        m.fused_nvfp4_qdq(x.detach(), amax.double())
    with pytest.raises(ValueError, match="only supported by Four Over Six"):
        m.NVFP4QDQConfig(e4m3_max=256)
    monkeypatch.setenv("NVTE_USE_FAST_MATH", "1")
    with pytest.raises(ValueError, match="NVTE_USE_FAST_MATH=0"):
        m.current_nvfp4_qdq_config()


def test_nvfp4_fake_qat_switch_on_grouped_weights(oracle, monkeypatch):
    # miles/utils/nvfp4_fake_qat.py:10-23: one configuration for the whole list, every weight through the fused q-dq
    from miles_amd.utils import nvfp4_fake_qat as qat

    for name in ("NVTE_USE_FAST_MATH", "NVTE_NVFP4_4OVER6", "NVTE_NVFP4_4OVER6_E4M3_USE_256"):
        monkeypatch.delenv(name, raising=False)
    cpu = [W.gaussian_outliers((64, 256), std=0.02, p_outlier=0.001, gain=20.0, seed=970 + i) for i in range(3)]
    weights = [torch.nn.Parameter(w.to(DEV)) for w in cpu]
    monkeypatch.setenv(qat.NVFP4_FAKE_QAT_FLAG, "1")
    out = qat.maybe_fake_quantize_nvfp4_weight_tensors(weights)
    assert len(out) == 3 and all(o.requires_grad for o in out)
    for o, w in zip(out, cpu):
        _assert_same(o.detach(), oracle.fused_nvfp4_qdq(w), "fake-quantized weight")
    sum(o.float().sum() for o in out).backward()
    assert all(torch.equal(w.grad, torch.ones_like(w)) for w in weights)


# ---------------------------------------------------------------------------------------------------
# NVFP4 Four Over Six block scaling (NVTE_NVFP4_4OVER6; miles/kernels/quant/nvfp4_qdq.py:893-990)
_FOS_CASES = [(448, "MAE", False), (256, "MAE", False), (256, "MSE", False), (256, "MAE", True), (448, "MSE", True)]


def _fos_env(monkeypatch, e4m3_max, mode, fp16):
    monkeypatch.setenv("NVTE_NVFP4_4OVER6", "weights")
    monkeypatch.setenv("NVTE_NVFP4_4OVER6_E4M3_USE_256", "all" if e4m3_max == 256 else "none")
    monkeypatch.setenv("NVTE_NVFP4_4OVER6_ERR_MODE", mode)
    monkeypatch.setenv("NVTE_NVFP4_4OVER6_ERR_USE_FAST_MATH", "1" if fp16 else "0")
    monkeypatch.delenv("NVTE_USE_FAST_MATH", raising=False)


@pytest.mark.parametrize("e4m3_max,mode,fp16", _FOS_CASES)
@pytest.mark.parametrize("shape", [(1, 16), (3, 48), (64, 128), (128, 1024), (512, 7168)])
@pytest.mark.parametrize("kind", ["random", "boundary", "zeros", "signed_zeros", "maxes"])
def test_nvfp4_four_over_six_quantizer(oracle, monkeypatch, shape, kind, e4m3_max, mode, fp16):
    from miles_amd.utils.nvfp4 import nvfp4_quantize_1d, nvfp4_quantize_1d_pair

    if shape[0] > 500 and kind != "random":
        pytest.skip("the large tensor is checked on random data")
    _fos_env(monkeypatch, e4m3_max, mode, fp16)
    flags = oracle.NVFP4_4OVER6 | (oracle.NVFP4_ERR_MSE if mode == "MSE" else 0) | (oracle.NVFP4_ERR_FP16 if fp16 else 0)
    w = W.reference_pattern(kind, shape, spread=12.0)
    if kind == "random" and shape[0] > 1:
        w[0].zero_()
    q, s, g = nvfp4_quantize_1d(w.to(DEV))
    q_o, s_o, g_o = oracle.nvfp4_quantize_1d(w, e4m3_max=e4m3_max, flags=flags)
    _assert_same(s, s_o, "block scales")
    _assert_same(q, q_o, "codes")
    _assert_same(g, g_o, "global scale")
    if shape == (64, 128):
        up = 3 * W.reference_pattern("random", (32, 128), spread=12.0, seed=2)
        (gq, gs, gg), (uq, us, ug) = nvfp4_quantize_1d_pair(w.to(DEV), up.to(DEV))
        (gq_o, gs_o, gg_o), (uq_o, us_o, ug_o) = oracle.nvfp4_quantize_1d_pair(w, up, e4m3_max=e4m3_max, flags=flags)
        for a, b, what in ((gq, gq_o, "pair codes"), (gs, gs_o, "pair scales"), (uq, uq_o, "pair up codes"), (us, us_o, "pair up scales"),
                           (gg, gg_o, "pair global"), (ug, ug_o, "pair up global")):
            _assert_same(a, b, what)


@pytest.mark.parametrize("e4m3_max,mode,fp16", _FOS_CASES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_nvfp4_four_over_six_qdq_and_other_dtypes(oracle, monkeypatch, dtype, e4m3_max, mode, fp16):
    from miles_amd.kernels.quant import nvfp4_qdq as m
    from miles_amd.utils.nvfp4 import nvfp4_quantize_1d

    _fos_env(monkeypatch, e4m3_max, mode, fp16)
    flags = oracle.NVFP4_4OVER6 | (oracle.NVFP4_ERR_MSE if mode == "MSE" else 0) | (oracle.NVFP4_ERR_FP16 if fp16 else 0)
    x = W.reference_pattern("random", (96, 256), dtype=dtype, spread=12.0, seed=5)
    x[1].zero_()
    cfg = m.current_nvfp4_qdq_config()
    assert cfg.use_4over6 and cfg.e4m3_max == e4m3_max and cfg.error_use_fast_math == fp16 and cfg.error_mode.name == mode
    got = m.fused_nvfp4_qdq(x.to(DEV), m.compute_nvfp4_amax(x.to(DEV)), cfg)
    _assert_same(got, oracle.fused_nvfp4_qdq(x, e4m3_max=e4m3_max, flags=flags), "dequantized values")
    # an amax handed in from elsewhere (a calibrated one, say) may use all 24 bits of its mantissa: value x scale x amax is
    # then no longer exact in any order, and the kernel keeps the reference's order of the two multiplications
    wide = torch.tensor(float(x.abs().max()) * 1.0001234, dtype=torch.float32)
    assert int(wide.view(torch.int32)) & 0xFFF
    got = m.fused_nvfp4_qdq(x.to(DEV), wide.to(DEV), cfg)
    _assert_same(got, oracle.fused_nvfp4_qdq(x, amax=wide, e4m3_max=e4m3_max, flags=flags), "dequantized values (24-bit amax)")
    # fp16 / fp32 weights take the one-lane-per-block quantizer kernel
    xf = x.float() if dtype == torch.float16 else x.half()
    q, s, g = nvfp4_quantize_1d(xf.to(DEV))
    q_o, s_o, g_o = oracle.nvfp4_quantize_1d(xf, e4m3_max=e4m3_max, flags=flags)
    _assert_same(s, s_o, "block scales (generic kernel)")
    _assert_same(q, q_o, "codes (generic kernel)")


@pytest.mark.parametrize("sym", [True, False])
@pytest.mark.parametrize("shape,block", [((64, 96), (32, 1)), ((70, 33), (32, 1)), ((16, 64), (4, 8)), ((18, 40), (2, 16)),
                                          ((40, 64), (8, 32)), ((5, 200), (1, 64)), ((256, 512), (32, 1))])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_fake_int4_quant_general_blocks(oracle, shape, block, sym, dtype):
    from miles_amd.kernels.quant.int4_fake import fake_int4_quant_cuda

    w = W.gaussian_outliers(shape, std=0.015, p_outlier=0.001, gain=30.0, seed=4003, dtype=dtype)
    w[0] = 0
    out, scale, zero = fake_int4_quant_cuda(w.to(DEV), block, sym)
    out_o, scale_o, zero_o = oracle.fake_int4_quant(w, block, sym)
    assert scale.shape == (-(-shape[0] // block[0]), -(-shape[1] // block[1]))
    _assert_same(out, out_o, "values")
    _assert_same(scale, scale_o, "scales")
    if not sym:
        _assert_same(zero, zero_o, "zero points")


@pytest.mark.parametrize("shape", W.SMALL_REFERENCE_SHAPES + [(130, 257), (256, 384), (4096, 2560)])
@pytest.mark.parametrize("kind", W.PATTERNS)
def test_fp8_power_of_two_scales(oracle, shape, kind):
    from miles_amd.kernels.quant.fp8_blockwise import per_block_cast_to_fp8

    if shape[0] > 1000 and kind != "random":
        pytest.skip("the full-size tensor is checked on random data")
    x = W.reference_pattern(kind, shape, spread=512.0, amplitude=16.0)
    y, s = per_block_cast_to_fp8(x.to(DEV))
    y_o, s_o = oracle.per_block_cast_to_fp8(x)
    assert y.dtype == torch.float8_e4m3fn and s.dtype == torch.float32
    _assert_same(s, s_o, "scales")
    _assert_same(y, y_o, "codes")
    if shape == (256, 384):     # fp32 input and a row-strided view take the generic kernel
        xf = torch.cat((x.float(), x.float()), dim=1)[:, :384]
        y2, s2 = per_block_cast_to_fp8(xf.to(DEV))
        y2_o, s2_o = oracle.per_block_cast_to_fp8(xf)
        _assert_same(s2, s2_o, "scales (fp32, strided)")
        _assert_same(y2, y2_o, "codes (fp32, strided)")


@pytest.mark.parametrize("shape,mn", [((1, 1), 1), ((2, 5), 200), ((3, 4), 384), ((3, 2, 7), 130), ((1, 3, 8), 128),
                                      ((2, 4), 250), ((76, 20), 9728), ((4, 3), 300)])
def test_transform_scale_ue8m0(oracle, shape, mn):
    from miles_amd.kernels.quant.fp8_blockwise import transform_scale_ue8m0

    g = torch.Generator().manual_seed(43)
    sf = torch.exp2(torch.randint(-40, 20, shape, generator=g).float())
    got, want = transform_scale_ue8m0(sf.to(DEV), mn), oracle.transform_scale_ue8m0(sf, mn)
    assert got.dtype == torch.int32 and got.shape == want.shape and got.stride() == want.stride()
    assert torch.equal(got.cpu(), want)
    # the padding rows of the storage are written too (zeros), as in the published construction
    amn, kw = -(-mn // 4) * 4, got.shape[-1]
    batch = got.shape[0] if got.dim() == 3 else 1
    whole = torch.as_strided(got, (batch, amn, kw), (kw * amn, 1, amn), got.storage_offset())
    assert torch.all(whole[:, mn:, :] == 0)
    with pytest.raises(IndexError):
        transform_scale_ue8m0(sf.to(DEV), 128 * shape[-2] + 1)
    # the contiguous form of the same words (what a flattened payload holds)
    from miles_amd import _lib
    sfd = sf.to(DEV).reshape(batch, shape[-2], shape[-1])
    dense = torch.full((batch, mn, kw), -1, dtype=torch.int32, device=DEV)
    _lib.check(_lib.load().mq_ue8m0_pack_scales(sfd.data_ptr(), dense.data_ptr(), batch, mn, shape[-1], shape[-2], 1,
                                                _lib.stream_ptr(dense.device)))
    assert torch.equal(dense.cpu().reshape(want.shape), want.contiguous())


@pytest.mark.parametrize("shape", [(256, 384), (130, 257), (3, 256, 128), (2, 2, 128, 256)])
def test_quant_weight_ue8m0(oracle, shape):
    from miles_amd.kernels.quant.fp8_blockwise import quant_weight_ue8m0

    x = W.reference_pattern("random", (int(torch.tensor(shape[:-1]).prod()), shape[-1]), spread=512.0, amplitude=16.0)
    y, s = quant_weight_ue8m0(x.view(shape).to(DEV), [128, 128])
    y_o, s_o = oracle.per_block_cast_to_fp8(x)
    assert y.shape == shape and s.shape == (*shape[:-2], -(-shape[-2] // 128), -(-shape[-1] // 128))
    _assert_same(y.view(-1, shape[-1]), y_o, "codes")
    _assert_same(s.reshape(s_o.shape), s_o, "scales")
    with pytest.raises(AssertionError):
        quant_weight_ue8m0(x.to(DEV), [128, 64])
    with pytest.raises(AssertionError):
        quant_weight_ue8m0(x.float().to(DEV), [128, 128])


# ---------------------------------------------------------------------------------------------------
# act_quant / fp8_simulate (miles/kernels/quant/fp8_act_quant.py, miles_plugins/models/deepseek_v4/ops/qat.py)
def _act_input(dtype, shape=(5, 37, 1024), seed=0):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(*shape, generator=g) * torch.logspace(-6, 4, shape[-1])).to(dtype)
    x[0, 0, :128] = 0
    x[0, 1, :4] = torch.tensor([448.0, -448.0, -0.0, 1e-6]).to(dtype)
    x[0, 2, :128] = -0.0
    x[0, 3, :128] = 2.0 ** -20
    x[0, 4, :128] = torch.finfo(dtype).max if dtype != torch.float32 else 1e38
    return x


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("block", [16, 32, 64, 128, 256, 8])
@pytest.mark.parametrize("scale_fmt", [None, "ue8m0"])
def test_act_quant_codes_scales_and_inplace(oracle, dtype, block, scale_fmt):
    from miles_amd.kernels.quant.fp8_act_quant import act_quant, fp8_simulate

    x = _act_input(dtype)
    y, s = act_quant(x.to(DEV), block, scale_fmt)
    y_o, s_o = oracle.act_quant(x, block, scale_fmt)
    assert y.dtype == F8 and y.shape == x.shape and s.dtype == torch.float32 and s.shape == (5, 37, 1024 // block)
    _assert_same(s, s_o, f"act_quant scales block {block}")
    _assert_same(y, y_o, f"act_quant codes block {block}")
    xd = x.to(DEV)
    out = act_quant(xd, block, scale_fmt, inplace=True)
    assert out is xd
    _assert_same(xd, oracle.act_quant(x, block, scale_fmt, inplace=True), f"act_quant inplace block {block}")
    if scale_fmt is not None:
        y8, s8 = act_quant(x.to(DEV), block, scale_fmt, scale_dtype=torch.float8_e8m0fnu)
        assert s8.dtype == torch.float8_e8m0fnu
        _assert_same(s8.view(torch.uint8), oracle.act_quant(x, block, scale_fmt, scale_dtype=torch.float8_e8m0fnu)[1].view(torch.uint8), "e8m0 scales")
        _assert_same(y8, y_o, "codes with e8m0 scales")
        src = x.to(DEV)
        sim = fp8_simulate(src, block)
        assert torch.equal(src.cpu(), x)                      # the input is left alone
        _assert_same(sim, oracle.fp8_simulate(x, block), f"fp8_simulate block {block}")


def test_act_quant_views_errors_and_straight_through(oracle):
    from miles_amd.kernels.quant.fp8_act_quant import act_quant, fp8_simulate_qat

    x = _act_input(torch.bfloat16, shape=(2, 16, 576))
    # the reference's callers quantize a slice of the last dimension in place (compressor.py:170): a strided view
    xd = x.to(DEV)
    act_quant(xd[..., :512], 64, "ue8m0", inplace=True)
    want = x.clone()
    want[..., :512] = oracle.act_quant(x[..., :512], 64, "ue8m0", inplace=True)
    _assert_same(xd, want, "in-place on a slice")
    # an unaligned base address takes the plain kernel
    flat = torch.zeros(64 * 128 + 1, dtype=torch.bfloat16)
    flat[1:] = x.reshape(-1)[: 64 * 128]
    y, s = act_quant(flat.to(DEV)[1:].view(64, 128), 128)
    y_o, s_o = oracle.act_quant(flat[1:].view(64, 128), 128)
    _assert_same(y, y_o, "unaligned codes")
    _assert_same(s, s_o, "unaligned scales")
    with pytest.raises(AssertionError):
        act_quant(torch.zeros(4, 100, device=DEV, dtype=torch.bfloat16), 64)
    with pytest.raises(ValueError):
        act_quant(torch.zeros(4, 128, device=DEV, dtype=torch.bfloat16), 64, scale_dtype=torch.float8_e8m0fnu)
    kv = torch.randn(8, 256, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    grad = torch.randn_like(kv)
    fp8_simulate_qat(kv, 64).backward(grad)
    assert torch.equal(kv.grad, grad)


def test_act_quant_full_size_round_trip(oracle):
    # size-independent properties on a large activation: |qdq - x| <= scale * 2^-4 * |code| grid step, scales
    # are powers of two, and quantizing the result again is the identity (idempotence)
    from miles_amd.kernels.quant.fp8_act_quant import act_quant, fp8_simulate

    x = torch.randn(16384, 7168, device=DEV, dtype=torch.bfloat16)
    y, s = act_quant(x, 128, "ue8m0")
    assert torch.all((s.view(torch.int32) & 0x7FFFFF) == 0)
    sim = fp8_simulate(x, 128)
    again = fp8_simulate(sim, 128)
    assert torch.equal(sim, again)
    err = (sim.float() - x.float()).abs().view(16384, -1, 128)
    assert torch.all(err <= s.unsqueeze(-1) * 448 * 2.0 ** -4)
    head = x[:64].cpu()
    _assert_same(sim[:64], oracle.fp8_simulate(head, 128), "full-size head rows")


@pytest.mark.parametrize("sym", [True, False])
@pytest.mark.parametrize("G", [32, 64, 128, 256])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_fake_int4_quant_row_blocks_edge_values(oracle, sym, G, dtype):
    # the row-block kernel: signed zeros, an all-zero block, a constant block (range 0 -> scale floor), blocks that are
    # all positive / all negative (clamped zero points), magnitudes near the top of the dtype, ragged row count
    from miles_amd.kernels.quant.int4_fake import fake_int4_quant_cuda

    big = {torch.bfloat16: 3.0e38, torch.float16: 6.0e4, torch.float32: 3.0e38}[dtype]
    w = W.gaussian_outliers((37, 512), std=0.02, p_outlier=0.002, gain=25.0, seed=4100 + G, dtype=dtype)
    w[0] = 0
    w[1, :128] = torch.tensor([-0.0, 0.0] * 64).to(dtype)
    w[2, :128] = 0.37
    w[3, :128] = w[3, :128].abs() + 0.5
    w[4, :128] = -(w[4, :128].abs()) - 0.5
    w[5, :4] = torch.tensor([big, -big, 1e-30, -1e-30]).to(dtype)
    w[6, :128] = torch.linspace(-7, 7, 128).to(dtype)          # exact ties of rint(x / 1)
    out, scale, zero = fake_int4_quant_cuda(w.to(DEV), (1, G), sym)
    out_o, scale_o, zero_o = oracle.fake_int4_quant(w, (1, G), sym)
    _assert_same(scale, scale_o, "scales")
    _assert_same(out, out_o, "values")
    if not sym:
        _assert_same(zero, zero_o, "zero points")


def test_fake_int4_quant_full_size_tensor(oracle):
    from miles_amd.kernels.quant.int4_fake import fake_int4_quant_cuda

    w = W.c4_expert(0, 0)                                      # [2048, 7168] bf16
    for sym in (True, False):
        out, scale, zero = fake_int4_quant_cuda(w.to(DEV), (1, 128), sym)
        out_o, scale_o, zero_o = oracle.fake_int4_quant(w, (1, 128), sym)
        _assert_same(out, out_o, "values")
        _assert_same(scale, scale_o, "scales")
        if not sym:
            _assert_same(zero, zero_o, "zero points")


# ---------------------------------------------------------------------------------------------------
# several host threads at once: the converters call the quantizers from a ThreadPoolExecutor
# (tools/convert_hf_to_fp8.py:175-184, tools/convert_hf_to_int4_direct.py:220-236)
def test_quantizers_from_concurrent_host_threads(oracle):
    from concurrent.futures import ThreadPoolExecutor

    from miles_amd import launch
    from miles_amd.kernels.quant.fp8_blockwise import fp8_blockwise_cast
    from miles_amd.kernels.quant.int4_fake import pack_layer
    from miles_amd.tools.convert_hf_to_fp8 import block_fp8, quant_fp8
    from miles_amd.utils.mxfp8 import mxfp8_quantize
    from miles_amd.utils.nvfp4 import nvfp4_quantize_1d

    cpu = [W.gaussian_outliers((128 + 8 * i, 256), std=0.02, p_outlier=0.001, gain=20.0, seed=900 + i) for i in range(8)]
    dev = [w.to(DEV) for w in cpu]
    torch.cuda.synchronize()

    def work(i):
        x = dev[i]
        out = {}
        for rep in range(10):
            out["block"] = block_fp8(x, [128, 128])
            out["tensor"] = quant_fp8(x, "tensor")
            out["mxfp8"] = mxfp8_quantize(x)
            out["nvfp4"] = nvfp4_quantize_1d(x)
            with launch.deferred() as batch:       # batches are per thread: only this thread's two jobs land here
                out["cast"] = fp8_blockwise_cast(x)
                out["int4"] = pack_layer(x, 128)[:2]
                assert len(batch) == 2
        torch.cuda.synchronize()
        return out

    with ThreadPoolExecutor(max_workers=8) as pool:
        results = list(pool.map(work, range(8)))
    for i, out in enumerate(results):
        x = cpu[i]
        want = {"block": oracle.block_fp8(x, (128, 128)), "tensor": oracle.tensor_fp8(x), "mxfp8": oracle.mxfp8_quantize(x),
                "nvfp4": oracle.nvfp4_quantize_1d(x), "cast": oracle.fp8_blockwise_cast(x), "int4": oracle.pack_layer(x, 128)[:2]}
        for name, got in out.items():
            for j, (g_, w_) in enumerate(zip(got, want[name])):
                _assert_same(g_, w_, f"thread {i} {name} output {j}")


# ---------------------------------------------------------------------------------------------------
# more than 2^31 elements in one tensor: every offset computed by the kernels has to be 64-bit.  The tensor is one
# [4096, 8192] block repeated down the rows, and every quantizer here works on row-local groups (tiles of 128 rows,
# row segments), so each repetition must come out as the block alone does; NVFP4 shares one amax, equal by construction.
def test_tensors_beyond_2_to_31_elements(oracle):
    from miles_amd.kernels.quant.fp8_blockwise import fp8_blockwise_cast
    from miles_amd.kernels.quant.int4_fake import pack_layer
    from miles_amd.tools.convert_hf_to_fp8 import block_fp8
    from miles_amd.tools.fp8_cast_bf16 import weight_dequant
    from miles_amd.utils.mxfp4 import quantize_mxfp4
    from miles_amd.utils.mxfp8 import mxfp8_quantize
    from miles_amd.utils.nvfp4 import nvfp4_quantize_1d

    reps, block_rows, cols, tail = 64, 4096, 8192, 128
    base_cpu = W.gaussian_outliers((block_rows, cols), std=0.02, p_outlier=0.001, gain=20.0, seed=31)
    base = base_cpu.to(DEV)
    rows = reps * block_rows + tail
    assert rows * cols > 2**31
    x = torch.empty((rows, cols), dtype=torch.bfloat16, device=DEV)
    x[: reps * block_rows].view(reps, block_rows, cols).copy_(base.unsqueeze(0).expand(reps, -1, -1))
    x[reps * block_rows:] = base[:tail]

    def repeats(full, small, what):
        full, small = full.view(torch.uint8) if full.element_size() == 1 else full, small.view(torch.uint8) if small.element_size() == 1 else small
        per = small.shape[0]
        body = full[: reps * per].view(reps, *small.shape)
        assert bool((body == small.unsqueeze(0)).all()), f"{what}: a repetition differs from the block alone"
        assert torch.equal(full[reps * per:], small[: full.shape[0] - reps * per]), f"{what}: tail differs"

    for name, fn in (("fp8_blockwise_cast", fp8_blockwise_cast), ("block_fp8", lambda t: block_fp8(t, [128, 128])),
                     ("mxfp8", mxfp8_quantize), ("int4", lambda t: pack_layer(t, 128)[:2]),
                     ("mxfp4", lambda t: quantize_mxfp4(t, 32)), ("nvfp4", lambda t: nvfp4_quantize_1d(t)[:2])):
        big, small = fn(x), fn(base)
        for j, (b_, s_) in enumerate(zip(big, small)):
            repeats(b_, s_, f"{name} output {j}")
        if name == "fp8_blockwise_cast":
            q_o, s_o = oracle.fp8_blockwise_cast(base_cpu)
            _assert_same(small[0], q_o, "block codes")
            _assert_same(small[1], s_o, "block scales")
            repeats(weight_dequant(big[0], big[1]), weight_dequant(small[0], small[1]), "weight_dequant")
        del big, small
    torch.cuda.synchronize()


# ---------------------------------------------------------------------------------------------------
# empty tensors (no rows, or no columns): torch hands them a null data pointer; every wrapper returns outputs of the
# shapes the reference's torch code would, and the reductions torch refuses over nothing raise the same way
@pytest.mark.parametrize("shape", [(0, 256), (4, 0)])
def test_empty_tensors(oracle, shape):
    from miles_amd.kernels.quant import fake_quant as fq
    from miles_amd.kernels.quant.fp8_act_quant import act_quant, fp8_simulate
    from miles_amd.kernels.quant.fp8_blockwise import fp8_blockwise_cast, per_block_cast_to_fp8
    from miles_amd.kernels.quant.int4_fake import fake_int4_quant_cuda, pack_layer
    from miles_amd.kernels.quant.nvfp4_qdq import compute_nvfp4_amax
    from miles_amd.tools.convert_hf_to_fp8 import block_fp8, quant_fp8
    from miles_amd.tools.fp8_cast_bf16 import weight_dequant
    from miles_amd.utils.mxfp4 import dequantize_mxfp4, quantize_mxfp4
    from miles_amd.utils.mxfp8 import mxfp8_quantize
    from miles_amd.utils.nvfp4 import nvfp4_quantize_1d, nvfp4_quantize_1d_pair

    x = torch.empty(shape, dtype=torch.bfloat16, device=DEV)
    xc = x.cpu()
    for name, got, want in (
            ("block_fp8", block_fp8(x, [128, 128]), oracle.block_fp8(xc, (128, 128))),
            ("fp8_blockwise_cast", fp8_blockwise_cast(x), oracle.fp8_blockwise_cast(xc)),
            ("per_block_cast_to_fp8", per_block_cast_to_fp8(x), oracle.per_block_cast_to_fp8(xc)),
            ("mxfp4", quantize_mxfp4(x, 32), oracle.quantize_mxfp4(xc, 32)),
            ("pack_layer", pack_layer(x, 128)[:2], oracle.pack_layer(xc, 128)[:2]),
            ("fake_int4", fake_int4_quant_cuda(x, (1, 128), False), oracle.fake_int4_quant(xc, (1, 128), False)),
            ("nvfp4", nvfp4_quantize_1d(x), oracle.nvfp4_quantize_1d(xc)),
            ("fake_quant", (fq.fake_quant_fp8_forward(x),), (oracle.fake_quant(xc, "fp8"),)),
            ("act_quant", act_quant(x, 128), oracle.act_quant(xc, 128)),
            ("fp8_simulate", (fp8_simulate(x, 128),), (oracle.fp8_simulate(xc, 128),))):
        for j, (g_, w_) in enumerate(zip(got, want)):
            assert g_.shape == w_.shape and g_.dtype == w_.dtype, f"{name} output {j}: {tuple(g_.shape)} {g_.dtype}"
            _assert_same(g_, w_, f"{name} output {j}")       # 0-dim NVFP4 global scale: the value of an all-zero tensor
    q, s = mxfp8_quantize(x)
    assert q.shape == shape and q.dtype == torch.float8_e4m3fn and s.shape == (shape[0], shape[1] // 32) and s.dtype == torch.uint8
    a, b = nvfp4_quantize_1d_pair(x, x.clone())
    assert a[0].shape == (shape[0], shape[1] // 2) and b[1].shape == (shape[0], shape[1] // 16) and torch.equal(a[2], b[2])
    p, s4 = quantize_mxfp4(x, 32)
    assert dequantize_mxfp4(p, s4, 32).shape == shape
    if shape[0] == 0:
        q8, s8 = block_fp8(x, [128, 128])
        assert weight_dequant(q8, s8).shape == shape
        cq, cs = quant_fp8(x, "channel")
        assert cq.shape == shape and cs.shape == (0, 1)
        packed, scale, zp = pack_layer(x, 128, sym=False)
        assert packed.shape == (0, 32) and scale.shape == (0, 2) and zp.shape == (2, 0)
    else:
        with pytest.raises(RuntimeError, match="non-zero size"):
            quant_fp8(x, "channel")
    with pytest.raises(RuntimeError, match="numel\\(\\) == 0"):
        quant_fp8(x, "tensor")
    with pytest.raises(ValueError, match="empty tensor"):
        compute_nvfp4_amax(x)
    torch.cuda.synchronize()


# ---------------------------------------------------------------------------------------------------
# NVFP4 with the amax carried over from the previous run of the same job list: one pass when the amax did not move,
# a second quantization of exactly the tensors whose amax did -- the results must never depend on which happened
@pytest.mark.parametrize("fos", [None, (448, "MAE", False), (256, "MSE", False), (256, "MAE", True)],
                         ids=["standard", "fos448", "fos256mse", "fos256f16err"])
def test_nvfp4_reads_fp16(oracle, monkeypatch, fos):
    """fp16 tensors take the packed NVFP4 kernels' fp16 instances (amax pass, quantizer, Four Over Six): blocks of
    subnormals, of zeros, the format's extremes, every block its own magnitude; single calls, a gate / up pair, and a
    recorded list of more than 64 jobs (device table where the mode has one) in which bf16 and fp16 tensors alternate,
    run twice and then with the amax carried over."""
    from miles_amd import launch
    from miles_amd.utils.nvfp4 import nvfp4_quantize_1d, nvfp4_quantize_1d_pair

    for name in ("NVTE_NVFP4_4OVER6", "NVTE_NVFP4_4OVER6_E4M3_USE_256", "NVTE_NVFP4_4OVER6_ERR_MODE",
                 "NVTE_NVFP4_4OVER6_ERR_USE_FAST_MATH", "NVTE_USE_FAST_MATH"):
        monkeypatch.delenv(name, raising=False)
    kw = {}
    if fos:
        _fos_env(monkeypatch, *fos)
        kw = {"e4m3_max": fos[0], "flags": oracle.NVFP4_4OVER6 | (oracle.NVFP4_ERR_MSE if fos[1] == "MSE" else 0)
              | (oracle.NVFP4_ERR_FP16 if fos[2] else 0)}

    def case(shape, seed, top):
        g = torch.Generator().manual_seed(seed)
        rows, cols = shape
        ex = torch.randint(-14, 1, (rows, cols // 16, 1), generator=g).float()
        w = (torch.randn(rows, cols // 16, 16, generator=g) * torch.exp2(ex)).reshape(rows, cols) * top
        w = w.clamp(-65504, 65504).to(torch.float16)
        w[0, :16] = 0
        w[0, 16:32] = torch.arange(1, 17, dtype=torch.int16).view(torch.float16)      # a block of subnormals
        if rows > 2:
            w[2, 5] = 65504.0 if top > 100 else w[2, 5]
            w[1] = 0
        return w

    for shape, top in (((1, 32), 1.0), ((64, 128), 1.0), ((200, 1024), 3000.0), ((37, 7168), 0.01)):
        w = case(shape, 77 + shape[1], top)
        got, want = nvfp4_quantize_1d(w.to(DEV)), oracle.nvfp4_quantize_1d(w, **kw)
        for k, (a, b) in enumerate(zip(got, want)):
            _assert_same(a, b, f"{shape} output {k}")
    gate, up = case((96, 256), 5, 1.0), case((96, 256), 6, 40.0)
    got, want = nvfp4_quantize_1d_pair(gate.to(DEV), up.to(DEV)), oracle.nvfp4_quantize_1d_pair(gate, up, **kw)
    for half in range(2):
        for k, (a, b) in enumerate(zip(got[half], want[half])):
            _assert_same(a, b, f"pair half {half} output {k}")
    tensors = []
    for i in range(80):
        t = case((24 + i % 5, 256), 300 + i, 1.0 + i % 7)
        tensors.append(t if (i % 3 == 0 or i >= 50) else t.float().to(torch.bfloat16))
    dev = [t.to(DEV) for t in tensors]
    with launch.recording() as batch:
        outs = [nvfp4_quantize_1d(t) for t in dev]
    batch.device = torch.device(DEV)
    batch.freeze()
    want = [oracle.nvfp4_quantize_1d(t, **kw) for t in tensors]
    for what in ("first run", "second run", "carried"):
        if what == "carried":
            assert batch.carry_amax() == len(tensors)
        for o in outs:
            for t in o[:2]:
                t.view(torch.uint8).fill_(0x5A)
        batch.run()
        torch.cuda.synchronize()
        for i, (o, wnt) in enumerate(zip(outs, want)):
            for k, (a, b) in enumerate(zip(o, wnt)):
                _assert_same(a, b, f"list tensor {i} ({tensors[i].dtype}) output {k}, {what}")
    dev[3].mul_(2.0)            # an fp16 tensor's amax moves: quantized again with the new one
    dev[60].mul_(0.5)
    batch.run()
    torch.cuda.synchronize()
    for i in (3, 4, 60, 79):
        for k, (a, b) in enumerate(zip(outs[i], oracle.nvfp4_quantize_1d(dev[i].cpu(), **kw))):
            _assert_same(a, b, f"list tensor {i} output {k}, after its amax moved")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("four_over_six", [False, True])
def test_nvfp4_carried_amax_hits_and_misses(oracle, monkeypatch, four_over_six, dtype):
    from miles_amd import launch
    from miles_amd.utils.nvfp4 import nvfp4_quantize_1d, nvfp4_quantize_1d_pair

    for name in ("NVTE_NVFP4_4OVER6", "NVTE_NVFP4_4OVER6_E4M3_USE_256", "NVTE_NVFP4_4OVER6_ERR_MODE"):
        monkeypatch.delenv(name, raising=False)
    kw = {}
    if four_over_six:
        monkeypatch.setenv("NVTE_NVFP4_4OVER6", "weights")
        kw = {"e4m3_max": 256, "flags": 1}
    shapes = [(256, 512), (384, 1024), (100, 256), (64, 2048), (512, 512), (128, 7168)]
    cpu = [W.gaussian_outliers(s, std=0.02, p_outlier=0.001, gain=20.0, seed=1200 + i, dtype=dtype) for i, s in enumerate(shapes)]
    pair_cpu = [W.gaussian_outliers((320, 768), std=0.02, p_outlier=0.001, gain=20.0, seed=1250 + i, dtype=dtype) for i in range(2)]
    dev, pair_dev = [w.to(DEV) for w in cpu], [w.to(DEV) for w in pair_cpu]
    with launch.recording() as batch:
        outs = [nvfp4_quantize_1d(w) for w in dev[:3]]
        pair_out = nvfp4_quantize_1d_pair(*pair_dev)
        outs += [nvfp4_quantize_1d(w) for w in dev[3:]]
    batch.device = torch.device(DEV)

    def check(what):
        batch.run()
        torch.cuda.synchronize()
        for i, (w, got) in enumerate(zip(dev, outs)):
            for j, (g_, w_) in enumerate(zip(got, oracle.nvfp4_quantize_1d(w.cpu(), **kw))):
                _assert_same(g_, w_, f"{what}: tensor {i} output {j}")
        want = oracle.nvfp4_quantize_1d_pair(pair_dev[0].cpu(), pair_dev[1].cpu(), **kw)
        for half in range(2):
            for j, (g_, w_) in enumerate(zip(pair_out[half], want[half])):
                _assert_same(g_, w_, f"{what}: pair half {half} output {j}")

    from miles_amd import _lib

    def state():
        """(second pass ran, marked volatile) per record, in job order: tensors 0-2, the pair, tensors 3-5"""
        recs = [r.cpu() for r in batch.amax_records()]
        return [int(r[_lib.RECORD_REDO_WORD]) for r in recs], [int(r[_lib.RECORD_VOLATILE_WORD]) for r in recs]

    check("first run (two passes)")
    assert batch.carry_amax() == len(shapes) + 2
    assert len(batch.amax_records()) == len(shapes) + 1
    check("same weights (every amax carried)")
    assert state() == ([0] * 7, [0] * 7)
    check("same weights again")
    for w in dev + pair_dev:                       # new values everywhere, every amax as before
        top = w.abs().flatten().argmax()
        keep = w.flatten()[top].clone()
        w.mul_(0.75)
        w.view(-1)[top] = keep
    check("changed data, same amax")
    assert state() == ([0] * 7, [0] * 7)
    dev[1].mul_(3.0)                               # these amax move: tensor 1 up, tensor 4 down, the pair through its second half
    dev[4].mul_(0.25)
    pair_dev[1].mul_(5.0)
    check("three amax moved")
    moved = [0, 1, 0, 1, 0, 1, 0]                  # records: tensors 0, 1, 2, the pair, tensors 3, 4, 5
    assert state() == (moved, [0] * 7)             # quantized twice; one move alone does not mark a record
    check("and stayed")
    assert state() == ([0] * 7, [0] * 7)           # the single pass with the new amax held
    dev[1].mul_(0.5)
    check("tensor 1 moved")
    assert state() == ([0, 1, 0, 0, 0, 0, 0], [0] * 7)
    dev[1].mul_(0.5)
    dev[3].mul_(2.0)
    check("tensor 1 moved again, tensor 3 for the first time")
    assert state() == ([0, 1, 0, 0, 1, 0, 0], [0, 1, 0, 0, 0, 0, 0])      # twice in a row: marked
    dev[1].mul_(2.0)
    check("tensor 1 moved while marked: the single pass only collected its amax, the second pass quantized it")
    assert state() == ([0, 1, 0, 0, 0, 0, 0], [0, 1, 0, 0, 0, 0, 0])
    check("tensor 1 stayed: the two-pass form once more, and the mark is gone")
    assert state() == ([0, 1, 0, 0, 0, 0, 0], [0] * 7)
    check("settled")
    assert state() == ([0] * 7, [0] * 7)
    dev[2].zero_()                                 # amax 0
    dev[0].view(-1)[7] = float("inf")              # amax inf
    check("zero tensor and an infinity")
    dev[0].view(-1)[7] = 1.0
    check("back to finite")


def test_tensor_fp8_jobs_grouped_and_with_carried_amax(oracle):
    # per-tensor FP8 as a job of the batched driver: several tensors per launch, and later runs of the same list with the
    # amax carried over (one pass, a second quantization only where the amax moved)
    from miles_amd import launch
    from miles_amd.tools.convert_hf_to_fp8 import quant_fp8

    shapes = [(256, 512), (100, 264), (3, 8), (1024, 1024), (64, 7168), (129, 1000)]
    cpu = [W.gaussian_outliers(s, std=0.02, p_outlier=0.001, gain=20.0, seed=1300 + i) for i, s in enumerate(shapes)]
    dev = [w.to(DEV) for w in cpu]
    with launch.recording() as batch:
        outs = [quant_fp8(w, "tensor") for w in dev]
    assert len(batch) == len(shapes) and batch.direct_calls == 0
    batch.device = torch.device(DEV)

    def check(what):
        batch.run()
        torch.cuda.synchronize()
        for i, (w, (q, sc)) in enumerate(zip(dev, outs)):
            q_o, s_o = oracle.tensor_fp8(w.cpu())
            _assert_same(sc, s_o, f"{what}: tensor {i} scale")
            _assert_same(q, q_o, f"{what}: tensor {i} codes")

    check("first run (two passes)")
    assert batch.carry_amax() == len(shapes)
    check("same weights")
    for w in dev:                                    # new values, every amax as before
        top = w.abs().flatten().argmax()
        keep = w.flatten()[top].clone()
        w.mul_(0.5)
        w.view(-1)[top] = keep
    check("changed data, same amax")
    dev[0].mul_(3.0)
    dev[3].mul_(0.125)
    check("two amax moved")
    dev[2].zero_()                                   # amax below the 1e-12 floor
    dev[4].view(-1)[5] = float("nan")                # NaN amax: scale and every code NaN
    check("zero tensor and a NaN")
    dev[4].view(-1)[5] = 0.5
    check("back to finite")
    # tensors the packed kernels do not take still go through the direct two-pass entry point
    odd = torch.randn(16, 12, device=DEV).to(torch.bfloat16)
    with launch.recording() as b2:
        q, sc = quant_fp8(odd, "tensor")
    assert len(b2) == 0 and b2.direct_calls == 1
    q_o, s_o = oracle.tensor_fp8(odd.cpu())
    _assert_same(sc, s_o, "odd width scale")
    _assert_same(q, q_o, "odd width codes")
