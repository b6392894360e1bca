"""Seeded random shapes, dtypes and placements for every quantizer, against the oracle.

The shape lists of the other GPU tests come from the reference's tests and from the benchmark configurations; this file
adds what they do not enumerate: odd row counts, column counts at every residue the API allows, tensors that start in
the middle of a larger allocation (so the 16-byte-aligned kernels and the plain ones both get exercised), fp16 and
fp32 inputs, and values spread over many binades.  Everything is deterministic: the case list is generated from a
fixed seed at collection time.
"""

import os
import random

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F8 = torch.float8_e4m3fn
_DTYPES = (torch.bfloat16, torch.bfloat16, torch.float16, torch.float32)     # bf16 twice as likely


def _bits(t):
    t = t.detach().cpu().contiguous()
    return t.view({1: torch.uint8, 2: torch.int16, 4: torch.int32}[t.element_size()])


def _same(got, want, what):
    g, w = _bits(got), _bits(want)
    assert g.shape == w.shape, f"{what}: shape {tuple(g.shape)} vs {tuple(w.shape)}"
    if not torch.equal(g, w):
        bad = (g != w).nonzero()
        i = tuple(bad[0].tolist())
        raise AssertionError(f"{what}: {bad.shape[0]} of {g.numel()} differ; first at {i}: got {g[i].item()} want {w[i].item()}")


def _tensor(seed, shape, dtype, offset):
    """Values over ~12 binades with a few zeros; on the device the tensor starts `offset` elements into its storage."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=g) * torch.exp2(torch.randint(-8, 4, shape, generator=g).float())
    x = torch.where(torch.rand(shape, generator=g) < 0.02, torch.zeros(()), x).to(dtype)
    n = x.numel()
    flat = torch.zeros(n + offset, dtype=dtype, device=DEV)
    flat[offset:] = x.reshape(-1).to(DEV)
    return x, flat[offset:].view(shape)


# MQ_RANDOM_SCALE=10 runs ten times as many random cases (the extra ones continue the same seeded sequence)
_SCALE = max(1, int(os.environ.get("MQ_RANDOM_SCALE", "1")))


def _cases(name, count, columns_multiple_of, max_rows=300, max_cols=1100):
    rng = random.Random(f"miles-quant-{name}")
    out = []
    for i in range(count * _SCALE):
        rows = rng.choice([1, 2, 3, 5, 31, 64, 127, 128, 129, 200, rng.randint(1, max_rows)])
        cols = columns_multiple_of * rng.randint(1, max(1, max_cols // columns_multiple_of))
        dtype = rng.choice(_DTYPES)
        offset = rng.choice([0, 0, 0, 1, 3, 8, 24])          # elements: 0 keeps the allocator's 256-byte alignment
        out.append(pytest.param(i, (rows, cols), dtype, offset, id=f"{name}{i}-{rows}x{cols}-{str(dtype)[6:]}-o{offset}"))
    return out


@pytest.mark.parametrize("seed,shape,dtype,offset", _cases("fp8", 40, 1))
def test_random_fp8_block_and_blockwise(oracle, seed, shape, dtype, offset):
    from miles_amd.kernels.quant.fp8_blockwise import fp8_blockwise_cast, per_block_cast_to_fp8
    from miles_amd.tools.convert_hf_to_fp8 import block_fp8, quant_fp8
    from miles_amd.tools.fp8_cast_bf16 import weight_dequant

    x, xd = _tensor(1000 + seed, shape, dtype, offset)
    for name, fn, ref in (("block_fp8", lambda t: block_fp8(t, [128, 128]), lambda t: oracle.block_fp8(t, (128, 128))),
                          ("fp8_blockwise_cast", fp8_blockwise_cast, oracle.fp8_blockwise_cast)):
        q, s = fn(xd)
        q_o, s_o = ref(x)
        _same(s, s_o, f"{name} scales")
        _same(q, q_o, f"{name} codes")
    if dtype == torch.bfloat16:
        q, s = per_block_cast_to_fp8(xd)
        q_o, s_o = oracle.per_block_cast_to_fp8(x)
        _same(s, s_o, "power-of-two scales")
        _same(q, q_o, "power-of-two codes")
        _same(weight_dequant(q.contiguous(), s.contiguous()), oracle.weight_dequant(q_o, s_o), "dequant")
    for strategy, ref in (("tensor", oracle.tensor_fp8), ("channel", oracle.channel_fp8)):
        q, s = quant_fp8(xd, strategy)
        q_o, s_o = ref(x)
        _same(s, s_o, f"{strategy} scale")
        _same(q, q_o, f"{strategy} codes")


@pytest.mark.parametrize("seed,shape,dtype,offset", _cases("mx", 40, 32))
def test_random_mxfp8_mxfp4_and_row_block_fake_quant(oracle, seed, shape, dtype, offset):
    from miles_amd.kernels.quant import fake_quant as fq
    from miles_amd.kernels.quant.fp8_act_quant import act_quant, fp8_simulate
    from miles_amd.utils.mxfp4 import dequantize_mxfp4, quantize_mxfp4
    from miles_amd.utils.mxfp8 import mxfp8_quantize

    x, xd = _tensor(2000 + seed, shape, dtype, offset)
    q, s = mxfp8_quantize(xd)
    q_o, s_o = oracle.mxfp8_quantize(x)
    _same(s, s_o, "mxfp8 scales")
    _same(q, q_o, "mxfp8 codes")
    p, s4 = quantize_mxfp4(xd, 32)
    p_o, s4_o = oracle.quantize_mxfp4(x, 32)
    _same(s4, s4_o, "mxfp4 scales")
    _same(p, p_o, "mxfp4 codes")
    _same(dequantize_mxfp4(p, s4, 32), oracle.dequantize_mxfp4(p_o, s4_o, 32), "mxfp4 dequant")
    for kind, fn in (("fp8", fq.fake_quant_fp8_forward), ("fp4", fq.fake_quant_fp4_forward),
                     ("compressed_kv", fq.fake_quant_compressed_kv_forward)):
        _same(fn(xd), oracle.fake_quant(x, kind), f"fake_quant {kind}")
    for fmt in (None, "ue8m0"):
        y, sc = act_quant(xd, 32, fmt)
        y_o, sc_o = oracle.act_quant(x, 32, fmt)
        if shape[1] % 64 == 0:
            _same(act_quant(xd, 64, fmt)[0], oracle.act_quant(x, 64, fmt)[0], f"act_quant codes, block 64 {fmt}")
        _same(sc, sc_o, f"act_quant scales {fmt}")
        _same(y, y_o, f"act_quant codes {fmt}")
    _same(fp8_simulate(xd, 32), oracle.fp8_simulate(x, 32), "fp8_simulate")


@pytest.mark.parametrize("seed,shape,dtype,offset", _cases("int4", 40, 128, max_cols=1600))
def test_random_int4(oracle, seed, shape, dtype, offset):
    from miles_amd.kernels.quant.int4_fake import fake_int4_quant_cuda, pack_layer
    from miles_amd.tools.convert_kimi_int4_to_bf16 import _dequantize_tensor

    x, xd = _tensor(3000 + seed, shape, dtype, offset)
    G = (32, 64, 128)[seed % 3]
    for sym in (True, False):
        out, scale, zero = fake_int4_quant_cuda(xd.contiguous(), (1, G), sym)
        out_o, scale_o, zero_o = oracle.fake_int4_quant(x, (1, G), sym)
        _same(scale, scale_o, f"fake int4 scales sym={sym}")
        _same(out, out_o, f"fake int4 values sym={sym}")
        if not sym:
            _same(zero, zero_o, "fake int4 zero points")
    if dtype == torch.float32:
        return                                  # pack_layer is defined on 16-bit weights
    packed, scale, _ = pack_layer(xd, G)
    packed_o, scale_o, _ = oracle.pack_layer(x, G)
    _same(scale, scale_o, "pack_layer scales")
    _same(packed, packed_o, "pack_layer words")
    _same(_dequantize_tensor(packed, scale, shape, G), oracle.int4_unpack_dequant(packed_o, scale_o, shape, G), "unpack")
    if shape[0] % 8 == 0:
        got = pack_layer(xd, G, sym=False)
        want = oracle.pack_layer(x, G, sym=False)
        for g, w, what in zip(got, want, ("asym words", "asym scales", "asym packed zero points")):
            _same(g, w, what)


@pytest.mark.parametrize("seed,shape,dtype,offset", _cases("nv", 40, 16))
def test_random_nvfp4(oracle, monkeypatch, seed, shape, dtype, offset):
    from miles_amd.kernels.quant.nvfp4_qdq import NVFP4QDQConfig, compute_nvfp4_amax, fused_nvfp4_qdq
    from miles_amd.utils.nvfp4 import nvfp4_quantize_1d, nvfp4_quantize_1d_pair

    x, xd = _tensor(4000 + seed, shape, dtype, offset)
    if seed % 4 == 3:      # Four Over Six, alternating error modes, through the environment switches the reference reads
        monkeypatch.setenv("NVTE_NVFP4_4OVER6", "weights")
        monkeypatch.setenv("NVTE_NVFP4_4OVER6_ERR_MODE", "MSE" if seed % 8 == 7 else "MAE")
        flags = 1 | (2 if seed % 8 == 7 else 0)
        q, s, g = nvfp4_quantize_1d(xd)
        q_o, s_o, g_o = oracle.nvfp4_quantize_1d(x, e4m3_max=256, flags=flags)
        _same(g, g_o, "global scale (4/6)")
        _same(s, s_o, "block scales (4/6)")
        _same(q, q_o, "codes (4/6)")
        return
    q, s, g = nvfp4_quantize_1d(xd)
    q_o, s_o, g_o = oracle.nvfp4_quantize_1d(x)
    _same(g, g_o, "global scale")
    _same(s, s_o, "block scales")
    _same(q, q_o, "codes")
    y, yd = _tensor(4500 + seed, shape, dtype, offset)
    for got, want in zip(nvfp4_quantize_1d_pair(xd, yd), oracle.nvfp4_quantize_1d_pair(x, y)):
        for a, b, what in zip(got, want, ("pair codes", "pair block scales", "pair global scale")):
            _same(a, b, what)
    if dtype != torch.float32:
        amax = compute_nvfp4_amax(xd)
        if xd.data_ptr() % 16:
            with pytest.raises(ValueError, match="16-byte-aligned"):      # the reference's contract (nvfp4_qdq.py:1147-1149)
                fused_nvfp4_qdq(xd, amax, NVFP4QDQConfig())
        else:
            _same(fused_nvfp4_qdq(xd, amax, NVFP4QDQConfig()), oracle.fused_nvfp4_qdq(x), "fused qdq")


@pytest.mark.parametrize("seed", range(6))
def test_random_mxfp4_to_fp8(oracle, seed):
    from miles_amd.tools.convert_mxfp4_to_fp8 import cast_e2m1fn_to_e4m3fn

    rng = random.Random(f"miles-quant-recode-{seed}")
    out_dim, in_dim, offset = 128 * rng.randint(1, 3), 128 * rng.randint(1, 5), rng.choice([0, 1, 16, 40])
    g = torch.Generator().manual_seed(5000 + seed)
    packed = torch.randint(-128, 128, (out_dim, in_dim // 2), dtype=torch.int8, generator=g)
    scale = torch.randint(100, 140, (out_dim, in_dim // 32), dtype=torch.uint8, generator=g)
    scale[0, 0] = 0                                            # 2^-127: far below the tile maximum
    flat = torch.zeros(packed.numel() + offset, dtype=torch.int8, device=DEV)
    flat[offset:] = packed.reshape(-1).to(DEV)
    y, ts = cast_e2m1fn_to_e4m3fn(flat[offset:].view(out_dim, in_dim // 2), scale.to(DEV).view(torch.float8_e8m0fnu))
    y_o, ts_o = oracle.cast_e2m1fn_to_e4m3fn(packed, scale.view(torch.float8_e8m0fnu))
    _same(ts, ts_o, "tile scales")
    _same(y, y_o, "codes")


@pytest.mark.parametrize("seed", range(4))
def test_random_job_lists_in_one_submission(oracle, seed):
    """150 jobs of mixed kinds and sizes recorded in random order and submitted with one call: the native driver has to cut
    the list into launches by kind, size class, NVFP4 pairing and group limit, and every job must come out as if alone."""
    from miles_amd import launch
    from miles_amd.kernels.quant.fp8_blockwise import fp8_blockwise_cast
    from miles_amd.kernels.quant.int4_fake import pack_layer
    from miles_amd.tools.convert_hf_to_fp8 import block_fp8, tensor_fp8
    from miles_amd.utils.mxfp4 import quantize_mxfp4
    from miles_amd.utils.mxfp8 import mxfp8_quantize
    from miles_amd.utils.nvfp4 import nvfp4_quantize_1d, nvfp4_quantize_1d_pair

    rng = random.Random(f"miles-jobs-{seed}")
    kinds = ["cast", "block", "mxfp8", "int4", "nvfp4", "pair", "mxfp4", "tensor"]
    plan = []
    for i in range(150):
        kind = rng.choice(kinds) if rng.random() < 0.5 or not plan else plan[-1][0]       # runs of one kind and switches
        shape = (rng.choice([1, 8, 64, 128, 200, 384]), 128 * rng.randint(1, 6))
        plan.append((kind, shape, i))
    cpu, dev = {}, {}
    for kind, shape, i in plan:
        for tag in ("a", "b") if kind == "pair" else ("a",):
            g = torch.Generator().manual_seed(6000 + 1000 * seed + 2 * i + (tag == "b"))
            cpu[i, tag] = (torch.randn(shape, generator=g) * 0.05).to(torch.bfloat16)
            dev[i, tag] = cpu[i, tag].to(DEV)
    results = {}
    with launch.recording() as batch:
        for kind, shape, i in plan:
            x = dev[i, "a"]
            results[i] = {"cast": lambda: fp8_blockwise_cast(x), "block": lambda: block_fp8(x, [128, 128]),
                          "mxfp8": lambda: mxfp8_quantize(x), "int4": lambda: pack_layer(x, 128)[:2],
                          "nvfp4": lambda: nvfp4_quantize_1d(x), "mxfp4": lambda: quantize_mxfp4(x, 32),
                          "tensor": lambda: tensor_fp8(x), "pair": lambda: nvfp4_quantize_1d_pair(x, dev[i, "b"])}[kind]()
        assert len(batch) == sum(2 if k == "pair" else 1 for k, _, _ in plan)
    batch.device = torch.device(DEV)
    batch.run()
    _check_job_list(oracle, plan, cpu, results, "first submission")
    # the same list again with the amax of the NVFP4 / per-tensor FP8 jobs carried over: unchanged inputs, then every third
    # tensor doubled (its amax moves) and every fourth replaced by new values under the old maximum
    batch.carry_amax()
    batch.run()
    _check_job_list(oracle, plan, cpu, results, "second submission, same inputs")
    for n, (key, x) in enumerate(sorted(dev.items())):
        if n % 3 == 0:
            x.mul_(2.0)
        elif n % 4 == 0:
            top = x.abs().flatten().argmax()
            keep = x.flatten()[top].clone()
            x.mul_(0.5)
            x.view(-1)[top] = keep
        cpu[key] = x.cpu()
    batch.run()
    _check_job_list(oracle, plan, cpu, results, "third submission, changed inputs")


def _check_job_list(oracle, plan, cpu, results, what):
    torch.cuda.synchronize()
    for kind, shape, i in plan:
        x = cpu[i, "a"]
        want = {"cast": lambda: oracle.fp8_blockwise_cast(x), "block": lambda: oracle.block_fp8(x, (128, 128)),
                "mxfp8": lambda: oracle.mxfp8_quantize(x), "int4": lambda: oracle.pack_layer(x, 128)[:2],
                "nvfp4": lambda: oracle.nvfp4_quantize_1d(x), "mxfp4": lambda: oracle.quantize_mxfp4(x, 32),
                "tensor": lambda: oracle.tensor_fp8(x), "pair": lambda: oracle.nvfp4_quantize_1d_pair(x, cpu[i, "b"])}[kind]()
        got = results[i]
        if kind == "pair":
            got, want = [t for half in got for t in half], [t for half in want for t in half]
        for j, (g_, w_) in enumerate(zip(got, want)):
            _same(g_, w_, f"{what}: job {i} ({kind} {shape}) output {j}")


# ---------------------------------------------------------------------------------------------------------------------
# non-finite and extreme values scattered over random data: NaN of both signs, infinities, signed zeros, the largest and
# the smallest magnitudes of the dtype, whole rows of zeros / NaN / one infinity
def _special_tensor(seed, shape, dtype, non_finite):
    g = torch.Generator().manual_seed(seed)
    rows, cols = shape
    x = (torch.randn(shape, generator=g) * torch.exp2(torch.randint(-6, 6, shape, generator=g).float())).to(dtype)
    fi = torch.finfo(dtype)
    pool = torch.tensor([0.0, -0.0, fi.max, -fi.max, fi.tiny, -fi.tiny, fi.smallest_normal * 0.5, 448.0, 464.0, 480.0, 6.0, 5.0,
                         1e-10, 7.0], dtype=torch.float32).to(dtype)
    hits = torch.rand(shape, generator=g) < 0.01
    picks = pool[torch.randint(0, pool.numel(), shape, generator=g)]
    x = torch.where(hits, picks, x)
    x[1 % rows] = 0.0
    x[3 % rows, : cols // 2] = 0.0
    x[5 % rows] = -0.0
    x[6 % rows, cols // 2:] = fi.max
    if non_finite:      # a few poisoned places only, so that most tiles / rows / blocks stay finite
        x[2 % rows] = float("nan")
        x[4 % rows, cols // 3] = float("inf")
        x[7 % rows, 5] = -float("inf")
        x[7 % rows, cols - 3] = float("nan")
        bits = x.view(torch.int16 if dtype != torch.float32 else torch.int32)
        bits[7 % rows, cols - 3] |= (-0x8000 if dtype != torch.float32 else -0x80000000)        # a NaN with the sign bit set
        x[(rows - 1), 17 % cols] = float("nan")
        x[(rows - 1), 18 % cols] = float("inf")
    return x


def _same_float(got, want, what):
    """Bit equality except that any NaN matches any NaN, for outputs held in a floating-point type of two bytes or more."""
    g, w = got.detach().cpu().contiguous(), want.detach().cpu().contiguous()
    assert g.shape == w.shape and g.dtype == w.dtype, f"{what}: {tuple(g.shape)} {g.dtype} vs {tuple(w.shape)} {w.dtype}"
    gn, wn = torch.isnan(g.float()), torch.isnan(w.float())
    assert torch.equal(gn, wn), f"{what}: NaN in different places ({int(gn.sum())} vs {int(wn.sum())})"
    _same(torch.where(gn, torch.zeros((), dtype=g.dtype), g), torch.where(wn, torch.zeros((), dtype=w.dtype), w), what)


def _same_any(got, want, what):
    if got.is_floating_point() and got.element_size() >= 2:
        _same_float(got, want, what)
    elif got.dtype == F8:       # the two NaN codes 0x7F / 0xFF count as one: which sign a NaN carries is the host FPU's choice
        g, w = _bits(got).clone(), _bits(want).clone()
        g[(g & 0x7F) == 0x7F] = 0x7F
        w[(w & 0x7F) == 0x7F] = 0x7F
        _same(g, w, what)
    else:
        _same(got, want, what)


@pytest.mark.parametrize("non_finite", [False, True], ids=["finite", "nonfinite"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=["bf16", "f16", "f32"])
@pytest.mark.parametrize("seed", range(4 * _SCALE))
def test_random_special_values(oracle, monkeypatch, seed, dtype, non_finite):
    from miles_amd.kernels.quant import fake_quant as fq
    from miles_amd.kernels.quant.fp8_act_quant import act_quant, fp8_simulate
    from miles_amd.kernels.quant.fp8_blockwise import fp8_blockwise_cast, per_block_cast_to_fp8
    from miles_amd.kernels.quant.int4_fake import fake_int4_quant_cuda, pack_layer
    from miles_amd.kernels.quant.nvfp4_qdq import NVFP4QDQConfig, compute_nvfp4_amax, fused_nvfp4_qdq
    from miles_amd.tools.convert_hf_to_fp8 import block_fp8, quant_fp8
    from miles_amd.tools.fp8_cast_bf16 import weight_dequant
    from miles_amd.utils.mxfp4 import dequantize_mxfp4, quantize_mxfp4
    from miles_amd.utils.mxfp8 import mxfp8_quantize
    from miles_amd.utils.nvfp4 import nvfp4_quantize_1d

    for name in ("NVTE_USE_FAST_MATH", "NVTE_NVFP4_4OVER6", "NVTE_NVFP4_4OVER6_E4M3_USE_256"):
        monkeypatch.delenv(name, raising=False)
    shape = [(136, 384), (64, 1024), (8, 256), (200, 128)][seed % 4]
    x = _special_tensor(7000 + seed, shape, dtype, non_finite)
    xd = x.to(DEV)
    failures = []

    def check(what, got, want):
        got, want = (got, want) if isinstance(got, (tuple, list)) else ((got,), (want,))
        for i, (g_, w_) in enumerate(zip(got, want)):
            if g_ is None and w_ is None:
                continue
            try:
                _same_any(g_, w_, f"{what}[{i}]")
            except AssertionError as e:
                failures.append(str(e))

    # Functions whose reference is a chain of torch floating-point ops, or CUDA code whose fmaxf / fminf reductions skip
    # NaN by definition, have a defined result for non-finite input and are held to it.  The rest of the list runs on
    # finite data only: there the reference's result for a NaN or an infinity hangs on a float -> integer conversion of
    # NaN (undefined in torch), on which NaN rule its Triton / TileLang compiler picks for max and clamp, or on a
    # third-party kernel outside the reference tree.
    check("block_fp8", block_fp8(xd, [128, 128]), oracle.block_fp8(x, (128, 128)))
    check("tensor_fp8", quant_fp8(xd, "tensor"), oracle.tensor_fp8(x))
    check("channel_fp8", quant_fp8(xd, "channel"), oracle.channel_fp8(x))
    for sym in (True, False):
        got = fake_int4_quant_cuda(xd, (1, 128), sym)
        want = oracle.fake_int4_quant(x, (1, 128), sym)
        check(f"fake_int4 sym={sym}", got[: 2 if sym else 3], want[: 2 if sym else 3])
    if dtype == torch.bfloat16:
        q_o, s_o = oracle.block_fp8(x, (128, 128))
        check("weight_dequant", weight_dequant(q_o.to(DEV), s_o.to(DEV)), oracle.weight_dequant(q_o, s_o))
    # fp8_blockwise_cast: Triton's max / maximum / clamp without propagate_nan return the operand that is not NaN
    check("fp8_blockwise_cast", fp8_blockwise_cast(xd), oracle.fp8_blockwise_cast(x))
    if dtype == torch.bfloat16:     # the published SGLang function is a torch chain
        check("per_block_cast_to_fp8", per_block_cast_to_fp8(xd), oracle.per_block_cast_to_fp8(x))
    # MXFP8: the published kernel takes the group maximum with fmaxf (a NaN is skipped, an infinity is not) and converts
    # with saturation (NaN -> the NaN code)
    check("mxfp8", mxfp8_quantize(xd), oracle.mxfp8_quantize(x))
    if non_finite:
        assert not failures, "\n".join(failures)
        return
    p, s4 = quantize_mxfp4(xd, 32)
    p_o, s4_o = oracle.quantize_mxfp4(x, 32)
    check("mxfp4", (p, s4), (p_o, s4_o))
    check("mxfp4 dequant", dequantize_mxfp4(p_o.to(DEV), s4_o.to(DEV), 32), oracle.dequantize_mxfp4(p_o, s4_o, 32))
    check("nvfp4", nvfp4_quantize_1d(xd), oracle.nvfp4_quantize_1d(x))
    for kind, fn in (("fp8", fq.fake_quant_fp8_forward), ("fp4", fq.fake_quant_fp4_forward),
                     ("compressed_kv", fq.fake_quant_compressed_kv_forward)):
        check(f"fake_quant {kind}", fn(xd), oracle.fake_quant(x, kind))
    for fmt in (None, "ue8m0"):
        check(f"act_quant {fmt}", act_quant(xd, 128, fmt), oracle.act_quant(x, 128, fmt))
    check("fp8_simulate", fp8_simulate(xd, 128), oracle.fp8_simulate(x, 128))
    if dtype != torch.float32:
        check("pack_layer", pack_layer(xd, 128)[:2], oracle.pack_layer(x, 128)[:2])
        check("pack_layer asym", pack_layer(xd, 128, sym=False), oracle.pack_layer(x, 128, sym=False))
        check("nvfp4 qdq", fused_nvfp4_qdq(xd, compute_nvfp4_amax(xd), NVFP4QDQConfig()), oracle.fused_nvfp4_qdq(x))
    assert not failures, "\n".join(failures)


# ---------------------------------------------------------------------------------------------------------------------
# strided and N-dimensional views: the reference's functions take them (they call .contiguous() or index by stride), so
# each must give what the contiguous copy gives
_VIEWS = {
    "transposed": lambda t: t.t(),
    "column_slice": lambda t: t[:, 128:384],
    "every_other_row": lambda t: t[::2],
    "every_other_column": lambda t: t[:, ::2],
    "3d": lambda t: t.view(2, 128, 512),
    "4d": lambda t: t.view(2, 2, 64, 512),
    "1d": lambda t: t.reshape(-1)[:1024],
}


@pytest.mark.parametrize("view", list(_VIEWS))
def test_strided_and_nd_views(oracle, view):
    from miles_amd.kernels.quant import fake_quant as fq
    from miles_amd.kernels.quant.fp8_act_quant import act_quant, fp8_simulate
    from miles_amd.kernels.quant.fp8_blockwise import fp8_blockwise_cast, per_block_cast_to_fp8
    from miles_amd.kernels.quant.int4_fake import fake_int4_quant_cuda, pack_layer
    from miles_amd.kernels.quant.nvfp4_qdq import NVFP4QDQConfig, compute_nvfp4_amax, fused_nvfp4_qdq
    from miles_amd.megatron_to_hf.processors.quantizer_nvfp4 import quantize_nvfp4
    from miles_amd.tools.convert_hf_to_fp8 import block_fp8, quant_fp8
    from miles_amd.utils.mxfp4 import quantize_mxfp4
    from miles_amd.utils.mxfp8 import mxfp8_quantize
    from miles_amd.utils.nvfp4 import nvfp4_quantize_1d

    g = torch.Generator().manual_seed(8000)
    base = (torch.randn(256, 512, generator=g) * 0.05).to(torch.bfloat16)
    xc, xd = _VIEWS[view](base), _VIEWS[view](base.to(DEV))
    cc = xc.contiguous()
    rows = cc.reshape(-1, cc.shape[-1])

    def check(what, got, want):
        got, want = (got, want) if isinstance(got, (tuple, list)) else ((got,), (want,))
        for j, (g_, w_) in enumerate(zip(got, want)):
            if g_ is not None:
                _same(g_, w_.reshape(g_.shape), f"{what} output {j} on a {view} view")

    if xc.dim() == 2:
        check("block_fp8", block_fp8(xd, [128, 128]), oracle.block_fp8(cc, (128, 128)))
        check("fp8_blockwise_cast", fp8_blockwise_cast(xd), oracle.fp8_blockwise_cast(cc))
        check("per_block_cast_to_fp8", per_block_cast_to_fp8(xd), oracle.per_block_cast_to_fp8(cc))
        check("tensor_fp8", quant_fp8(xd, "tensor"), oracle.tensor_fp8(cc))
        check("channel_fp8", quant_fp8(xd, "channel"), oracle.channel_fp8(cc))
        check("pack_layer", pack_layer(xd, 128)[:2], oracle.pack_layer(cc, 128)[:2])
        check("pack_layer asym", pack_layer(xd, 128, sym=False), oracle.pack_layer(cc, 128, sym=False))
        check("fake_int4", fake_int4_quant_cuda(xd, (1, 128), True)[:2], oracle.fake_int4_quant(cc, (1, 128), True)[:2])
        check("nvfp4", nvfp4_quantize_1d(xd), oracle.nvfp4_quantize_1d(cc))
        if not xd.is_contiguous():
            with pytest.raises(ValueError, match="contiguous"):      # the reference's contract for the fused q-dq
                fused_nvfp4_qdq(xd, compute_nvfp4_amax(xd), NVFP4QDQConfig())
    check("mxfp8", mxfp8_quantize(xd), oracle.mxfp8_quantize(rows))
    check("mxfp4", quantize_mxfp4(xd, 32), oracle.quantize_mxfp4(rows, 32))
    check("fake_quant", fq.fake_quant_fp8_forward(xd), oracle.fake_quant(rows, "fp8"))
    check("act_quant", act_quant(xd, 128), oracle.act_quant(rows, 128))
    check("fp8_simulate", fp8_simulate(xd, 128), oracle.fp8_simulate(rows, 128))
    if xc.dim() == 3:
        want = tuple(torch.stack(f) for f in zip(*[oracle.nvfp4_quantize_1d(cc[i]) for i in range(cc.shape[0])]))
        check("quantize_nvfp4 on a stack", quantize_nvfp4(xd), want)


# rows of 256 elements whose flat grids (2048, 4096 or 8192 elements per workgroup, by kernel) come to workgroup counts
# that select every run length the flat kernels deal to the XCDs: 1, 2, 3, 4, 6, 8, 12, 16, 24, 32, 48, 64
_RUN_LENGTH_ROWS = [16, 128, 192, 376, 512, 568, 752, 1024, 1136, 1519, 1520, 2048, 3024, 3040, 4096, 5999, 6000, 7984, 12000]


@pytest.mark.parametrize("rows", _RUN_LENGTH_ROWS)
def test_flat_kernels_on_every_xcd_run_length(oracle, rows):
    """A flat kernel remaps its workgroup ids so that an XCD takes runs of consecutive blocks; the run length is picked
    from the workgroup count (a power of two or three times one).  A wrong remap skips or repeats blocks, so every
    quantizer's bytes are compared with the oracle's on sizes that select every run length, ragged ends included."""
    from miles_amd import workloads as W
    from miles_amd.kernels.quant.int4_fake import pack_layer
    from miles_amd.tools.convert_hf_to_fp8 import block_fp8
    from miles_amd.tools.convert_kimi_int4_to_bf16 import _dequantize_tensor
    from miles_amd.tools.fp8_cast_bf16 import weight_dequant
    from miles_amd.utils.mxfp4 import dequantize_mxfp4, quantize_mxfp4
    from miles_amd.utils.mxfp8 import mxfp8_quantize, requantize_fp8_block_to_mxfp8
    from miles_amd.utils.nvfp4 import nvfp4_quantize_1d

    w = W.gaussian_outliers((rows, 256), std=0.02, p_outlier=0.001, gain=20.0, seed=4000 + rows)
    d = w.to(DEV)

    def same(got, want, what):
        for k, (g_, w_) in enumerate(zip(got, want)):
            if g_ is not None and w_ is not None:
                _same(g_, w_, f"{what}, output {k}, {rows} rows")

    same(mxfp8_quantize(d), oracle.mxfp8_quantize(w), "MXFP8")
    same(pack_layer(d, 128)[:2], oracle.pack_layer(w, 128)[:2], "INT4 g128")
    if rows % 8 == 0:           # the packed zero points take eight rows per word
        same(pack_layer(d, 32, sym=False), oracle.pack_layer(w, 32, sym=False), "INT4 g32 asymmetric")
    same(quantize_mxfp4(d, 32), oracle.quantize_mxfp4(w, 32), "MXFP4")
    same(nvfp4_quantize_1d(d), oracle.nvfp4_quantize_1d(w), "NVFP4")
    q, s = block_fp8(d, [128, 128])
    q_o, s_o = oracle.block_fp8(w, [128, 128])
    same((q, s), (q_o, s_o), "FP8 128 x 128")
    same((weight_dequant(q, s),), (oracle.weight_dequant(q_o, s_o),), "FP8 dequantize")
    same(requantize_fp8_block_to_mxfp8(q, s), oracle.fp8_block_to_mxfp8(q_o, s_o), "FP8 -> MXFP8")
    p4, s4 = oracle.quantize_mxfp4(w, 32)
    same((dequantize_mxfp4(p4.to(DEV), s4.to(DEV), 32),), (oracle.dequantize_mxfp4(p4, s4, 32),), "MXFP4 dequantize")
    pk, sc, _ = oracle.pack_layer(w, 128)
    same((_dequantize_tensor(pk.to(DEV), sc.to(DEV), (rows, 256), 128),), (oracle.int4_unpack_dequant(pk, sc, (rows, 256), 128),),
         "INT4 unpack")
