"""What Triton makes, on this GPU, of the expressions the reference's two Triton kernels on this path are written in:
the sync path's FP8 quantizer (its two fp32 divisions first of all) and the FP8 block dequantizer.

The reference's `_fp8_blockwise_cast_kernel` (miles/kernels/quant/fp8_blockwise.py:51-54) computes, per tile,
`_absmax = maximum(max|x|, eps)`, `x_s = _absmax / fp8_max` and `s_inv = 1.0 / x_s` with Triton's `/` on fp32 scalars
(`eps`, `fp8_max` are run-time arguments).  The oracle and the HIP kernel take both as IEEE divisions.  Triton does not
promise a correctly rounded quotient, so this file measures it: a probe of its own (not the reference's kernel) runs the
same three expressions on every tile maximum a bf16 or fp16 tensor can have and compares them with IEEE division.

A second probe is a whole 128 x 128 tile quantizer written for this file from the same expressions (maximum floored at
eps, the two divisions, clamp of the product, cast to e4m3): its bytes are compared with the HIP kernel's on finite data,
on tiles holding infinities and NaN, and on one Qwen3-4B layer at full size.

The counts are printed (and written to the directory MQ_PROBE_REPORT_DIR names, if any).  Every test is skipped, with the reason,
where Triton cannot compile for the GPU.
"""

import json
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _keep_report(name, report):
    """The counts also go to a file when MQ_PROBE_REPORT_DIR names a directory."""
    out_dir = os.environ.get("MQ_PROBE_REPORT_DIR")
    if out_dir and os.path.isdir(out_dir):
        with open(os.path.join(out_dir, name), "w") as f:
            json.dump(report, f, indent=1)


def _tile_maxima():
    """Every positive finite bf16 and fp16 value as fp32 (the tile maximum is exact in fp32), duplicates removed."""
    bf = torch.arange(1, 0x7F80, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()
    fp = torch.arange(1, 0x7C00, dtype=torch.int32).to(torch.int16).view(torch.float16).float()
    return torch.unique(torch.cat([bf, fp])), bf.numel(), fp.numel()


def _probe():
    try:
        import triton
        import triton.language as tl
    except Exception as exc:              # pragma: no cover - depends on the image
        pytest.skip(f"triton is not importable: {exc!r}")

    @triton.jit
    def elementwise(a_ptr, xs_ptr, sinv_ptr, n, eps, fp8_max, BLOCK: tl.constexpr):
        offs = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
        mask = offs < n
        a = tl.load(a_ptr + offs, mask=mask, other=1.0)
        absmax = tl.maximum(a, eps)
        x_s = absmax / fp8_max
        s_inv = 1.0 / x_s
        tl.store(xs_ptr + offs, x_s, mask=mask)
        tl.store(sinv_ptr + offs, s_inv, mask=mask)

    @triton.jit
    def per_tile(a_ptr, xs_ptr, sinv_ptr, eps, fp8_max, BLOCK: tl.constexpr):
        # the reference's shape of the computation: a reduction to a scalar, then scalar divisions
        pid = tl.program_id(0)
        x = tl.load(a_ptr + pid + tl.zeros([BLOCK], dtype=tl.int32))
        absmax = tl.maximum(tl.max(tl.abs(x)), eps)
        x_s = absmax / fp8_max
        s_inv = 1.0 / x_s
        tl.store(xs_ptr + pid, x_s)
        tl.store(sinv_ptr + pid, s_inv)

    return triton, elementwise, per_tile


def _ulps(a, b):
    return (a.view(torch.int32).to(torch.int64) - b.view(torch.int32).to(torch.int64)).abs()


def test_triton_division_against_ieee(oracle):
    triton, elementwise, per_tile = _probe()
    amax, n_bf16, n_fp16 = _tile_maxima()
    n = amax.numel()
    eps, fp8_max = 1e-10, float(torch.finfo(torch.float8_e4m3fn).max)
    a = amax.to(DEV)
    results = {}
    try:
        xs, sinv = torch.empty_like(a), torch.empty_like(a)
        elementwise[(triton.cdiv(n, 256),)](a, xs, sinv, n, eps, fp8_max, BLOCK=256)
        torch.cuda.synchronize()
        results["elementwise"] = (xs.cpu(), sinv.cpu())
        xs2, sinv2 = torch.empty_like(a), torch.empty_like(a)
        per_tile[(n,)](a, xs2, sinv2, eps, fp8_max, BLOCK=64)
        torch.cuda.synchronize()
        results["per_tile_scalar"] = (xs2.cpu(), sinv2.cpu())
    except Exception as exc:              # pragma: no cover - depends on the image
        pytest.skip(f"triton could not compile or launch on this GPU: {type(exc).__name__}: {str(exc)[:200]}")

    # IEEE: numpy's float32 division, and the oracle's own x_s for the same maxima (one 1 x 8 block per value)
    floor = np.maximum(amax.numpy(), np.float32(eps))
    want_xs = torch.from_numpy(floor / np.float32(fp8_max))
    want_sinv = torch.from_numpy(np.float32(1.0) / want_xs.numpy())
    sample = amax[:: max(n // 4096, 1)]
    _y, oracle_xs = oracle.fp8_blockwise_cast(sample.reshape(-1, 1).repeat(1, 8).contiguous(), (1, 8))
    sample_want = torch.from_numpy(np.maximum(sample.numpy(), np.float32(eps)) / np.float32(fp8_max))
    assert torch.equal(oracle_xs.reshape(-1).view(torch.int32), sample_want.view(torch.int32)), "the oracle's x_s is not numpy's IEEE quotient"

    report = {"tile_maxima": n, "bf16_patterns": n_bf16, "fp16_patterns": n_fp16, "triton": triton.__version__}
    for form, (got_xs, got_sinv) in results.items():
        d_xs, d_sinv = _ulps(got_xs, want_xs), _ulps(got_sinv, want_sinv)
        # s_inv as Triton would have it from the IEEE x_s cannot be separated from its own x_s: also compare s_inv with
        # the IEEE reciprocal of Triton's own x_s, which isolates the second division
        own = torch.from_numpy(np.float32(1.0) / got_xs.numpy())
        d_own = _ulps(got_sinv, own)
        report[form] = {"x_s_differ": int((d_xs != 0).sum()), "x_s_max_ulp": int(d_xs.max()),
                        "s_inv_differ": int((d_sinv != 0).sum()), "s_inv_max_ulp": int(d_sinv.max()),
                        "s_inv_differ_from_ieee_reciprocal_of_own_x_s": int((d_own != 0).sum())}
        # what a differing s_inv does to the codes: every bf16 x with |x| <= amax through clamp(x * s_inv) -> e4m3
        bad = (d_sinv != 0).nonzero().reshape(-1)
        changed = total = 0
        for i in bad[:: max(bad.numel() // 64, 1)].tolist():
            x = torch.arange(0, 0x7F80, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()
            x = x[x <= amax[i]]
            ya = (x * got_sinv[i]).clamp(-fp8_max, fp8_max).to(torch.float8_e4m3fn).view(torch.uint8)
            yb = (x * want_sinv[i]).clamp(-fp8_max, fp8_max).to(torch.float8_e4m3fn).view(torch.uint8)
            changed += int((ya != yb).sum())
            total += x.numel()
        report[form]["codes_changed_of_sampled_inputs"] = [changed, total]
    print("TRITON_DIVISION", json.dumps(report))
    _keep_report("triton_division.json", report)
    for form in results:
        assert report[form]["x_s_max_ulp"] <= 1 and report[form]["s_inv_max_ulp"] <= 2, report


def _tile_probe():
    """A 128 x 128 tile quantizer written for this test from the reference's expressions (maximum of |x| floored at eps,
    the two divisions, clamp of the product, cast to e4m3): what Triton makes of them on this GPU, end to end."""
    try:
        import triton
        import triton.language as tl
    except Exception as exc:              # pragma: no cover - depends on the image
        pytest.skip(f"triton is not importable: {exc!r}")

    @triton.jit
    def tile_quant(x_ptr, y_ptr, s_ptr, rows, cols, tiles_across, eps, lo, hi, B: tl.constexpr):
        t = tl.program_id(0)
        r = (t // tiles_across) * B + tl.arange(0, B)
        c = (t % tiles_across) * B + tl.arange(0, B)
        inside = (r < rows)[:, None] & (c < cols)[None, :]
        at = r[:, None].to(tl.int64) * cols + c[None, :]
        x = tl.load(x_ptr + at, mask=inside, other=0.0).to(tl.float32)
        top = tl.maximum(tl.max(tl.abs(x)), eps)
        scale = top / hi
        inv = 1.0 / scale
        y = tl.clamp(x * inv, lo, hi).to(y_ptr.dtype.element_ty)
        tl.store(y_ptr + at, y, mask=inside)
        tl.store(s_ptr + t, scale)

    def run(x):
        rows, cols = x.shape
        tr, tc = -(-rows // 128), -(-cols // 128)
        y = torch.empty((rows, cols), dtype=torch.float8_e4m3fn, device=x.device)
        s = torch.empty((tr, tc), dtype=torch.float32, device=x.device)
        hi = float(torch.finfo(torch.float8_e4m3fn).max)
        tile_quant[(tr * tc,)](x, y, s, rows, cols, tc, 1e-10, -hi, hi, B=128, num_warps=8)
        torch.cuda.synchronize()
        return y, s

    return run


def _cases():
    from miles_amd import workloads as W

    gate = W.gaussian_outliers((384, 640), std=0.02, p_outlier=0.001, gain=20.0, seed=2001)
    gate[128:256, 128:256] = 0                                   # an all-zero tile: the eps floor
    yield "bf16 gaussian with outliers and a zero tile", gate
    yield "bf16 ragged", W.gaussian_outliers((130, 264), std=0.02, p_outlier=0.001, gain=20.0, seed=5)
    yield "fp16", W.gaussian_outliers((256, 384), std=0.02, p_outlier=0.001, gain=20.0, seed=6, dtype=torch.float16)
    for kind in W.PATTERNS:
        yield f"bf16 {kind}", W.reference_pattern(kind, (256, 128), spread=512.0, amplitude=16.0)
    g = torch.Generator().manual_seed(7)
    wide = (torch.randn((256, 256), generator=g) * torch.exp(torch.randn((256, 256), generator=g) * 8)).to(torch.bfloat16)
    yield "bf16 sixty binades in one tile", wide
    tiny = (torch.randn((128, 256), generator=g) * 1e-12).to(torch.bfloat16)
    yield "bf16 below the eps floor", tiny


def test_triton_tile_quantizer_gives_the_hip_kernels_bytes(oracle):
    """The whole sync-path quantizer, as Triton compiles its expressions for this GPU, against the HIP kernel and the
    oracle on finite inputs: scales and codes byte for byte."""
    from miles_amd.kernels.quant.fp8_blockwise import fp8_blockwise_cast

    run = _tile_probe()
    report = {}
    for what, x in _cases():
        try:
            ty, ts = run(x.to(DEV))
        except Exception as exc:          # pragma: no cover - depends on the image
            pytest.skip(f"triton could not compile or launch on this GPU: {type(exc).__name__}: {str(exc)[:200]}")
        hy, hs = fp8_blockwise_cast(x.to(DEV))
        oy, os_ = oracle.fp8_blockwise_cast(x)
        ty, ts = ty.cpu().view(torch.uint8), ts.cpu().view(torch.int32)
        codes = int((ty != hy.cpu().view(torch.uint8)).sum())
        scales = int((ts != hs.cpu().view(torch.int32)).sum())
        report[what] = {"codes_differ": codes, "scales_differ": scales, "elements": x.numel()}
        assert torch.equal(hy.cpu().view(torch.uint8), oy.view(torch.uint8)) and torch.equal(hs.cpu().view(torch.int32), os_.view(torch.int32)), what
    print("TRITON_TILE_QUANTIZER", json.dumps(report))
    _keep_report("triton_tile_quantizer.json", report)
    assert all(v["codes_differ"] == 0 and v["scales_differ"] == 0 for v in report.values()), report


def test_triton_tile_quantizer_on_non_finite_inputs():
    """Where the HIP kernel's handling of infinities and NaN rests on a reading of Triton's max / maximum / clamp (the
    operand that is not NaN is returned): the same probe on tiles that hold them.  The two e4m3 NaN codes count as one."""
    from miles_amd.kernels.quant.fp8_blockwise import fp8_blockwise_cast

    run = _tile_probe()
    g = torch.Generator().manual_seed(9)
    base = (torch.randn((128, 384), generator=g) * 0.02).to(torch.bfloat16)
    base[3, 5] = float("nan")                 # tile 0: a NaN among ordinary values
    base[7, 128 + 9] = float("inf")           # tile 1: an infinity
    base[9, 256 + 1], base[11, 256 + 2] = float("-inf"), float("nan")   # tile 2: both
    try:
        ty, ts = run(base.to(DEV))
    except Exception as exc:              # pragma: no cover - depends on the image
        pytest.skip(f"triton could not compile or launch on this GPU: {type(exc).__name__}: {str(exc)[:200]}")
    hy, hs = fp8_blockwise_cast(base.to(DEV))
    ty, hy = ty.cpu().view(torch.uint8), hy.cpu().view(torch.uint8)
    fold = lambda c: torch.where((c & 0x7F) == 0x7F, torch.full_like(c, 0x7F), c)
    report = {}
    for j, what in enumerate(("nan_in_tile", "inf_in_tile", "inf_and_nan_in_tile")):
        cols = slice(128 * j, 128 * (j + 1))
        report[what] = {"codes_differ": int((fold(ty[:, cols]) != fold(hy[:, cols])).sum()),
                        "scale_triton": ts[0, j].item(), "scale_hip": hs[0, j].item()}
    print("TRITON_TILE_NONFINITE", json.dumps(report))
    _keep_report("triton_tile_nonfinite.json", report)
    for what, r in report.items():
        assert r["codes_differ"] == 0 and (r["scale_triton"] == r["scale_hip"]), (what, r)


def test_triton_tile_quantizer_on_one_qwen3_4b_layer():
    """The seven quantized tensors of one Qwen3-4B layer at full size (q, k, v, o, gate, up, down of the headline
    workload's generator): Triton's bytes against the HIP kernel's."""
    from miles_amd import workloads as W
    from miles_amd.kernels.quant.fp8_blockwise import fp8_blockwise_cast

    run = _tile_probe()
    gen = torch.Generator(device=DEV)
    gen.manual_seed(2001)
    shapes = [(4096, 2560), (1024, 2560), (1024, 2560), (2560, 4096), (9728, 2560), (9728, 2560), (2560, 9728)]
    for shape in shapes:
        x = W.device_gaussian_outliers(shape, gen, std=0.02, p_outlier=0.001, gain=20.0)
        try:
            ty, ts = run(x)
        except Exception as exc:          # pragma: no cover - depends on the image
            pytest.skip(f"triton could not compile or launch on this GPU: {type(exc).__name__}: {str(exc)[:200]}")
        hy, hs = fp8_blockwise_cast(x)
        assert torch.equal(ts.view(torch.int32), hs.view(torch.int32)), f"{shape}: scales"
        assert torch.equal(ty.view(torch.uint8), hy.view(torch.uint8)), f"{shape}: codes"


def test_triton_dequantizer_gives_the_hip_kernels_bytes(oracle):
    """The FP8 block dequantizer of the reference is a Triton kernel too (tools/fp8_cast_bf16.py:15-27): decode the code
    to fp32, one multiplication by the tile's scale, a store that rounds to bf16.  A probe written for this test from
    those expressions (flat over the elements, the scale found per element) against the HIP kernel: every code byte
    times scales over eighty binades, subnormal products and NaN codes included (any bf16 NaN counts as NaN)."""
    from miles_amd.tools.fp8_cast_bf16 import weight_dequant

    try:
        import triton
        import triton.language as tl
    except Exception as exc:              # pragma: no cover - depends on the image
        pytest.skip(f"triton is not importable: {exc!r}")

    @triton.jit
    def decode_scale_store(code_ptr, scale_ptr, out_ptr, count, cols, tiles_across, BLOCK: tl.constexpr, TILE: tl.constexpr):
        at = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
        live = at < count
        value = tl.load(code_ptr + at, mask=live).to(tl.float32)
        scale = tl.load(scale_ptr + (at // cols) // TILE * tiles_across + (at % cols) // TILE, mask=live)
        tl.store(out_ptr + at, value * scale, mask=live)

    g = torch.Generator().manual_seed(17)
    rows, cols = 384, 640
    codes = torch.arange(256, dtype=torch.uint8).repeat(rows, 3)[:, :cols].contiguous()
    codes[200:] = torch.randint(0, 256, (rows - 200, cols), generator=g, dtype=torch.int32).to(torch.uint8)
    scale = torch.exp(torch.randn((3, 5), generator=g) * 12).float()
    scale[0, 0], scale[1, 1], scale[2, 2], scale[0, 4] = 0.0, -2.5, 2.0 ** -130, 2.0 ** 100
    x, s = codes.view(torch.float8_e4m3fn).to(DEV), scale.to(DEV)
    out = torch.empty((rows, cols), dtype=torch.bfloat16, device=DEV)
    try:
        decode_scale_store[(triton.cdiv(rows * cols, 1024),)](x, s, out, rows * cols, cols, 5, BLOCK=1024, TILE=128)
        torch.cuda.synchronize()
    except Exception as exc:              # pragma: no cover - depends on the image
        pytest.skip(f"triton could not compile or launch on this GPU: {type(exc).__name__}: {str(exc)[:200]}")
    hip = weight_dequant(x, s)
    want = oracle.weight_dequant(codes.view(torch.float8_e4m3fn), scale)
    assert torch.equal(hip.cpu().view(torch.int16), want.view(torch.int16)), "the HIP dequantizer differs from the oracle"
    t, h = out.cpu(), hip.cpu()
    nan = torch.isnan(h)
    assert torch.equal(torch.isnan(t), nan), "NaN in different places"
    differ = int((t.view(torch.int16)[~nan] != h.view(torch.int16)[~nan]).sum())
    print("TRITON_DEQUANTIZER", json.dumps({"elements": rows * cols, "nan_elements": int(nan.sum()), "values_differ": differ}))
    assert differ == 0


@pytest.mark.parametrize("kind", ["fp8", "fp4", "compressed_kv"])
def test_triton_fake_quantizers_give_the_hip_kernels_values(oracle, kind):
    """The training-forward fake quantizers of the reference are one Triton kernel (miles/kernels/quant/fake_quant.py:
    24-61): per group of 32 (16 for the compressed-KV form) the largest magnitude, a scale -- a power of two from the
    bits of `amax / fmax`, or an e4m3 value -- a division by it (`/`, or `div_rn`), a clamp, a rounding to the e4m3 or
    e2m1 grid (a cast, or `rint` of magnitude over step) and the product with the scale, stored in the input's dtype.  A
    probe written for this test from those expressions against the HIP kernel on bf16, fp16 and fp32 data over many
    binades: what Triton makes of the casts, `div_rn`, the maxima and the rounding to an integer on this GPU.  Triton
    3.6.0's ROCm `libdevice` has no `rint` (the reference's own kernel does not compile with it in the two e2m1 modes); the
    probe then takes `nearbyint`, the same function of its argument (nearest integer, ties to even)."""
    from miles_amd.kernels.quant import fake_quant as fq

    try:
        import triton
        import triton.language as tl
        from triton.language.extra import libdevice
    except Exception as exc:              # pragma: no cover - depends on the image
        pytest.skip(f"triton is not importable: {exc!r}")

    import triton.language.extra.hip.libdevice as rocm_libdevice
    to_integer = libdevice.rint if hasattr(rocm_libdevice, "rint") else libdevice.nearbyint

    @triton.jit
    def group_round_trip(src, dst, groups, TOP: tl.constexpr, FLOOR: tl.constexpr, GRID4: tl.constexpr,
                         BYTE_SCALE: tl.constexpr, WIDTH: tl.constexpr, TALL: tl.constexpr):
        g = tl.program_id(0) * TALL + tl.arange(0, TALL)
        at = g[:, None] * WIDTH + tl.arange(0, WIDTH)[None, :]
        live = (g < groups)[:, None]
        v = tl.load(src + at, mask=live, other=0.0).to(tl.float32)
        top = tl.max(tl.abs(v), axis=1)
        if BYTE_SCALE:
            s = tl.minimum(tl.maximum(top * (1.0 / TOP), FLOOR), 448.0).to(tl.float8e4nv).to(tl.float32)
            w = tl.div_rn(v, s[:, None])
        else:
            bits = (tl.maximum(top, FLOOR) * (1.0 / TOP)).to(tl.int32, bitcast=True)
            e = ((bits >> 23) & 0xFF) + ((bits & 0x7FFFFF) != 0).to(tl.int32)
            s = (e << 23).to(tl.float32, bitcast=True)
            w = v / s[:, None]
        w = tl.minimum(tl.maximum(w, -TOP), TOP)
        if GRID4:
            m = tl.abs(w)
            step = tl.where(m < 2.0, 0.5, tl.where(m < 4.0, 1.0, 2.0))
            r = to_integer(m / step) * step * tl.where(w > 0, 1.0, tl.where(w < 0, -1.0, 0.0))
        else:
            r = w.to(tl.float8e4nv).to(tl.float32)
        tl.store(dst + at, (r * s[:, None]).to(dst.dtype.element_ty), mask=live)

    width = 16 if kind == "compressed_kv" else 32
    top, floor = {"fp8": (448.0, 1e-4), "fp4": (6.0, 6 * 2.0 ** -126), "compressed_kv": (6.0, 2.0 ** -9)}[kind]
    hip_fn = {"fp8": fq.fake_quant_fp8_forward, "fp4": fq.fake_quant_fp4_forward,
              "compressed_kv": fq.fake_quant_compressed_kv_forward}[kind]
    g = torch.Generator().manual_seed(23)
    report = {}
    for dtype in (torch.bfloat16, torch.float16, torch.float32):
        groups = 40_000
        x = torch.randn((groups, width), generator=g) * torch.exp(torch.randn((groups, 1), generator=g) * 6)
        x[:64] = 0.0                                              # all-zero groups
        x[64:128] *= 1e-30                                        # far below every floor
        x[128:192, ::3] = 0.0
        x[192:256] = torch.round(x[192:256] * 4) / 4              # ties of the e2m1 grid
        if dtype == torch.float16:
            x = x.clamp(-6e4, 6e4)
        x = x.to(dtype)
        xd = x.to(DEV)
        out = torch.empty_like(xd)
        try:
            group_round_trip[(triton.cdiv(groups, 64),)](xd, out, groups, TOP=top, FLOOR=floor, GRID4=kind != "fp8",
                                                         BYTE_SCALE=kind == "compressed_kv", WIDTH=width, TALL=64)
            torch.cuda.synchronize()
        except Exception as exc:              # pragma: no cover - depends on the image
            pytest.skip(f"triton could not compile or launch on this GPU: {type(exc).__name__}: {str(exc)[:200]}")
        hip = hip_fn(xd).cpu()
        want = oracle.fake_quant(x, kind)
        bits = {torch.bfloat16: torch.int16, torch.float16: torch.int16, torch.float32: torch.int32}[dtype]
        assert torch.equal(hip.view(bits), want.view(bits)), f"{dtype}: the HIP kernel differs from the oracle"
        t = out.cpu()
        differ = t.view(bits) != hip.view(bits)
        # (+0 and -0 count as one value: the reference multiplies by an explicit sign, the probe with it)
        differ &= ~((t == 0) & (hip == 0))
        report[str(dtype)] = {"elements": x.numel(), "values_differ": int(differ.sum())}
    print("TRITON_FAKE_QUANT", kind, json.dumps(report))
    _keep_report(f"triton_fake_quant_{kind}.json", report)
    assert all(v["values_differ"] == 0 for v in report.values()), report
