"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py from PyTorch's CPU kernels running
the reference's op chains) against the C oracle (CPU tests) and against the HIP library (GPU tests).

The GPU tests do not involve the oracle at all: the expected bytes come from the files.
"""

import json
import os

import numpy as np
import pytest
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
DEV = "cuda:0"
_DT = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32, "bfloat16": torch.bfloat16,
       "float16": torch.float16, "float32": torch.float32}

with open(os.path.join(GOLDEN, "manifest.json")) as _f:
    MANIFEST = {fam["file"][:-4]: fam for fam in json.load(_f)["families"]}
_CACHE = {}


def _npz(family):
    if family not in _CACHE:
        _CACHE[family] = np.load(os.path.join(GOLDEN, f"{family}.npz"), allow_pickle=False)
    return _CACHE[family]


def _cases(family, prefix=""):
    return [c["case"] for c in MANIFEST[family]["cases"] if c["case"].startswith(prefix)]


def _info(family, case):
    return next(c for c in MANIFEST[family]["cases"] if c["case"] == case)


def _t(family, case, key, dtype=None):
    """Array `case.key` as a tensor; 16-bit and 8-bit float types are rebuilt from their stored bit patterns."""
    a = _npz(family)[f"{case}.{key}"]
    if a.dtype == np.uint16:
        t = torch.from_numpy(a.view(np.int16).copy())
        return t.view(dtype or torch.bfloat16)
    t = torch.from_numpy(a.copy())
    if dtype is not None and t.dtype != dtype:
        t = t.view(dtype)
    return t


def _bits(t):
    t = t.detach().cpu().contiguous()
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16)
    if t.dtype == torch.float32:
        return t.view(torch.int32)
    if t.dtype == torch.float8_e4m3fn:
        return t.view(torch.uint8)
    return t


def _same(got, want, what):
    g, w = _bits(got), _bits(want)
    assert g.shape == w.shape, f"{what}: shape {tuple(g.shape)} != {tuple(w.shape)}"
    if not torch.equal(g, w):
        bad = (g != w).nonzero()
        raise AssertionError(f"{what}: {bad.shape[0]} mismatches, first at {bad[0].tolist()}: "
                             f"got {g[tuple(bad[0])].item()} want {w[tuple(bad[0])].item()}")


def test_manifest_lists_every_array():
    for family, fam in MANIFEST.items():
        keys = set(_npz(family).files)
        cases = {k.rsplit(".", 1)[0] for k in keys}
        assert cases == {c["case"] for c in fam["cases"]}, family


# ----------------------------------------------------------------------------------------------------
# implementations under test: name -> callable taking CPU tensors (oracle) or GPU tensors (HIP wrappers)
# ----------------------------------------------------------------------------------------------------
class _OracleImpl:
    def __init__(self, oracle):
        self.o = oracle
        self.dev = "cpu"

    def block_fp8(self, w, block):
        return self.o.block_fp8(w, tuple(block))

    def fp8_blockwise_cast(self, x):
        return self.o.fp8_blockwise_cast(x)

    def weight_dequant(self, q, s):
        return self.o.weight_dequant(q, s)

    def mxfp8(self, w):
        return self.o.mxfp8_quantize(w)

    def quantize_mxfp4(self, w, g):
        return self.o.quantize_mxfp4(w, g)

    def dequantize_mxfp4(self, p, s, g):
        return self.o.dequantize_mxfp4(p, s, g)

    def fake_int4(self, w, g, sym):
        return self.o.fake_int4_quant(w, (1, g), sym)

    def pack_layer(self, w, g, sym):
        return self.o.pack_layer(w, g, sym=sym)

    def nvfp4(self, w):
        return self.o.nvfp4_quantize_1d(w)

    def fake_quant(self, x, kind):
        return self.o.fake_quant(x, kind)

    def nvfp4_pair(self, a, b):
        return self.o.nvfp4_quantize_1d_pair(a, b)

    def act_quant(self, x, block, fmt, inplace=False):
        return self.o.act_quant(x, block, fmt, inplace=inplace)

    def _each(self, fn, weight, scale):
        """The oracle takes one matrix at a time: apply to every matrix of a stacked tensor."""
        n, k = weight.shape[-2:]
        outs = [fn(w, s) for w, s in zip(weight.reshape(-1, n, k), scale.reshape(-1, *scale.shape[-2:]))]
        return outs, weight.shape[:-2]

    def fp8_block_to_mxfp8(self, codes, scale):
        outs, lead = self._each(self.o.fp8_block_to_mxfp8, codes, scale)
        return (torch.stack([q for q, _ in outs]).reshape(codes.shape),
                torch.stack([s for _, s in outs]).reshape(*lead, codes.shape[-2], codes.shape[-1] // 32))

    def expand_tile_scales(self, weight, scale):
        outs, lead = self._each(self.o.expand_tile_scales_e8m0, weight, scale)
        return torch.stack(outs).reshape(*lead, weight.shape[-2], weight.shape[-1] // 32)

    def scales_pow2(self, weight, scale):
        outs, _ = self._each(self.o.fp8_scales_are_pow2, weight, scale)
        return all(outs)


class _HipImpl:
    dev = DEV

    def block_fp8(self, w, block):
        from miles_amd.tools.convert_hf_to_fp8 import block_fp8
        return block_fp8(w, tuple(block))

    def fp8_blockwise_cast(self, x):
        from miles_amd.kernels.quant.fp8_blockwise import fp8_blockwise_cast
        return fp8_blockwise_cast(x)

    def weight_dequant(self, q, s):
        from miles_amd.tools.fp8_cast_bf16 import weight_dequant
        return weight_dequant(q, s)

    def mxfp8(self, w):
        from miles_amd.utils.mxfp8 import mxfp8_quantize
        return mxfp8_quantize(w)

    def quantize_mxfp4(self, w, g):
        from miles_amd.utils.mxfp4 import quantize_mxfp4
        return quantize_mxfp4(w, g)

    def dequantize_mxfp4(self, p, s, g):
        from miles_amd.utils.mxfp4 import dequantize_mxfp4
        return dequantize_mxfp4(p, s, g)

    def fake_int4(self, w, g, sym):
        from miles_amd.kernels.quant.int4_fake import fake_int4_quant_cuda
        return fake_int4_quant_cuda(w, (1, g), sym)

    def pack_layer(self, w, g, sym):
        from miles_amd.kernels.quant.int4_fake import pack_layer
        return pack_layer(w, g, sym)

    def nvfp4(self, w):
        from miles_amd.utils.nvfp4 import nvfp4_quantize_1d
        return nvfp4_quantize_1d(w)

    def fake_quant(self, x, kind):
        from miles_amd.kernels.quant import fake_quant as fq
        return {"fp8": fq.fake_quant_fp8_forward, "fp4": fq.fake_quant_fp4_forward,
                "compressed_kv": fq.fake_quant_compressed_kv_forward}[kind](x)

    def nvfp4_pair(self, a, b):
        from miles_amd.utils.nvfp4 import nvfp4_quantize_1d_pair
        return nvfp4_quantize_1d_pair(a, b)

    def act_quant(self, x, block, fmt, inplace=False):
        from miles_amd.kernels.quant.fp8_act_quant import act_quant
        return act_quant(x.clone(), block, fmt, inplace=inplace)

    def fp8_block_to_mxfp8(self, codes, scale):
        from miles_amd.utils.mxfp8 import requantize_fp8_block_to_mxfp8
        return requantize_fp8_block_to_mxfp8(codes, scale)

    def expand_tile_scales(self, weight, scale):
        from miles_amd.utils.mxfp8 import expand_tile_scales_e8m0
        return expand_tile_scales_e8m0(weight, scale)

    def scales_pow2(self, weight, scale):
        from miles_amd.utils.mxfp8 import fp8_tile_scales_pow2
        return fp8_tile_scales_pow2([(weight, scale)])[0]


def _check_fp8_block(impl, case):
    info = _info("fp8_block", case)
    w = _t("fp8_block", case, "w", _DT[info["dtype"]]).to(impl.dev)
    q, s = impl.block_fp8(w, info["block"])
    _same(s, _t("fp8_block", case, "scale"), f"{case} scales")
    _same(q, _t("fp8_block", case, "q"), f"{case} codes")


def _check_fp8_blockwise(impl, case):
    x = _t("fp8_blockwise_cast", case, "x").to(impl.dev)
    y, s = impl.fp8_blockwise_cast(x)
    _same(s, _t("fp8_blockwise_cast", case, "scale"), f"{case} scales")
    _same(y, _t("fp8_blockwise_cast", case, "y"), f"{case} codes")


def _check_fp8_dequant(impl, case):
    q = _t("fp8_dequant", case, "q").view(torch.float8_e4m3fn).to(impl.dev)
    s = _t("fp8_dequant", case, "scale").to(impl.dev)
    _same(impl.weight_dequant(q, s), _t("fp8_dequant", case, "y"), f"{case} values")


def _check_mxfp8(impl, case):
    w = _t("mxfp8", case, "w").to(impl.dev)
    q, s = impl.mxfp8(w)
    _same(s, _t("mxfp8", case, "scale"), f"{case} E8M0 scales")
    _same(q, _t("mxfp8", case, "q"), f"{case} codes")


def _check_mxfp4(impl, case):
    info = _info("mxfp4", case)
    if case.startswith("quant_"):
        w = _t("mxfp4", case, "w", _DT[info["dtype"]]).to(impl.dev)
        p, s = impl.quantize_mxfp4(w, info["group"])
        _same(s, _t("mxfp4", case, "scale"), f"{case} E8M0 scales")
        _same(p, _t("mxfp4", case, "packed"), f"{case} packed codes")
    else:
        p, s = _t("mxfp4", case, "packed").to(impl.dev), _t("mxfp4", case, "scale").to(impl.dev)
        _same(impl.dequantize_mxfp4(p, s, info["group"]), _t("mxfp4", case, "y"), f"{case} values")


def _check_int4(impl, case):
    info = _info("int4", case)
    w = _t("int4", case, "w").to(impl.dev)
    g, sym = info["group"], info["sym"]
    out, scale, zero = impl.fake_int4(w, g, sym)
    _same(out, _t("int4", case, "fake_out"), f"{case} fake-quant values")
    _same(scale, _t("int4", case, "fake_scale"), f"{case} fake-quant scales")
    if not sym:
        _same(zero, _t("int4", case, "fake_zero"), f"{case} fake-quant zero points")
    packed, pscale, pzp = impl.pack_layer(w, g, sym)
    _same(packed, _t("int4", case, "packed"), f"{case} packed words")
    _same(pscale, _t("int4", case, "scale"), f"{case} scales")
    if sym:
        assert pzp is None
    else:
        _same(pzp, _t("int4", case, "packed_zp"), f"{case} packed zero points")


def _check_nvfp4(impl, case):
    if case.startswith("global_scale_vectors"):
        return
    if case.startswith("pair_"):
        gate, up = _t("nvfp4", case, "gate").to(impl.dev), _t("nvfp4", case, "up").to(impl.dev)
        (gq, gs, gg), (uq, us, ug) = impl.nvfp4_pair(gate, up)
        _same(gq, _t("nvfp4", case, "gate_q"), "pair gate codes")
        _same(uq, _t("nvfp4", case, "up_q"), "pair up codes")
        _same(gs, _t("nvfp4", case, "gate_scale"), "pair gate block scales")
        _same(us, _t("nvfp4", case, "up_scale"), "pair up block scales")
        want = _t("nvfp4", case, "global_scale").reshape(())
        _same(gg, want, "pair gate global scale")
        _same(ug, want, "pair up global scale")
        return
    w = _t("nvfp4", case, "w").to(impl.dev)
    q, s, g = impl.nvfp4(w)
    _same(s, _t("nvfp4", case, "block_scale"), f"{case} block scales")
    _same(q, _t("nvfp4", case, "q"), f"{case} codes")
    _same(g, _t("nvfp4", case, "global_scale").reshape(()), f"{case} global scale")


def _check_fake_quant(impl, case):
    info = _info("fake_quant", case)
    x = _t("fake_quant", case, "x", _DT[info["dtype"]]).to(impl.dev)
    got = impl.fake_quant(x, info["kind"]).cpu()
    want = _t("fake_quant", case, "y", _DT[info["dtype"]])
    # the reference statement multiplies by torch.sign, which erases the sign of results that round to zero
    assert torch.equal(got.float(), want.float()), f"{case} values"
    nz = want != 0
    assert torch.equal(_bits(got)[nz], _bits(want)[nz]), f"{case} bits"


def _check_act_quant(impl, case):
    info = _info("fp8_act_quant", case)
    dt = _DT[info["dtype"]]
    x = _t("fp8_act_quant", case, "x", dt).to(impl.dev)
    fmt = "ue8m0" if info["round_scale"] else None
    y, s = impl.act_quant(x, info["block"], fmt)
    _same(s, _t("fp8_act_quant", case, "scale"), f"{case} scales")
    _same(y.view(torch.uint8), _t("fp8_act_quant", case, "y"), f"{case} codes")
    _same(impl.act_quant(x, info["block"], fmt, inplace=True), _t("fp8_act_quant", case, "qdq", dt), f"{case} quantize-dequantize")


def _check_fp8_to_mxfp8(impl, case):
    fam = "fp8_to_mxfp8"
    shape = _info(fam, case)["shape"]
    want_pow2 = bool(_t(fam, case, "pow2").item())
    if case.startswith("requant_"):
        codes = _t(fam, case, "codes").view(torch.float8_e4m3fn).to(impl.dev)
        tile_scale = _t(fam, case, "tile_scale").to(impl.dev)
        assert impl.scales_pow2(codes, tile_scale) == want_pow2, f"{case} power-of-two test"
        q, s = impl.fp8_block_to_mxfp8(codes, tile_scale)
        _same(s, _t(fam, case, "scale"), f"{case} E8M0 scales")
        _same(q, _t(fam, case, "q"), f"{case} codes")
        return
    f32 = _t(fam, case, "scale_f32").to(impl.dev)
    weight = torch.empty(shape, dtype=torch.uint8, device=impl.dev).view(torch.float8_e4m3fn)
    if case.startswith("pow2_test_"):
        weight = torch.empty((f32.shape[0] * 128, f32.shape[1] * 128), dtype=torch.uint8, device=impl.dev)
        assert impl.scales_pow2(weight, f32) == want_pow2, f"{case} power-of-two test"
        return
    assert impl.scales_pow2(weight, f32) == want_pow2, f"{case} power-of-two test"
    want = _t(fam, case, "expanded")
    _same(impl.expand_tile_scales(weight, f32), want, f"{case} group scales from fp32 powers of two")
    _same(impl.expand_tile_scales(weight, _t(fam, case, "scale_u8").to(impl.dev)), want, f"{case} group scales from bytes")


_CHECKS = [("fp8_to_mxfp8", _check_fp8_to_mxfp8), ("fp8_block", _check_fp8_block), ("fp8_blockwise_cast", _check_fp8_blockwise), ("fp8_dequant", _check_fp8_dequant),
           ("mxfp8", _check_mxfp8), ("mxfp4", _check_mxfp4), ("int4", _check_int4), ("nvfp4", _check_nvfp4), ("fake_quant", _check_fake_quant),
           ("fp8_act_quant", _check_act_quant)]
_PARAMS = [pytest.param(fam, fn, case, id=f"{fam}-{case}") for fam, fn in _CHECKS for case in _cases(fam)]


@pytest.mark.parametrize("family,check,case", _PARAMS)
def test_oracle_matches_golden(oracle, family, check, case):
    check(_OracleImpl(oracle), case)


@pytest.mark.gpu
@pytest.mark.parametrize("family,check,case", _PARAMS)
def test_hip_matches_golden(family, check, case):
    check(_HipImpl(), case)


@pytest.mark.parametrize("e4m3_max", [256, 448])
def test_oracle_nvfp4_global_scale_vectors(oracle, e4m3_max):
    case = f"global_scale_vectors_{e4m3_max}"
    amax, enc, dec = (_t("nvfp4", case, k) for k in ("amax", "encode", "decode"))
    for a, e, d in zip(amax.tolist(), enc.tolist(), dec.tolist()):
        assert oracle.nvfp4_global_encode_scale(a, e4m3_max) == e
        assert oracle.nvfp4_global_decode_scale(a, e4m3_max) == d


@pytest.mark.gpu
@pytest.mark.parametrize("e4m3_max", [256, 448])
def test_hip_nvfp4_global_scale_vectors(e4m3_max):
    from miles_amd.utils.nvfp4 import nvfp4_global_decode_scale_te, nvfp4_global_encode_scale_te

    case = f"global_scale_vectors_{e4m3_max}"
    amax, enc, dec = (_t("nvfp4", case, k) for k in ("amax", "encode", "decode"))
    got_e = nvfp4_global_encode_scale_te(amax.to(DEV), e4m3_max)
    got_d = nvfp4_global_decode_scale_te(amax.to(DEV), e4m3_max)
    _same(got_e, enc, "encode scales")
    _same(got_d, dec, "decode scales")
