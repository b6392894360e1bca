"""Writes the golden fixtures in this directory:  python tests/golden/make_fixtures.py

Every expected output is produced by PyTorch's CPU kernels running the reference's op chain
(tests/golden/torch_chains.py) on seeded inputs -- never by the C oracle and never by the HIP library -- so the
files are an independent third party for both.  Inputs reuse the reference's own test generators:
shape list and `random / boundary / zeros / maxes` patterns of tests/fast-gpu/test_mxfp8_quantizer.py:26-59 and
tests/fast-gpu/test_nvfp4_quantizer.py:43-76, the global-scale vectors of :108-143 and the MXFP4 golden bytes of
tests/fast/backends/megatron_utils/test_quantizer_mxfp4.py:6-16.

One compressed .npz per quantizer (arrays only, loadable with allow_pickle=False; bf16 / fp16 / fp8 tensors are
stored as their raw uint16 / uint8 bit patterns) plus manifest.json naming every case, its generator and the
chain that produced it.
"""

import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from miles_amd import workloads as W  # noqa: E402
from tests.golden import torch_chains as T  # noqa: E402

SHAPES = [(1, 64), (3, 128), (16, 64), (64, 128), (128, 64), (256, 128), (128, 1024)]
_BITS = {torch.bfloat16: torch.int16, torch.float16: torch.int16, torch.float8_e4m3fn: torch.uint8}


def raw(t: torch.Tensor) -> np.ndarray:
    """Bit pattern of a tensor as a numpy array (uint16 for bf16/fp16, uint8 for fp8)."""
    t = t.contiguous()
    if t.dtype in _BITS:
        t = t.view(_BITS[t.dtype])
    a = t.numpy()
    return a.view(np.uint16) if a.dtype == np.int16 else a


class Family:
    def __init__(self, name: str, chain: str, pinned: str):
        self.name, self.arrays, self.cases = name, {}, []
        self.meta = {"file": f"{name}.npz", "chain": chain, "pinned": pinned}

    def add(self, case: str, info: dict, **tensors):
        for key, t in tensors.items():
            self.arrays[f"{case}.{key}"] = raw(t) if isinstance(t, torch.Tensor) else np.asarray(t)
        self.cases.append({"case": case, **info})

    def save(self) -> dict:
        np.savez_compressed(os.path.join(HERE, f"{self.name}.npz"), **self.arrays)
        return {**self.meta, "cases": self.cases}


def fp8_block() -> dict:
    fam = Family("fp8_block", "torch_block_fp8 = tools/convert_hf_to_fp8.py:39-70",
                 "torch CPU kernels running the reference's op chain")
    for shape in SHAPES + [(130, 257)]:
        for kind in W.PATTERNS:
            w = W.reference_pattern(kind, shape, spread=512.0, amplitude=16.0)
            q, s = T.torch_block_fp8(w, (128, 128))
            fam.add(f"{shape[0]}x{shape[1]}_{kind}", {"shape": list(shape), "pattern": kind, "dtype": "bf16", "block": [128, 128]},
                    w=w, q=q, scale=s)
    gate = W.gaussian_outliers((9728, 2560), std=0.02, p_outlier=0.001, gain=20.0, seed=1001)[:256, :384].contiguous()
    gate[128:256, 128:256] = 0                           # the all-zero tile (1, 1) of the first config
    q, s = T.torch_block_fp8(gate, (128, 128))
    fam.add("c1_gate_slice_zero_tile", {"shape": [256, 384], "pattern": "c1 generator, tile (1,1) zero", "dtype": "bf16",
                                        "block": [128, 128]}, w=gate, q=q, scale=s)
    w = W.gaussian_outliers((96, 160), std=0.02, p_outlier=0.001, gain=20.0, seed=77, dtype=torch.float16)
    q, s = T.torch_block_fp8(w, (64, 32))
    fam.add("96x160_fp16_block64x32", {"shape": [96, 160], "pattern": "gaussian_outliers seed 77", "dtype": "fp16",
                                       "block": [64, 32]}, w=w, q=q, scale=s)
    return fam.save()


def fp8_blockwise() -> dict:
    fam = Family("fp8_blockwise_cast", "torch_fp8_blockwise_cast = miles/kernels/quant/fp8_blockwise.py:43-58, IEEE division",
                 "closed form; the reference's Triton device division is unpinned")
    for shape in SHAPES + [(130, 257)]:
        for kind in W.PATTERNS:
            x = W.reference_pattern(kind, shape, spread=512.0, amplitude=16.0)
            y, s = T.torch_fp8_blockwise_cast(x)
            fam.add(f"{shape[0]}x{shape[1]}_{kind}", {"shape": list(shape), "pattern": kind, "dtype": "bf16"}, x=x, y=y, scale=s)
    return fam.save()


def fp8_dequant() -> dict:
    fam = Family("fp8_dequant", "torch_dequant_fp8_block = tools/fp8_cast_bf16.py:15-40 = tools/convert_mimo_v2_to_bf16.py:44-47",
                 "torch CPU kernels running the reference's op chain")
    g = torch.Generator().manual_seed(21)
    codes = torch.arange(256, dtype=torch.uint8).repeat(300, 2)[:, :400].contiguous()
    codes = torch.where((codes & 0x7F) == 0x7F, torch.zeros_like(codes), codes)     # NaN codes are checked by property
    s = torch.exp(torch.randn((3, 4), generator=g) * 4).float()
    fam.add("all_codes_300x400", {"shape": [300, 400], "block": 128}, q=codes, scale=s,
            y=T.torch_dequant_fp8_block(codes.view(T.F8), s))
    w = W.gaussian_outliers((256, 384), std=0.02, p_outlier=0.001, gain=20.0, seed=78)
    q, s = T.torch_block_fp8(w, (128, 128))
    fam.add("round_trip_256x384", {"shape": [256, 384], "block": 128}, q=q, scale=s, y=T.torch_dequant_fp8_block(q, s))
    return fam.save()


def mxfp8() -> dict:
    fam = Family("mxfp8", "torch_mxfp8 = OCP-MX closed form; layout miles/utils/mxfp8.py:51-78",
                 "closed form; parity unpinned against Transformer Engine")
    for shape in SHAPES:
        for kind in W.PATTERNS:
            w = W.reference_pattern(kind, shape, spread=512.0, amplitude=16.0)
            q, s = T.torch_mxfp8(w)
            fam.add(f"{shape[0]}x{shape[1]}_{kind}", {"shape": list(shape), "pattern": kind, "dtype": "bf16"}, w=w, q=q, scale=s)
    w = W.student_t_rows((96, 2048), std=0.02, seed=3001)
    q, s = T.torch_mxfp8(w)
    fam.add("c3_student_t_96x2048", {"shape": [96, 2048], "pattern": "student_t_rows seed 3001", "dtype": "bf16"}, w=w, q=q, scale=s)
    return fam.save()


def mxfp4() -> dict:
    fam = Family("mxfp4", "torch_quantize_mxfp4 / torch_dequantize_mxfp4 = miles/utils/mxfp4.py:11-59",
                 "torch CPU kernels running the reference's op chain + the reference's golden bytes")
    for shape, G, dt in [((16, 64), 32, torch.bfloat16), ((64, 64), 32, torch.bfloat16), ((8, 2048), 32, torch.bfloat16),
                         ((4, 64), 16, torch.float16), ((5, 24), 4, torch.float32)]:
        w = W.student_t_rows(shape, std=0.02, seed=6001).to(dt)
        w[0, :G] = 0
        w[1, :4] = torch.tensor([0.75, 1.75, 3.5, -0.0]).to(dt)
        p, s = T.torch_quantize_mxfp4(w, G)
        fam.add(f"quant_{shape[0]}x{shape[1]}_g{G}_{str(dt).split('.')[-1]}",
                {"shape": list(shape), "group": G, "dtype": str(dt).split(".")[-1]}, w=w, packed=p, scale=s)
    packed = torch.tensor([[0x10, 0x32, 0x54, 0x76]], dtype=torch.uint8)
    scales = torch.tensor([127, 128], dtype=torch.uint8)
    fam.add("dequant_reference_golden", {"group": 4, "source": "tests/fast/backends/megatron_utils/test_quantizer_mxfp4.py:6-16"},
            packed=packed, scale=scales, y=torch.tensor([[0.0, 0.5, 1.0, 1.5, 4.0, 6.0, 8.0, 12.0]], dtype=torch.bfloat16))
    packed = torch.arange(256, dtype=torch.uint8).repeat(255, 1)
    scales = torch.arange(255, dtype=torch.uint8).repeat_interleave(16)
    fam.add("dequant_all_bytes_all_scales", {"group": 32}, packed=packed, scale=scales,
            y=T.torch_dequantize_mxfp4(packed, scales, 32))
    return fam.save()


def int4() -> dict:
    fam = Family("int4", "torch_fake_int4_{sym,asym} = fake_int4_quant_cuda.cu:159-259; torch_pack_layer_*_python_half = "
                         "quantizer_compressed_tensors.py:137-265",
                 "torch CPU kernels running the reference's op chain (the .cu half as fp32 tensor ops)")
    for shape, G in [((8, 128), 128), ((16, 256), 128), ((64, 1024), 128), ((16, 256), 32)]:
        w = W.gaussian_outliers(shape, std=0.015, p_outlier=0.0005, gain=30.0, seed=4001)
        w[0] = 0
        w[1] = w[1].abs() + 0.25
        w[2] = -w[2].abs() - 0.25
        w[3, :G] = 3e-6
        out, scale = T.torch_fake_int4_sym(w, G)
        packed, pscale = T.torch_pack_layer_python_half(out, scale, G)
        fam.add(f"sym_{shape[0]}x{shape[1]}_g{G}", {"shape": list(shape), "group": G, "sym": True, "dtype": "bf16"},
                w=w, fake_out=out, fake_scale=scale, packed=packed, scale=pscale)
        out, scale, zero = T.torch_fake_int4_asym(w, G)
        packed, pscale, pzp = T.torch_pack_layer_asym_python_half(out, scale, zero, G)
        fam.add(f"asym_{shape[0]}x{shape[1]}_g{G}", {"shape": list(shape), "group": G, "sym": False, "dtype": "bf16"},
                w=w, fake_out=out, fake_scale=scale, fake_zero=zero, packed=packed, scale=pscale, packed_zp=pzp)
    return fam.save()


def nvfp4() -> dict:
    fam = Family("nvfp4", "torch_nvfp4 = block arithmetic of miles/kernels/quant/nvfp4_qdq.py:716-743,859-889; global scale "
                          "miles/utils/nvfp4.py:19-39",
                 "pinned by the in-tree restatement's source, not by Transformer Engine vectors; global-scale vectors are "
                 "the reference's (tests/fast-gpu/test_nvfp4_quantizer.py:108-143)")
    for shape in SHAPES + [(1, 16), (3, 48), (31, 128)]:
        for kind in ["random", "boundary", "zeros", "signed_zeros", "maxes"]:
            w = W.reference_pattern(kind, shape, spread=12.0)
            q, s = T.torch_nvfp4(w)
            amax = w.float().abs().max()
            enc = torch.div(2688.0, amax).clamp_max(torch.finfo(torch.float32).max)
            enc = torch.where(enc == 0.0, 1.0, enc)
            fam.add(f"{shape[0]}x{shape[1]}_{kind}", {"shape": list(shape), "pattern": kind, "dtype": "bf16"},
                    w=w, q=q, block_scale=s, global_scale=torch.div(1.0, enc).reshape(1))
    gate = W.reference_pattern("random", (16, 64), spread=12.0, seed=1)
    up = 3 * W.reference_pattern("random", (24, 64), spread=12.0, seed=2)
    amax = torch.cat((gate, up)).float().abs().max()
    gq, gs = T.torch_nvfp4(gate, amax)
    uq, us = T.torch_nvfp4(up, amax)
    fam.add("pair_16x64_24x64", {"pattern": "gate/up pair sharing one amax"}, gate=gate, up=up, gate_q=gq, gate_scale=gs,
            up_q=uq, up_scale=us, global_scale=(amax / 2688.0).reshape(1))
    for e4m3_max in (256, 448):
        values = torch.tensor([0.0, 1.0, 3.5, torch.finfo(torch.float32).tiny, torch.finfo(torch.float32).max,
                               float("inf"), -float("inf")], dtype=torch.float32)
        expected = torch.div(torch.tensor(float(e4m3_max)) * torch.tensor(6.0), values)
        expected = torch.min(expected, torch.tensor(torch.finfo(torch.float32).max))
        expected = torch.where(expected == 0.0, torch.ones_like(expected), expected)
        fam.add(f"global_scale_vectors_{e4m3_max}", {"e4m3_max": e4m3_max}, amax=values, encode=expected,
                decode=torch.div(1.0, expected))
    return fam.save()


def fake_quant() -> dict:
    fam = Family("fake_quant", "torch_fake_quant_reference = the torch statement of tests/fast-gpu/kernels/quant/test_fake_quant.py:24-49",
                 "the reference's own test statement, run by torch CPU kernels (zero signs compared by value)")
    for dt in (torch.bfloat16, torch.float32):
        g = torch.Generator().manual_seed(0)
        x = (torch.randn(3, 8, 512, generator=g) * torch.logspace(-3, 3, 512)).to(dt)
        x[0, 0, :32] = 0
        x[1, 1, :8] = torch.tensor([448.0, -448.0, 6.0, -6.0, 3.5, 2.5, 0.75, 1.25]).to(dt)
        for kind in ("fp8", "fp4", "compressed_kv"):
            fam.add(f"{kind}_{str(dt).split('.')[-1]}", {"kind": kind, "dtype": str(dt).split(".")[-1], "shape": [3, 8, 512]},
                    x=x, y=T.torch_fake_quant_reference(x, kind))
    return fam.save()


def fp8_act_quant() -> dict:
    fam = Family("fp8_act_quant", "torch_act_quant = miles/kernels/quant/fp8_act_quant.py:49-137 as torch CPU ops",
                 "fp32 division, clamp and float8_e4m3fn cast of torch's CPU kernels (the device kernel of the reference is "
                 "TileLang; parity with it is unpinned)")
    for dt in (torch.bfloat16, torch.float32):
        g = torch.Generator().manual_seed(11)
        x = (torch.randn(6, 512, generator=g) * torch.logspace(-6, 4, 512)).to(dt)
        x[0, :128] = 0
        x[1, :4] = torch.tensor([448.0, -448.0, -0.0, 1e-6]).to(dt)
        x[2, :128] = -0.0
        name = str(dt).split(".")[-1]
        for block in (64, 128):
            for round_scale in (False, True):
                y, s = T.torch_act_quant(x, block, round_scale, False)
                qdq, _ = T.torch_act_quant(x, block, round_scale, True)
                fam.add(f"b{block}_{'pow2' if round_scale else 'plain'}_{name}",
                        {"block": block, "round_scale": round_scale, "dtype": name, "shape": [6, 512]},
                        x=x, y=y, scale=s, qdq=qdq)
    return fam.save()


def fp8_to_mxfp8() -> dict:
    fam = Family("fp8_to_mxfp8", "torch_fp8_block_to_mxfp8 / torch_source_fp8_to_mxfp8_scale_u8 / torch_scales_pow2 = "
                                 "tools/convert_hf_to_mxfp8.py:56-102,180-195 (block_quant_dequant is SGLang's: repeat, crop, "
                                 "one fp32 multiply)",
                 "torch CPU kernels running the reference's op chain; MXFP8 arithmetic as in the mxfp8 family (parity "
                 "unpinned against Transformer Engine and SGLang)")
    g = torch.Generator().manual_seed(31)
    for shape in [(128, 256), (256, 384), (130, 288), (64, 96), (3, 2, 130, 160)]:
        n, k = shape[-2:]
        w = (torch.randn(shape, generator=g) * 0.02 * torch.exp(torch.randn(shape[:-1] + (1,), generator=g))).to(torch.bfloat16)
        flat = w.reshape(-1, n, k)
        pairs = [T.torch_block_fp8(m, (128, 128)) for m in flat]
        codes = torch.stack([q for q, _ in pairs]).reshape(shape)
        scale = torch.stack([s for _, s in pairs]).reshape(*shape[:-2], -(-n // 128), -(-k // 128))
        q, s = T.torch_fp8_block_to_mxfp8(codes, scale)
        name = "x".join(map(str, shape))
        fam.add(f"requant_{name}_amax_scales", {"shape": list(shape), "scales": "amax / 448 of a bf16 tensor"},
                codes=codes, tile_scale=scale, q=q, scale=s, pow2=np.asarray([int(T.torch_scales_pow2(scale))]))
    # every code except the two NaN bytes, scales over forty binades (fp32-subnormal products included), a grid larger
    # than the weight needs (the reference crops it)
    codes = torch.arange(256, dtype=torch.uint8).repeat(260, 2)[:, :416].contiguous()
    codes = torch.where((codes & 0x7F) == 0x7F, torch.zeros_like(codes), codes)
    scale = torch.exp(torch.randn((4, 5), generator=g) * 9).float()
    scale[0, 1], scale[1, 0], scale[2, 3] = 0.0, -scale[1, 0], 2.0 ** -140
    q, s = T.torch_fp8_block_to_mxfp8(codes.view(T.F8), scale)
    fam.add("requant_all_codes_260x416_wide_grid", {"shape": [260, 416], "scales": "lognormal, zero, negative, subnormal; grid 4x5"},
            codes=codes, tile_scale=scale, q=q, scale=s, pow2=np.asarray([0]))
    # power-of-two sources: the codes stay, the exponent bytes are repeated per 1x32 group
    for shape in [(130, 288), (256, 512), (2, 140, 160)]:
        n, k = shape[-2:]
        grid = (*shape[:-2], -(-n // 128), -(-k // 128))
        exps = torch.randint(100, 140, grid, generator=g)
        f32 = torch.ldexp(torch.ones(grid), exps - 127).float()
        u8 = exps.to(torch.uint8)
        name = "x".join(map(str, shape))
        fam.add(f"relabel_{name}", {"shape": list(shape)}, scale_f32=f32, scale_u8=u8,
                expanded=T.torch_source_fp8_to_mxfp8_scale_u8(shape, u8),
                bytes_from_f32=T.torch_source_scale_bytes(f32), pow2=np.asarray([int(T.torch_scales_pow2(f32))]))
    for label, value in (("negative_pow2", -0.5), ("mantissa_bit", 1.0000001), ("zero", 0.0)):
        f32 = torch.ldexp(torch.ones((2, 3)), torch.randint(-20, 5, (2, 3), generator=g)).float()
        f32[1, 2] = value
        fam.add(f"pow2_test_{label}", {"shape": [2, 3]}, scale_f32=f32, pow2=np.asarray([int(T.torch_scales_pow2(f32))]))
    return fam.save()


FAMILIES = (fp8_block, fp8_blockwise, fp8_dequant, mxfp8, mxfp4, int4, nvfp4, fake_quant, fp8_act_quant, fp8_to_mxfp8)


def main() -> None:
    """All families, or only those named on the command line (their entries replace the manifest's)."""
    wanted = set(sys.argv[1:])
    path = os.path.join(HERE, "manifest.json")
    if wanted:
        with open(path) as f:
            manifest = json.load(f)
        fresh = {fam["file"]: fam for fam in (f() for f in FAMILIES if f.__name__ in wanted)}
        kept = [fresh.pop(fam["file"], fam) for fam in manifest["families"]]
        manifest["families"] = kept + list(fresh.values())
    else:
        manifest = {"generator": "tests/golden/make_fixtures.py", "torch": torch.__version__,
                    "families": [f() for f in FAMILIES]}
    with open(path, "w") as f:
        json.dump(manifest, f, indent=1)
    total = sum(os.path.getsize(os.path.join(HERE, fam["file"])) for fam in manifest["families"])
    print(f"wrote {len(manifest['families'])} fixture files, {total / 1e6:.2f} MB, "
          f"{sum(len(fam['cases']) for fam in manifest['families'])} cases")


if __name__ == "__main__":
    main()
