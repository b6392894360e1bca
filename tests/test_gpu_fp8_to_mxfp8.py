"""FP8 128x128 block-scaled sources -> MXFP8 on the GPU (tools/convert_hf_to_mxfp8.py:56-102,180-215) against the CPU
oracle: the one-pass re-quantizer, the exponent expansion of a power-of-two source, the power-of-two test, through the
Python wrappers, the batched driver and the raw C ABI, and the converter end to end with every kind of source."""

import ctypes
import json

import pytest
import safetensors
import safetensors.torch
import torch

from miles_amd import workloads as W

pytestmark = pytest.mark.gpu
F8 = torch.float8_e4m3fn
DEV = "cuda:0"


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


def _source(oracle, shape, seed, spread=1.0):
    """An FP8 block-scaled tensor as a checkpoint holds it: block_fp8 of a bf16 matrix whose rows differ in magnitude."""
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(shape, generator=g) * 0.02 * torch.exp(spread * torch.randn((shape[0], 1), generator=g))).to(torch.bfloat16)
    return oracle.block_fp8(w, (128, 128))


def _requant(codes, scale):
    from miles_amd.utils.mxfp8 import requantize_fp8_block_to_mxfp8

    return requantize_fp8_block_to_mxfp8(codes.to(DEV), scale.to(DEV))


def _check_requant(oracle, codes, scale, what):
    q, s = _requant(codes, scale)
    want_q, want_s = oracle.fp8_block_to_mxfp8(codes, scale)
    _assert_same(s, want_s, f"{what}: E8M0 scales")
    _assert_same(q, want_q, f"{what}: codes")


@pytest.mark.parametrize("shape", [(128, 256), (256, 384), (130, 288), (1, 32), (5, 96), (127, 160), (384, 2048), (200, 7168)])
def test_requantize_general_scales(oracle, shape):
    codes, scale = _source(oracle, shape, seed=sum(shape))
    _check_requant(oracle, codes, scale, f"{shape}")


def test_requantize_every_code_nan_codes_and_extreme_scales(oracle):
    g = torch.Generator().manual_seed(5)
    codes = torch.randint(0, 256, (384, 640), generator=g, dtype=torch.int32).to(torch.uint8)     # 0x7F / 0xFF (NaN) included
    codes[0:4, :] = torch.arange(256, dtype=torch.uint8).repeat(4, 3)[:, :640]
    scale = torch.exp(torch.randn((3, 5), generator=g) * 6).float()
    scale[0, 0], scale[0, 1], scale[0, 2] = 0.0, -0.0, -3.5
    scale[1, 0], scale[1, 1], scale[1, 2] = 2.0 ** -140, 2.0 ** -126, 1e-38
    scale[2, 0], scale[2, 1], scale[2, 2] = 2.0 ** 118, 2.0 ** 119, 3e38           # products up to and past FLT_MAX
    scale[2, 3], scale[2, 4] = float("inf"), float("nan")
    _check_requant(oracle, codes.view(F8), scale, "random bytes")
    clean = torch.where((codes & 0x7F) == 0x7F, torch.zeros_like(codes), codes)
    _check_requant(oracle, clean.view(F8), scale, "no NaN bytes")


def test_requantize_wide_grid_views_batches_and_unaligned_tensors(oracle):
    from miles_amd.utils.mxfp8 import requantize_fp8_block_to_mxfp8

    codes, scale = _source(oracle, (260, 416), seed=9)
    wide = torch.full((5, 7), 123.0)
    wide[:3, :4] = scale
    q, s = requantize_fp8_block_to_mxfp8(codes.to(DEV), wide.to(DEV))           # a grid larger than the weight needs
    want_q, want_s = oracle.fp8_block_to_mxfp8(codes, scale)
    _assert_same(q, want_q, "wide grid codes"), _assert_same(s, want_s, "wide grid scales")
    q, s = requantize_fp8_block_to_mxfp8(codes.to(DEV), wide.to(DEV)[:3, :4])   # the cropped view, rows 7 apart
    _assert_same(q, want_q, "grid view codes"), _assert_same(s, want_s, "grid view scales")
    # codes that start one byte into an allocation take the byte-wise kernel
    flat = torch.zeros(codes.numel() + 16, dtype=torch.uint8, device=DEV)
    flat[1:1 + codes.numel()] = codes.view(torch.uint8).flatten().to(DEV)
    q, s = requantize_fp8_block_to_mxfp8(flat[1:1 + codes.numel()].view(260, 416).view(F8), scale.to(DEV))
    _assert_same(q, want_q, "unaligned codes"), _assert_same(s, want_s, "unaligned scales")
    # stacked experts [E, N, K] with a scale grid [E, nt, kt]
    pairs = [_source(oracle, (130, 160), seed=20 + e) for e in range(3)]
    stack_c, stack_s = torch.stack([c for c, _ in pairs]), torch.stack([s for _, s in pairs])
    q, s = requantize_fp8_block_to_mxfp8(stack_c.to(DEV), stack_s.to(DEV))
    for e, (c, sc) in enumerate(pairs):
        want_q, want_s = oracle.fp8_block_to_mxfp8(c, sc)
        _assert_same(q[e], want_q, f"expert {e} codes"), _assert_same(s[e], want_s, f"expert {e} scales")
    with pytest.raises(ValueError, match="divisible by 32"):
        requantize_fp8_block_to_mxfp8(torch.zeros((4, 48), dtype=torch.uint8, device=DEV).view(F8), torch.ones((1, 1), device=DEV))
    q, s = requantize_fp8_block_to_mxfp8(torch.zeros((0, 64), dtype=torch.uint8, device=DEV).view(F8), torch.ones((0, 1), device=DEV))
    assert q.shape == (0, 64) and s.shape == (0, 2)


def test_requantize_job_lists_share_launches(oracle):
    """Many tensors recorded inside one deferred block: grouped launches of up to 64, sizes mixed."""
    from miles_amd import launch
    from miles_amd.utils.mxfp8 import expand_tile_scales_e8m0, requantize_fp8_block_to_mxfp8

    shapes = [(128, 256)] * 70 + [(256, 384), (130, 288), (5, 96), (384, 2048), (128, 256)]
    sources = [_source(oracle, shape, seed=100 + i) for i, shape in enumerate(shapes)]
    device = [(c.to(DEV), s.to(DEV)) for c, s in sources]
    with launch.deferred():
        outs = [requantize_fp8_block_to_mxfp8(c, s) for c, s in device]
        pow2 = expand_tile_scales_e8m0(device[0][0], torch.full((1, 2), 0.25, device=DEV))
    for i, ((c, s), (q, e)) in enumerate(zip(sources, outs)):
        want_q, want_e = oracle.fp8_block_to_mxfp8(c, s)
        _assert_same(q, want_q, f"job {i} codes"), _assert_same(e, want_e, f"job {i} scales")
    assert pow2.unique().tolist() == [125]


@pytest.mark.parametrize("shape", [(2048, 7168), (7168, 2048)])
def test_requantize_full_size_expert(oracle, shape):
    codes, scale = _source(oracle, shape, seed=77)
    _check_requant(oracle, codes, scale, f"{shape}")


@pytest.mark.parametrize("shape", [(130, 288), (256, 512), (1, 32), (129, 160), (2, 140, 160)])
def test_expand_tile_scales_and_pow2_test(oracle, shape):
    from miles_amd.utils.mxfp8 import expand_tile_scales_e8m0, exponent_bytes_to_fp32, fp8_tile_scales_pow2

    g = torch.Generator().manual_seed(3)
    n, k = shape[-2:]
    grid = (*shape[:-2], -(-n // 128), -(-k // 128))
    u8 = torch.randint(0, 256, grid, generator=g, dtype=torch.int32).to(torch.uint8)
    f32 = (u8.to(torch.int32) << 23).view(torch.float32)
    weight = torch.zeros(shape, dtype=torch.uint8, device=DEV).view(F8)
    mats_w = weight.cpu().reshape(-1, n, k)
    want = torch.stack([oracle.expand_tile_scales_e8m0(w, s) for w, s in zip(mats_w, u8.reshape(-1, *grid[-2:]))]).reshape(*shape[:-1], k // 32)
    _assert_same(expand_tile_scales_e8m0(weight, u8.to(DEV)), want, "from bytes")
    _assert_same(expand_tile_scales_e8m0(weight, f32.to(DEV)), want, "from fp32 powers of two")
    _assert_same(exponent_bytes_to_fp32(u8.to(DEV)), f32, "bytes as fp32")
    assert fp8_tile_scales_pow2([(weight, f32.to(DEV))]) == [True]
    for bad in (-1.0, 1.5, 1.0000001, float("nan")):
        broken = f32.clone()
        broken.view(-1)[broken.numel() // 2] = bad
        assert fp8_tile_scales_pow2([(weight, broken.to(DEV)), (weight, f32.to(DEV))]) == [False, True], bad
    # only the part of a larger grid that the weight uses counts
    wide = torch.full((*grid[:-2], grid[-2] + 1, grid[-1] + 2), 1.5)
    wide[..., :grid[-2], :grid[-1]] = f32
    assert fp8_tile_scales_pow2([(weight, wide.to(DEV))]) == [True]
    _assert_same(expand_tile_scales_e8m0(weight, wide.to(DEV)), want, "from a wider grid")


def test_c_abi_entry_points(oracle):
    from miles_amd import _lib

    lib = _lib.load()
    codes, scale = _source(oracle, (256, 384), seed=1)
    x, s = codes.to(DEV), scale.to(DEV)
    q = torch.empty((256, 384), dtype=torch.uint8, device=DEV)
    e = torch.empty((256, 12), dtype=torch.uint8, device=DEV)
    assert lib.mq_fp8_block_to_mxfp8(x.data_ptr(), s.data_ptr(), 3, q.data_ptr(), e.data_ptr(), 256, 384, None) == 0
    want_q, want_e = oracle.fp8_block_to_mxfp8(codes, scale)
    _assert_same(q, want_q, "C ABI codes"), _assert_same(e, want_e, "C ABI scales")
    assert lib.mq_fp8_block_to_mxfp8(x.data_ptr(), s.data_ptr(), 3, q.data_ptr(), e.data_ptr(), 256, 48, None) == -1
    assert b"divisible by 32" in lib.mq_last_error()
    assert lib.mq_fp8_block_to_mxfp8(x.data_ptr(), s.data_ptr(), 2, q.data_ptr(), e.data_ptr(), 256, 384, None) == -1   # rows of the grid overlap
    assert lib.mq_fp8_block_to_mxfp8(None, s.data_ptr(), 3, q.data_ptr(), e.data_ptr(), 256, 384, None) == -1
    flag = torch.full((2,), 7, dtype=torch.int32, device=DEV)
    pow2 = torch.tensor([[0.5, 2.0, 1.0], [4.0, 0.25, 8.0]], device=DEV)
    assert lib.mq_fp8_scales_pow2_flag(pow2.data_ptr(), 2, 3, 3, flag.data_ptr(), None) == 0
    assert lib.mq_fp8_scales_pow2_flag(s.data_ptr(), 2, 3, 3, flag.data_ptr() + 4, None) == 0
    assert flag.tolist() == [1, 0]
    out = torch.empty((256, 12), dtype=torch.uint8, device=DEV)
    assert lib.mq_e8m0_expand_tile_scales(pow2.data_ptr(), 1, 3, out.data_ptr(), 256, 12, None) == 0
    _assert_same(out, oracle.expand_tile_scales_e8m0(codes, pow2.cpu()), "C ABI expansion")
    assert lib.mq_e8m0_expand_tile_scales(pow2.data_ptr(), 1, 2, out.data_ptr(), 256, 12, None) == -1
    one = (_lib.Job * 1)(_lib.Job(_lib.JOB_FP8_TO_MXFP8, 0, x.data_ptr(), q.data_ptr(), e.data_ptr(), None, None, 256, 384, 3, 0, 0, 0, 0))
    assert lib.mq_run_jobs(one, 1, None) == -1 and b"tile scales" in lib.mq_last_error()
    assert ctypes.sizeof(_lib.Job) == 96


# ---- the converter, end to end -------------------------------------------------------------------------------------
def _checkpoint(root, shards, config):
    root.mkdir(parents=True)
    (root / "config.json").write_text(json.dumps(config))
    weight_map = {}
    for i, tensors in enumerate(shards):
        name = f"model-{i:05d}-of-{len(shards):05d}.safetensors"
        safetensors.torch.save_file(tensors, root / name, metadata={"format": "pt"})
        weight_map.update({k: name for k in tensors})
    (root / "model.safetensors.index.json").write_text(json.dumps({"weight_map": weight_map, "metadata": {}}))
    return root


def _load_all(path):
    out = {}
    for f in sorted(path.glob("*.safetensors")):
        with safetensors.safe_open(f, framework="pt", device="cpu") as h:
            for k in h.keys():
                out[k] = h.get_tensor(k)
    return out


def test_convert_mxfp8_from_every_kind_of_fp8_source(oracle, tmp_path):
    """One checkpoint holding a source of each kind: general fp32 scales (re-quantized), fp32 powers of two and stored
    exponent bytes (relabelled), a scale tensor that lives in another shard, a grid larger than its weight needs, stacked
    experts, and modules that stay in bf16 (dequantized with fp32 and with byte scales)."""
    from miles_amd.tools.convert_hf_to_mxfp8 import convert_mxfp8

    g = torch.Generator().manual_seed(8)
    general_c, general_s = _source(oracle, (256, 384), seed=11)
    other_c, other_s = _source(oracle, (130, 288), seed=12)
    wide = torch.full((3, 4), 9.0)
    wide[:2, :3] = other_s
    pow2_c = torch.randint(0, 127, (256, 384), generator=g, dtype=torch.int32).to(torch.uint8).view(F8)
    pow2_s = torch.tensor([[0.5, 2.0, 1.0], [4.0, 0.25, 8.0]])
    bytes_c = torch.randint(0, 127, (140, 160), generator=g, dtype=torch.int32).to(torch.uint8).view(F8)
    bytes_s = torch.tensor([[120, 131], [127, 118]], dtype=torch.uint8)
    experts = [_source(oracle, (130, 160), seed=30 + e) for e in range(2)]
    stack_c, stack_s = torch.stack([c for c, _ in experts]), torch.stack([s for _, s in experts])
    router_c, router_s = _source(oracle, (8, 256), seed=13)
    p = "model.layers.0."
    shard0 = {p + "self_attn.q_proj.weight": general_c, p + "self_attn.q_proj.weight_scale_inv": general_s,
              p + "self_attn.o_proj.weight": other_c,                     # its scales are in the other shard
              p + "mlp.down_proj.weight": pow2_c, p + "mlp.down_proj.weight_scale_inv": pow2_s,
              p + "mlp.gate.weight": router_c, p + "mlp.gate.weight_scale_inv": router_s,
              p + "input_layernorm.weight": torch.ones(256, dtype=torch.bfloat16)}
    shard1 = {p + "self_attn.o_proj.weight_scale_inv": wide,
              p + "mlp.up_proj.weight": bytes_c, p + "mlp.up_proj.weight_scale_inv": bytes_s,
              p + "mlp.experts.w13.weight": stack_c, p + "mlp.experts.w13.weight_scale_inv": stack_s,
              p + "mlp.shared_experts.up_proj.weight": bytes_c.clone(), p + "mlp.shared_experts.up_proj.weight_scale_inv": bytes_s.clone(),
              p + "self_attn.k_proj.weight": W.gaussian_outliers((64, 256), std=0.02, p_outlier=0.001, gain=20.0, seed=3)}
    model = _checkpoint(tmp_path / "src", [shard0, shard1], {"num_hidden_layers": 1, "quantization_config": {
        "quant_method": "fp8", "weight_block_size": [128, 128], "scale_fmt": "ue8m0"}})
    out = tmp_path / "mx"
    convert_mxfp8(str(model), str(out), "cuda:0", extra_high_precision_layers_hf=(".shared_experts.",))
    got = _load_all(out)

    def expect_requant(key, codes, scale):
        q, s = oracle.fp8_block_to_mxfp8(codes, scale)
        _assert_same(got[key], q, key), _assert_same(got[key + "_scale_inv"], s, key + " scales")

    expect_requant(p + "self_attn.q_proj.weight", general_c, general_s)
    expect_requant(p + "self_attn.o_proj.weight", other_c, other_s)
    for e, (c, s) in enumerate(experts):
        q, sc = oracle.fp8_block_to_mxfp8(c, s)
        _assert_same(got[p + "mlp.experts.w13.weight"][e], q, f"expert {e}")
        _assert_same(got[p + "mlp.experts.w13.weight_scale_inv"][e], sc, f"expert {e} scales")
    _assert_same(got[p + "mlp.down_proj.weight"], pow2_c, "fp32 powers of two: codes kept")
    _assert_same(got[p + "mlp.down_proj.weight_scale_inv"], oracle.expand_tile_scales_e8m0(pow2_c, pow2_s), "fp32 powers of two: exponents")
    _assert_same(got[p + "mlp.up_proj.weight"], bytes_c, "stored bytes: codes kept")
    _assert_same(got[p + "mlp.up_proj.weight_scale_inv"], oracle.expand_tile_scales_e8m0(bytes_c, bytes_s), "stored bytes: exponents")
    _assert_same(got[p + "mlp.gate.weight"], oracle.weight_dequant(router_c, router_s), "router to bf16")
    bytes_f32 = (bytes_s.to(torch.int32) << 23).view(torch.float32)
    _assert_same(got[p + "mlp.shared_experts.up_proj.weight"], oracle.weight_dequant(bytes_c, bytes_f32), "byte-scaled module to bf16")
    q, s = oracle.mxfp8_quantize(shard1[p + "self_attn.k_proj.weight"])
    _assert_same(got[p + "self_attn.k_proj.weight"], q, "bf16 tensor of an FP8 checkpoint")
    _assert_same(got[p + "self_attn.k_proj.weight_scale_inv"], s, "its scales")
    assert p + "mlp.gate.weight_scale_inv" not in got and p + "mlp.shared_experts.up_proj.weight_scale_inv" not in got
    cfg = json.loads((out / "config.json").read_text())["quantization_config"]
    assert cfg["quant_method"] == "mxfp8" and cfg["modules_to_not_convert"] == [
        "model.layers.0.input_layernorm", "model.layers.0.mlp.gate", "model.layers.0.mlp.shared_experts.up_proj"]
    index = json.loads((out / "model.safetensors.index.json").read_text())
    assert index["metadata"]["total_size"] == sum(t.numel() * t.element_size() for t in got.values())
