"""Offline converters end to end on the GPU: tiny sharded checkpoints in, converted checkpoints out, every
tensor compared with the oracle.  The cross-shard / same-shard gated-pair cases restate
tests/fast-gpu/test_nvfp4_quantizer.py:286-366."""

import json

import pytest
import safetensors
import safetensors.torch
import torch

from miles_amd import workloads as W

pytestmark = pytest.mark.gpu
F8 = torch.float8_e4m3fn


def _load_all(path):
    out = {}
    for f in sorted(path.glob("*.safetensors")):
        with safetensors.safe_open(f, framework="pt", device="cpu") as h:
            for k in h.keys():
                out[k] = h.get_tensor(k)
    return out


def _bits(t):
    t = t.contiguous()
    return t.view({1: torch.uint8, 2: torch.int16, 4: torch.int32}[t.element_size()])


def _same(a, b, what):
    assert a.shape == b.shape and torch.equal(_bits(a), _bits(b)), f"{what} differs"


def _checkpoint(tmp_path, shards, config=None):
    model = tmp_path / "model"
    model.mkdir()
    (model / "config.json").write_text(json.dumps(config or {"num_hidden_layers": 2}))
    (model / "tokenizer.json").write_text("{}")
    weight_map = {}
    for i, tensors in enumerate(shards):
        name = f"model-{i:05d}-of-{len(shards):05d}.safetensors"
        safetensors.torch.save_file(tensors, model / name, metadata={"format": "pt"})
        weight_map.update({k: name for k in tensors})
    (model / "model.safetensors.index.json").write_text(json.dumps({"weight_map": weight_map, "metadata": {}}))
    return model


def _rand(shape, seed, dtype=torch.bfloat16):
    return W.gaussian_outliers(shape, std=0.02, p_outlier=0.001, gain=20.0, seed=seed, dtype=dtype)


def _dense_shards():
    a = {"model.embed_tokens.weight": _rand((64, 256), 1), "model.layers.0.input_layernorm.weight": _rand((256,), 2),
         "model.layers.0.self_attn.q_proj.weight": _rand((384, 256), 3), "model.layers.0.mlp.gate.weight": _rand((8, 256), 4),
         "model.layers.0.self_attn.q_proj.bias": _rand((384,), 5)}
    b = {"model.layers.1.mlp.down_proj.weight": _rand((256, 640), 6), "model.layers.1.mlp.experts.0.up_proj.weight": _rand((130, 256), 7),
         "lm_head.weight": _rand((64, 256), 8)}
    return [a, b]


def test_convert_fp8_block_and_back(oracle, tmp_path):
    from miles_amd.tools.convert_hf_to_fp8 import convert_fp8
    from miles_amd.tools.fp8_cast_bf16 import main as fp8_cast_bf16

    shards = _dense_shards()
    model = _checkpoint(tmp_path, shards)
    out = tmp_path / "fp8"
    convert_fp8(str(model), str(out), "block", [128, 128], max_workers=2)
    got = _load_all(out)
    src = {k: v for s in shards for k, v in s.items()}
    quantized = ["model.layers.0.self_attn.q_proj.weight", "model.layers.1.mlp.down_proj.weight",
                 "model.layers.1.mlp.experts.0.up_proj.weight"]
    for k in quantized:
        q, s = oracle.block_fp8(src[k], (128, 128))
        _same(got[k], q, k)
        _same(got[k.replace(".weight", ".weight_scale_inv")], s, k + " scale")
    for k in set(src) - set(quantized):
        _same(got[k], src[k], k)
    cfg = json.loads((out / "config.json").read_text())["quantization_config"]
    assert cfg["quant_method"] == "fp8" and cfg["weight_block_size"] == [128, 128] and cfg["fmt"] == "e4m3"
    assert set(cfg["modules_to_not_convert"]) == {"model.embed_tokens", "model.layers.0.input_layernorm", "lm_head",
                                                  "model.layers.0.mlp.gate", "model.layers.0.self_attn.q_proj.bias"}
    index = json.loads((out / "model.safetensors.index.json").read_text())
    assert set(index["weight_map"]) == set(got) and (out / "tokenizer.json").exists()
    # and back to bf16: weights whose scales sit in the same or another shard
    back = tmp_path / "bf16"
    fp8_cast_bf16(str(out), str(back))
    rt = _load_all(back)
    assert not any(k.endswith("_scale_inv") for k in rt)
    for k in quantized:
        _same(rt[k], oracle.weight_dequant(*oracle.block_fp8(src[k], (128, 128))), k + " round trip")
    assert not any(k.endswith("_scale_inv") for k in json.loads((back / "model.safetensors.index.json").read_text())["weight_map"])


@pytest.mark.parametrize("strategy", ["tensor", "channel"])
def test_convert_fp8_tensor_and_channel(oracle, tmp_path, strategy):
    from miles_amd.tools.convert_hf_to_fp8 import convert_fp8

    shards = _dense_shards()
    model = _checkpoint(tmp_path, shards)
    out = tmp_path / "fp8"
    convert_fp8(str(model), str(out), strategy, None, max_workers=1)
    got = _load_all(out)
    k = "model.layers.1.mlp.down_proj.weight"
    q, s = (oracle.tensor_fp8 if strategy == "tensor" else oracle.channel_fp8)(shards[1][k])
    _same(got[k], q, k)
    _same(got[k.replace(".weight", ".weight_scale")], s, k + " scale")


def _moe_shards():
    a, b = {}, {}
    for e in range(3):
        a[f"model.layers.0.mlp.experts.{e}.gate_proj.weight"] = _rand((96, 256), 10 + e)
        (a if e < 2 else b)[f"model.layers.0.mlp.experts.{e}.up_proj.weight"] = _rand((96, 256), 20 + e)   # expert 2: pair split over shards
        b[f"model.layers.0.mlp.experts.{e}.down_proj.weight"] = _rand((256, 96), 30 + e)
    a["model.layers.0.mlp.gate.weight"] = _rand((3, 256), 40)
    a["model.layers.0.self_attn.o_proj.weight"] = _rand((256, 256), 41)
    b["model.layers.1.mlp.experts.0.down_proj.weight"] = _rand((256, 96), 42)      # layer 1: kept in bf16 below
    b["model.layers.0.mlp.shared_experts.down_proj.weight"] = _rand((256, 96), 43)
    return [a, b]


def test_convert_nvfp4_pairs_across_shards(oracle, tmp_path):
    from miles_amd.tools.convert_hf_to_nvfp4 import convert_nvfp4

    shards = _moe_shards()
    model = _checkpoint(tmp_path, shards)
    out = tmp_path / "nvfp4"
    convert_nvfp4(str(model), str(out), device="cuda:0", num_layers_at_end_in_bf16=1)
    got = _load_all(out)
    src = {k: v for s in shards for k, v in s.items()}
    for e in range(3):
        base = f"model.layers.0.mlp.experts.{e}"
        (gq, gs, gg), (uq, us, ug) = oracle.nvfp4_quantize_1d_pair(src[base + ".gate_proj.weight"], src[base + ".up_proj.weight"])
        dq, ds, dg = oracle.nvfp4_quantize_1d(src[base + ".down_proj.weight"])
        for proj, (q, s, g) in (("gate_proj", (gq, gs, gg)), ("up_proj", (uq, us, ug)), ("down_proj", (dq, ds, dg))):
            _same(got[f"{base}.{proj}.weight"], q, f"{base}.{proj} codes")
            _same(got[f"{base}.{proj}.weight_scale"], s, f"{base}.{proj} block scales")
            _same(got[f"{base}.{proj}.weight_scale_2"], g, f"{base}.{proj} global scale")
            assert got[f"{base}.{proj}.input_scale"].item() == 1.0
        assert got[base + ".gate_proj.weight_scale_2"].item() == got[base + ".up_proj.weight_scale_2"].item()
    for k in ("model.layers.1.mlp.experts.0.down_proj.weight", "model.layers.0.mlp.shared_experts.down_proj.weight",
              "model.layers.0.self_attn.o_proj.weight", "model.layers.0.mlp.gate.weight"):
        _same(got[k], src[k], k)
    ignore = json.loads((out / "config.json").read_text())["quantization_config"]["ignore"]
    assert "model.layers.1." in ignore and "model.layers.1.mlp.experts" in ignore and "model.layers.0.self_attn.o_proj" in ignore
    hf = json.loads((out / "hf_quant_config.json").read_text())["quantization"]
    assert hf["quant_algo"] == "NVFP4" and hf["exclude_modules"] == ignore
    # the up tensor of expert 2 was written into the shard that holds it in the source
    index = json.loads((out / "model.safetensors.index.json").read_text())["weight_map"]
    assert index["model.layers.0.mlp.experts.2.up_proj.weight"] == "model-00001-of-00002.safetensors"
    assert index["model.layers.0.mlp.experts.2.gate_proj.weight"] == "model-00000-of-00002.safetensors"


def test_convert_nvfp4_stacked_expert_weight(oracle, tmp_path):
    """A checkpoint that stores its routed experts as one 3-D tensor: every matrix of the stack is quantized with its
    own global scale.  The converter works inside a deferred batch, so the stacked results must be written by the jobs
    themselves (nothing may be gathered before the batch has run)."""
    from miles_amd.tools.convert_hf_to_nvfp4 import convert_nvfp4

    stack = torch.stack([_rand((256, 96), 60 + e) * (1.0 + e) for e in range(4)])
    shards = [{"model.layers.0.mlp.experts.down_proj.weight": stack, "model.layers.0.mlp.gate.weight": _rand((4, 256), 70)}]
    model = _checkpoint(tmp_path, shards)
    out = tmp_path / "nvfp4"
    convert_nvfp4(str(model), str(out), device="cuda:0")
    got = _load_all(out)
    want = [oracle.nvfp4_quantize_1d(stack[e].contiguous()) for e in range(4)]
    base = "model.layers.0.mlp.experts.down_proj"
    _same(got[base + ".weight"], torch.stack([w[0] for w in want]), "stacked codes")
    _same(got[base + ".weight_scale"], torch.stack([w[1] for w in want]), "stacked block scales")
    _same(got[base + ".weight_scale_2"], torch.stack([w[2] for w in want]), "stacked global scales")
    assert got[base + ".weight_scale_2"].unique().numel() == 4
    assert torch.equal(got[base + ".input_scale"], torch.ones(4))


def test_convert_mxfp8_from_bf16_and_from_pow2_fp8(oracle, tmp_path):
    from miles_amd.tools.convert_hf_to_mxfp8 import convert_mxfp8

    shards = _moe_shards()
    model = _checkpoint(tmp_path, shards)
    out = tmp_path / "mx"
    convert_mxfp8(str(model), str(out), "cuda:0", num_layers_at_end_in_bf16=1, extra_high_precision_layers_hf=(".shared_experts.",))
    got = _load_all(out)
    src = {k: v for s in shards for k, v in s.items()}
    for k in (f"model.layers.0.mlp.experts.{e}.{p}.weight" for e in range(3) for p in ("gate_proj", "up_proj", "down_proj")):
        q, s = oracle.mxfp8_quantize(src[k])
        _same(got[k], q, k)
        _same(got[k.replace(".weight", ".weight_scale_inv")], s, k + " scale")
    q, s = oracle.mxfp8_quantize(src["model.layers.0.self_attn.o_proj.weight"])
    _same(got["model.layers.0.self_attn.o_proj.weight"], q, "o_proj")
    for k in ("model.layers.1.mlp.experts.0.down_proj.weight", "model.layers.0.mlp.shared_experts.down_proj.weight",
              "model.layers.0.mlp.gate.weight"):
        _same(got[k], src[k], k)
    cfg = json.loads((out / "config.json").read_text())["quantization_config"]
    assert cfg["quant_method"] == "mxfp8" and cfg["weight_block_size"] == [1, 32] and cfg["scale_fmt"] == "ue8m0"
    assert cfg["modules_to_not_convert"] == ["model.layers.0.mlp.gate", "model.layers.0.mlp.shared_experts.down_proj", "model.layers.1."]
    # FP8 source with power-of-two tile scales: codes are kept, exponents are repeated per 1x32 group
    codes = torch.randint(0, 120, (256, 384), dtype=torch.int32).to(torch.uint8).view(F8)
    tile_scale = torch.tensor([[0.5, 2.0, 1.0], [4.0, 0.25, 8.0]])
    (tmp_path / "x").mkdir()
    fp8_model = _checkpoint(tmp_path / "x", [{"model.layers.0.mlp.down_proj.weight": codes,
                                               "model.layers.0.mlp.down_proj.weight_scale_inv": tile_scale,
                                               "model.layers.0.mlp.gate.weight": codes.clone(),
                                               "model.layers.0.mlp.gate.weight_scale_inv": tile_scale.clone()}],
                            config={"num_hidden_layers": 1, "quantization_config": {
                                "quant_method": "fp8", "weight_block_size": [128, 128], "scale_fmt": "ue8m0"}})
    out2 = tmp_path / "mx2"
    convert_mxfp8(str(fp8_model), str(out2), "cuda:0")
    got2 = _load_all(out2)
    _same(got2["model.layers.0.mlp.down_proj.weight"], codes, "relabelled codes")
    want = tile_scale.view(torch.int32).bitwise_right_shift(23).to(torch.uint8).repeat_interleave(128, 0).repeat_interleave(4, 1)
    _same(got2["model.layers.0.mlp.down_proj.weight_scale_inv"], want, "relabelled exponents")
    # the router stays out of MXFP8 and is dequantized to bf16 with its tile scales
    _same(got2["model.layers.0.mlp.gate.weight"], oracle.weight_dequant(codes, tile_scale), "router dequant")
    assert "model.layers.0.mlp.gate.weight_scale_inv" not in got2


def test_convert_int4_direct(oracle, tmp_path):
    from miles_amd.tools.convert_hf_to_int4_direct import DEFAULT_IGNORE_RULES, convert_int4

    shards = _moe_shards()
    model = _checkpoint(tmp_path, shards)
    out = tmp_path / "int4"
    convert_int4(str(model), str(out), 32, True, DEFAULT_IGNORE_RULES, max_workers=2)
    got = _load_all(out)
    src = {k: v for s in shards for k, v in s.items()}
    for k, w in src.items():
        if ".experts." in k and "shared" not in k:
            p, s, _ = oracle.pack_layer(w, 32)
            _same(got[k.replace(".weight", ".weight_packed")], p, k + " packed")
            _same(got[k.replace(".weight", ".weight_scale")], s, k + " scale")
            assert got[k.replace(".weight", ".weight_shape")].tolist() == list(w.shape)
            assert k not in got
        else:
            _same(got[k], w, k)
    cfg = json.loads((out / "config.json").read_text())["quantization_config"]
    assert cfg["format"] == "pack-quantized" and cfg["config_groups"]["group_0"]["weights"]["group_size"] == 32


def test_convert_kimi_int4_to_bf16(tmp_path, oracle):
    from miles_amd.kernels.quant.int4_fake import pack_layer
    from miles_amd.tools import convert_kimi_int4_to_bf16 as tool

    cfg = {"text_config": {"hidden_size": 256, "moe_intermediate_size": 128,
                           "quantization_config": {"config_groups": {"group_0": {"weights": {"group_size": 32}}}}}}
    shard = {"model.embed_tokens.weight": _rand((64, 256), 1)}
    originals = {}
    for e in range(2):
        for proj, shape in (("gate_proj", (128, 256)), ("up_proj", (128, 256)), ("down_proj", (256, 128))):
            w = _rand(shape, 40 + 3 * e + len(proj))
            packed, scale, _ = pack_layer(w.cuda(), 32)
            base = f"model.layers.0.mlp.experts.{e}.{proj}"
            shard[f"{base}.weight_packed"] = packed.cpu()
            shard[f"{base}.weight_scale"] = scale.cpu()
            shard[f"{base}.weight_shape"] = torch.tensor(shape, dtype=torch.int32)
            originals[base] = (packed.cpu(), scale.cpu(), shape)
    # an incomplete triple and a shared expert stay as they are
    shard["model.layers.0.mlp.experts.9.up_proj.weight_packed"] = torch.zeros((4, 4), dtype=torch.int32)
    shard["model.layers.0.mlp.shared_experts.up_proj.weight_packed"] = torch.ones((4, 4), dtype=torch.int32)
    model = _checkpoint(tmp_path, [shard], cfg)
    out = tmp_path / "bf16"
    tool.main(["--model-dir", str(model), "--output-dir", str(out)])
    got = _load_all(out)
    for base, (packed, scale, shape) in originals.items():
        want = oracle.int4_unpack_dequant(packed, scale.float(), shape, 32)
        _same(got[f"{base}.weight"], want, base)
        assert f"{base}.weight_packed" not in got and f"{base}.weight_scale" not in got
    assert "model.layers.0.mlp.experts.9.up_proj.weight_packed" in got
    assert "model.layers.0.mlp.shared_experts.up_proj.weight_packed" in got
    _same(got["model.embed_tokens.weight"], shard["model.embed_tokens.weight"], "embed")
    index = json.loads((out / "model.safetensors.index.json").read_text())
    assert set(index["weight_map"]) == set(got) and (out / "tokenizer.json").exists()


def test_convert_mxfp4_to_bf16(tmp_path, oracle):
    from miles_amd.tools import convert_mxfp4_to_bf16 as tool

    cfg = {"num_hidden_layers": 1,
           "quantization_config": {"format": "mxfp4-pack-quantized",
                                   "config_groups": {"group_0": {"weights": {"group_size": 32, "type": "float", "num_bits": 4,
                                                                             "scale_dtype": "torch.uint8"}}}}}
    g = torch.Generator().manual_seed(5)
    shards = []
    for i in range(2):
        shards.append({f"model.layers.0.mlp.experts.{i}.w1.weight_packed": torch.randint(0, 256, (64, 128), dtype=torch.uint8, generator=g),
                       f"model.layers.0.mlp.experts.{i}.w1.weight_scale": torch.randint(100, 140, (64, 8), dtype=torch.uint8, generator=g),
                       f"model.layers.0.norm{i}.weight": _rand((256,), 60 + i)})
    model = _checkpoint(tmp_path, shards, cfg)
    out = tmp_path / "bf16"
    tool.main(["--model-dir", str(model), "--save-dir", str(out)])
    got = _load_all(out)
    for i, shard in enumerate(shards):
        base = f"model.layers.0.mlp.experts.{i}.w1"
        want = oracle.dequantize_mxfp4(shard[f"{base}.weight_packed"], shard[f"{base}.weight_scale"], 32)
        _same(got[f"{base}.weight"], want, base)
        assert f"{base}.weight_packed" not in got and f"{base}.weight_scale" not in got
        _same(got[f"model.layers.0.norm{i}.weight"], shard[f"model.layers.0.norm{i}.weight"], "norm")
    assert "quantization_config" not in json.loads((out / "config.json").read_text())
    index = json.loads((out / "model.safetensors.index.json").read_text())
    assert set(index["weight_map"]) == set(got)
    assert index["metadata"]["total_size"] == sum(t.numel() * t.element_size() for t in got.values())


def test_convert_mxfp4_to_fp8(tmp_path, oracle):
    from miles_amd.tools import convert_mxfp4_to_fp8 as tool

    g = torch.Generator().manual_seed(9)

    def expert(seed):
        packed = torch.randint(0, 256, (128, 128), dtype=torch.uint8, generator=g).view(torch.int8)
        scale = torch.randint(118, 126, (128, 8), dtype=torch.uint8, generator=g).view(torch.float8_e8m0fnu)
        return packed, scale

    (p0, s0), (p1, s1) = expert(0), expert(1)
    shards = [{"model.layers.0.mlp.experts.0.w1.weight": p0, "model.layers.0.mlp.experts.0.w1.scale": s0,
               "model.layers.0.mlp.experts.1.w1.weight": p1, "model.norm.weight": _rand((256,), 70)},
              {"model.layers.0.mlp.experts.1.w1.scale": s1, "lm_head.weight": _rand((64, 256), 71)}]   # scale in another shard
    model = _checkpoint(tmp_path, shards, {"expert_dtype": "fp4", "quantization_config": {"expert_dtype": "fp4", "quant_method": "fp8"}})
    out = tmp_path / "fp8"
    tool.main(str(model), str(out), "cuda")
    got = _load_all(out)
    for i, (p, s) in enumerate(((p0, s0), (p1, s1))):
        y, ts = oracle.cast_e2m1fn_to_e4m3fn(p, s)
        _same(got[f"model.layers.0.mlp.experts.{i}.w1.weight"], y, f"expert {i} codes")
        _same(got[f"model.layers.0.mlp.experts.{i}.w1.scale"], ts, f"expert {i} tile scales")
    _same(got["lm_head.weight"], shards[1]["lm_head.weight"], "lm_head")
    cfg = json.loads((out / "config.json").read_text())
    assert "expert_dtype" not in cfg and "expert_dtype" not in cfg["quantization_config"]
    index = json.loads((out / "model.safetensors.index.json").read_text())
    assert index["weight_map"]["model.layers.0.mlp.experts.1.w1.scale"] == index["weight_map"]["model.layers.0.mlp.experts.1.w1.weight"]
    assert set(index["weight_map"]) == set(got) and (out / "tokenizer.json").exists()


# ---------------------------------------------------------------------------------------------------------------------
# MiMo-V2 -> BF16 (tools/convert_mimo_v2_to_bf16.py); expectations come from torch CPU ops in tests/mimo_fixture.py
def test_mimo_dequant_mxfp4_matches_the_closed_form():
    from miles_amd.tools.convert_mimo_v2_to_bf16 import dequant_mxfp4
    from tests import mimo_fixture as MF

    g = torch.Generator().manual_seed(3)
    codes = torch.randint(0, 16, (8, 64), generator=g)
    exps = torch.randint(120, 134, (8, 2), dtype=torch.uint8, generator=g)
    want = (MF.FP4_VALUES[codes] * torch.exp2(exps.float() - 127).repeat_interleave(32, dim=1)).to(torch.bfloat16)
    got = dequant_mxfp4(MF.pack_nibbles(codes).cuda(), exps.cuda()).cpu()
    _same(got, want, "mxfp4 dequant")          # bit for bit, the sign of -0 codes included


def test_mimo_fused_qkv_scales_belong_to_their_shard():
    from miles_amd.tools.convert_mimo_v2_to_bf16 import dequant_fused_qkv
    from tests import mimo_fixture as MF

    # shards of 224 rows are not 128-aligned: each one has two scale rows of its own
    w = torch.randn(2 * 224, 256, generator=torch.Generator().manual_seed(4))
    halves = [MF.quantize_fp8_blocks(part) for part in w.chunk(2)]
    q, s = torch.cat([h[0] for h in halves]), torch.cat([h[1] for h in halves])
    assert s.shape == (4, 2)
    got = dequant_fused_qkv(q.cuda(), s.cuda(), 2).cpu()
    _same(got, torch.cat([MF.dequantize_fp8_blocks(*h) for h in halves]), "fused qkv")
    assert (got.float() - w).abs().max() < 0.07 * w.abs().max()


@pytest.mark.parametrize("layers,num_experts", [(None, None), ([1], 2)])
def test_mimo_conversion_end_to_end(tmp_path, layers, num_experts):
    from miles_amd.tools import convert_mimo_v2_to_bf16 as M
    from tests import mimo_fixture as MF

    src, dst = tmp_path / "src", tmp_path / "dst"
    src.mkdir()
    expected = MF.write(src)
    M.main(str(src), str(dst), layers, num_experts, keep_quant=False, device="cuda")
    config = json.loads((dst / "config.json").read_text())
    out = _load_all(dst)
    assert set(json.loads((dst / "model.safetensors.index.json").read_text())["weight_map"]) == set(out)
    assert "quantization_config" not in config and "attention_projection_layout" not in config
    assert (dst / "tokenizer_config.json").exists()
    assert not any(n.endswith(("weight_scale", "weight_scale_inv", "qkv_proj.weight")) for n in out)
    renumber = {old: new for new, old in enumerate(layers)} if layers else {0: 0, 1: 1}
    experts_kept = num_experts or 4
    assert config["num_hidden_layers"] == len(renumber) and config["n_routed_experts"] == experts_kept
    assert config["hybrid_layer_pattern"] == config["moe_layer_freq"] == list(renumber)
    checked = 0
    for name, want in expected.items():
        parts = name.split(".")
        layer = int(parts[2])
        if layer not in renumber or (parts[4] == "experts" and int(parts[5]) >= experts_kept):
            continue
        _same(out[".".join(["model", "layers", str(renumber[layer]), *parts[3:]])], want, name)
        checked += 1
    assert checked == (6 if 0 in renumber else 0) + 3 + 3 * experts_kept
    moe = renumber[1]
    assert sum(".experts." in n for n in out) == 3 * experts_kept
    assert out[f"model.layers.{moe}.mlp.gate.weight"].shape[0] == experts_kept
    assert out[f"model.layers.{moe}.mlp.gate.e_score_correction_bias"].dtype == torch.float32
