"""Converter shells on the CPU: name scopes, config / index emitters, scale relabelling.  Cases with reference
counterparts restate tests/fast-gpu/test_nvfp4_quantizer.py:233-283 (HF name scope, compact MoE prefixes)."""

import json

import pytest
import safetensors.torch
import torch

from miles_amd.tools import _checkpoint as ckpt
from miles_amd.tools import convert_hf_to_fp8 as FP8
from miles_amd.tools import convert_hf_to_int4_direct as INT4
from miles_amd.tools import convert_hf_to_mxfp8 as MX
from miles_amd.tools import convert_hf_to_nvfp4 as NV


def test_fp8_name_filter_matches_the_reference_list():
    keep = ["model.layers.0.self_attn.q_proj.weight", "model.layers.3.mlp.experts.7.down_proj.weight",
            "model.layers.0.mlp.shared_experts.up_proj.weight"]
    skip = ["model.embed_tokens.weight", "model.norm.weight", "lm_head.weight", "model.layers.0.input_layernorm.weight",
            "model.layers.0.mlp.gate.weight", "model.layers.0.mlp.router.weight", "model.layers.0.self_attn.q_proj.bias",
            "model.layers.61.eh_proj.weight", "vision_tower.blocks.0.attn.weight", "model.layers.0.self_attn.indexer.weights_proj.weight",
            "model.layers.0.self_attn.wo_a.weight", "model.layers.0.ffn.gate.weight", "model.layers.0.attn.compressor.wkv.weight"]
    assert all(FP8.should_quantize_fp8(k) for k in keep)
    assert not any(FP8.should_quantize_fp8(k) for k in skip)


def test_fp8_quantization_config_variants():
    r = ckpt.ShardResults(size_in_bytes=False)
    r.add("a.safetensors", {"model.layers.0.self_attn.indexer.wq_b.weight": torch.zeros(4, 2)}, ["model.norm", "model.norm"])
    cfg = FP8.fp8_quantization_config("block", [128, 128], r)
    assert cfg == {"activation_scheme": "dynamic", "fmt": "e4m3", "quant_method": "fp8", "weight_block_size": [128, 128],
                   "scale_fmt": "ue8m0", "modules_to_not_convert": ["model.norm"]}
    assert r.total_size == 4      # the FP8 tool counts len(tensor), not bytes
    r2 = ckpt.ShardResults(size_in_bytes=False)
    assert FP8.fp8_quantization_config("tensor", None, r2) == {"activation_scheme": "dynamic", "fmt": "e4m3", "quant_method": "fp8"}
    ch = FP8.fp8_quantization_config("channel", None, r2)
    assert ch["quant_method"] == "compressed-tensors" and ch["format"] == "float-quantized"
    assert ch["config_groups"]["group_0"]["weights"]["strategy"] == "channel"
    assert ch["config_groups"]["group_0"]["input_activations"]["strategy"] == "token"


def test_int4_ignore_rules_and_config():
    rules = INT4.DEFAULT_IGNORE_RULES
    assert INT4.is_ignored("model.layers.0.self_attn.q_proj.weight", rules)
    assert INT4.is_ignored("model.layers.0.mlp.gate_proj.weight", rules) and INT4.is_ignored("lm_head.weight", rules)
    assert INT4.is_ignored("model.layers.1.mlp.shared_experts.down_proj.weight", rules)
    assert not INT4.is_ignored("model.layers.1.mlp.experts.3.down_proj.weight", rules)
    assert INT4.is_ignored("abc.def", ["abc"]) and INT4.is_ignored("abc", ["abc"]) and not INT4.is_ignored("xabc", ["abc"])
    cfg = INT4.int4_quantization_config(128, True, ["re:.*norm.*"])
    w = cfg["config_groups"]["group_0"]["weights"]
    assert (cfg["format"], cfg["quant_method"], w["num_bits"], w["group_size"], w["strategy"], w["symmetric"], w["type"]) == \
        ("pack-quantized", "compressed-tensors", 4, 128, "group", True, "int")
    assert cfg["ignore"] == ["re:.*norm.*"] and cfg["kv_cache_scheme"] is None


def test_nvfp4_name_scope():
    w = torch.zeros(4, 16, dtype=torch.bfloat16)
    name = "model.layers.0.mlp.experts.0.gate_proj.weight"
    assert NV.should_quantize(name, w)
    assert not NV.should_quantize(name, w, skip_weight_substrings=("mlp.experts.0",))
    assert NV.should_quantize(name, w, skip_weight_substrings=("mlp.experts.1",))
    assert not NV.should_quantize(name, w, num_hidden_layers=0)                      # MTP layers appended after the decoder
    assert NV.should_quantize("language_model.model.layers.2.mlp.experts.1.w2.weight", w, num_hidden_layers=3)
    assert not NV.should_quantize("model.layers.0.mlp.shared_experts.gate_proj.weight", w)
    assert not NV.should_quantize("model.layers.0.mlp.gate_proj.weight", w)
    assert not NV.should_quantize("vision_tower.layers.0.mlp.experts.0.gate_proj.weight", w)
    assert not NV.should_quantize(name, w.to(torch.int8))
    with pytest.raises(ValueError, match="must be divisible by 16"):
        NV.should_quantize(name, torch.zeros(4, 24, dtype=torch.bfloat16))


def test_nvfp4_ignore_list_and_configs(tmp_path):
    got = NV._augment_ignore_list(["model.layers.0.self_attn.q_proj", "model.layers.0.mlp.experts.3.down_proj",
                                   "model.layers.1.mlp.experts.gate_up_proj", "model.norm"])
    assert got == sorted({"model.layers.0.self_attn.q_proj", "model.layers.0.self_attn.qkv_proj",
                          "model.layers.0.mlp.experts.3.down_proj", "model.layers.0.mlp.experts",
                          "model.layers.1.mlp.experts.gate_up_proj", "model.layers.1.mlp.experts", "model.norm"})
    cfg = {"text_config": {"quantization_config": {}}, "quantization_config": {"config_groups": {"g": {"weights": {}}}}}
    NV._update_quantization_config(cfg, ["a"])
    q = cfg["quantization_config"]
    assert (q["quant_algo"], q["quant_method"], q["group_size"], q["ignore"]) == ("NVFP4", "modelopt", 16, ["a"])
    assert q["kv_cache_scheme"] == {"dynamic": False, "num_bits": 8, "type": "float"}
    assert q["config_groups"]["g"]["weights"] == {"dynamic": False, "num_bits": 4, "type": "float", "group_size": 16}
    assert cfg["text_config"]["quantization_config"]["quant_algo"] == "NVFP4"
    NV._write_hf_quant_config(str(tmp_path), ["a"], str(tmp_path))
    doc = json.loads((tmp_path / "hf_quant_config.json").read_text())
    assert doc == {"producer": {"name": "modelopt"}, "quantization": {"quant_algo": "NVFP4", "kv_cache_quant_algo": "FP8",
                                                                        "group_size": 16, "exclude_modules": ["a"]}}


def test_nvfp4_converter_uses_compact_bf16_moe_prefixes(tmp_path):
    # every layer kept in bf16: nothing is quantized, so the conversion runs without a GPU
    model_dir, save_dir = tmp_path / "model", tmp_path / "converted"
    model_dir.mkdir()
    (model_dir / "config.json").write_text('{"num_hidden_layers": 1}')
    weights = {f"model.layers.0.mlp.experts.{e}.{p}.weight": torch.ones((1, 16), dtype=torch.bfloat16)
               for e in range(128) for p in ("gate_proj", "up_proj", "down_proj")}
    weights["model.layers.0.input_layernorm.weight"] = torch.ones(16, dtype=torch.bfloat16)
    safetensors.torch.save_file(weights, model_dir / "model.safetensors", metadata={"format": "pt"})
    NV.convert_nvfp4(str(model_dir), str(save_dir), device="cpu", num_layers_at_end_in_bf16=1)
    expected = ["model.layers.0.", "model.layers.0.input_layernorm", "model.layers.0.mlp.experts"]
    assert json.loads((save_dir / "config.json").read_text())["quantization_config"]["ignore"] == expected
    assert json.loads((save_dir / "hf_quant_config.json").read_text())["quantization"]["exclude_modules"] == expected
    with safetensors.safe_open(save_dir / "model.safetensors", framework="pt", device="cpu") as f:
        assert all("weight_scale" not in k for k in f.keys())
        assert f.get_tensor("model.layers.0.mlp.experts.127.down_proj.weight").dtype == torch.bfloat16
    index = json.loads((save_dir / "model.safetensors.index.json").read_text())
    assert index["metadata"]["total_size"] == sum(t.numel() * 2 for t in weights.values())   # bytes for this tool


def test_mxfp8_source_detection_and_scale_lookup():
    assert MX._source_kind({}) == "bf16" and MX._source_kind({"quantization_config": {"quant_method": "bf16"}}) == "bf16"
    fp8 = {"quantization_config": {"quant_method": "fp8", "weight_block_size": [128, 128], "scale_fmt": "ue8m0"}}
    assert MX._source_kind(fp8) == "fp8_ue8m0"
    with pytest.raises(ValueError, match="Unsupported source quantization_config"):
        MX._source_kind({"quantization_config": {"quant_method": "fp8", "weight_block_size": [128, 128]}})
    # a weight's tile scales are looked up under `<name>.weight_scale_inv`, in this shard's tensors when they are there
    scales = torch.tensor([[0.5, 2.0, 1.0], [4.0, 0.25, 8.0]])
    weights = {"a.weight": torch.zeros(200, 288, dtype=torch.uint8), "a.weight_scale_inv": scales}
    got, key = MX._source_scale(weights, "a.weight", {"a.weight_scale_inv": "s"}, ".", "cpu", "s")
    assert key == "a.weight_scale_inv" and got is scales
    with pytest.raises(ValueError, match="Expected key ending"):
        MX._strip_weight_suffix("a.bias")


# ---------------------------------------------------------------------------------------------------------------------
# NVFP4 checkpoint scope, the scenarios of the reference's tests/fast/test_nvfp4_scope.py with the numeric kernels
# replaced by shape-correct stand-ins (the kernels themselves are covered by the GPU parity tests)
LAYER_ROOTS = ("model.layers", "language_model.model.layers", "model.language_model.layers", "language_model.layers")


@pytest.fixture
def stand_in_quantizers(monkeypatch):
    calls = []

    def result(w):
        rows, cols = w.shape
        return (torch.zeros((rows, cols // 2), dtype=torch.uint8), torch.ones((rows, cols // 16)).to(torch.float8_e4m3fn),
                torch.tensor(1.0))

    monkeypatch.setattr(NV, "quantize_nvfp4", lambda w: (calls.append("single"), result(w))[1])
    monkeypatch.setattr(NV, "nvfp4_quantize_1d_pair", lambda g, u: (calls.append("pair"), (result(g), result(u)))[1])
    return calls


def _run_nvfp4_conversion(tmp_path, config, shards, **kwargs):
    src, dst = tmp_path / "src", tmp_path / "dst"
    src.mkdir()
    (src / "config.json").write_text(json.dumps(config))
    for filename, tensors in shards.items():
        safetensors.torch.save_file(tensors, src / filename)
    NV.convert_nvfp4(str(src), str(dst), "cpu", **kwargs)
    index = json.loads((dst / "model.safetensors.index.json").read_text())
    out = {}
    for filename in set(index["weight_map"].values()):
        tensors = safetensors.torch.load_file(dst / filename)
        assert all(index["weight_map"][n] == filename for n in tensors)
        out.update(tensors)
    assert set(index["weight_map"]) == set(out)
    assert index["metadata"]["total_size"] == sum(t.numel() * t.element_size() for t in out.values())
    cfg = json.loads((dst / "config.json").read_text())
    ignore = cfg["quantization_config"]["ignore"]
    assert ignore == json.loads((dst / "hf_quant_config.json").read_text())["quantization"]["exclude_modules"]
    return out, ignore, cfg


def _kept_as_is(out, name, original, ignore):
    assert out[name].dtype == original.dtype and torch.equal(out[name], original)
    module = name.removesuffix(".weight")
    assert not any(f"{module}.{s}" in out for s in ("weight_scale", "weight_scale_2", "input_scale"))
    assert any(module == rule or module.startswith(rule.rstrip(".") + ".") for rule in ignore)


@pytest.mark.parametrize("root", LAYER_ROOTS)
def test_nvfp4_selector_stays_inside_the_language_decoder(root):
    w = torch.ones((2, 16), dtype=torch.bfloat16)
    e = ".mlp.experts.0."
    assert NV.should_quantize(f"{root}.69{e}down_proj.weight", w, num_hidden_layers=70)
    assert not NV.should_quantize(f"{root}.70{e}down_proj.weight", w, num_hidden_layers=70)
    assert not NV.should_quantize(f"{root}.0.mlp.shared_experts.down_proj.weight", w)
    assert not NV.should_quantize(f"{root}.0.mlp.shared_expert.experts.0.down_proj.weight", w)
    assert not NV.should_quantize(f"{root}.0.mlp.down_proj.weight", w)
    assert not NV.should_quantize(f"{root}.0{e}down_proj.weight", w, ("down_proj",))


@pytest.mark.parametrize("root", ["model.mtp.layers", "model.mtp_layers", "mtp.layers", "visual.layers", "audio_encoder.layers",
                                  "speech_embeddings.layers", "vision.model.layers", "model.visual.layers"])
def test_nvfp4_selector_never_validates_other_towers(root):
    # 7 columns would raise inside the decoder; an excluded tower must be turned away before that check
    assert not NV.should_quantize(f"{root}.0.mlp.experts.0.gate_proj.weight", torch.ones((2, 7)))


def test_nvfp4_multimodal_checkpoint_with_a_pair_split_over_two_shards(tmp_path, stand_in_quantizers):
    config = {"model_type": "mimo_v2", "num_hidden_layers": 70, "num_nextn_predict_layers": 1, "vision_config": {},
              "audio_config": {}}
    e = ".mlp.experts.0."
    gate, up, down = (f"model.layers.69{e}{p}.weight" for p in ("gate_proj", "up_proj", "down_proj"))
    outside = [f"model.mtp.layers.0{e}gate_proj.weight", f"model.layers.70{e}gate_proj.weight",
               f"visual.layers.0{e}gate_proj.weight", f"audio_encoder.layers.0{e}gate_proj.weight",
               f"speech_embeddings.layers.0{e}gate_proj.weight", "model.mtp.layers.0.block_sparse_moe.experts.0.w1.weight",
               "audio_encoder.layers.0.moe.experts.0.w2.weight", "model.layers.69.mlp.shared_experts.gate_proj.weight",
               "model.layers.69.self_attn.q_proj.weight", "lm_head.weight"]
    kept = {n: torch.full((2, 16), i + 1, dtype=torch.bfloat16) for i, n in enumerate(outside)}
    kept["model.mtp.layers.0.mlp.experts.gate_up_proj.weight"] = torch.ones((2, 2, 16), dtype=torch.bfloat16)
    w = torch.ones((2, 16), dtype=torch.bfloat16)
    out, ignore, cfg = _run_nvfp4_conversion(tmp_path, config, {"a.safetensors": {gate: w, down: w.clone(), **kept},
                                                                "b.safetensors": {up: w}})
    assert sorted(stand_in_quantizers) == ["pair", "single"]
    assert cfg["model_type"] == "mimo_v2" and cfg["num_hidden_layers"] == 70
    for name in (gate, up, down):
        module = name.removesuffix(".weight")
        assert out[name].dtype == torch.uint8 and out[name].shape == (2, 8)
        assert all(f"{module}.{s}" in out for s in ("weight_scale", "weight_scale_2", "input_scale"))
        assert not any(module == rule or module.startswith(rule.rstrip(".") + ".") for rule in ignore)
    for name, original in kept.items():
        _kept_as_is(out, name, original, ignore)
        if ".experts." in name:
            assert name.split(".experts.", 1)[0] + ".experts" in ignore


@pytest.mark.parametrize("root", LAYER_ROOTS[1:])
def test_nvfp4_depth_comes_from_the_nested_text_config(tmp_path, stand_in_quantizers, root):
    config = {"num_hidden_layers": 99, "text_config": {"num_hidden_layers": 3, "quantization_config": {"quant_method": "fp8"}}}
    tensors = {f"{root}.{i}.mlp.experts.0.down_proj.weight": torch.full((2, 16), i + 1, dtype=torch.bfloat16) for i in range(4)}
    out, ignore, cfg = _run_nvfp4_conversion(tmp_path, config, {"model.safetensors": tensors},
                                             num_layers_at_start_in_bf16=1, num_layers_at_end_in_bf16=1)
    assert stand_in_quantizers == ["single"]
    nested = cfg["text_config"]["quantization_config"]
    assert nested["ignore"] == ignore and nested["quant_algo"] == "NVFP4" and nested["quant_method"] == "modelopt"
    for name, original in tensors.items():
        if name == f"{root}.1.mlp.experts.0.down_proj.weight":
            assert out[name].dtype == torch.uint8
        else:
            _kept_as_is(out, name, original, ignore)
    assert {f"{root}.0.", f"{root}.2."}.issubset(ignore)
    assert not any(rule.startswith("model.layers.") for rule in ignore)


@pytest.mark.parametrize("prefix,eligible", [
    ("decoder", True), ("module.module.decoder", True), ("language_model.decoder", True),
    ("module.language_model.decoder", True), ("mtp", False), ("module.module.mtp", False), ("mtp.decoder", False),
    ("mtp.layers.0.transformer_layer.decoder", False), ("vision_model.decoder", False), ("audio_encoder.decoder", False),
    ("module.vision_model.decoder", False)])
def test_runtime_nvfp4_quantizer_only_takes_the_main_language_decoder(monkeypatch, prefix, eligible):
    from miles_amd.megatron_to_hf.processors import quantizer_nvfp4 as Q

    original, converted = [], [("quantized", torch.zeros(1))]
    monkeypatch.setattr(Q, "_quantize_moe_params", lambda *_: converted)
    got = Q.quantize_params_nvfp4(None, f"{prefix}.layers.0.mlp.experts.linear_fc2.weight0", original, {"quant_method": "nvfp4"})
    assert got is (converted if eligible else original)


# ---------------------------------------------------------------------------------------------------------------------
# MiMo-V2 -> BF16: the host-side parts (names, config, head order, --keep-quant, which needs no kernel)
def test_mimo_split_fused_qkv_restores_head_order():
    from miles_amd.tools.convert_mimo_v2_to_bf16 import split_fused_qkv
    from tests import mimo_fixture as MF

    config = {"num_key_value_heads": 2, "swa_num_attention_heads": 8, "swa_num_key_value_heads": 4, "swa_head_dim": 3, "swa_v_head_dim": 2}
    q, k, v = torch.randn(8 * 3, 5), torch.randn(4 * 3, 5), torch.randn(4 * 2, 5)
    for got, want in zip(split_fused_qkv(MF.interleave(q, k, v, 2), config, is_swa=True), (q, k, v), strict=True):
        assert torch.equal(got, want)
    with pytest.raises(AssertionError):
        split_fused_qkv(torch.zeros(10, 5), config, is_swa=True)


def test_mimo_names_and_config_when_layers_and_experts_are_dropped():
    from miles_amd.tools import convert_mimo_v2_to_bf16 as M
    from tests import mimo_fixture as MF

    assert M.output_name("lm_head.weight", {1: 0}, 2) == "lm_head.weight"
    assert M.output_name("model.layers.0.mlp.up_proj.weight", {1: 0}, None) is None
    assert M.output_name("model.layers.1.mlp.experts.1.up_proj.weight", {1: 0}, 2) == "model.layers.0.mlp.experts.1.up_proj.weight"
    assert M.output_name("model.layers.1.mlp.experts.2.up_proj.weight", {1: 0}, 2) is None
    assert M.output_name("model.layers.1.mlp.experts.2.up_proj.weight", None, None) == "model.layers.1.mlp.experts.2.up_proj.weight"
    cfg = M.convert_config(MF.CONFIG, {1: 0}, 2, keep_quant=False)
    assert (cfg["num_hidden_layers"], cfg["hybrid_layer_pattern"], cfg["moe_layer_freq"], cfg["n_routed_experts"]) == (1, [1], [1], 2)
    assert "quantization_config" not in cfg and "attention_projection_layout" not in cfg
    assert MF.CONFIG["num_hidden_layers"] == 2                                  # the input is not modified
    kept = M.convert_config(MF.CONFIG, {1: 0}, None, keep_quant=True)
    assert kept["quantization_config"]["ignored_layers"] == ["model.layers.0.self_attn.o_proj"]
    with pytest.raises(AssertionError):
        M.convert_config(MF.CONFIG, None, 1, keep_quant=False)                  # fewer experts than are routed to per token
    with pytest.raises(AssertionError, match="experts"):
        M.check_output({"model.layers.0.input_layernorm.weight": "f"}, cfg)            # the kept layer is the MoE layer
    dense_only = M.convert_config(MF.CONFIG, {0: 0}, None, keep_quant=False)
    with pytest.raises(AssertionError, match="is missing"):
        M.check_output({"model.layers.0.input_layernorm.weight": "f"}, dense_only)


def test_mimo_keep_quant_renumbers_and_copies_on_the_cpu(tmp_path, monkeypatch):
    from miles_amd.tools import convert_mimo_v2_to_bf16 as M
    from tests import mimo_fixture as MF

    src, dst = tmp_path / "src", tmp_path / "dst"
    src.mkdir()
    MF.write(src)
    # an interrupted side-file copy must not leave an index behind (the index is what marks a finished conversion)
    real_copy = M.shutil.copy2
    monkeypatch.setattr(M.shutil, "copy2", lambda *_: (_ for _ in ()).throw(OSError("interrupted auxiliary copy")))
    with pytest.raises(OSError, match="interrupted auxiliary copy"):
        M.main(str(src), str(dst), [1], None, keep_quant=True, device="cpu")
    assert not (dst / "model.safetensors.index.json").exists()
    monkeypatch.setattr(M.shutil, "copy2", real_copy)
    M.main(str(src), str(dst), [1], None, keep_quant=True, device="cpu")
    config = json.loads((dst / "config.json").read_text())
    assert config["quantization_config"]["ignored_layers"] == ["model.layers.0.self_attn.o_proj"]
    assert config["attention_projection_layout"] == "fused_qkv" and config["num_hidden_layers"] == 1
    index = json.loads((dst / "model.safetensors.index.json").read_text())
    out = safetensors.torch.load_file(dst / "model-00001.safetensors")
    assert set(index["weight_map"]) == set(out)
    assert out["model.layers.0.self_attn.qkv_proj.weight"].dtype == torch.float8_e4m3fn       # stored formats survive
    assert out["model.layers.0.mlp.experts.3.down_proj.weight"].dtype == torch.uint8
    assert not any(name.startswith("model.layers.1.") for name in out)
    assert (dst / "tokenizer_config.json").read_text() == "{}"
