"""The weightless MXFP8 rollout schema (`miles_amd/utils/hf_rollout_schema.py`): the expectations of the reference's
tests/fast/utils/test_hf_rollout_schema.py, restated on checkpoints written here.  Host logic only."""

import json

import pytest
import torch
from safetensors.torch import save_file

from miles_amd.tools import convert_hf_to_mxfp8
from miles_amd.utils.hf_rollout_schema import build_mxfp8_quantization_config, create_mxfp8_rollout_schema

EXPERT = "model.layers.0.mlp.experts.0.gate_proj.weight"


def _mixed_checkpoint(root):
    root.mkdir()
    f8, bf16 = torch.float8_e4m3fn, torch.bfloat16
    tensors = {"model.embed_tokens.weight": torch.zeros(32, 64, dtype=bf16),
               "model.layers.0.input_layernorm.weight": torch.zeros(64, dtype=bf16),
               "model.layers.0.self_attn.wq_a.weight": torch.zeros(64, 64, dtype=f8),
               "model.layers.0.self_attn.wo_a.weight": torch.zeros(64, 64, dtype=f8),
               "model.layers.10.self_attn.wo_a.weight": torch.zeros(64, 64, dtype=f8),
               "model.layers.2.self_attn.wo_a.weight": torch.zeros(64, 64, dtype=f8),
               EXPERT: torch.zeros(64, 32, dtype=torch.int8),          # packed MXFP4: 64 logical columns
               "model.layers.0.self_attn.wq_a.weight_scale_inv": torch.zeros(1, 1),
               "lm_head.weight": torch.zeros(32, 64, dtype=bf16)}
    shard = "model-00001-of-00001.safetensors"
    save_file(tensors, root / shard)
    (root / "config.json").write_text(json.dumps({"architectures": ["TestForCausalLM"], "expert_dtype": "fp4",
                                                  "quantization_config": {"quant_method": "fp8"}}))
    (root / "model.safetensors.index.json").write_text(json.dumps({"weight_map": dict.fromkeys(tensors, shard)}))
    (root / "tokenizer.json").write_text("{}")
    return root


def test_config_lists_what_stays_unquantized_from_headers_alone(tmp_path):
    config = build_mxfp8_quantization_config(_mixed_checkpoint(tmp_path / "src"))
    assert {k: v for k, v in config.items() if k != "modules_to_not_convert"} == {
        "activation_scheme": "dynamic", "fmt": "e4m3", "quant_method": "mxfp8", "weight_block_size": [1, 32],
        "scale_fmt": "ue8m0"}
    kept = config["modules_to_not_convert"]
    # natural order: layer 2 before layer 10; names without the ".weight" suffix; non-weights never listed
    assert kept == ["lm_head", "model.embed_tokens", "model.layers.0.input_layernorm", "model.layers.0.self_attn.wo_a",
                    "model.layers.2.self_attn.wo_a", "model.layers.10.self_attn.wo_a"]
    assert "model.layers.0.self_attn.wq_a" not in kept              # an FP8 source matrix is re-scaled, so quantized
    assert not any("experts" in name for name in kept)               # packed int8 experts count as quantizable


def test_schema_directory_has_metadata_and_no_weights(tmp_path):
    source = _mixed_checkpoint(tmp_path / "src")
    made = create_mxfp8_rollout_schema(source, tmp_path / "schema")
    assert made == (tmp_path / "schema").resolve()
    assert sorted(p.name for p in made.iterdir()) == ["config.json", "tokenizer.json"]
    config = json.loads((made / "config.json").read_text())
    assert config["expert_dtype"] == "fp8" and config["architectures"] == ["TestForCausalLM"]
    assert config["quantization_config"] == build_mxfp8_quantization_config(source)
    assert (made / "config.json").read_text().endswith("}\n")


def test_schema_refuses_the_source_itself_and_a_directory_with_weights(tmp_path):
    source = _mixed_checkpoint(tmp_path / "src")
    with pytest.raises(ValueError, match="must differ from the source"):
        create_mxfp8_rollout_schema(source, source)
    target = tmp_path / "schema"
    target.mkdir()
    (target / "left_over.safetensors").write_bytes(b"payload")
    with pytest.raises(ValueError, match="containing weight payloads"):
        create_mxfp8_rollout_schema(source, target)
    assert not (target / "config.json").exists()


@pytest.mark.parametrize("dtype,width,valid", [(torch.int8, 16, True), (torch.int8, 24, False),
                                               (torch.bfloat16, 48, False), (torch.int32, 32, False),
                                               (torch.bfloat16, 64, True), (torch.float8_e4m3fn, 32, True)])
def test_an_expert_that_cannot_be_quantized_is_an_error(tmp_path, dtype, width, valid):
    (tmp_path / "config.json").write_text(json.dumps({"architectures": ["TestForCausalLM"]}))
    save_file({EXPERT: torch.zeros(32, width, dtype=dtype)}, tmp_path / "model.safetensors")
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {EXPERT: "model.safetensors"}}))
    if valid:
        assert build_mxfp8_quantization_config(tmp_path)["modules_to_not_convert"] == []
    else:
        with pytest.raises(ValueError, match="Unsupported MXFP8 expert"):
            build_mxfp8_quantization_config(tmp_path)


def test_checkpoint_without_an_index_and_the_cli_flag(tmp_path):
    source = tmp_path / "src"
    source.mkdir()
    (source / "config.json").write_text(json.dumps({"architectures": ["TestForCausalLM"]}))
    save_file({"model.embed_tokens.weight": torch.zeros(32, 32, dtype=torch.bfloat16)}, source / "model.safetensors")
    # the command line takes the same route and needs no device
    convert_hf_to_mxfp8.main(["--model-dir", str(source), "--save-dir", str(tmp_path / "schema"), "--metadata-only"])
    config = json.loads((tmp_path / "schema" / "config.json").read_text())
    assert config["quantization_config"]["modules_to_not_convert"] == ["model.embed_tokens"]
    assert not list((tmp_path / "schema").glob("*.safetensors"))


def test_errors_of_a_broken_checkpoint(tmp_path):
    with pytest.raises(FileNotFoundError, match="config.json"):
        build_mxfp8_quantization_config(tmp_path)
    (tmp_path / "config.json").write_text("{}")
    with pytest.raises(FileNotFoundError, match="No safetensors weights"):
        build_mxfp8_quantization_config(tmp_path)
    save_file({"a.weight": torch.zeros(32, 32)}, tmp_path / "one.safetensors")
    save_file({"a.weight": torch.zeros(32, 32)}, tmp_path / "two.safetensors")
    with pytest.raises(ValueError, match="Duplicate tensor a.weight"):
        build_mxfp8_quantization_config(tmp_path)
    (tmp_path / "two.safetensors").unlink()
    (tmp_path / "model.safetensors.index.json").write_text(
        json.dumps({"weight_map": {"a.weight": "one.safetensors", "b.weight": "one.safetensors"}}))
    with pytest.raises(KeyError, match="b.weight is listed"):
        build_mxfp8_quantization_config(tmp_path)


def test_a_name_table_is_applied_before_the_predicate(tmp_path):
    (tmp_path / "config.json").write_text("{}")
    save_file({"embed.weight": torch.zeros(32, 32, dtype=torch.bfloat16),
               "blk.weight": torch.zeros(32, 32, dtype=torch.bfloat16)}, tmp_path / "model.safetensors")
    table = {"embed.weight": "model.embed_tokens.weight", "blk.weight": "model.layers.0.mlp.up_proj.weight"}
    assert build_mxfp8_quantization_config(tmp_path, table.get)["modules_to_not_convert"] == ["model.embed_tokens"]
