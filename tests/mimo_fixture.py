"""A two-layer checkpoint in the official MiMo-V2 layout (layer 0: global attention + dense MLP, layer 1: sliding-window
attention + four routed experts) for the converter tests; the scenario follows the reference's
tests/fast/tools/test_convert_mimo_v2_to_bf16.py:84-146.  Built with torch CPU ops only."""

import json

import torch
from safetensors.torch import save_file

FP4_VALUES = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0])

CONFIG = {
    "architectures": ["MiMoV2ForCausalLM"], "attention_projection_layout": "fused_qkv", "num_hidden_layers": 2,
    "hybrid_layer_pattern": [0, 1], "moe_layer_freq": [0, 1], "hybrid_block_size": None,
    "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 64, "v_head_dim": 32,
    "swa_num_attention_heads": 4, "swa_num_key_value_heads": 4, "swa_head_dim": 64, "swa_v_head_dim": 32,
    "add_swa_attention_sink_bias": True, "n_routed_experts": 4, "num_experts_per_tok": 2,
    "quantization_config": {"quant_method": "fp8", "store_dtype": "mxfp4", "ignored_layers": ["model.layers.1.self_attn.o_proj"]},
}


def pack_nibbles(codes: torch.Tensor) -> torch.Tensor:
    """[out, in] e2m1 codes -> [out, in / 2] bytes, even elements in the low nibble."""
    return (codes[:, 0::2] | (codes[:, 1::2] << 4)).to(torch.uint8)


def quantize_fp8_blocks(w: torch.Tensor):
    """128x128 block FP8 of one matrix whose rows are padded to whole blocks: (e4m3 [rows, cols], fp32 scale grid)."""
    rows, cols = w.shape
    grid_r, grid_c = -(-rows // 128), -(-cols // 128)
    padded = torch.zeros(grid_r * 128, grid_c * 128)
    padded[:rows, :cols] = w
    tiles = padded.view(grid_r, 128, grid_c, 128)
    scale = tiles.abs().amax(dim=(1, 3)).clamp(min=1e-12) / 448.0
    q = (tiles / scale[:, None, :, None]).reshape(grid_r * 128, grid_c * 128)[:rows, :cols].to(torch.float8_e4m3fn)
    return q, scale


def dequantize_fp8_blocks(q: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    rows, cols = q.shape
    full = scale.float().repeat_interleave(128, 0)[:rows].repeat_interleave(128, 1)[:, :cols]
    return (q.float() * full).to(torch.bfloat16)


def dequantize_mxfp4(packed: torch.Tensor, exponents: torch.Tensor) -> torch.Tensor:
    codes = torch.stack([packed & 0xF, packed >> 4], dim=-1).reshape(packed.shape[0], -1).long()
    return (FP4_VALUES[codes] * torch.exp2(exponents.float() - 127).repeat_interleave(32, dim=1)).to(torch.bfloat16)


def interleave(q, k, v, shards):
    """Shard i of the fused projection is [q_i | k_i | v_i]."""
    return torch.cat([torch.cat(piece) for piece in zip(q.chunk(shards), k.chunk(shards), v.chunk(shards))])


def write(path, seed=0):
    """Writes the checkpoint; returns {output tensor name: expected bf16 tensor} for everything that gets dequantized."""
    g = torch.Generator().manual_seed(seed)
    rnd = lambda *shape: torch.randn(*shape, generator=g)   # noqa: E731
    expected, tensors = {}, {"model.embed_tokens.weight": rnd(16, 128).bfloat16()}
    for layer, kv_heads in ((0, 2), (1, 4)):
        p = f"model.layers.{layer}."
        q, k, v = rnd(4 * 64, 128), rnd(kv_heads * 64, 128), rnd(kv_heads * 32, 128)
        halves = [quantize_fp8_blocks(part) for part in interleave(q, k, v, 2).chunk(2)]
        tensors[p + "self_attn.qkv_proj.weight"] = torch.cat([h[0] for h in halves])
        tensors[p + "self_attn.qkv_proj.weight_scale_inv"] = torch.cat([h[1] for h in halves])
        fused = torch.cat([dequantize_fp8_blocks(*h) for h in halves])
        sizes = [4 // 2 * 64, kv_heads // 2 * 64, kv_heads // 2 * 32]
        for letter, piece in zip("qkv", fused.view(2, sum(sizes), 128).split(sizes, dim=1)):
            expected[p + f"self_attn.{letter}_proj.weight"] = piece.reshape(-1, 128)
        tensors[p + "input_layernorm.weight"] = torch.ones(128).bfloat16()
        tensors[p + "post_attention_layernorm.weight"] = torch.ones(128).bfloat16()
        tensors[p + "self_attn.o_proj.weight"] = rnd(128, 4 * 32).bfloat16()
    tensors["model.layers.1.self_attn.attention_sink_bias"] = torch.zeros(4).bfloat16()
    for proj, shape in (("gate_proj", (256, 128)), ("up_proj", (256, 128)), ("down_proj", (128, 256))):
        q8, s = quantize_fp8_blocks(rnd(*shape))
        tensors[f"model.layers.0.mlp.{proj}.weight"], tensors[f"model.layers.0.mlp.{proj}.weight_scale_inv"] = q8, s
        expected[f"model.layers.0.mlp.{proj}.weight"] = dequantize_fp8_blocks(q8, s)
    tensors["model.layers.1.mlp.gate.weight"] = rnd(4, 128).bfloat16()
    tensors["model.layers.1.mlp.gate.e_score_correction_bias"] = rnd(4)
    for e in range(4):
        for proj, (rows, cols) in (("gate_proj", (64, 128)), ("up_proj", (64, 128)), ("down_proj", (128, 64))):
            name = f"model.layers.1.mlp.experts.{e}.{proj}."
            packed = pack_nibbles(torch.randint(0, 16, (rows, cols), generator=g))
            exps = torch.randint(124, 130, (rows, cols // 32), dtype=torch.uint8, generator=g)
            tensors[name + "weight"], tensors[name + "weight_scale"] = packed, exps
            expected[name + "weight"] = dequantize_mxfp4(packed, exps)
    save_file(tensors, str(path / "model-00001.safetensors"))
    (path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": dict.fromkeys(tensors, "model-00001.safetensors")}))
    (path / "config.json").write_text(json.dumps(CONFIG))
    (path / "tokenizer_config.json").write_text("{}")
    return expected
