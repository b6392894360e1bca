"""FP8 (e4m3) quantization of HF-named tensors on the weight-sync path.

Same interface and decisions as the reference's
miles/backends/megatron_utils/megatron_to_hf/processors/quantizer_fp8.py:
`quantize_params_fp8` (:16-128) decides from the Megatron parameter name, `_quantize_param` (:131-159)
quantizes one HF tensor and names its scale.  The 128x128 cast is the gfx950 kernel behind
`fp8_blockwise_cast`; the power-of-two-scale variants the reference takes from SGLang (`per_block_cast_to_fp8`,
`quant_weight_ue8m0` + `transform_scale_ue8m0`) are third-party code outside the reference tree, restated here from
their published algorithms.
"""

from __future__ import annotations

import os

from miles_amd.kernels.quant.fp8_blockwise import (fp8_blockwise_cast, per_block_cast_to_fp8, quant_weight_ue8m0,
                                                   transform_scale_ue8m0)
from miles_amd.tools.convert_hf_to_fp8 import tensor_fp8

from ._names import parse_layer_param

_DECODER = r"module\.module\.decoder\.layers\.(\d+)\.(.+)"
_MTP = r"module\.module\.mtp\.layers\.(\d+)\.(.+)"

# dense / attention linears stored as FP8 by the rollout engine
_FP8_LINEARS = frozenset({
    "self_attention.linear_proj.weight",
    "self_attention.linear_qkv.weight",
    "mlp.linear_fc1.weight",
    "mlp.linear_fc2.weight",
    # MLA
    "self_attention.linear_q_proj.weight",
    "self_attention.linear_q_down_proj.weight",
    "self_attention.linear_q_up_proj.weight",
    "self_attention.linear_kv_down_proj.weight",
    "self_attention.linear_kv_up_proj.weight",
    # DSA indexer
    "self_attention.wq_b.weight",
    # linear attention
    "self_attention.linear_attn.in_proj_qkv.weight",
    "self_attention.linear_attn.in_proj_z.weight",
    "self_attention.linear_attn.out_proj.weight",
    # DeepSeek V4 attention
    "self_attention.linear_kv_proj.weight",
    "self_attention.core_attention.indexer.linear_wq_b.weight",
})
# only when the indexer keeps wk as a standalone FP8 parameter (no rope interleave)
_FP8_INDEXER_WK = frozenset({
    "self_attention.wk.weight",
    "self_attention.core_attention.indexer.linear_wk.weight",
})


def is_layer_skipped(prefix: str, ignored_layers: list[str], fused_mapping: dict | None = None) -> bool:
    """Whether the checkpoint keeps module `prefix` unquantized.

    Restates the contract of SGLang's `is_layer_skipped` (third party, imported by the reference at
    miles/backends/megatron_utils/sglang.py:20): a module is skipped when it is listed; a fused module is
    skipped when all of its shards are listed, and a partial listing is an error.
    """
    fused_mapping = fused_mapping or {}
    proj = prefix.split(".")[-1]
    if proj in fused_mapping and fused_mapping[proj] != [proj]:
        flags = {prefix.replace(proj, shard) in ignored_layers for shard in fused_mapping[proj]}
        if len(flags) > 1:
            raise ValueError(f"Detected some but not all shards of {prefix} are quantized. "
                             "All shards of fused layers must have the same precision.")
        return flags.pop()
    return prefix in ignored_layers


def _wants(args, rest: str) -> bool:
    if rest in _FP8_LINEARS:
        return True
    return not getattr(args, "indexer_rope_interleave", False) and rest in _FP8_INDEXER_WK


def quantize_params_fp8(args, megatron_name, converted_named_params, quantization_config):
    assert quantization_config["quant_method"] == "fp8"
    fmt = quantization_config.get("fmt", "e4m3")
    assert fmt == "e4m3", f"Unsupported FP8 format: {fmt}"
    assert quantization_config["activation_scheme"] == "dynamic"
    weight_block_size = quantization_config.get("weight_block_size", None)
    ignored_layers: list[str] = []
    for name in quantization_config.get("ignored_layers", quantization_config.get("modules_to_not_convert", [])) or []:
        name = name.removeprefix("model.")
        ignored_layers.extend((name, f"model.{name}"))
    packed_modules_mapping = quantization_config.get("packed_modules_mapping") or {}

    p = parse_layer_param(megatron_name, decoder=_DECODER, mtp=_MTP, anchored=True)
    if p is None:
        return converted_named_params

    skip_scale_tensors = False
    if p.routed_expert_linear is not None:
        if p.routed_expert_linear not in ("linear_fc1", "linear_fc2"):
            return converted_named_params
        skip_scale_tensors = True  # bf16 checkpoints carry weight_scale / input_scale entries: drop them
    elif p.shared_expert_rest is not None and p.shared_expert_rest in ("linear_fc1.weight", "linear_fc2.weight"):
        pass
    elif not _wants(args, p.rest):
        return converted_named_params

    out = []
    for hf_name, param in converted_named_params:
        if skip_scale_tensors and hf_name.endswith("_scale"):
            continue
        out.extend(_quantize_param(args, hf_name, param, weight_block_size, ignored_layers, packed_modules_mapping))
    return out


def _quantize_param(args, name, weight, weight_block_size, ignored_layers, packed_modules_mapping):
    assert name.endswith(".weight"), f"Expected weight parameter, got {name}"
    prefix = name.removesuffix(".weight")
    if ".experts." in prefix:
        prefix = prefix.split(".experts.", 1)[0] + ".experts"  # one precision per fused MoE module
    if ignored_layers and is_layer_skipped(prefix, ignored_layers, fused_mapping=packed_modules_mapping):
        return [(name, weight)]
    if weight_block_size is not None:
        scale_format = _get_scale_format(args, name, weight_block_size)
        if scale_format == "ue8m0":
            if weight.dim() == 3 and getattr(args, "qkv_row_block_views", False):
                qweight, scale = per_block_cast_to_fp8(weight)      # a [groups, rows, hidden] view standing for a matrix
            else:
                qweight, scale = quant_weight_ue8m0(weight, weight_block_size=weight_block_size)
            scale = transform_scale_ue8m0(scale, mn=qweight.shape[-2])
        elif os.environ.get("NVTE_FP8_BLOCK_SCALING_FP32_SCALES", "1") == "0" and list(weight_block_size) == [128, 128]:
            qweight, scale = per_block_cast_to_fp8(weight)      # power-of-two scales, kept as fp32
        else:
            qweight, scale = fp8_blockwise_cast(weight, weight_block_size)
        return [(name, qweight), (name.replace(".weight", ".weight_scale_inv"), scale)]
    # per-tensor: scale = max(amax, 1e-12) / 448 with the quotient kept in the weight's dtype
    qweight, scale = tensor_fp8(weight)
    return [(name, qweight), (name.replace(".weight", ".weight_scale"), scale)]


def _get_scale_format(args, name, weight_block_size):
    """'ue8m0' when the engine's DeepGEMM path wants requantized power-of-two scales, else None.

    The reference asks SGLang (`should_deepgemm_weight_requant_ue8m0`); without SGLang the answer is the
    fp32-scale format unless the arguments explicitly request DeepGEMM requantization.
    """
    if not getattr(args, "deepgemm_weight_requant_ue8m0", False):
        return None
    if ".experts." not in name:
        return "ue8m0"
    backend = getattr(args, "sglang_moe_runner_backend", None)
    a2a = getattr(args, "sglang_moe_a2a_backend", None)
    return "ue8m0" if backend == "deep_gemm" or (backend == "auto" and a2a in ("deepep", "mooncake")) else None
