"""MXFP8 quantization of HF-named tensors on the weight-sync path.

Same interface and decisions as the reference's
miles/backends/megatron_utils/megatron_to_hf/processors/quantizer_mxfp8.py (`quantize_params_mxfp8` :6-107,
`_quantize_param` :110-114).
"""

from __future__ import annotations

from miles_amd.utils.mxfp8 import mxfp8_quantize

from ._names import in_bf16_head_or_tail, named_in_extra_high_precision, parse_layer_param

_DECODER = r"decoder\.layers\.(\d+)\.(.+)"
_MTP = r"mtp\.layers\.(\d+)\.(.+)"

_MXFP8_LINEARS = frozenset({
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
    "self_attention.wq_b.weight",
    # DeepSeek V4 attention
    "self_attention.linear_kv_proj.weight",
    "self_attention.core_attention.indexer.linear_wq_b.weight",
})
# an interleaved indexer fuses wk into a bf16 tensor whose loader would misread uint8 E8M0 scales
_MXFP8_INDEXER_WK = frozenset({
    "self_attention.wk.weight",
    "self_attention.core_attention.indexer.linear_wk.weight",
})


def quantize_params_mxfp8(args, megatron_name, converted_named_params, quantization_config):
    assert quantization_config["quant_method"] == "mxfp8"
    if named_in_extra_high_precision(args, megatron_name):
        return converted_named_params
    p = parse_layer_param(megatron_name, decoder=_DECODER, mtp=_MTP, anchored=False)
    if p is None:
        return converted_named_params
    # the BF16 head / tail applies to whichever layer index was parsed, as in the reference
    if in_bf16_head_or_tail(args, p.layer_idx):
        return converted_named_params

    skip_scale_tensors = False
    if p.routed_expert_linear is not None:
        if p.routed_expert_linear not in ("linear_fc1", "linear_fc2"):
            return converted_named_params
        skip_scale_tensors = True
    elif p.shared_expert_rest is not None and p.shared_expert_rest in ("linear_fc1.weight", "linear_fc2.weight"):
        pass
    elif p.rest in _MXFP8_LINEARS:
        pass
    elif not getattr(args, "indexer_rope_interleave", False) and p.rest in _MXFP8_INDEXER_WK:
        pass
    else:
        return converted_named_params

    out = []
    for hf_name, param in converted_named_params:
        if skip_scale_tensors and hf_name.endswith("_scale"):
            continue
        out.extend(_quantize_param(hf_name, param))
    return out


def _quantize_param(name, weight):
    assert name.endswith(".weight"), f"Expected weight parameter, got {name}"
    qweight, scale = mxfp8_quantize(weight)
    return [(name, qweight), (name.replace(".weight", ".weight_scale_inv"), scale)]
