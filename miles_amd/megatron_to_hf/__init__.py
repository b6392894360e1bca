"""Megatron parameter -> quantized HF tensors (reference: miles/backends/megatron_utils/megatron_to_hf/__init__.py)."""

from __future__ import annotations

from .name_maps import (convert_deepseekv3_to_hf, convert_glm4_to_hf, convert_glm4moe_to_hf, convert_llama_to_hf,
                        convert_mimo_to_hf, convert_qwen2_to_hf, convert_qwen3moe_to_hf)
from .processors import quantize_params, remove_padding

# substring of the lower-cased model name -> converter; first match wins, order as in the reference's
# _convert_to_hf_core (megatron_to_hf/__init__.py:37-83).  A family whose map is not built here keeps its place in the
# order with None, so that its name is refused and not taken by a later, shorter key ("qwen3next" contains "qwen3").
_CONVERTERS = (
    (("glm5_next", "glm5next"), None),
    (("kimi_k25", "kimi_k3", "kimivl"), None),      # ahead of "kimi_k2" below, which is a key of this table only
    (("glm4moelite", "deepseekv3", "glmmoedsa", "glm_moe_dsa", "kimi_k2", "kimik2"), convert_deepseekv3_to_hf),
    (("glm4moe",), convert_glm4moe_to_hf),
    (("glm4",), convert_glm4_to_hf),
    (("qwen3moe",), convert_qwen3moe_to_hf),
    (("qwen3next", "qwen3_8_next", "qwen4_exp", "qwen3.8_next", "qwen3_5", "qwen3_6"), None),
    (("qwen2", "qwen3"), convert_qwen2_to_hf),
    (("deepseekv41", "deepseekv4", "inkling"), None),
    (("llama",), convert_llama_to_hf),
    (("mimo",), convert_mimo_to_hf),
)


def _convert_to_hf_core(args, model_name, name, param):
    lowered = model_name.lower()
    for keys, fn in _CONVERTERS:
        if any(k in lowered for k in keys):
            if fn is None:
                break
            return fn(args, name, param)
    raise ValueError(f"Unsupported model: {lowered}")


def convert_to_hf(args, model_name, name, param, quantization_config=None, packed_weight_basenames=None):
    """One Megatron parameter -> the HF-named tensors it becomes, quantized per `quantization_config`
    (reference: megatron_to_hf/__init__.py:28-33)."""
    param = remove_padding(name, param, args.vocab_size)
    converted = _convert_to_hf_core(args, model_name, name, param)
    return quantize_params(args, name, converted, quantization_config, packed_weight_basenames)
