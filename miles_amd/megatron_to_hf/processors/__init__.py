"""Quantizer dispatch for HF-named tensors (reference: .../megatron_to_hf/processors/__init__.py:17-30)."""

from .padding_remover import remove_padding
from .quantizer_compressed_tensors import quantize_params_compressed_tensors
from .quantizer_fp8 import quantize_params_fp8
from .quantizer_mxfp8 import quantize_params_mxfp8
from .quantizer_nvfp4 import quantize_params_nvfp4

__all__ = [
    "remove_padding",
    "quantize_params",
    "quantize_params_fp8",
    "quantize_params_mxfp8",
    "quantize_params_nvfp4",
    "quantize_params_compressed_tensors",
]


def quantize_params(args, megatron_name, converted_named_params, quantization_config, packed_weight_basenames=None):
    """Returns `converted_named_params` itself (the same list object) when nothing is quantized."""
    if quantization_config is None:
        return converted_named_params
    method = quantization_config.get("quant_method")
    if method == "fp8":
        return quantize_params_fp8(args, megatron_name, converted_named_params, quantization_config)
    if method == "mxfp8":
        return quantize_params_mxfp8(args, megatron_name, converted_named_params, quantization_config)
    if quantization_config.get("quant_algo") == "NVFP4" or method == "nvfp4":
        return quantize_params_nvfp4(args, megatron_name, converted_named_params, quantization_config)
    if method == "compressed-tensors":
        assert packed_weight_basenames is not None, \
            "compressed-tensors quantization needs the checkpoint's packed weight names"
        return quantize_params_compressed_tensors(converted_named_params, quantization_config, packed_weight_basenames)
    return None
