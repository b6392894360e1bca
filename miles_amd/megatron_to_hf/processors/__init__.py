"""Quantizer dispatch for HF-named tensors (reference: .../megatron_to_hf/processors/__init__.py:17-30).

`quantize_params` keeps the reference's signature and its order of tests on the checkpoint's `quantization_config`:
`quant_method` "fp8", then "mxfp8", then NVFP4 (named by `quant_algo` or by the method), then "compressed-tensors",
which needs the names the checkpoint stores packed; any other configuration yields None, and no configuration at all
hands the input list back unchanged (the same object: callers test for it).
"""

from . import quantizer_compressed_tensors as _int4
from . import quantizer_fp8 as _fp8
from . import quantizer_mxfp8 as _mxfp8
from . import quantizer_nvfp4 as _nvfp4
from .padding_remover import remove_padding

quantize_params_fp8 = _fp8.quantize_params_fp8
quantize_params_mxfp8 = _mxfp8.quantize_params_mxfp8
quantize_params_nvfp4 = _nvfp4.quantize_params_nvfp4
quantize_params_compressed_tensors = _int4.quantize_params_compressed_tensors

__all__ = ["quantize_params", "quantize_params_compressed_tensors", "quantize_params_fp8", "quantize_params_mxfp8",
           "quantize_params_nvfp4", "remove_padding"]

# quantizers that take (args, megatron_name, named_params, config), by the method name that selects them
_PER_PARAMETER = {"fp8": quantize_params_fp8, "mxfp8": quantize_params_mxfp8, "nvfp4": quantize_params_nvfp4}


def _method_of(config: dict) -> str | None:
    method = config.get("quant_method")
    if method not in ("fp8", "mxfp8") and config.get("quant_algo") == "NVFP4":
        return "nvfp4"          # ModelOpt checkpoints say quant_method "modelopt" and name the algorithm
    return method


def quantize_params(args, megatron_name, converted_named_params, quantization_config, packed_weight_basenames=None):
    if quantization_config is None:
        return converted_named_params
    method = _method_of(quantization_config)
    if method in _PER_PARAMETER:
        return _PER_PARAMETER[method](args, megatron_name, converted_named_params, quantization_config)
    if method == "compressed-tensors":
        assert packed_weight_basenames is not None, \
            "compressed-tensors quantization needs the checkpoint's packed weight names"
        return quantize_params_compressed_tensors(converted_named_params, quantization_config, packed_weight_basenames)
    return None
