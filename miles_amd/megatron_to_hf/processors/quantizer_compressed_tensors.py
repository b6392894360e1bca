"""compressed-tensors INT4 (pack-quantized, symmetric, group-wise) on the weight-sync path.

Same interface and output naming as the reference's
miles/backends/megatron_utils/megatron_to_hf/processors/quantizer_compressed_tensors.py
(`quantize_params_compressed_tensors` :268-303).  `pack_layer` (:235-265) is the fused gfx950 kernel.
"""

from __future__ import annotations

import torch

from miles_amd import launch
from miles_amd.kernels.quant.int4_fake import pack_layer
from miles_amd.utils.mxfp4 import quantize_mxfp4

__all__ = ["quantize_params_compressed_tensors", "pack_layer"]


def quantize_params_compressed_tensors(converted_named_params, quantization_config, packed_weight_basenames):
    weights_cfg = quantization_config["config_groups"]["group_0"]["weights"]
    group_size = weights_cfg["group_size"]
    symmetric = weights_cfg["symmetric"]
    is_mxfp4 = quantization_config["format"] == "mxfp4-pack-quantized"
    if is_mxfp4:
        assert weights_cfg["type"] == "float"
        assert weights_cfg["num_bits"] == 4
        assert weights_cfg["scale_dtype"] == "torch.uint8"
        assert symmetric

    out = []
    for name, param in converted_named_params:
        if not (name.endswith(".weight") and name.removesuffix(".weight") in packed_weight_basenames):
            out.append((name, param))
            continue
        if is_mxfp4:   # only the packed codes and the E8M0 scales are published for this format
            packed, scale = quantize_mxfp4(param, group_size)
            out.append((name.replace(".weight", ".weight_packed"), packed))
            out.append((name.replace(".weight", ".weight_scale"), scale))
            continue
        packed, scale, zero_point = pack_layer(param, group_size, symmetric)
        shape = torch.tensor(param.shape, dtype=torch.int32, device=param.device)
        launch.note_constant(shape)
        if zero_point is not None:
            out.append((name.replace(".weight", ".weight_zero_point"), zero_point))
        out.append((name.replace(".weight", ".weight_packed"), packed))
        out.append((name.replace(".weight", ".weight_scale"), scale))
        out.append((name.replace(".weight", ".weight_shape"), shape))
    return out
