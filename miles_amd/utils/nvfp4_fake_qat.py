"""Switch that puts NVFP4 fake quantization in front of grouped-linear weights during training.

Same surface as the reference's miles/utils/nvfp4_fake_qat.py:10-23: with OPEN_TRAINING_NVFP4_FAKE_QAT_FLAG=1 every
weight of the list is replaced by its quantize-dequantize image (straight-through gradient), with one configuration
read from the environment for the whole list; with any other value the list comes back as the same object.
"""

from __future__ import annotations

import os

import torch

NVFP4_FAKE_QAT_FLAG = "OPEN_TRAINING_NVFP4_FAKE_QAT_FLAG"


def maybe_fake_quantize_nvfp4_weight_tensors(weight_tensors: list[torch.Tensor]) -> list[torch.Tensor]:
    if os.environ.get(NVFP4_FAKE_QAT_FLAG, "0") != "1":
        return weight_tensors
    # resolved at call time, so that processes which never enable the switch do not load the kernels
    from miles_amd.kernels.quant import nvfp4_qdq

    config = nvfp4_qdq.current_nvfp4_qdq_config()
    return [nvfp4_qdq.fake_nvfp4_quantization_ste(w, config) for w in weight_tensors]


__all__ = ["NVFP4_FAKE_QAT_FLAG", "maybe_fake_quantize_nvfp4_weight_tensors"]
