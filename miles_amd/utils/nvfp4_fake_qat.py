"""Training-side switch: put NVFP4 fake quantization in front of the weights of a grouped linear layer.

Surface of the reference's miles/utils/nvfp4_fake_qat.py:10-23.  While the environment variable named by
NVFP4_FAKE_QAT_FLAG is "1", `maybe_fake_quantize_nvfp4_weight_tensors` swaps every weight of the list it is given
for its quantize-dequantize image (gradients pass straight through); the q-dq options are read from the environment
once per call, not once per weight.  With any other value the caller gets its own list object back untouched.
"""

from __future__ import annotations

import os

import torch

NVFP4_FAKE_QAT_FLAG = "OPEN_TRAINING_NVFP4_FAKE_QAT_FLAG"
__all__ = ["NVFP4_FAKE_QAT_FLAG", "maybe_fake_quantize_nvfp4_weight_tensors"]


def _switched_on() -> bool:
    return os.environ.get(NVFP4_FAKE_QAT_FLAG, "0") == "1"


def maybe_fake_quantize_nvfp4_weight_tensors(weight_tensors: list[torch.Tensor]) -> list[torch.Tensor]:
    if _switched_on():
        # looked up here, not at import: a process that never flips the switch never loads the kernels
        from miles_amd.kernels.quant import nvfp4_qdq as qdq

        options = qdq.current_nvfp4_qdq_config()
        weight_tensors = [qdq.fake_nvfp4_quantization_ste(weight, options) for weight in weight_tensors]
    return weight_tensors
