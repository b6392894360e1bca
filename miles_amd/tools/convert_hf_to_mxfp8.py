"""MXFP8 offline converter (UE8M0 scales, 1x32 groups).

    python -m miles_amd.tools.convert_hf_to_mxfp8 --model-dir SRC --save-dir DST [--device cuda]
        [--num-layers-at-start-in-bf16 N] [--num-layers-at-end-in-bf16 N] [--extra-high-precision-layers-hf ...]
        [--metadata-only]

Mirror of the reference's tools/convert_hf_to_mxfp8.py (`process_file` :123-228, `convert_mxfp8` :231-308).
Sources: BF16/FP16/FP32 checkpoints, and block-scaled FP8 checkpoints (`scale_fmt: ue8m0`, [128,128] scales stored
as exponent bytes or as fp32).  A tensor whose tile scales are powers of two keeps its codes and gets one exponent
byte per 1x32 group (`_source_fp8_to_mxfp8_scale_u8`, :98-102: `mq_e8m0_expand_tile_scales`); a tensor with any other
scale is dequantized to fp32 and quantized again in the reference (SGLang's `block_quant_dequant`, :187-190), which
`mq_fp8_block_to_mxfp8` does in one pass over the codes; a tensor that stays in bf16 goes through the FP8 block
dequantizer (:203-215).  The power-of-two test (:81-86) runs on the device, one flag per tensor, read once per shard.
"""

from __future__ import annotations

import argparse
import os
import re

import torch

from miles_amd import launch
from miles_amd.tools import _checkpoint as ckpt
from miles_amd.utils.hf_rollout_schema import create_mxfp8_rollout_schema
from miles_amd.utils.mxfp8 import (MXFP8_GROUP_SIZE, MXFP8_SKIP_WEIGHT_SUBSTRINGS, MXFP8_SOURCE_FP8_DTYPES,
                                   dequantize_fp8_source, expand_tile_scales_e8m0, exponent_bytes_to_fp32,
                                   fp8_tile_scales_pow2, requantize_fp8_block_to_mxfp8, should_use_mxfp8)
from miles_amd.utils.mxfp8 import mxfp8_quantize as quantize_mxfp8

SOURCE_FP8_BLOCK_SIZE = [128, 128]
TARGET_MXFP8_BLOCK_SIZE = [1, MXFP8_GROUP_SIZE]
SOURCE_FP8_SCALE_KEY_SUFFIX = ".weight_scale_inv"


def _strip_weight_suffix(weight_key: str) -> str:
    if not weight_key.endswith(".weight"):
        raise ValueError(f"Expected key ending with '.weight', got: {weight_key}")
    return weight_key[: -len(".weight")]


def _source_kind(cfg: dict) -> str:
    """'bf16' or 'fp8_ue8m0'; anything else is refused (reference :39-54, :245-254)."""
    qcfg = cfg.get("quantization_config", {}) if isinstance(cfg, dict) else {}
    if (isinstance(qcfg, dict) and qcfg.get("quant_method") == "fp8"
            and list(qcfg.get("weight_block_size", [])) == SOURCE_FP8_BLOCK_SIZE and qcfg.get("scale_fmt") == "ue8m0"):
        return "fp8_ue8m0"
    if not isinstance(qcfg, dict) or not qcfg or qcfg.get("quant_method") in (None, "", "bf16"):
        return "bf16"
    raise ValueError("Unsupported source quantization_config. Only BF16/FP16/FP32 sources and "
                     "{quant_method=fp8, weight_block_size=[128, 128], scale_fmt=ue8m0} sources are supported.")


def _source_scale(weights, weight_key, source_scale_index, input_path, device, current_filename):
    """(tile-scale tensor as stored -- uint8 exponents or fp32 --, its key) of a source FP8 weight; the tensor may sit in
    another shard (reference :65-72)."""
    scale_key = _strip_weight_suffix(weight_key) + SOURCE_FP8_SCALE_KEY_SUFFIX
    scale_file = source_scale_index[scale_key]
    if scale_file == current_filename and scale_key in weights:
        return weights[scale_key], scale_key
    return ckpt.load_tensor(input_path, scale_file, scale_key, device), scale_key


def process_file(input_path, output_path, filename, result_collector, device, num_hidden_layers,
                 num_layers_at_start_in_bf16, num_layers_at_end_in_bf16, source_is_block_fp8_ue8m0,
                 extra_high_precision_layers_hf, source_scale_index) -> None:
    weights = ckpt.load_shard(input_path, filename, device)
    out: dict[str, torch.Tensor] = {}
    bf16_layers = sorted({f"model.layers.{i}." for i in range(0, num_layers_at_start_in_bf16)} |
                         {f"model.layers.{i}." for i in range(num_hidden_layers - num_layers_at_end_in_bf16,
                                                             num_hidden_layers)})
    skipped: list[str] = list(bf16_layers) if (num_layers_at_end_in_bf16 > 0 or num_layers_at_start_in_bf16 > 0) else []
    skip_substrings = (*MXFP8_SKIP_WEIGHT_SUBSTRINGS, *extra_high_precision_layers_hf, *bf16_layers)

    # what becomes of every .weight tensor: "quantize" (a high-precision source), "keep" (passed through), or, for the
    # FP8 tensors of a block-scaled source, "relabel" (power-of-two tile scales: codes kept, one exponent per group),
    # "requantize" (any other scales) and "dequantize" (a module that stays in bf16)
    plan: dict[str, tuple] = {}
    undecided = []            # FP8 tensors with fp32 scales: relabel or requantize, by the power-of-two test
    for key, tensor in weights.items():
        if not key.endswith(".weight"):
            continue
        fp8_source = source_is_block_fp8_ue8m0 and tensor.dtype in MXFP8_SOURCE_FP8_DTYPES
        quantized = should_use_mxfp8(key, tuple(tensor.shape), tensor.dtype, skip_substrings=skip_substrings,
                                     allow_source_fp8=source_is_block_fp8_ue8m0)
        if not quantized and ".experts." not in key:
            skipped.append(_strip_weight_suffix(key))
        if not fp8_source:
            plan[key] = ("quantize" if quantized else "keep", None, None)
            continue
        scale, scale_key = _source_scale(weights, key, source_scale_index, input_path, device, filename)
        if not quantized:
            plan[key] = ("dequantize", scale if scale.dtype == torch.float32 else exponent_bytes_to_fp32(scale), None)
        elif scale.dtype == torch.uint8:
            plan[key] = ("relabel", scale, scale_key)
        else:
            assert scale.dtype == torch.float32
            plan[key] = ("requantize", scale, scale_key)
            undecided.append(key)
    for key, pow2 in zip(undecided, fp8_tile_scales_pow2((weights[k], plan[k][1]) for k in undecided)):
        if pow2:
            plan[key] = ("relabel", *plan[key][1:])

    with launch.deferred():
        for key, (action, scale, scale_key) in plan.items():
            tensor = weights[key]
            if action == "quantize":
                out[key], out[_strip_weight_suffix(key) + SOURCE_FP8_SCALE_KEY_SUFFIX] = quantize_mxfp8(tensor)
            elif action == "relabel":
                out[key], out[scale_key] = tensor.contiguous(), expand_tile_scales_e8m0(tensor, scale)
            elif action == "requantize":
                out[key], out[scale_key] = requantize_fp8_block_to_mxfp8(tensor, scale)
            elif action == "dequantize":
                out[key] = dequantize_fp8_source(tensor, scale)
            else:
                out[key] = tensor
    for key, tensor in weights.items():
        if key.endswith(".weight"):
            continue
        if source_is_block_fp8_ue8m0 and key.endswith(SOURCE_FP8_SCALE_KEY_SUFFIX):
            continue  # the source's block scales are replaced, not copied
        out[key] = tensor
    ckpt.save_shard(out, output_path, filename)
    result_collector.add(filename, out, skipped)


def _natural_key(s: str):
    return [int(t) if t.isdigit() else t for t in re.findall(r"\d+|\D+", s)]


def convert_mxfp8(model_dir, save_dir, device, num_layers_at_start_in_bf16=0, num_layers_at_end_in_bf16=0,
                  extra_high_precision_layers_hf=()) -> None:
    import json

    input_path, output_path = os.path.abspath(model_dir), os.path.abspath(save_dir)
    os.makedirs(output_path, exist_ok=True)
    cfg = ckpt.read_config(input_path)
    if cfg is None:
        raise FileNotFoundError(os.path.join(input_path, "config.json"))
    num_hidden_layers = int(cfg["num_hidden_layers"])
    from_fp8 = _source_kind(cfg) == "fp8_ue8m0"
    ckpt.copy_side_files(input_path, output_path)
    with open(os.path.join(input_path, "model.safetensors.index.json")) as f:
        weight_map = json.load(f)["weight_map"]
    scale_index = {k: v for k, v in weight_map.items() if k.endswith(SOURCE_FP8_SCALE_KEY_SUFFIX)} if from_fp8 else {}
    results = ckpt.ShardResults(size_in_bytes=True)
    for filename in sorted(set(weight_map.values())):
        process_file(input_path, output_path, filename, results, device, num_hidden_layers,
                     num_layers_at_start_in_bf16, num_layers_at_end_in_bf16, from_fp8,
                     tuple(extra_high_precision_layers_hf), scale_index)
    qcfg = {"activation_scheme": "dynamic", "fmt": "e4m3", "quant_method": "mxfp8",
            "weight_block_size": TARGET_MXFP8_BLOCK_SIZE, "scale_fmt": "ue8m0"}
    if results.modules_to_not_convert:
        qcfg["modules_to_not_convert"] = sorted(set(results.modules_to_not_convert), key=_natural_key)
    cfg["quantization_config"] = qcfg
    ckpt.write_config(output_path, cfg)
    ckpt.write_index(output_path, results.weight_map, results.total_size)


def main(argv=None) -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--model-dir", type=str, required=True, help="Path to HF safetensors model.")
    ap.add_argument("--save-dir", type=str, required=True, help="Path to save converted model.")
    ap.add_argument("--device", type=str, default="cuda")
    ap.add_argument("--num-layers-at-start-in-bf16", type=int, default=0)
    ap.add_argument("--num-layers-at-end-in-bf16", type=int, default=0)
    ap.add_argument("--extra-high-precision-layers-hf", type=str, nargs="*", default=())
    ap.add_argument("--metadata-only", action="store_true",
                    help="Write a weightless MXFP8 rollout schema (config + tokenizer) instead of converting weights.")
    args, _ = ap.parse_known_args(argv)
    if args.metadata_only:      # host work only: no device, no kernel (reference :359-362)
        schema = create_mxfp8_rollout_schema(args.model_dir, args.save_dir)
        print(f"Created metadata-only MXFP8 rollout schema at {schema}")
        return
    if not torch.cuda.is_available():
        raise RuntimeError("CUDA is not available, cannot run MXFP8 quantization.")
    device = torch.device(f"cuda:{args.device}" if args.device.isdigit() else args.device)
    if device.type != "cuda":
        raise RuntimeError("MXFP8 quantization requires a CUDA device.")
    if device.index is None:
        device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    if os.path.exists(args.save_dir) and not os.path.isdir(args.save_dir):
        raise ValueError("The save_dir should be a directory.")
    convert_mxfp8(args.model_dir, args.save_dir, str(device), args.num_layers_at_start_in_bf16,
                  args.num_layers_at_end_in_bf16,
                  tuple(s.strip() for s in args.extra_high_precision_layers_hf if isinstance(s, str) and s.strip()))


if __name__ == "__main__":
    main()
