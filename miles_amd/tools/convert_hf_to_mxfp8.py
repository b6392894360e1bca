"""MXFP8 offline converter (UE8M0 scales, 1x32 groups).

    python -m miles_amd.tools.convert_hf_to_mxfp8 --model-dir SRC --save-dir DST [--device cuda]
        [--num-layers-at-start-in-bf16 N] [--num-layers-at-end-in-bf16 N] [--extra-high-precision-layers-hf ...]

Mirror of the reference's tools/convert_hf_to_mxfp8.py (`process_file` :123-228, `convert_mxfp8` :231-308).
Sources: BF16/FP16/FP32 checkpoints, and block-scaled FP8 checkpoints whose [128,128] scales are powers of two
(`scale_fmt: ue8m0`): those are re-labelled without touching the codes (`_source_fp8_to_mxfp8_scale_u8`,
:98-102).  FP8 sources with general fp32 scales need SGLang's `block_quant_dequant` in the reference; here
they are dequantized by the FP8 block dequant kernel's arithmetic in fp32 torch ops on the device and
re-quantized.
"""

from __future__ import annotations

import argparse
import os
import re

import torch

from miles_amd import launch
from miles_amd.tools import _checkpoint as ckpt
from miles_amd.tools.fp8_cast_bf16 import weight_dequant
from miles_amd.utils.mxfp8 import (MXFP8_GROUP_SIZE, MXFP8_SKIP_WEIGHT_SUBSTRINGS, MXFP8_SOURCE_FP8_DTYPES,
                                   should_use_mxfp8)
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


def _tile_counts(weight: torch.Tensor) -> tuple[int, int]:
    n, k = weight.shape[-2], weight.shape[-1]
    return -(-n // SOURCE_FP8_BLOCK_SIZE[0]), -(-k // SOURCE_FP8_BLOCK_SIZE[1])


def _load_source_scale_u8(weights, weight_key, weight, source_scale_index, input_path, device, current_filename):
    """(fp32 scales, uint8 exponents or None, scale key) of a source FP8 weight."""
    scale_key = _strip_weight_suffix(weight_key) + SOURCE_FP8_SCALE_KEY_SUFFIX
    scale_file = source_scale_index[scale_key]
    scale = weights[scale_key] if scale_file == current_filename and scale_key in weights else \
        ckpt.load_tensor(input_path, scale_file, scale_key, device)
    nt, kt = _tile_counts(weight)
    if scale.dtype == torch.uint8:
        u8 = scale[..., :nt, :kt].contiguous()
        return (u8.to(torch.int32) << 23).view(torch.float32), u8, scale_key
    assert scale.dtype == torch.float32
    f32 = scale[..., :nt, :kt].contiguous()
    bits = f32.view(torch.int32)
    pow2 = not torch.any((bits & 0x007FFFFF) != 0).item() and not torch.any(bits < 0).item()
    return f32, (((bits >> 23) & 0xFF).to(torch.uint8) if pow2 else None), scale_key


def _source_fp8_to_mxfp8_scale_u8(weight: torch.Tensor, source_scale_u8: torch.Tensor) -> torch.Tensor:
    """One exponent per 128x128 tile -> one per 1x32 group (repeat 128 down, 4 across), cropped."""
    n, k = weight.shape[-2], weight.shape[-1]
    wide = source_scale_u8.repeat_interleave(SOURCE_FP8_BLOCK_SIZE[0], dim=-2).repeat_interleave(
        SOURCE_FP8_BLOCK_SIZE[1] // TARGET_MXFP8_BLOCK_SIZE[1], dim=-1)
    return wide[..., :n, : k // TARGET_MXFP8_BLOCK_SIZE[1]].contiguous()


def _dequant_fp32(weight: torch.Tensor, scale_fp32: torch.Tensor) -> torch.Tensor:
    n, k = weight.shape
    wide = scale_fp32.repeat_interleave(128, dim=0)[:n].repeat_interleave(128, dim=1)[:, :k]
    return (weight.float() * wide).contiguous()


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

    def source_scale(key, tensor):
        return _load_source_scale_u8(weights, key, tensor, source_scale_index, input_path, device, filename)

    with launch.deferred():
        for key, tensor in weights.items():
            if not key.endswith(".weight"):
                continue
            fp8_source = source_is_block_fp8_ue8m0 and tensor.dtype in MXFP8_SOURCE_FP8_DTYPES
            if should_use_mxfp8(key, tuple(tensor.shape), tensor.dtype, skip_substrings=skip_substrings,
                                allow_source_fp8=source_is_block_fp8_ue8m0):
                if fp8_source:
                    scale_f32, scale_u8, scale_key = source_scale(key, tensor)
                    if scale_u8 is not None:
                        out[key], out[scale_key] = tensor.contiguous(), _source_fp8_to_mxfp8_scale_u8(tensor, scale_u8)
                    else:
                        out[key], out[scale_key] = quantize_mxfp8(_dequant_fp32(tensor, scale_f32))
                else:
                    out[key], out[_strip_weight_suffix(key) + SOURCE_FP8_SCALE_KEY_SUFFIX] = quantize_mxfp8(tensor)
            else:
                if ".experts." not in key:
                    skipped.append(_strip_weight_suffix(key))
                if fp8_source:
                    scale_f32, _, _ = source_scale(key, tensor)
                    out[key] = weight_dequant(tensor.contiguous(), scale_f32)
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
    args, _ = ap.parse_known_args(argv)
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
