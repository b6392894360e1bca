"""compressed-tensors INT4 (pack-quantized, symmetric) MoE experts -> BF16 checkpoint.

    python -m miles_amd.tools.convert_kimi_int4_to_bf16 --model-dir SRC [--output-dir DST] [--files F ...]
                                                        [--config-path CFG] [--overwrite]

Mirror of the reference's tools/convert_kimi_int4_to_bf16.py: `_load_config` (:39-54), `_dequantize_tensor`
(:57-86), `_is_quantized_weight_key` (:89-98), `convert_file` (:101-157) and the CLI (:160-246).  The reference
unpacks with compressed-tensors' `unpack_from_int32` and multiplies by the repeated scales with torch ops;
here both are one gfx950 kernel.
"""

from __future__ import annotations

import argparse
import json
import os
import shutil
from collections import defaultdict

import torch
from safetensors.torch import safe_open, save_file

from miles_amd import _lib, launch


def _load_config(model_dir: str, config_path: str | None) -> tuple[int, int, int]:
    """hidden_size, moe_intermediate_size and the INT4 group size (default 128) from config.json."""
    with open(config_path or os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    loader = cfg.get("text_config", cfg)
    weights = loader.get("quantization_config", {}).get("config_groups", {}).get("group_0", {}).get("weights", {})
    return int(loader.get("hidden_size")), int(loader.get("moe_intermediate_size")), int(weights.get("group_size", 128))


def _dequantize_tensor(weight_packed: torch.Tensor, weight_scale: torch.Tensor, weight_shape, group_size: int) -> torch.Tensor:
    """int32 [M, ceil(K/8)] codes + [M, K/group_size] scales -> bfloat16 [M, K] = bf16((code - 8) * f32(scale))."""
    if isinstance(weight_shape, torch.Tensor):
        shape = tuple(int(v) for v in weight_shape.view(-1).tolist())
    else:
        shape = tuple(weight_shape)
    _lib.require_gpu(weight_packed, "_dequantize_tensor")
    if group_size <= 0:
        raise NotImplementedError("per-element scales (group_size <= 0) are not implemented on gfx950")
    M, K = shape
    packed = weight_packed.contiguous()
    if packed.dtype != torch.int32 or tuple(packed.shape) != (M, -(-K // 8)):
        raise ValueError(f"Packed shape {tuple(packed.shape)} / dtype {packed.dtype} incompatible with weight shape {shape}")
    scale = weight_scale.contiguous()
    if scale.dim() == 1:
        scale = scale.unsqueeze(1)
    if K % group_size != 0 or scale.numel() != M * (K // group_size):
        raise ValueError(f"Scale shape {tuple(scale.shape)} incompatible with weight shape {shape}")
    out = torch.empty((M, K), dtype=torch.bfloat16, device=packed.device)
    launch.note_direct_call()
    rc = _lib.load().mq_int4_unpack_dequant(packed.data_ptr(), scale.data_ptr(), _lib.dtype_code(scale, "_dequantize_tensor"),
                                            out.data_ptr(), M, K, int(group_size), _lib.stream_ptr(packed.device))
    _lib.check(rc)
    return out


def _is_quantized_weight_key(key: str) -> bool:
    """Routed-expert gate/up/down tensors stored as weight_packed / weight_scale / weight_shape."""
    if ".mlp.experts." not in key or ".shared_experts." in key:
        return False
    return any(key.endswith(f".{proj}.{suffix}") for proj in ("gate_proj", "up_proj", "down_proj")
               for suffix in ("weight_packed", "weight_scale", "weight_shape"))


def convert_file(input_path: str, output_path: str, group_size: int, skip_existing: bool = True, device: str = "cuda"):
    """One shard: every complete (packed, scale, shape) triple becomes `<prefix>.<proj>.weight` in bfloat16;
    incomplete triples and all other tensors are copied."""
    if skip_existing and os.path.exists(output_path):
        return
    tensors = {}
    experts = defaultdict(lambda: defaultdict(dict))
    with safe_open(input_path, framework="pt", device=device) as reader:
        for key in reader.keys():
            tensor = reader.get_tensor(key)
            parts = key.split(".")
            if not _is_quantized_weight_key(key) or "experts" not in parts:
                tensors[key] = tensor
                continue
            prefix = ".".join(parts[: parts.index("experts") + 2])
            experts[prefix][parts[-2]][parts[-1]] = tensor
    for prefix, components in experts.items():
        for proj in ("gate_proj", "up_proj", "down_proj"):
            data = components.get(proj, {})
            if not {"weight_packed", "weight_scale", "weight_shape"}.issubset(data):
                for suffix, value in data.items():
                    tensors[f"{prefix}.{proj}.{suffix}"] = value
                continue
            tensors[f"{prefix}.{proj}.weight"] = _dequantize_tensor(
                data["weight_packed"].to(torch.int32), data["weight_scale"].to(torch.float32), data["weight_shape"], group_size)
    os.makedirs(os.path.dirname(output_path), exist_ok=True)
    save_file({k: v.cpu().contiguous() for k, v in tensors.items()}, output_path)


def parse_args(argv=None) -> argparse.Namespace:
    parser = argparse.ArgumentParser(description="Convert INT4 pack-quantized MoE experts to BF16 weights.")
    parser.add_argument("--model-dir", required=True)
    parser.add_argument("--output-dir", default=None, help="default: <model-dir>_bf16")
    parser.add_argument("--files", nargs="+", default=None)
    parser.add_argument("--config-path", default=None)
    parser.add_argument("--overwrite", action="store_true")
    return parser.parse_args(argv)


def main(argv=None) -> None:
    args = parse_args(argv)
    model_dir = os.path.abspath(args.model_dir)
    output_dir = os.path.abspath(args.output_dir or f"{model_dir}_bf16")
    if not os.path.isdir(model_dir):
        raise FileNotFoundError(f"Model directory not found: {model_dir}")
    _, _, group_size = _load_config(model_dir, args.config_path)
    names = args.files or [n for n in sorted(os.listdir(model_dir)) if n.endswith(".safetensors")]
    if not names:
        print("No safetensors checkpoints found.")
        return
    for name in names:
        path = os.path.join(model_dir, name)
        if os.path.isfile(path):
            convert_file(path, os.path.join(output_dir, os.path.relpath(path, model_dir)), group_size,
                         skip_existing=not args.overwrite)
    for fname in os.listdir(model_dir):
        if fname == "model.safetensors.index.json":
            continue
        if fname.startswith("tokenizer") or fname.endswith((".json", ".py", ".jinja", ".model")):
            shutil.copy2(os.path.join(model_dir, fname), os.path.join(output_dir, fname))
    weight_map = {}
    for fname in sorted(os.listdir(output_dir)):
        if fname.endswith(".safetensors"):
            with safe_open(os.path.join(output_dir, fname), framework="pt") as reader:
                for key in reader.keys():
                    weight_map[key] = fname
    with open(os.path.join(output_dir, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {}, "weight_map": weight_map}, f, indent=2)
    print(f"\nSuccessful! Output saved to: {output_dir}")


if __name__ == "__main__":
    main()
