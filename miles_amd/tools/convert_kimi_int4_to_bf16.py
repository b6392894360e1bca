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
import re
import shutil

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
    M, K = shape
    if group_size <= 0:                 # one scale per element (:75-76): the same kernel with groups of one column
        if weight_scale.numel() != M * K:
            raise ValueError(f"Scale shape {tuple(weight_scale.shape)} incompatible with weight shape {shape}")
        weight_scale, group_size = weight_scale.reshape(M, K), 1
    packed = weight_packed.contiguous()
    if packed.dtype != torch.int32 or tuple(packed.shape) != (M, -(-K // 8)):
        raise ValueError(f"Packed shape {tuple(packed.shape)} / dtype {packed.dtype} incompatible with weight shape {shape}")
    scale = weight_scale.contiguous()
    if scale.dim() == 1:
        scale = scale.unsqueeze(1)
    if K % group_size != 0 or scale.numel() != M * (K // group_size):
        raise ValueError(f"Scale shape {tuple(scale.shape)} incompatible with weight shape {shape}")
    out = torch.empty((M, K), dtype=torch.bfloat16, device=packed.device)
    # a job of the batched driver: inside `launch.deferred()` the experts of a whole shard share grouped launches
    launch.submit(_lib.JOB_INT4_UNPACK, packed, out, None, scale, None, M, K, K, int(group_size),
                  dtype=_lib.dtype_code(scale, "_dequantize_tensor"))
    return out


_PROJECTIONS = ("gate_proj", "up_proj", "down_proj")
_FIELDS = ("weight_packed", "weight_scale", "weight_shape")
# <anything>.mlp.experts.<e>.<proj>.<field>, but nothing under a shared expert
_TRIPLE_MEMBER = re.compile(r"^(?P<expert>.*\.mlp\.experts\.[^.]+)(?:\..*)?\.(?P<proj>%s)\.(?P<field>%s)$"
                            % ("|".join(_PROJECTIONS), "|".join(_FIELDS)))


def _is_quantized_weight_key(key: str) -> bool:
    """A routed expert's gate / up / down projection stored as weight_packed / weight_scale / weight_shape."""
    return ".shared_experts." not in key and _TRIPLE_MEMBER.match(key) is not None


def convert_file(input_path: str, output_path: str, group_size: int, skip_existing: bool = True, device: str = "cuda"):
    """One shard: a projection whose three fields are all present becomes `<expert>.<proj>.weight` in bfloat16;
    everything else, fields of incomplete projections included, is carried over under its own name."""
    if skip_existing and os.path.exists(output_path):
        return
    carried: dict[str, torch.Tensor] = {}
    fields_of: dict[tuple[str, str], dict[str, torch.Tensor]] = {}
    with safe_open(input_path, framework="pt", device=device) as shard:
        for key in shard.keys():
            member = _TRIPLE_MEMBER.match(key) if _is_quantized_weight_key(key) else None
            if member is None:
                carried[key] = shard.get_tensor(key)
            else:
                module = (key[: member.start("proj") - 1], member["proj"])        # (expert prefix, projection)
                fields_of.setdefault(module, {})[member["field"]] = shard.get_tensor(key)
    with launch.deferred():         # the shard's projections are unpacked together when the block ends
        for (expert, proj), fields in fields_of.items():
            if len(fields) < len(_FIELDS):
                carried.update({f"{expert}.{proj}.{field}": value for field, value in fields.items()})
                continue
            carried[f"{expert}.{proj}.weight"] = _dequantize_tensor(fields["weight_packed"].to(torch.int32),
                                                                    fields["weight_scale"].to(torch.float32),
                                                                    fields["weight_shape"], group_size)
    os.makedirs(os.path.dirname(output_path), exist_ok=True)
    save_file({name: t.cpu().contiguous() for name, t in carried.items()}, output_path)


def parse_args(argv=None) -> argparse.Namespace:
    p = argparse.ArgumentParser(description="Convert INT4 pack-quantized MoE experts to BF16 weights.")
    p.add_argument("--model-dir", required=True)
    p.add_argument("--output-dir", default=None, help="default: <model-dir>_bf16")
    p.add_argument("--files", nargs="+", default=None)
    p.add_argument("--config-path", default=None)
    p.add_argument("--overwrite", action="store_true")
    return p.parse_args(argv)


_SIDE_FILE_SUFFIXES = (".json", ".py", ".jinja", ".model")


def _finish(model_dir: str, output_dir: str) -> None:
    """Tokenizer / config / code files next to the shards, and an index rebuilt from the shards that were written."""
    for name in os.listdir(model_dir):
        if name != "model.safetensors.index.json" and (name.startswith("tokenizer") or name.endswith(_SIDE_FILE_SUFFIXES)):
            shutil.copy2(os.path.join(model_dir, name), os.path.join(output_dir, name))
    owner = {}
    for name in sorted(n for n in os.listdir(output_dir) if n.endswith(".safetensors")):
        with safe_open(os.path.join(output_dir, name), framework="pt") as shard:
            owner.update(dict.fromkeys(shard.keys(), name))
    with open(os.path.join(output_dir, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {}, "weight_map": owner}, f, indent=2)


def main(argv=None) -> None:
    args = parse_args(argv)
    model_dir = os.path.abspath(args.model_dir)
    if not os.path.isdir(model_dir):
        raise FileNotFoundError(f"Model directory not found: {model_dir}")
    output_dir = os.path.abspath(args.output_dir or model_dir + "_bf16")
    group_size = _load_config(model_dir, args.config_path)[2]
    shards = args.files or sorted(n for n in os.listdir(model_dir) if n.endswith(".safetensors"))
    if not shards:
        print("No safetensors checkpoints found.")
        return
    for name in shards:
        source = os.path.join(model_dir, name)
        if os.path.isfile(source):
            convert_file(source, os.path.join(output_dir, os.path.relpath(source, model_dir)), group_size,
                         skip_existing=not args.overwrite)
    _finish(model_dir, output_dir)
    print(f"\nSuccessful! Output saved to: {output_dir}")


if __name__ == "__main__":
    main()
