"""MXFP4 routed experts -> uniform block-wise FP8 checkpoint.

    python -m miles_amd.tools.convert_mxfp4_to_fp8 --model-dir SRC --save-dir DST [--device cuda]

Mirror of the reference's tools/convert_mxfp4_to_fp8.py: `cast_e2m1fn_to_e4m3fn` (:30-49) re-codes packed e2m1
weights with 1x32 E8M0 scales as e4m3fn with one fp32 scale per 128x128 tile; `main` (:52-99) applies it to every
int8 `.weight` that has a `.scale` partner, copies everything else and drops `expert_dtype` from config.json.  The
reference expands the codes through a table and rescales with torch ops; here the cast is one gfx950 kernel.
"""

from __future__ import annotations

import glob
import json
import os
import shutil
from argparse import ArgumentParser
from pathlib import Path

import torch
from safetensors import safe_open
from safetensors.torch import load_file, save_file

from miles_amd import _lib, launch


def cast_e2m1fn_to_e4m3fn(x: torch.Tensor, scale: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """int8 [out, in/2] (two e2m1 codes per byte, even element low) + E8M0 scales [out, in/32]
    -> (float8_e4m3fn [out, in], float32 [out/128, in/128])."""
    assert x.dtype == torch.int8 and x.ndim == 2
    out_dim, in_dim = x.size(0), x.size(1) * 2
    assert out_dim % 128 == 0 and in_dim % 128 == 0
    assert scale.shape == (out_dim, in_dim // 32), f"{scale.shape=} {x.shape=}"
    _lib.require_gpu(x, "cast_e2m1fn_to_e4m3fn")
    if scale.element_size() != 1:
        raise _lib.MilesQuantError(f"cast_e2m1fn_to_e4m3fn expects one-byte E8M0 scales, got {scale.dtype}")
    packed, sbytes = x.contiguous(), scale.contiguous().view(torch.uint8)
    if packed.data_ptr() % 16:        # the kernel reads whole 16-byte pieces: a view that starts mid-allocation is moved first
        packed = packed.clone()
    y = torch.empty((out_dim, in_dim), dtype=torch.float8_e4m3fn, device=x.device)
    tile_scale = torch.empty((out_dim // 128, in_dim // 128), dtype=torch.float32, device=x.device)
    # a job of the batched driver: inside `launch.deferred()` the casts of a whole shard share grouped launches
    launch.submit(_lib.JOB_MXFP4_TO_FP8, packed, y, tile_scale, sbytes, None, out_dim, in_dim, in_dim)
    return y, tile_scale


def _copy_side_files(model_dir: Path, save_dir: Path) -> None:
    """config.json without `expert_dtype`, tokenizer / chat template / generation config as they are."""
    config = json.loads((model_dir / "config.json").read_text())
    for holder in (config, config.get("quantization_config")):
        if isinstance(holder, dict):
            holder.pop("expert_dtype", None)
    (save_dir / "config.json").write_text(json.dumps(config, indent=2) + "\n")
    for pattern in ("tokenizer*", "chat_template*", "generation_config.json"):
        for path in glob.glob(str(model_dir / pattern)):
            target = save_dir / os.path.basename(path)
            if os.path.isdir(path):
                shutil.copytree(path, target, dirs_exist_ok=True)
            else:
                shutil.copy(path, target)


def _packed_fp4_weights(model_dir: Path, shard_names: list[str]) -> set[str]:
    """Names of the int8 tensors (packed e2m1 pairs); the reference recognises them by dtype alone."""
    found = set()
    for shard_name in shard_names:
        with safe_open(str(model_dir / shard_name), framework="pt") as f:
            for name in f.keys():
                if f.get_slice(name).get_dtype() == "I8":
                    assert name.endswith(".weight"), f"unexpected int8 tensor {name}"
                    found.add(name)
    return found


def main(model_dir: str, save_dir: str, device: str = "cuda") -> None:
    src, dst = Path(model_dir), Path(save_dir)
    dst.mkdir(parents=True, exist_ok=True)
    _copy_side_files(src, dst)
    weight_map = dict(json.loads((src / "model.safetensors.index.json").read_text())["weight_map"])
    shard_names = sorted(set(weight_map.values()))
    fp4_weights = _packed_fp4_weights(src, shard_names)
    scale_of = {name: name.removesuffix(".weight") + ".scale" for name in fp4_weights}
    fp4_scales = set(scale_of.values())
    for shard_name in shard_names:
        state = load_file(str(src / shard_name), device=device)
        converted = {}
        with launch.deferred():     # the shard's casts are submitted together when the block ends
            for name, tensor in state.items():
                if name in fp4_scales:
                    continue            # re-emitted next to its weight
                if name not in fp4_weights:
                    converted[name] = tensor
                    continue
                scale_name = scale_of[name]
                scale = state[scale_name] if scale_name in state else \
                    load_file(str(src / weight_map[scale_name]), device=device)[scale_name]
                converted[name], converted[scale_name] = cast_e2m1fn_to_e4m3fn(tensor, scale)
                weight_map[scale_name] = shard_name
        save_file(converted, str(dst / shard_name))
    (dst / "model.safetensors.index.json").write_text(json.dumps({"metadata": {}, "weight_map": weight_map}, indent=2) + "\n")
    assert fp4_weights, "no packed-fp4 expert weights found; is this already an FP8 checkpoint?"
    print(f"cast {len(fp4_weights)} expert weights to fp8, saved to {save_dir}")


if __name__ == "__main__":
    parser = ArgumentParser()
    parser.add_argument("--model-dir", type=str, required=True)
    parser.add_argument("--save-dir", type=str, required=True)
    parser.add_argument("--device", type=str, default="cuda")
    args = parser.parse_args()
    main(args.model_dir, args.save_dir, args.device)
