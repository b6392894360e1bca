"""Weightless MXFP8 "rollout schema": the config / tokenizer directory an inference engine needs to allocate an MXFP8
model that the weight sync then fills, without converting a single tensor.

Host-only counterpart of the reference's `miles/utils/hf_rollout_schema.py` (`build_mxfp8_quantization_config` :46-85,
`create_mxfp8_rollout_schema` :88-117).  Everything is decided from safetensors headers (name, shape, dtype string) with
`should_use_mxfp8`, the same predicate the live quantizer and the offline converter use, so the allocation the engine
makes and the tensors the sync produces agree.  The reference renames checkpoint tensors through a model-specific table
that lives in SGLang (`hf_utils/weight_mapping.py:80-96`: identity for every model but native DeepSeek-V4 checkpoints);
here that table is the `remap` argument, identity by default.
"""

from __future__ import annotations

import json
import re
import shutil
from collections import defaultdict
from collections.abc import Callable
from pathlib import Path

import torch
from safetensors import safe_open

from miles_amd.utils.mxfp8 import MXFP8_GROUP_SIZE, should_use_mxfp8

WEIGHT_INDEX_NAME = "model.safetensors.index.json"

# safetensors header dtype strings of tensors that can be (or already are) MXFP8 sources; any other dtype is not
_DTYPE_OF_HEADER = {"BF16": torch.bfloat16, "F16": torch.float16, "F32": torch.float32,
                    "F8_E4M3": torch.float8_e4m3fn, "I8": torch.int8}


def checkpoint_weight_map(checkpoint: Path) -> dict[str, str]:
    """tensor name -> shard file, from the index when there is one, else from the headers of every `*.safetensors`
    (reference `hf_utils/weight_mapping.py:59-77`).  No payload is read."""
    index = checkpoint / WEIGHT_INDEX_NAME
    if index.is_file():
        return json.loads(index.read_text(encoding="utf-8"))["weight_map"]
    found: dict[str, str] = {}
    for shard in sorted(checkpoint.glob("*.safetensors")):
        with safe_open(shard, framework="pt", device="cpu") as reader:
            for name in reader.keys():
                if name in found:
                    raise ValueError(f"Duplicate tensor {name} in {found[name]} and {shard.name}")
                found[name] = shard.name
    if not found:
        raise FileNotFoundError(f"No safetensors weights or index under {checkpoint}")
    return found


def _header_layouts(checkpoint: Path, weight_map: dict[str, str]) -> dict[str, tuple[tuple[int, ...], str]]:
    """(shape, header dtype string) of every tensor of the map, shard by shard."""
    by_shard: dict[str, list[str]] = defaultdict(list)
    for name, shard in weight_map.items():
        by_shard[shard].append(name)
    layouts = {}
    for shard, names in by_shard.items():
        with safe_open(checkpoint / shard, framework="pt", device="cpu") as reader:
            present = set(reader.keys())
            for name in names:
                if name not in present:
                    raise KeyError(f"{name} is listed in {WEIGHT_INDEX_NAME} but missing from {shard}")
                piece = reader.get_slice(name)
                layouts[name] = (tuple(piece.get_shape()), piece.get_dtype())
    return layouts


def _digits_as_numbers(text: str) -> list:
    """Sort key under which `layers.2` precedes `layers.10`."""
    return [int(run) if run.isdigit() else run for run in re.findall(r"\d+|\D+", text)]


def build_mxfp8_quantization_config(source_dir: str | Path, remap: Callable[[str], str] = lambda name: name) -> dict:
    """The `quantization_config` of the MXFP8 model a sync of this checkpoint produces: every `.weight` the quantizer
    would leave alone is listed in `modules_to_not_convert`.  An expert weight that cannot be quantized is an error, not
    an entry: the engine's fused expert allocation does not read that list."""
    source = Path(source_dir)
    if not (source / "config.json").is_file():
        raise FileNotFoundError(f"Expected config.json under {source}")
    weight_map = checkpoint_weight_map(source)
    kept = set()
    for stored_name, (shape, header_dtype) in _header_layouts(source, weight_map).items():
        if not stored_name.endswith(".weight"):
            continue
        name = remap(stored_name)
        dtype = _DTYPE_OF_HEADER.get(header_dtype)
        routed = ".experts." in name
        # int8 experts hold two MXFP4 codes per byte: the logical row is twice the stored one
        if dtype is not None and should_use_mxfp8(name, shape, dtype, allow_source_fp8=True,
                                                  packed_mxfp4_experts=routed and dtype is torch.int8):
            continue
        if routed:
            raise ValueError(f"Unsupported MXFP8 expert {stored_name}: shape={shape}, dtype={header_dtype}; "
                             f"expected a quantizable expert with logical width divisible by {MXFP8_GROUP_SIZE} "
                             "and no high-precision exclusion")
        kept.add(name.removesuffix(".weight"))
    return {"activation_scheme": "dynamic", "fmt": "e4m3", "quant_method": "mxfp8",
            "weight_block_size": [1, MXFP8_GROUP_SIZE], "scale_fmt": "ue8m0",
            "modules_to_not_convert": sorted(kept, key=_digits_as_numbers)}


def create_mxfp8_rollout_schema(source_dir: str | Path, destination_dir: str | Path,
                                remap: Callable[[str], str] = lambda name: name) -> Path:
    """Write the schema directory: the checkpoint's non-weight files, and its config.json with the MXFP8
    `quantization_config` and `expert_dtype: "fp8"`.  Refuses the checkpoint's own directory and any destination that
    already holds weight files."""
    source, destination = Path(source_dir).resolve(), Path(destination_dir).resolve()
    if source == destination:
        raise ValueError("The rollout schema destination must differ from the source checkpoint")
    quantization_config = build_mxfp8_quantization_config(source, remap)
    destination.mkdir(parents=True, exist_ok=True)
    if next(destination.glob("*.safetensors"), None) is not None:
        raise ValueError(f"Refusing to use schema directory containing weight payloads: {destination}")
    for entry in source.iterdir():
        if entry.is_file() and entry.suffix != ".safetensors" and entry.name != WEIGHT_INDEX_NAME:
            shutil.copy2(entry, destination / entry.name)
    config = json.loads((source / "config.json").read_text(encoding="utf-8"))
    config.update(quantization_config=quantization_config, expert_dtype="fp8")
    (destination / "config.json").write_text(json.dumps(config, indent=2) + "\n", encoding="utf-8")
    return destination
