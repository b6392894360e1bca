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
from collections.abc import Callable, Iterator
from pathlib import Path

import torch
from safetensors import safe_open

from miles_amd.utils.mxfp8 import MXFP8_GROUP_SIZE, should_use_mxfp8

WEIGHT_INDEX_NAME = "model.safetensors.index.json"

# safetensors header dtype strings of tensors that can be (or already are) MXFP8 sources; any other dtype is not
_DTYPE_OF_HEADER = {"BF16": torch.bfloat16, "F16": torch.float16, "F32": torch.float32,
                    "F8_E4M3": torch.float8_e4m3fn, "I8": torch.int8}
_DIGIT_RUNS = re.compile(r"\d+|\D+")


def _identity(name: str) -> str:
    return name


class _Headers:
    """What the safetensors headers of a checkpoint directory say, read without touching a payload."""

    def __init__(self, directory: Path) -> None:
        self.directory = directory

    def shard_of_tensor(self) -> dict[str, str]:
        """tensor name -> shard file: the index when the checkpoint has one, else every `*.safetensors` it holds
        (reference `hf_utils/weight_mapping.py:59-77`)."""
        index = self.directory / WEIGHT_INDEX_NAME
        if index.is_file():
            return json.loads(index.read_text(encoding="utf-8"))["weight_map"]
        owner: dict[str, str] = {}
        for shard in sorted(self.directory.glob("*.safetensors")):
            with safe_open(shard, framework="pt", device="cpu") as reader:
                for name in reader.keys():
                    if name in owner:
                        raise ValueError(f"Duplicate tensor {name} in {owner[name]} and {shard.name}")
                    owner[name] = shard.name
        if not owner:
            raise FileNotFoundError(f"No safetensors weights or index under {self.directory}")
        return owner

    def layouts(self) -> Iterator[tuple[str, tuple[int, ...], str]]:
        """(name, shape, header dtype string) of every tensor, one shard opened at a time."""
        wanted: dict[str, list[str]] = {}
        for name, shard in self.shard_of_tensor().items():
            wanted.setdefault(shard, []).append(name)
        for shard, names in wanted.items():
            with safe_open(self.directory / shard, framework="pt", device="cpu") as reader:
                stored = frozenset(reader.keys())
                for name in names:
                    if name not in stored:
                        raise KeyError(f"{name} is listed in {WEIGHT_INDEX_NAME} but missing from {shard}")
                    header = reader.get_slice(name)
                    yield name, tuple(header.get_shape()), header.get_dtype()


def _natural(text: str) -> list:
    """Sort key under which `layers.2` precedes `layers.10`."""
    return [int(run) if run[0].isdigit() else run for run in _DIGIT_RUNS.findall(text)]


def _stays_high_precision(name: str, shape: tuple[int, ...], header_dtype: str, stored_as: str) -> bool:
    """True for a `.weight` the MXFP8 quantizer leaves alone; an expert weight among them is an error, not an answer:
    the engine's fused expert allocation reads no exclusion list."""
    dtype = _DTYPE_OF_HEADER.get(header_dtype)
    expert = ".experts." in name
    # int8 experts hold two MXFP4 codes per byte: the logical row is twice the stored one
    if dtype is not None and should_use_mxfp8(name, shape, dtype, allow_source_fp8=True,
                                              packed_mxfp4_experts=expert and dtype is torch.int8):
        return False
    if expert:
        raise ValueError(f"Unsupported MXFP8 expert {stored_as}: shape={shape}, dtype={header_dtype}; "
                         f"expected a quantizable expert with logical width divisible by {MXFP8_GROUP_SIZE} "
                         "and no high-precision exclusion")
    return True


def build_mxfp8_quantization_config(source_dir: str | Path, remap: Callable[[str], str] = _identity) -> dict:
    """The `quantization_config` of the MXFP8 model a sync of this checkpoint produces: every `.weight` the quantizer
    would leave alone is listed in `modules_to_not_convert` (without the suffix, in natural order)."""
    source = Path(source_dir)
    if not (source / "config.json").is_file():
        raise FileNotFoundError(f"Expected config.json under {source}")
    kept = set()
    for stored, shape, header_dtype in _Headers(source).layouts():
        if stored.endswith(".weight"):
            name = remap(stored)
            if _stays_high_precision(name, shape, header_dtype, stored):
                kept.add(name.removesuffix(".weight"))
    return {"activation_scheme": "dynamic", "fmt": "e4m3", "quant_method": "mxfp8",
            "weight_block_size": [1, MXFP8_GROUP_SIZE], "scale_fmt": "ue8m0",
            "modules_to_not_convert": sorted(kept, key=_natural)}


def create_mxfp8_rollout_schema(source_dir: str | Path, destination_dir: str | Path,
                                remap: Callable[[str], str] = _identity) -> Path:
    """Write the schema directory: the checkpoint's non-weight files, and its config.json with the MXFP8
    `quantization_config` and `expert_dtype: "fp8"`.  Refuses the checkpoint's own directory and any destination that
    already holds weight files."""
    source, destination = Path(source_dir).resolve(), Path(destination_dir).resolve()
    if source == destination:
        raise ValueError("The rollout schema destination must differ from the source checkpoint")
    quantization_config = build_mxfp8_quantization_config(source, remap)        # (raises where there is no config.json)
    config = json.loads((source / "config.json").read_text(encoding="utf-8"))
    config.update(quantization_config=quantization_config, expert_dtype="fp8")
    destination.mkdir(parents=True, exist_ok=True)
    if next(destination.glob("*.safetensors"), None) is not None:
        raise ValueError(f"Refusing to use schema directory containing weight payloads: {destination}")
    for entry in source.iterdir():
        if entry.is_file() and entry.suffix != ".safetensors" and entry.name != WEIGHT_INDEX_NAME:
            shutil.copy2(entry, destination / entry.name)
    (destination / "config.json").write_text(json.dumps(config, indent=2) + "\n", encoding="utf-8")
    return destination
