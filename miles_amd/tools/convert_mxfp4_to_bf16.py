"""`mxfp4-pack-quantized` compressed-tensors checkpoint -> BF16, dequantized on the GPU.

    python -m miles_amd.tools.convert_mxfp4_to_bf16 --model-dir SRC --save-dir DST [--files F ...]
                                                    [--shard-rank R --num-shards N] [--finalize-only] [--overwrite]

Behaviour of the reference's tools/convert_mxfp4_to_bf16.py: each `<name>.weight_packed` / `<name>.weight_scale`
pair of a shard turns into `<name>.weight` in bfloat16 (:66-103), all other tensors travel unchanged, the copied
`config.json` loses its `quantization_config` (:50-63; multimodal configs keep it under `text_config`) and the index
is rebuilt by scanning the written shards (:106-131).  Several processes can split the shard list between them
(`--shard-rank / --num-shards`); one final `--finalize-only` call then writes the side files and the index.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import shutil
from pathlib import Path

from safetensors.torch import safe_open, save_file

from miles_amd import launch
from miles_amd.utils.mxfp4 import dequantize_mxfp4

PACKED, SCALE = ".weight_packed", ".weight_scale"
_BYTES_PER_ELEMENT = {"BF16": 2, "F16": 2, "F32": 4, "F64": 8, "I32": 4, "I64": 8, "U8": 1}


def quantization_section(config: dict) -> dict:
    """The part of a config that holds `quantization_config` (the text sub-config of a multimodal model)."""
    return config["text_config"] if "text_config" in config else config


class Mxfp4Checkpoint:
    """One source directory and the directory its BF16 twin is written to."""

    def __init__(self, source: Path, target: Path, device: str = "cuda") -> None:
        self.source, self.target, self.device = source, target, device
        scheme = quantization_section(json.loads((source / "config.json").read_text()))["quantization_config"]
        assert scheme["format"] == "mxfp4-pack-quantized", scheme["format"]
        weights = scheme["config_groups"]["group_0"]["weights"]
        assert weights["type"] == "float"
        assert weights["num_bits"] == 4
        assert weights["scale_dtype"] == "torch.uint8"
        self.group_size = int(weights["group_size"])

    def shard_names(self) -> list[str]:
        return sorted(p.name for p in self.source.glob("*.safetensors"))

    def write_side_files(self) -> None:
        """Tokenizer, generation config and friends as they are; `config.json` without its quantization section."""
        self.target.mkdir(parents=True, exist_ok=True)
        for item in self.source.iterdir():
            if item.is_file() and item.suffix != ".safetensors" and not item.name.endswith(".index.json"):
                shutil.copy2(item, self.target / item.name)
        config = json.loads((self.target / "config.json").read_text())
        del quantization_section(config)["quantization_config"]
        (self.target / "config.json").write_text(json.dumps(config, indent=2))

    def convert_shard(self, name: str) -> None:
        """Dequantize the packed pairs of one shard; the result replaces the target file in one rename."""
        out = {}
        with safe_open(self.source / name, framework="pt", device="cpu") as shard:
            names = set(shard.keys())
            stems = sorted(n[: -len(PACKED)] for n in names if n.endswith(PACKED))
            scales = {n for n in names if n.endswith(SCALE)}
            with launch.deferred():         # the shard's tensors are unpacked together when the block ends
                for stem in stems:
                    assert stem + SCALE in scales, f"Missing scale for {stem + PACKED}"
                    scales.discard(stem + SCALE)
                    codes, exponents = shard.get_tensor(stem + PACKED), shard.get_tensor(stem + SCALE)
                    out[stem + ".weight"] = dequantize_mxfp4(codes.to(self.device), exponents.to(self.device), self.group_size)
            for stem in stems:
                out[stem + ".weight"] = out[stem + ".weight"].cpu()
            assert not scales, f"Orphan MXFP4 scales in {name}: {sorted(scales)}"
            consumed = {stem + suffix for stem in stems for suffix in (PACKED, SCALE)}
            for other in sorted(names - consumed):
                out[other] = shard.get_tensor(other)
        destination = self.target / name
        destination.parent.mkdir(parents=True, exist_ok=True)
        staging = destination.with_suffix(destination.suffix + ".tmp")
        save_file(out, staging)
        os.replace(staging, destination)

    def write_index(self) -> None:
        """`model.safetensors.index.json` from the headers of whatever shards the target directory holds."""
        owner, size = {}, 0
        for path in sorted(self.target.glob("*.safetensors")):
            with safe_open(path, framework="pt", device="cpu") as shard:
                for tensor in shard.keys():
                    assert tensor not in owner, f"Duplicate tensor: {tensor}"
                    owner[tensor] = path.name
                    header = shard.get_slice(tensor)
                    assert header.get_dtype() in _BYTES_PER_ELEMENT, f"Unsupported safetensors dtype: {header.get_dtype()}"
                    size += math.prod(header.get_shape()) * _BYTES_PER_ELEMENT[header.get_dtype()]
        (self.target / "model.safetensors.index.json").write_text(
            json.dumps({"metadata": {"total_size": size}, "weight_map": owner}, indent=2))


def parse_args(argv=None) -> argparse.Namespace:
    p = argparse.ArgumentParser(description="Convert MXFP4-packed compressed-tensors weights to BF16.")
    p.add_argument("--model-dir", type=Path, required=True)
    p.add_argument("--save-dir", type=Path, required=True)
    p.add_argument("--device", choices=("cuda",), default="cuda")
    p.add_argument("--files", nargs="+")
    p.add_argument("--shard-rank", type=int)
    p.add_argument("--num-shards", type=int)
    p.add_argument("--finalize-only", action="store_true")
    p.add_argument("--overwrite", action="store_true")
    return p.parse_args(argv)


def main(argv=None) -> None:
    args = parse_args(argv)
    assert args.model_dir.is_dir(), args.model_dir
    assert args.save_dir != args.model_dir
    split = args.num_shards is not None
    assert split == (args.shard_rank is not None)
    if split:
        assert args.num_shards > 0 and 0 <= args.shard_rank < args.num_shards
        assert args.files is None, "--files cannot be combined with sharded conversion"
    job = Mxfp4Checkpoint(args.model_dir, args.save_dir, args.device)
    args.save_dir.mkdir(parents=True, exist_ok=True)
    if args.finalize_only:
        job.write_side_files()
        job.write_index()
        return
    if not split or args.shard_rank == 0:
        job.write_side_files()
    todo = args.files or job.shard_names()
    if split:
        todo = todo[args.shard_rank::args.num_shards]
    assert todo, "No safetensors files found"
    for name in todo:
        assert (args.model_dir / name).is_file(), args.model_dir / name
        if (args.save_dir / name).exists() and not args.overwrite:
            print(f"Skipping existing {args.save_dir / name}", flush=True)
            continue
        print(f"Converting {args.model_dir / name} -> {args.save_dir / name}", flush=True)
        job.convert_shard(name)
    if not split:
        job.write_index()


if __name__ == "__main__":
    main()
