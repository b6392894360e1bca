"""Shard-level plumbing shared by the offline converters: safetensors in / out, side files, config and index
emitters.  (The reference repeats this code in each tool: tools/convert_hf_to_fp8.py:98-247,
tools/convert_hf_to_mxfp8.py:105-303, tools/convert_hf_to_int4_direct.py:154-271,
tools/convert_hf_to_nvfp4.py:170-470.)"""

from __future__ import annotations

import json
import os
import shutil
import threading

import safetensors
import safetensors.torch
import torch


def copy_side_files(src: str, dst: str) -> None:
    """Everything that is neither a safetensors shard nor a directory travels unchanged."""
    for name in os.listdir(src):
        path = os.path.join(src, name)
        if not name.endswith(".safetensors") and not os.path.isdir(path):
            shutil.copyfile(path, os.path.join(dst, name))


def list_shards(src: str) -> list[str]:
    return [f for f in os.listdir(src) if f.endswith(".safetensors")]


def load_shard(src: str, filename: str, device: str) -> dict[str, torch.Tensor]:
    with safetensors.safe_open(os.path.join(src, filename), framework="pt", device=device) as f:
        return {k: f.get_tensor(k) for k in f.keys()}


def load_tensor(src: str, filename: str, key: str, device: str) -> torch.Tensor:
    with safetensors.safe_open(os.path.join(src, filename), framework="pt", device=device) as f:
        return f.get_tensor(key)


_PT_FORMAT = {"format": "pt"}


def save_shard(tensors: dict[str, torch.Tensor], dst: str, filename: str, metadata: dict | None = _PT_FORMAT) -> None:
    """One safetensors file; the converters tag theirs `format: pt` as the reference's tools do, the snapshot export
    writes none (`metadata=None`)."""
    safetensors.torch.save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(dst, filename),
                                metadata=metadata)


def read_config(src: str) -> dict | None:
    path = os.path.join(src, "config.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        return json.load(f)


def write_config(dst: str, cfg: dict) -> None:
    with open(os.path.join(dst, "config.json"), "w") as f:
        json.dump(cfg, f, indent=2)


def write_index(dst: str, weight_map: dict[str, str], total_size: int) -> None:
    with open(os.path.join(dst, "model.safetensors.index.json"), "w") as f:
        json.dump({"weight_map": weight_map, "metadata": {"total_size": total_size}}, f, indent=2)


class ShardResults:
    """Collects the per-shard outcome; safe to fill from several worker threads."""

    def __init__(self, *, size_in_bytes: bool) -> None:
        self._lock = threading.Lock()
        self._size_in_bytes = size_in_bytes
        self.weight_map: dict[str, str] = {}
        self.total_size = 0
        self.modules_to_not_convert: list[str] = []
        self.has_dsa_layers = False

    def add(self, filename: str, tensors: dict[str, torch.Tensor], modules: list[str] = ()) -> None:
        with self._lock:
            for key, t in tensors.items():
                self.weight_map[key] = filename
                # the FP8 and INT4 tools of the reference count len(tensor) (first dimension), the MXFP8 and
                # NVFP4 tools count bytes; each converter keeps its tool's convention
                self.total_size += t.numel() * t.element_size() if self._size_in_bytes else len(t)
                if "indexer" in key:
                    self.has_dsa_layers = True
            self.modules_to_not_convert.extend(modules)
