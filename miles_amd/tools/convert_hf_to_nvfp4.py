"""NVFP4 offline converter: routed-expert weights of the main language decoder only.

    python -m miles_amd.tools.convert_hf_to_nvfp4 --model-dir SRC --save-dir DST [--device cuda]
        [--num-layers-at-start-in-bf16 N] [--num-layers-at-end-in-bf16 N] [--extra-high-precision-layers-hf ...]

Mirror of the reference's tools/convert_hf_to_nvfp4.py: name scope (`should_quantize` :104-128), gate/up pairs
that may live in different shards (`_collect_gated_pair_locations` :264-291, deferred outputs in `process_file`
:313-403), `quantization_config` / `hf_quant_config.json` emitters (:185-238), ignore-list augmentation
(:241-255).  Tensor names: `.weight` (packed e2m1), `.weight_scale` (e4m3 1x16), `.weight_scale_2` (fp32 global),
`.input_scale` (ones).
"""

from __future__ import annotations

import argparse
import json
import os
import re

import torch

from miles_amd import launch
from miles_amd.megatron_to_hf.processors.quantizer_nvfp4 import GATED_PAIR_SUFFIXES, _split_gated_pair_name, quantize_nvfp4
from miles_amd.tools import _checkpoint as ckpt
from miles_amd.utils.nvfp4 import NVFP4_GROUP_SIZE, nvfp4_quantize_1d_pair

__all__ = ["convert_nvfp4", "quantize_nvfp4", "should_quantize", "GATED_PAIR_SUFFIXES"]

DEFAULT_KV_CACHE_SCHEME = {"dynamic": False, "num_bits": 8, "type": "float"}
DEFAULT_KV_CACHE_QUANT_ALGO = "FP8"
EXPERT_WEIGHT_SUFFIXES = (".w1.weight", ".w2.weight", ".w3.weight", ".gate_proj.weight", ".up_proj.weight",
                          ".down_proj.weight", ".gate_up_proj.weight")
ROUTED_EXPERT_NAME_MARKERS = (".experts.", "block_sparse_moe.experts.", ".moe.experts.")
SHARED_EXPERT_NAME_MARKERS = (".shared_expert.", ".shared_experts.")
LANGUAGE_MODEL_LAYER_PREFIXES = ("model.layers", "language_model.model.layers", "model.language_model.layers",
                                 "language_model.layers")
LANGUAGE_MODEL_LAYER_PATTERN = re.compile(
    r"^(?:" + "|".join(re.escape(p) for p in LANGUAGE_MODEL_LAYER_PREFIXES) + r")\.(\d+)\.")
FUSED_QKV_SUFFIXES = (".q_proj", ".k_proj", ".v_proj")


def _is_routed_expert_weight_name(name: str) -> bool:
    return (name.endswith(".weight") and not any(m in name for m in SHARED_EXPERT_NAME_MARKERS)
            and any(m in name for m in ROUTED_EXPERT_NAME_MARKERS) and name.endswith(EXPERT_WEIGHT_SUFFIXES))


def _get_num_hidden_layers(model_dir: str) -> int:
    cfg = ckpt.read_config(model_dir)
    if cfg is None:
        raise ValueError("config.json is required to identify the main language decoder layers.")
    text = cfg.get("text_config")
    n = text.get("num_hidden_layers") if isinstance(text, dict) else None
    if n is None:
        n = cfg.get("num_hidden_layers")
    if n is None:
        raise ValueError("num_hidden_layers not found in config.json.")
    return int(n)


def _get_bf16_layer_prefixes(num_hidden_layers: int, num_at_start: int, num_at_end: int) -> tuple[str, ...]:
    idx = set(range(num_at_start)) | set(range(num_hidden_layers - num_at_end, num_hidden_layers))
    return tuple(sorted(f"{p}.{i}." for p in LANGUAGE_MODEL_LAYER_PREFIXES for i in idx))


def should_quantize(name: str, weight: torch.Tensor, skip_weight_substrings: tuple[str, ...] = (), *,
                    num_hidden_layers: int | None = None) -> bool:
    """Allowlist: routed experts inside `model.layers.<i>` with i below the decoder depth (MTP layers appended
    to model.layers and modality towers stay out)."""
    m = LANGUAGE_MODEL_LAYER_PATTERN.match(name)
    if m is None or (num_hidden_layers is not None and int(m.group(1)) >= num_hidden_layers):
        return False
    if any(s in name for s in skip_weight_substrings) or not _is_routed_expert_weight_name(name):
        return False
    if weight.dtype not in (torch.float16, torch.bfloat16, torch.float32) or weight.dim() < 2:
        return False
    if weight.shape[-1] % NVFP4_GROUP_SIZE != 0:
        raise ValueError(f"Last dim {weight.shape[-1]} must be divisible by {NVFP4_GROUP_SIZE} "
                         f"for NVFP4 quantization ({name}).")
    return True


_GROUP_DEFAULTS = {"dynamic": False, "num_bits": 4, "type": "float"}


def _update_quantization_config(cfg: dict, ignore_list: list[str]) -> None:
    """Stamp the NVFP4 policy on `quantization_config` (created if missing or malformed), keep what the source said
    about the KV cache, bring every compressed-tensors style group to 1x16 float4, and repeat for a nested
    `text_config` that carries a policy of its own (a composite config must not keep a stale one)."""
    policy = cfg["quantization_config"] if isinstance(cfg.get("quantization_config"), dict) else {}
    policy["quant_algo"], policy["quant_method"] = "NVFP4", "modelopt"
    policy["group_size"], policy["ignore"] = NVFP4_GROUP_SIZE, ignore_list
    policy.setdefault("kv_cache_scheme", DEFAULT_KV_CACHE_SCHEME)
    groups = policy.get("config_groups")
    for group in (groups.values() if isinstance(groups, dict) else ()):
        if isinstance(group, dict):
            group.setdefault("targets", ["Linear"])
            for side in ("input_activations", "weights"):
                if isinstance(group.get(side), dict):
                    for field, default in _GROUP_DEFAULTS.items():
                        group[side].setdefault(field, default)
                    group[side]["group_size"] = NVFP4_GROUP_SIZE
    cfg["quantization_config"] = policy
    nested = cfg.get("text_config")
    if isinstance(nested, dict) and "quantization_config" in nested:
        _update_quantization_config(nested, ignore_list)


def _write_hf_quant_config(output_path: str, ignore_list: list[str], input_path: str) -> None:
    """`hf_quant_config.json` in modelopt's layout, starting from the source's file when it has one."""
    existing = os.path.join(input_path, "hf_quant_config.json")
    doc = {"producer": {"name": "modelopt"}}
    if os.path.exists(existing):
        with open(existing) as f:
            doc = json.load(f)
    block = doc["quantization"] if isinstance(doc.get("quantization"), dict) else {}
    block["quant_algo"], block["kv_cache_quant_algo"] = "NVFP4", DEFAULT_KV_CACHE_QUANT_ALGO
    block["group_size"], block["exclude_modules"] = NVFP4_GROUP_SIZE, ignore_list
    doc["quantization"] = block
    with open(os.path.join(output_path, "hf_quant_config.json"), "w") as f:
        json.dump(doc, f, indent=2)


def _augment_ignore_list(ignore_list: list[str]) -> list[str]:
    """Add the fused names loaders look for: `<attn>.qkv_proj` and the `<...>.experts` container."""
    extra = set()
    for name in ignore_list:
        for suffix in FUSED_QKV_SUFFIXES:
            if name.endswith(suffix):
                extra.add(name[: -len(suffix)] + ".qkv_proj")
                break
        m = re.fullmatch(r"(.*\.experts)(?:\.\d+)?\.(gate_proj|up_proj|down_proj|gate_up_proj|w1|w2|w3)", name)
        if m:
            extra.add(m.group(1))
    return sorted(set(ignore_list) | extra)


def _quantized_entries(key: str, codes, block_scale, global_scale) -> dict[str, torch.Tensor]:
    """The four tensors a quantized `<module>.weight` becomes in a modelopt checkpoint."""
    stem = key[: -len("weight")]
    return {key: codes, stem + "weight_scale": block_scale, stem + "weight_scale_2": global_scale,
            stem + "input_scale": torch.ones_like(global_scale, dtype=torch.float32)}


class _Run:
    """One conversion: which tensors are in scope, where the halves of every gate/up pair live, and the outputs of
    pairs whose halves sit in different shards (quantized when the first half is met, written with each half's own
    shard)."""

    def __init__(self, src: str, dst: str, device: str, bf16_at_start: int, bf16_at_end: int, extra_skips) -> None:
        self.src, self.dst, self.device = src, dst, device
        self.depth = _get_num_hidden_layers(src)
        self.bf16_prefixes = _get_bf16_layer_prefixes(self.depth, bf16_at_start, bf16_at_end)
        self.skips = (*extra_skips, *sorted(self.bf16_prefixes))
        self.shards = ckpt.list_shards(src)
        self.results = ckpt.ShardResults(size_in_bytes=True)
        self.pair_homes: dict[str, dict[str, tuple[str, str]]] = {}
        self.pairs_done: set[str] = set()
        self.waiting: dict[str, dict[str, dict[str, torch.Tensor]]] = {}     # shard -> key -> entries

    def in_scope(self, key: str, tensor: torch.Tensor) -> bool:
        return should_quantize(key, tensor, skip_weight_substrings=self.skips, num_hidden_layers=self.depth)

    def locate_pairs(self) -> None:
        """A first pass over every shard: expert prefix -> {"gate": (shard, key), "up": (shard, key)}, complete pairs only."""
        seen: dict[str, dict[str, tuple[str, str]]] = {}
        for shard in self.shards:
            for key, tensor in ckpt.load_shard(self.src, shard, self.device).items():
                if not self.in_scope(key, tensor):
                    continue
                prefix, role = _split_gated_pair_name(key)
                if prefix is None:
                    continue
                homes = seen.setdefault(prefix, {})
                if role in homes:
                    raise ValueError(f"NVFP4 requires a single complete gate/up pair per converted checkpoint; "
                                     f"found duplicate {role} tensor for {prefix}.")
                homes[role] = (shard, key)
        self.pair_homes = {prefix: homes for prefix, homes in seen.items() if len(homes) == 2}

    def _kept_in_high_precision(self, key: str) -> list[str]:
        """Ignore-list entries for a `.weight` that stays as it is: its module, or for an expert of a BF16 layer the
        layer prefix and the experts container (loaders decide per fused MoE module)."""
        if not key.endswith(".weight"):
            return []
        layers = [p for p in self.bf16_prefixes if key.startswith(p)]
        module = key[: -len(".weight")]
        if layers and ".experts." in key:
            return layers + [module.split(".experts.", 1)[0] + ".experts"]
        return layers + [module]

    def _quantize_pair(self, prefix: str, shard: str, key: str, tensor: torch.Tensor, out: dict) -> None:
        if prefix in self.pairs_done:
            raise ValueError(f"Missing deferred NVFP4 output for already processed gated pair {prefix}.")
        homes = [self.pair_homes[prefix]["gate"], self.pair_homes[prefix]["up"]]
        halves = [tensor if k == key else ckpt.load_tensor(self.src, f, k, self.device) for f, k in homes]
        for (home_shard, home_key), result in zip(homes, nvfp4_quantize_1d_pair(*halves)):
            entries = _quantized_entries(home_key, *result)
            if home_shard == shard:
                out.update(entries)
            else:
                self.waiting.setdefault(home_shard, {})[home_key] = entries
        self.pairs_done.add(prefix)

    def convert_shard(self, shard: str) -> None:
        out: dict[str, torch.Tensor] = {}
        ignored: list[str] = []
        with launch.deferred():
            for key, tensor in ckpt.load_shard(self.src, shard, self.device).items():
                if key in out:
                    continue
                ready = self.waiting.get(shard, {}).pop(key, None)
                if ready is not None:
                    out.update(ready)
                elif not self.in_scope(key, tensor):
                    ignored += self._kept_in_high_precision(key)
                    out[key] = tensor
                else:
                    prefix = _split_gated_pair_name(key)[0]
                    if prefix in self.pair_homes:
                        self._quantize_pair(prefix, shard, key, tensor, out)
                    else:
                        out.update(_quantized_entries(key, *quantize_nvfp4(tensor)))
        ckpt.save_shard(out, self.dst, shard)
        self.results.add(shard, out, ignored)

    def finish(self) -> None:
        stranded = {shard: sorted(entries) for shard, entries in self.waiting.items() if entries}
        if stranded:
            raise RuntimeError(f"Unwritten deferred NVFP4 gated-pair entries: {stranded}")
        ignore_list = _augment_ignore_list(self.results.modules_to_not_convert)
        cfg = ckpt.read_config(self.src)
        if cfg is not None:
            _update_quantization_config(cfg, ignore_list)
            ckpt.write_config(self.dst, cfg)
        _write_hf_quant_config(self.dst, ignore_list, self.src)
        ckpt.write_index(self.dst, self.results.weight_map, self.results.total_size)


def convert_nvfp4(model_dir, save_dir, device, num_layers_at_start_in_bf16=0, num_layers_at_end_in_bf16=0,
                  extra_high_precision_layers_hf=()) -> None:
    src, dst = os.path.abspath(model_dir), os.path.abspath(save_dir)
    os.makedirs(dst, exist_ok=True)
    ckpt.copy_side_files(src, dst)
    run = _Run(src, dst, device, num_layers_at_start_in_bf16, num_layers_at_end_in_bf16,
               tuple(extra_high_precision_layers_hf))
    run.locate_pairs()
    for shard in run.shards:
        run.convert_shard(shard)
    run.finish()


def main(argv=None) -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--model-dir", type=str, required=True, help="Path to HF safetensors model.")
    ap.add_argument("--save-dir", type=str, required=True, help="Path to save converted model.")
    ap.add_argument("--device", type=str, default="cuda")
    ap.add_argument("--num-layers-at-start-in-bf16", type=int, default=0)
    ap.add_argument("--num-layers-at-end-in-bf16", type=int, default=0)
    ap.add_argument("--extra-high-precision-layers-hf", type=str, nargs="*", default=[])
    args, _ = ap.parse_known_args(argv)
    device = torch.device(f"cuda:{args.device}" if args.device.isdigit() else args.device)
    if device.type == "cuda":
        if not torch.cuda.is_available():
            raise RuntimeError("CUDA is not available, cannot run NVFP4 quantization.")
        if device.index is None:
            device = torch.device("cuda:0")
        torch.cuda.set_device(device)
    if os.path.exists(args.save_dir) and not os.path.isdir(args.save_dir):
        raise ValueError("The save_dir should be a directory.")
    convert_nvfp4(args.model_dir, args.save_dir, str(device), args.num_layers_at_start_in_bf16,
                  args.num_layers_at_end_in_bf16,
                  tuple(s.strip() for s in args.extra_high_precision_layers_hf if isinstance(s, str) and s.strip()))


if __name__ == "__main__":
    main()
