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


def _update_quantization_config(cfg: dict, ignore_list: list[str]) -> None:
    q = cfg.get("quantization_config")
    if not isinstance(q, dict):
        q = {}
    q.update(quant_algo="NVFP4", quant_method="modelopt", group_size=NVFP4_GROUP_SIZE, ignore=ignore_list)
    q.setdefault("kv_cache_scheme", DEFAULT_KV_CACHE_SCHEME)
    groups = q.get("config_groups")
    if isinstance(groups, dict):
        for group in groups.values():
            if not isinstance(group, dict):
                continue
            group.setdefault("targets", ["Linear"])
            for key in ("input_activations", "weights"):
                section = group.get(key)
                if isinstance(section, dict):
                    section.setdefault("dynamic", False)
                    section.setdefault("num_bits", 4)
                    section.setdefault("type", "float")
                    section["group_size"] = NVFP4_GROUP_SIZE
    cfg["quantization_config"] = q
    text = cfg.get("text_config")
    if isinstance(text, dict) and "quantization_config" in text:
        _update_quantization_config(text, ignore_list)   # composite configs must not keep a stale policy


def _write_hf_quant_config(output_path: str, ignore_list: list[str], input_path: str) -> None:
    src = os.path.join(input_path, "hf_quant_config.json")
    if os.path.exists(src):
        with open(src) as f:
            doc = json.load(f)
    else:
        doc = {"producer": {"name": "modelopt"}}
    section = doc.get("quantization")
    if not isinstance(section, dict):
        section = {}
    section.update(quant_algo="NVFP4", kv_cache_quant_algo=DEFAULT_KV_CACHE_QUANT_ALGO, group_size=NVFP4_GROUP_SIZE,
                   exclude_modules=ignore_list)
    doc["quantization"] = section
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


def _collect_gated_pair_locations(*, input_path, safetensors_files, device, skip_weight_substrings, num_hidden_layers):
    """base name -> {'gate': (file, key), 'up': (file, key)} for every complete pair in the checkpoint."""
    pairs: dict[str, dict[str, tuple[str, str]]] = {}
    for filename in safetensors_files:
        for key, tensor in ckpt.load_shard(input_path, filename, device).items():
            if not should_quantize(key, tensor, skip_weight_substrings=skip_weight_substrings,
                                   num_hidden_layers=num_hidden_layers):
                continue
            base, role = _split_gated_pair_name(key)
            if base is None:
                continue
            roles = pairs.setdefault(base, {})
            if role in roles:
                raise ValueError(f"NVFP4 requires a single complete gate/up pair per converted checkpoint; "
                                 f"found duplicate {role} tensor for {base}.")
            roles[role] = (filename, key)
    return {b: r for b, r in pairs.items() if set(r) == {"gate", "up"}}


def _nvfp4_quantized_entries(key, qweight, block_scale, weight_scale_2) -> dict[str, torch.Tensor]:
    return {key: qweight, key.replace(".weight", ".weight_scale"): block_scale,
            key.replace(".weight", ".weight_scale_2"): weight_scale_2,
            key.replace(".weight", ".input_scale"): torch.ones_like(weight_scale_2, dtype=torch.float32)}


def process_file(input_path, output_path, filename, result_collector, device, num_hidden_layers,
                 num_layers_at_start_in_bf16, num_layers_at_end_in_bf16, extra_high_precision_layers_hf,
                 gated_pair_locations, processed_gated_pairs, deferred_quantized_entries) -> None:
    if not filename.endswith(".safetensors"):
        return
    skipped: list[str] = []
    out: dict[str, torch.Tensor] = {}
    bf16_prefixes = _get_bf16_layer_prefixes(num_hidden_layers, num_layers_at_start_in_bf16, num_layers_at_end_in_bf16)
    skip_substrings = (*extra_high_precision_layers_hf, *sorted(bf16_prefixes))
    with launch.deferred():
        for key, tensor in ckpt.load_shard(input_path, filename, device).items():
            if key in out:
                continue
            parked = deferred_quantized_entries.get(filename, {}).pop(key, None)
            if parked is not None:      # quantized earlier together with its partner from another shard
                out.update(parked)
                continue
            if not should_quantize(key, tensor, skip_weight_substrings=skip_substrings, num_hidden_layers=num_hidden_layers):
                if key.endswith(".weight"):
                    module = key[: -len(".weight")]
                    in_bf16_layers = [p for p in bf16_prefixes if key.startswith(p)]
                    skipped.extend(in_bf16_layers)
                    if ".experts." in key and in_bf16_layers:
                        skipped.append(module.split(".experts.", 1)[0] + ".experts")   # the FusedMoE container
                    else:
                        skipped.append(module)
                out[key] = tensor
                continue
            base, _role = _split_gated_pair_name(key)
            if base not in gated_pair_locations:
                out.update(_nvfp4_quantized_entries(key, *quantize_nvfp4(tensor)))
                continue
            if base in processed_gated_pairs:
                raise ValueError(f"Missing deferred NVFP4 output for already processed gated pair {base}.")
            (gate_file, gate_key), (up_file, up_key) = gated_pair_locations[base]["gate"], gated_pair_locations[base]["up"]
            gate = tensor if key == gate_key else ckpt.load_tensor(input_path, gate_file, gate_key, device)
            up = tensor if key == up_key else ckpt.load_tensor(input_path, up_file, up_key, device)
            for (fname, k), result in zip(((gate_file, gate_key), (up_file, up_key)), nvfp4_quantize_1d_pair(gate, up)):
                entries = _nvfp4_quantized_entries(k, *result)
                if fname == filename:
                    out.update(entries)
                else:
                    deferred_quantized_entries.setdefault(fname, {})[k] = entries
            processed_gated_pairs.add(base)
    ckpt.save_shard(out, output_path, filename)
    result_collector.add(filename, out, skipped)


def convert_nvfp4(model_dir, save_dir, device, num_layers_at_start_in_bf16=0, num_layers_at_end_in_bf16=0,
                  extra_high_precision_layers_hf=()) -> None:
    input_path, output_path = os.path.abspath(model_dir), os.path.abspath(save_dir)
    os.makedirs(output_path, exist_ok=True)
    ckpt.copy_side_files(input_path, output_path)
    shards = ckpt.list_shards(input_path)
    num_hidden_layers = _get_num_hidden_layers(input_path)
    bf16_prefixes = _get_bf16_layer_prefixes(num_hidden_layers, num_layers_at_start_in_bf16, num_layers_at_end_in_bf16)
    pairs = _collect_gated_pair_locations(input_path=input_path, safetensors_files=shards, device=device,
                                          skip_weight_substrings=(*extra_high_precision_layers_hf, *sorted(bf16_prefixes)),
                                          num_hidden_layers=num_hidden_layers)
    done: set[str] = set()
    parked: dict[str, dict[str, dict[str, torch.Tensor]]] = {}
    results = ckpt.ShardResults(size_in_bytes=True)
    for filename in shards:
        process_file(input_path, output_path, filename, results, device, num_hidden_layers, num_layers_at_start_in_bf16,
                     num_layers_at_end_in_bf16, tuple(extra_high_precision_layers_hf), pairs, done, parked)
    left = {f: sorted(e) for f, e in parked.items() if e}
    if left:
        raise RuntimeError(f"Unwritten deferred NVFP4 gated-pair entries: {left}")
    ignore_list = _augment_ignore_list(results.modules_to_not_convert)
    cfg = ckpt.read_config(input_path)
    if cfg is not None:
        _update_quantization_config(cfg, ignore_list)
        ckpt.write_config(output_path, cfg)
    _write_hf_quant_config(output_path, ignore_list, input_path)
    ckpt.write_index(output_path, results.weight_map, results.total_size)


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
