"""INT4 (compressed-tensors pack-quantized, round-to-nearest, group-wise) offline converter.

    python -m miles_amd.tools.convert_hf_to_int4_direct --model-dir SRC --save-dir DST [--group-size 32]
                                                        [--ignore-rules ...] [--max-workers N]

Mirror of the reference's tools/convert_hf_to_int4_direct.py (`process_file` :167-202, `convert_int4`
:205-271, CLI :274-320); `pack_layer` is the fused gfx950 kernel.
"""

from __future__ import annotations

import argparse
import os
import re
from concurrent.futures import ThreadPoolExecutor

import torch

from miles_amd import launch
from miles_amd.kernels.quant.int4_fake import pack_layer
from miles_amd.tools import _checkpoint as ckpt

DEFAULT_IGNORE_RULES = [
    "re:.*lm_head.*", "re:.*norm.*", "re:.*embed.*", "re:.*self_attn.*", "re:.*shared_experts.*",
    "re:.*mlp\\.(gate|up|gate_up|down)_proj.*", "re:.*mlp\\.gate\\.*", "re:vision_tower.*", "re:mm_projector.*",
]


def is_ignored(name: str, ignore_rules) -> bool:
    """A rule is a regex (prefix `re:`, matched from the start of the name), an exact name or a name prefix."""
    return any((r.startswith("re:") and re.match(r[3:], name)) or r == name or name.startswith(r) for r in ignore_rules)


def process_file(input_path, output_path, filename, group_size, is_symmetric, ignore_rules, result_collector,
                 device="cuda"):
    weights = ckpt.load_shard(input_path, filename, device)
    out: dict[str, torch.Tensor] = {}
    with launch.deferred():
        for name, weight in weights.items():
            if is_ignored(name, ignore_rules) or not name.endswith(".weight") or weight.dim() < 2:
                out[name] = weight
                continue
            packed, scale, zero_point = pack_layer(weight, group_size, is_symmetric)
            if zero_point is not None:
                out[name.replace(".weight", ".weight_zero_point")] = zero_point
            out[name.replace(".weight", ".weight_packed")] = packed
            out[name.replace(".weight", ".weight_scale")] = scale
            out[name.replace(".weight", ".weight_shape")] = torch.tensor(weight.shape, dtype=torch.int32, device=weight.device)
    ckpt.save_shard(out, output_path, filename)
    result_collector.add(filename, out)


def int4_quantization_config(group_size, is_symmetric, ignore_rules) -> dict:
    weights = {"actorder": None, "block_structure": None, "dynamic": False, "group_size": group_size, "num_bits": 4,
               "observer": "minmax", "observer_kwargs": {}, "strategy": "group", "symmetric": is_symmetric, "type": "int"}
    group = {"input_activations": None, "output_activations": None, "targets": ["Linear"], "weights": weights}
    return {"config_groups": {"group_0": group}, "format": "pack-quantized", "ignore": ignore_rules,
            "kv_cache_scheme": None, "quant_method": "compressed-tensors", "quantization_status": "compressed"}


def convert_int4(input_path, output_path, group_size, is_symmetric, ignore_rules, max_workers, device="cuda"):
    input_path = os.path.abspath(input_path)
    os.makedirs(output_path, exist_ok=True)
    ckpt.copy_side_files(input_path, output_path)
    results = ckpt.ShardResults(size_in_bytes=False)
    with ThreadPoolExecutor(max_workers=max_workers) as pool:
        futures = [pool.submit(process_file, input_path, output_path, f, group_size, is_symmetric, ignore_rules,
                               results, device) for f in ckpt.list_shards(input_path)]
        for fut in futures:
            fut.result()
    cfg = ckpt.read_config(input_path)
    if cfg is not None:
        cfg["quantization_config"] = int4_quantization_config(group_size, is_symmetric, ignore_rules)
        ckpt.write_config(output_path, cfg)
    ckpt.write_index(output_path, results.weight_map, results.total_size)
    return output_path


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--model-dir", type=str, required=True, help="local BF16 path")
    ap.add_argument("--save-dir", type=str, required=True)
    ap.add_argument("--group-size", type=int, default=32, help="Group Size")
    ap.add_argument("--is-symmetric", type=bool, default=True, help="Is Symmetric")
    ap.add_argument("--ignore-rules", nargs="+", default=DEFAULT_IGNORE_RULES, help="Ignore Rules")
    ap.add_argument("--max-workers", type=int, default=1, help="Number of worker threads for parallel processing")
    args = ap.parse_args(argv)
    if os.path.exists(args.save_dir) and not os.path.isdir(args.save_dir):
        raise ValueError("The save_dir should be a directory.")
    os.makedirs(args.save_dir, exist_ok=True)
    convert_int4(args.model_dir, args.save_dir, args.group_size, args.is_symmetric, args.ignore_rules, args.max_workers)
    print(f"Conversion complete, output saved to {args.save_dir}")


if __name__ == "__main__":
    main()
