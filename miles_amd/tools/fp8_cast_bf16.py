"""FP8 block-scale -> BF16 checkpoint converter.

    python -m miles_amd.tools.fp8_cast_bf16 --input-fp8-hf-path SRC --output-bf16-hf-path DST

Mirror of the reference's tools/fp8_cast_bf16.py: `weight_dequant` (:30-40; Triton kernel :15-27) and `main`
(:43-125).  The reference renames tensors through `get_param_name_remap` (a model-specific table outside this
path); `main` takes the renaming function as an argument and defaults to the identity.
"""

from __future__ import annotations

import argparse
import glob
import json
import os
import shutil

import torch
from safetensors.torch import load_file, save_file

from miles_amd import _lib, launch


def weight_dequant(x: torch.Tensor, s: torch.Tensor, block_size: int = 128) -> torch.Tensor:
    """x e4m3 [M, N], s float32 [ceil(M/B), ceil(N/B)] -> bfloat16 [M, N] = bf16(float(x) * s[i//B, j//B]).

    The reference allocates the output in the default dtype, which its tool sets to bfloat16 before the
    first call (tools/fp8_cast_bf16.py:44); this function always writes bfloat16.
    """
    assert x.is_contiguous() and s.is_contiguous()
    assert x.dim() == 2 and s.dim() == 2
    _lib.require_gpu(x, "weight_dequant")
    if s.dtype != torch.float32:
        raise _lib.MilesQuantError(f"weight_dequant expects float32 scales, got {s.dtype}")
    M, N = x.size()
    y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    launch.submit(_lib.JOB_FP8_DEQUANT, x, y, None, s, None, M, N, N, int(block_size), 0)
    return y


def main(fp8_path, bf16_path, remap=lambda name: name, device="cuda"):
    """Dequantize every 1-byte weight that has a `<name>_scale_inv` partner (possibly in another shard); copy
    the rest; drop the scale tensors from the shards and from the index."""
    os.makedirs(bf16_path, exist_ok=True)
    for pattern in ("config.json", "*.py", "tokenizer*", "chat_template*"):
        for path in glob.glob(os.path.join(fp8_path, pattern)):
            shutil.copy(path, bf16_path)
    with open(os.path.join(fp8_path, "model.safetensors.index.json")) as f:
        weight_map_raw = json.load(f)["weight_map"]
    weight_map, raw_of = {}, {}
    for raw, fname in weight_map_raw.items():
        new = remap(raw)
        assert new not in raw_of, f"Remapped tensor name collision: {new} from {raw} and {raw_of.get(new)}"
        weight_map[new], raw_of[new] = fname, raw

    loaded: dict[str, dict[str, torch.Tensor]] = {}

    def get_tensor(name):
        raw = raw_of[name]
        fname = weight_map_raw[raw]
        if fname not in loaded:
            loaded[fname] = load_file(os.path.join(fp8_path, fname), device=device)
        return loaded[fname][raw]

    dequantized = []
    for path in sorted(glob.glob(os.path.join(fp8_path, "*.safetensors"))):
        fname = os.path.basename(path)
        state = load_file(path, device=device)
        loaded[fname] = state
        out = {}
        with launch.deferred():
            for raw, weight in state.items():
                name = remap(raw)
                if name.endswith("_scale_inv"):
                    continue
                if weight.element_size() != 1:
                    out[name] = weight
                    continue
                try:
                    scale_inv = get_tensor(f"{name}_scale_inv")
                except KeyError:
                    print(f"Warning: Missing scale_inv tensor for {name}, skipping conversion")
                    out[name] = weight
                else:
                    dequantized.append(name)
                    out[name] = weight_dequant(weight.contiguous(), scale_inv.float().contiguous())
        save_file(out, os.path.join(bf16_path, fname))
        if len(loaded) > 2:      # keep the two most recently used shards
            del loaded[next(iter(loaded))]
    for name in dequantized:
        weight_map.pop(f"{name}_scale_inv", None)
    with open(os.path.join(bf16_path, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {}, "weight_map": weight_map}, f, indent=2)


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--input-fp8-hf-path", type=str, required=True)
    ap.add_argument("--output-bf16-hf-path", type=str, required=True)
    a = ap.parse_args()
    main(a.input_fp8_hf_path, a.output_bf16_hf_path)
