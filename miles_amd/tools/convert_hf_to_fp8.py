"""FP8 e4m3 offline converter: quantizers and the checkpoint shell around them.

    python -m miles_amd.tools.convert_hf_to_fp8 --model-dir SRC --save-dir DST [--strategy block|channel|tensor]
                                                [--block-size 128 128] [--max-workers N]

Mirror of the reference's tools/convert_hf_to_fp8.py: `block_fp8` (:39-70), `channel_fp8` (:73-78),
`tensor_fp8` (:81-86), `quant_fp8` (:89-95), `process_file` (:116-160), `convert_fp8` (:163-247).  The chain of
~8 full-tensor PyTorch kernels per weight there is one gfx950 kernel here, and all weights of a shard are
submitted as one batched call.
"""

from __future__ import annotations

import argparse
import os
from concurrent.futures import ThreadPoolExecutor

import torch

from miles_amd import _lib, launch
from miles_amd.tools import _checkpoint as ckpt

FP8_INFO = torch.finfo(torch.float8_e4m3fn)
FP8_MAX, FP8_MIN = FP8_INFO.max, FP8_INFO.min


def ceildiv(a, b):
    return -(-a // b)


def block_fp8(weight: torch.Tensor, block_size):
    """weight [N, K] -> (float8_e4m3fn [N, K], float32 [ceil(N/bn), ceil(K/bk)]).

    Per (zero-padded) tile: scale = amax / 448 with a true division, q = e4m3(clamp(w / scale, +-448)).
    An all-zero tile keeps the reference's CPU result: scale 0 and every byte 0xFF.
    """
    _lib.require_gpu(weight, "block_fp8")
    bn, bk = int(block_size[0]), int(block_size[1])
    n, k = weight.shape
    w = weight if weight.stride(1) == 1 else weight.contiguous()
    q = torch.empty((n, k), dtype=torch.float8_e4m3fn, device=w.device)
    scale = torch.empty((ceildiv(n, bn), ceildiv(k, bk)), dtype=torch.float32, device=w.device)
    _lib.dtype_code(w, "block_fp8")
    launch.submit(_lib.JOB_FP8_BLOCK, w, q, scale, None, None, n, k, w.stride(0), bn, bk)
    return q, scale


_AMAX_RECORD_WORDS = 1280   # MQ_NVFP4_RECORD_WORDS: partial maxima of a tensor on the device, then its folded amax


def _scaled_fp8(weight: torch.Tensor, per_channel: bool):
    _lib.require_gpu(weight, "channel_fp8" if per_channel else "tensor_fp8")
    n, k = weight.shape
    # the reference reduces with weight.abs().max() / .amax(dim=1): torch refuses a reduction over nothing
    if not per_channel and weight.numel() == 0:
        raise RuntimeError("max(): Expected reduction dim to be specified for input.numel() == 0. Specify the reduction dim with the 'dim' argument.")
    if per_channel and k == 0:
        raise RuntimeError("amax(): Expected reduction dim 1 to have non-zero size.")
    w = weight if weight.stride(1) == 1 else weight.contiguous()
    q = torch.empty((n, k), dtype=torch.float8_e4m3fn, device=w.device)
    scale = torch.empty((n, 1) if per_channel else (1,), dtype=torch.float32, device=w.device)
    floor = float(torch.tensor(1e-12, dtype=w.dtype).float())  # clamp(min=1e-12) acts in the weight dtype
    if not per_channel and w.dtype in (torch.bfloat16, torch.float16) and w.is_contiguous() and k % 8 == 0 and w.data_ptr() % 16 == 0:
        # a job of the batched driver (grouped launches, replayable): amax record as for NVFP4
        record = torch.empty(_AMAX_RECORD_WORDS, dtype=torch.int32, device=w.device)
        floor_bits = int(torch.tensor(floor, dtype=torch.float32).view(torch.int32))
        launch.submit(_lib.JOB_FP8_TENSOR, w, q, scale, record, None, n, k, k, floor_bits, 0)
        return q, scale
    ws = torch.empty(max(n, 1), dtype=torch.int32, device=w.device)
    launch.note_direct_call()
    rc = _lib.load().mq_fp8_scaled_quant(w.data_ptr(), _lib.dtype_code(w, "fp8"), w.stride(0), q.data_ptr(),
                                         scale.data_ptr(), ws.data_ptr(), n, k, int(per_channel), floor,
                                         _lib.stream_ptr(w.device))
    _lib.check(rc)
    return q, scale


def channel_fp8(weight: torch.Tensor):
    """One scale per output channel: (float8_e4m3fn [N, K], float32 [N, 1])."""
    return _scaled_fp8(weight, True)


def tensor_fp8(weight: torch.Tensor):
    """One scale per tensor: (float8_e4m3fn [N, K], float32 [1])."""
    return _scaled_fp8(weight, False)


def quant_fp8(weight, strategy, block_size=None):
    if strategy == "tensor":
        return tensor_fp8(weight)
    if strategy == "channel":
        return channel_fp8(weight)
    return block_fp8(weight, block_size)


# substrings of tensor names that stay in high precision (reference: tools/convert_hf_to_fp8.py:129-146)
FP8_SKIP_SUBSTRINGS = ("layernorm", "embed", "router", "mlp.gate.", "norm", "lm_head", "eh_proj", "weights_proj",
                       "head.", "wo_a", "ffn.gate.", "compressor.", "vision_tower", "mm_projector")


def should_quantize_fp8(key: str) -> bool:
    return "weight" in key and not any(s in key for s in FP8_SKIP_SUBSTRINGS)


def process_file(input_path, output_path, filename, strategy, block_size, result_collector, device="cuda"):
    """Quantize one shard: `<name>.weight` -> e4m3 plus `<name>.weight_scale_inv` (block) or `.weight_scale`."""
    if not filename.endswith(".safetensors"):
        return
    weights = ckpt.load_shard(input_path, filename, device)
    out: dict[str, torch.Tensor] = {}
    skipped: list[str] = []
    with launch.deferred():
        for key, tensor in weights.items():
            if should_quantize_fp8(key):
                q, scale = quant_fp8(tensor, strategy, block_size)
                out[key] = q
                out[key.replace(".weight", ".weight_scale_inv" if block_size else ".weight_scale")] = scale
            else:
                skipped.append(key.replace(".weight", ""))
                out[key] = tensor
    ckpt.save_shard(out, output_path, filename)
    result_collector.add(filename, out, skipped)


def fp8_quantization_config(strategy, block_size, results) -> dict:
    """`quantization_config` entry of config.json (reference: tools/convert_hf_to_fp8.py:186-236)."""
    skipped = list(set(results.modules_to_not_convert))
    if strategy in ("block", "tensor"):
        cfg = {"activation_scheme": "dynamic", "fmt": "e4m3", "quant_method": "fp8"}
        if block_size:
            cfg["weight_block_size"] = block_size
            if results.has_dsa_layers:
                cfg["scale_fmt"] = "ue8m0"
        if skipped:
            cfg["modules_to_not_convert"] = skipped
        return cfg
    common = {"actorder": None, "block_structure": None, "group_size": None, "num_bits": 8, "observer_kwargs": {},
              "symmetric": True, "type": "float"}
    group = {
        "input_activations": {**common, "dynamic": True, "observer": None, "strategy": "token"},
        "output_activations": None,
        "targets": ["Linear"],
        "weights": {**common, "dynamic": False, "observer": "minmax", "strategy": strategy},
    }
    return {"config_groups": {"group_0": group}, "format": "float-quantized", "ignore": skipped,
            "quant_method": "compressed-tensors", "quantization_status": "compressed"}


def convert_fp8(input_path, output_path, strategy, block_size=None, max_workers=4, device="cuda"):
    input_path = os.path.abspath(input_path)
    os.makedirs(output_path, exist_ok=True)
    ckpt.copy_side_files(input_path, output_path)
    results = ckpt.ShardResults(size_in_bytes=False)
    with ThreadPoolExecutor(max_workers=max_workers) as pool:
        futures = [pool.submit(process_file, input_path, output_path, f, strategy, block_size, results, device)
                   for f in ckpt.list_shards(input_path)]
        for fut in futures:
            fut.result()
    cfg = ckpt.read_config(input_path)
    if cfg is not None:
        cfg["quantization_config"] = fp8_quantization_config(strategy, block_size, results)
        ckpt.write_config(output_path, cfg)
    ckpt.write_index(output_path, results.weight_map, results.total_size)


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--model-dir", type=str, help="Path to the directory of the HF safetensors model.")
    ap.add_argument("--save-dir", type=str, help="Path to the directory to save the converted model.")
    ap.add_argument("--strategy", type=str, default="block", choices=["block", "channel", "tensor"])
    ap.add_argument("--block-size", type=int, nargs="*", default=None, help="eg. --block-size 32 32")
    ap.add_argument("--max-workers", type=int, default=1, help="Number of worker threads for parallel processing")
    args = ap.parse_args(argv)
    if os.path.exists(args.save_dir) and not os.path.isdir(args.save_dir):
        raise ValueError("The save_dir should be a directory.")
    os.makedirs(args.save_dir, exist_ok=True)
    convert_fp8(args.model_dir, args.save_dir, args.strategy, args.block_size, args.max_workers)


if __name__ == "__main__":
    main()
