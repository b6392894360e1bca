"""Official MiMo-V2 checkpoint (`MiMoV2ForCausalLM`) -> plain BF16 with separate q / k / v projections.

    python -m miles_amd.tools.convert_mimo_v2_to_bf16 --model-dir SRC --save-dir DST [--layers 0,1,5] [--num-experts 32]
                                                      [--keep-quant] [--device cuda]

Mirror of the reference's tools/convert_mimo_v2_to_bf16.py.  The source keeps `self_attn.qkv_proj` fused and
interleaved over `num_key_value_heads` shards (shard i = [q_i | k_i | v_i]), block-FP8 quantized shard by shard with
every shard padded to whole 128-row blocks (:59-66), the dense and MTP linears in block FP8 (:44-47) and the routed
experts as packed e2m1 with one E8M0 scale per 32 inputs (:50-56).  Everything is dequantized to BF16 on the GPU
(`mq_fp8_block_dequant`, `mq_mxfp4_dequant`), qkv is split back into head order (:69-81), layers / experts can be
thinned out (:84-121) and `quantization_config` / `attention_projection_layout` leave the config.  `--keep-quant`
only renumbers layers and copies every tensor as stored, which needs no GPU.

One difference: an E8M0 scale byte of 255 is NaN here (the format's definition, as in miles/utils/mxfp4.py) while the
reference tool's `exp2(255 - 127)` makes it infinity; no checkpoint stores that byte.
"""

from __future__ import annotations

import argparse
import json
import re
import shutil
from pathlib import Path

import torch
from safetensors import safe_open
from safetensors.torch import save_file

FP8_BLOCK = 128
MXFP4_BLOCK = 32
SHARD_BYTES = 5 * 1024**3
SCALE_SUFFIXES = ("weight_scale_inv", "weight_scale")
ROUTER_KEYS = ("mlp.gate.weight", "mlp.gate.e_score_correction_bias")

_LAYER = re.compile(r"^model\.layers\.(\d+)\.(.+)$")
_EXPERT = re.compile(r"^mlp\.experts\.(\d+)\.")


# ---------------------------------------------------------------------------------------------------------------------
# tensor transforms
def dequant_fp8_block(weight: torch.Tensor, scale_inv: torch.Tensor) -> torch.Tensor:
    """e4m3 [rows, cols] x fp32 [ceil(rows/128), ceil(cols/128)] -> bf16(float(weight) * scale of the 128x128 block)."""
    from miles_amd.tools.fp8_cast_bf16 import weight_dequant

    return weight_dequant(weight.contiguous(), scale_inv.float().contiguous(), FP8_BLOCK)


def dequant_mxfp4(packed: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """packed e2m1 pairs [out, in/2] (element 2i in the low nibble) x E8M0 bytes [out, in/32] -> bf16 [out, in]."""
    from miles_amd.utils.mxfp4 import dequantize_mxfp4

    out_dim, in_dim = packed.shape[0], packed.shape[1] * 2
    assert scale.shape == (out_dim, in_dim // MXFP4_BLOCK), f"{packed.shape=} {scale.shape=}"
    return dequantize_mxfp4(packed.view(torch.uint8).contiguous(), scale.view(torch.uint8).contiguous(), MXFP4_BLOCK)


def dequant_fused_qkv(weight: torch.Tensor, scale_inv: torch.Tensor, shards: int) -> torch.Tensor:
    """Every kv-head shard of the fused projection was quantized by itself, its rows padded to whole blocks: shard i
    owns rows [i * rows, (i + 1) * rows) of the weight and ceil(rows / 128) rows of the scale grid."""
    rows = weight.shape[0] // shards
    scale_rows = -(-rows // FP8_BLOCK)
    assert scale_inv.shape[0] == shards * scale_rows, f"{weight.shape=} {scale_inv.shape=} {shards=}"
    parts = [dequant_fp8_block(weight[i * rows:(i + 1) * rows], scale_inv[i * scale_rows:(i + 1) * scale_rows])
             for i in range(shards)]
    return torch.cat(parts)


def split_fused_qkv(qkv: torch.Tensor, config: dict, is_swa: bool) -> list[torch.Tensor]:
    """[q, k, v] in head order from the shard-interleaved fused projection."""
    shards = config["num_key_value_heads"]
    key = "swa_" if is_swa else ""
    heads, kv_heads = config[key + "num_attention_heads"], config[key + "num_key_value_heads"]
    assert heads % shards == 0 and kv_heads % shards == 0, f"{heads=} {kv_heads=} {shards=}"
    per_shard = [heads // shards * config[key + "head_dim"], kv_heads // shards * config[key + "head_dim"],
                 kv_heads // shards * config[key + "v_head_dim"]]
    assert qkv.shape[0] == shards * sum(per_shard), f"{qkv.shape=} does not match {shards=} x {per_shard=}"
    by_shard = qkv.view(shards, sum(per_shard), qkv.shape[1])
    return [piece.reshape(-1, qkv.shape[1]) for piece in by_shard.split(per_shard, dim=1)]


# ---------------------------------------------------------------------------------------------------------------------
# names and config
def output_name(name: str, layer_map: dict[int, int] | None, num_experts: int | None) -> str | None:
    """Where a source tensor goes, or None when its layer or expert is dropped."""
    hit = _LAYER.match(name)
    if hit is None:
        return name
    layer, rest = int(hit.group(1)), hit.group(2)
    if layer_map is not None and layer not in layer_map:
        return None
    expert = _EXPERT.match(rest)
    if expert is not None and num_experts is not None and int(expert.group(1)) >= num_experts:
        return None
    return f"model.layers.{layer if layer_map is None else layer_map[layer]}.{rest}"


def convert_config(config: dict, layer_map: dict[int, int] | None, num_experts: int | None, keep_quant: bool) -> dict:
    out = json.loads(json.dumps(config))
    if layer_map is not None:
        assert out.get("hybrid_block_size") is None, "per-layer schedules must be explicit lists"
        kept = list(layer_map)
        out["num_hidden_layers"] = len(kept)
        for schedule in ("hybrid_layer_pattern", "moe_layer_freq"):
            out[schedule] = [out[schedule][layer] for layer in kept]
    if num_experts is not None:
        assert out["num_experts_per_tok"] <= num_experts <= out["n_routed_experts"], num_experts
        out["n_routed_experts"] = num_experts
    if not keep_quant:
        out.pop("quantization_config", None)
        out.pop("attention_projection_layout", None)
        return out
    quant = out["quantization_config"]
    renamed = (output_name(module + ".weight", layer_map, num_experts) for module in quant.get("ignored_layers", []))
    quant["ignored_layers"] = [name.removesuffix(".weight") for name in renamed if name is not None]
    return out


_ALWAYS = ("input_layernorm.weight", "post_attention_layernorm.weight", "self_attn.o_proj.weight")
_SPLIT_ATTENTION = tuple(f"self_attn.{p}_proj.weight" for p in "qkv")
_DENSE_MLP = tuple(f"mlp.{p}_proj.weight" for p in ("gate", "up", "down"))


def _required_tensors(config: dict, layer: int, have: set[str]) -> set[str]:
    need = set(_ALWAYS)
    if "self_attn.qkv_proj.weight" not in have:
        need.update(_SPLIT_ATTENTION)
    if config["hybrid_layer_pattern"][layer] == 1 and config.get("add_swa_attention_sink_bias"):
        need.add("self_attn.attention_sink_bias")
    need.update(ROUTER_KEYS if config["moe_layer_freq"][layer] else _DENSE_MLP)
    return need


def check_output(weight_map: dict[str, str], config: dict) -> None:
    """Every kept decoder layer has the tensors its attention and MLP variant need, and all its routed experts."""
    per_layer: dict[int, set[str]] = {layer: set() for layer in range(config["num_hidden_layers"])}
    for name in weight_map:
        hit = _LAYER.match(name)
        if hit is not None and int(hit.group(1)) in per_layer:
            per_layer[int(hit.group(1))].add(hit.group(2))
    for layer, have in per_layer.items():
        if config["moe_layer_freq"][layer]:
            experts = {int(m.group(1)) for name in have if (m := _EXPERT.match(name))}
            assert experts == set(range(config["n_routed_experts"])), f"layer {layer}: experts {sorted(experts)[:4]}..."
        missing = _required_tensors(config, layer, have) - have
        assert not missing, f"layer {layer} is missing {sorted(missing)}"


# ---------------------------------------------------------------------------------------------------------------------
class ShardWriter:
    """Collects tensors on the host and writes a safetensors shard whenever 5 GiB have accumulated."""

    def __init__(self, save_dir: Path) -> None:
        self.save_dir = save_dir
        self.pending: dict[str, torch.Tensor] = {}
        self.pending_bytes = 0
        self.num_shards = 0
        self.total_bytes = 0
        self.weight_map: dict[str, str] = {}

    def add(self, name: str, tensor: torch.Tensor) -> None:
        assert name not in self.weight_map and name not in self.pending, f"duplicate tensor {name}"
        self.pending[name] = tensor.contiguous().cpu()
        self.pending_bytes += tensor.numel() * tensor.element_size()
        if self.pending_bytes >= SHARD_BYTES:
            self.flush()

    def flush(self) -> None:
        if not self.pending:
            return
        self.num_shards += 1
        filename = f"model-{self.num_shards:05d}.safetensors"
        save_file(self.pending, str(self.save_dir / filename), metadata={"format": "pt"})
        for name in self.pending:
            self.weight_map[name] = filename
        self.total_bytes += self.pending_bytes
        self.pending, self.pending_bytes = {}, 0


class _Source:
    """Read access to the tensors of a sharded safetensors checkpoint by name."""

    def __init__(self, root: Path, device: str) -> None:
        self.root, self.device = root, device
        self.shard_of: dict[str, str] = json.loads((root / "model.safetensors.index.json").read_text())["weight_map"]
        self._open: dict[str, object] = {}

    def tensor(self, name: str) -> torch.Tensor:
        shard = self.shard_of[name]
        if shard not in self._open:
            self._open[shard] = safe_open(str(self.root / shard), framework="pt", device="cpu")
        return self._open[shard].get_tensor(name).to(self.device)

    def names_in_shard_order(self):
        """Tensor names grouped by shard file (files in sorted order, names in index order inside a file)."""
        grouped: dict[str, list[str]] = {}
        for name, shard in self.shard_of.items():
            grouped.setdefault(shard, []).append(name)
        for shard in sorted(grouped):
            yield from grouped[shard]


class _Conversion:
    """State of one run: the source, the shard writer and the tallies printed at the end."""

    def __init__(self, source: _Source, writer: ShardWriter, config: dict, layer_map, num_experts, keep_quant) -> None:
        self.source, self.writer, self.config = source, writer, config
        self.layer_map, self.num_experts, self.keep_quant = layer_map, num_experts, keep_quant
        self.fused_qkv = config.get("attention_projection_layout") == "fused_qkv"
        self.tally = {"fp8": 0, "mxfp4": 0, "qkv_split": 0, "copied": 0}

    def run(self) -> None:
        for name in self.source.names_in_shard_order():
            target = output_name(name, self.layer_map, self.num_experts)
            if target is None:
                continue
            if self.keep_quant:
                self._emit(target, self.source.tensor(name))
            elif not name.endswith(SCALE_SUFFIXES):       # scales are consumed together with their weights
                self._dequantized(name, target)
        self.writer.flush()

    def _emit(self, target: str, tensor: torch.Tensor) -> None:
        self.writer.add(target, tensor)
        self.tally["copied"] += 1

    def _dequantized(self, name: str, target: str) -> None:
        tensor = self.source.tensor(name)
        if self.fused_qkv and target.endswith("self_attn.qkv_proj.weight"):
            self._fused_attention(name, target, tensor)
            return
        if tensor.dtype == torch.float8_e4m3fn:
            tensor = dequant_fp8_block(tensor, self.source.tensor(name + "_scale_inv"))
            self.tally["fp8"] += 1
        elif tensor.dtype == torch.uint8:
            tensor = dequant_mxfp4(tensor, self.source.tensor(name.removesuffix("weight") + "weight_scale"))
            self.tally["mxfp4"] += 1
        if self.num_experts is not None and target.endswith(ROUTER_KEYS):
            tensor = tensor[: self.num_experts]
        self._emit(target, tensor)

    def _fused_attention(self, name: str, target: str, tensor: torch.Tensor) -> None:
        layer = _LAYER.match(name)
        sliding = layer is None or self.config["hybrid_layer_pattern"][int(layer.group(1))] == 1
        if tensor.dtype == torch.float8_e4m3fn:
            tensor = dequant_fused_qkv(tensor, self.source.tensor(name + "_scale_inv"), self.config["num_key_value_heads"])
            self.tally["fp8"] += 1
        for letter, piece in zip("qkv", split_fused_qkv(tensor, self.config, sliding), strict=True):
            self.writer.add(target.replace("qkv_proj", letter + "_proj"), piece)
        self.tally["qkv_split"] += 1


def _copy_side_files(src: Path, dst: Path, keep_drafter: bool) -> None:
    for path in src.iterdir():
        if path.name.startswith("."):          # a download cache, say
            continue
        if path.is_dir():
            # the DFlash drafter reads hidden states of fixed layers of the full model: only valid with every layer kept
            if path.name != "dflash" or keep_drafter:
                shutil.copytree(path, dst / path.name, dirs_exist_ok=True)
        elif path.suffix != ".safetensors" and path.name not in ("config.json", "model.safetensors.index.json"):
            shutil.copy2(path, dst / path.name)


def main(model_dir: str, save_dir: str, layers: list[int] | None, num_experts: int | None, keep_quant: bool,
         device: str) -> None:
    src, dst = Path(model_dir), Path(save_dir)
    dst.mkdir(parents=True, exist_ok=True)
    config = json.loads((src / "config.json").read_text())
    assert config["architectures"] == ["MiMoV2ForCausalLM"], config["architectures"]
    layer_map = None if layers is None else {old: new for new, old in enumerate(layers)}
    assert layer_map is None or all(0 <= layer < config["num_hidden_layers"] for layer in layer_map), layers
    assert not (keep_quant and num_experts is not None), "--num-experts needs the dequantized output"

    writer = ShardWriter(dst)
    job = _Conversion(_Source(src, device), writer, config, layer_map, num_experts, keep_quant)
    job.run()

    new_config = convert_config(config, layer_map, num_experts, keep_quant)
    if not keep_quant:
        check_output(writer.weight_map, new_config)
    (dst / "config.json").write_text(json.dumps(new_config, indent=2) + "\n")
    _copy_side_files(src, dst, keep_drafter=layer_map is None)
    # the index appears last and in one rename: a conversion interrupted before this point leaves no index behind
    index_path = dst / "model.safetensors.index.json"
    staging = index_path.with_suffix(".json.tmp")
    staging.write_text(json.dumps({"metadata": {"total_size": writer.total_bytes}, "weight_map": writer.weight_map},
                                  indent=2) + "\n")
    staging.replace(index_path)
    print(f"{job.tally}; {len(writer.weight_map)} tensors, {writer.total_bytes / 1e9:.2f} GB in {writer.num_shards} "
          f"shards -> {dst}")


def cli(argv=None) -> None:
    parser = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    parser.add_argument("--model-dir", type=str, required=True)
    parser.add_argument("--save-dir", type=str, required=True)
    parser.add_argument("--layers", type=str, default=None, help="Comma-separated source layer indices to keep, in order.")
    parser.add_argument("--num-experts", type=int, default=None, help="Keep only the first N routed experts per MoE layer.")
    parser.add_argument("--keep-quant", action="store_true", help="Renumber layers but keep the source tensor formats.")
    parser.add_argument("--device", type=str, default="cuda", help="Dequantization runs on the GPU; --keep-quant works on cpu.")
    args = parser.parse_args(argv)
    layers = [int(x) for x in args.layers.split(",")] if args.layers else None
    main(args.model_dir, args.save_dir, layers, args.num_experts, args.keep_quant, args.device)


if __name__ == "__main__":
    cli()
