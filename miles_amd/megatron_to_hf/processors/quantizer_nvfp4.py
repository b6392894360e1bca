"""NVFP4 quantization of routed-expert tensors on the weight-sync path.

Same interface and decisions as the reference's
miles/backends/megatron_utils/megatron_to_hf/processors/quantizer_nvfp4.py: ignore rules (:17-50),
`quantize_params_nvfp4` (:53-98), gate/up pairing in `_quantize_moe_params` (:101-156),
`quantize_nvfp4` for 2-D / 3-D weights (:185-204).
"""

from __future__ import annotations

import re
from functools import lru_cache

import torch

from miles_amd.utils.nvfp4 import NVFP4_GROUP_SIZE, nvfp4_quantize_1d, nvfp4_quantize_1d_pair

from ._names import in_bf16_head_or_tail, named_in_extra_high_precision, parse_layer_param

GATED_PAIR_SUFFIXES = {
    ".gate_proj.weight": "gate",
    ".up_proj.weight": "up",
    ".w1.weight": "gate",
    ".w3.weight": "up",
}

# only the main language decoder: MTP layers and modality towers stay in high precision
_DECODER = r"(?:module\.)*(?:language_model\.)?decoder\.layers\.(\d+)\.(.+)"


def _as_list(value) -> list[str]:
    if not value:
        return []
    return [value] if isinstance(value, str) else list(value)


def _get_ignore_rules(quantization_config) -> list[str]:
    rules = _as_list(quantization_config.get("ignore", []))
    return rules + [r for r in _as_list(quantization_config.get("exclude_modules", [])) if r not in rules]


@lru_cache(maxsize=16)
def _literal_ignore_rules(ignore_rules: tuple[str, ...]) -> frozenset[str] | None:
    """A hashable set when no rule is a regex (then matching is a walk up the dotted name)."""
    if any(rule.startswith("re:") for rule in ignore_rules):
        return None
    return frozenset(ignore_rules)


def _is_ignored(name: str, ignore_rules: list[str], literal_rules: frozenset[str] | None = None) -> bool:
    if literal_rules is not None:
        while True:
            if name in literal_rules:
                return True
            name, dot, _ = name.rpartition(".")
            if not dot:
                return False
    for rule in ignore_rules:
        if rule.startswith("re:"):
            if re.match(rule[3:], name):
                return True
        elif name == rule or name.startswith(f"{rule}."):
            return True
    return False


def quantize_params_nvfp4(args, megatron_name, converted_named_params, quantization_config):
    assert quantization_config is not None
    assert quantization_config.get("quant_algo") == "NVFP4" or quantization_config.get("quant_method") == "nvfp4"
    if args is not None and bool(getattr(args, "fp4_param", False) or getattr(args, "fp4_param_gather", False)):
        raise NotImplementedError("fp4-param-gather is unsupported for Miles NVFP4 checkpoint export.")
    if named_in_extra_high_precision(args, megatron_name):
        return converted_named_params
    p = parse_layer_param(megatron_name, decoder=_DECODER, mtp=None, anchored=True)
    if p is None or in_bf16_head_or_tail(args, p.layer_idx):
        return converted_named_params
    if p.routed_expert_linear in ("linear_fc1", "linear_fc2"):
        return _quantize_moe_params(converted_named_params, _get_ignore_rules(quantization_config))
    return converted_named_params


def _quantize_moe_params(converted_named_params, ignore_rules):
    literal_rules = _literal_ignore_rules(tuple(ignore_rules))
    wanted = [_should_quantize_param(n, t, ignore_rules, literal_rules) for n, t in converted_named_params]

    # gate/up tensors of one expert share one global amax: collect complete pairs first
    pairs: dict[str, dict[str, tuple[str, torch.Tensor]]] = {}
    for (name, tensor), want in zip(converted_named_params, wanted):
        base, role = _split_gated_pair_name(name)
        if base is None or not want:
            continue
        roles = pairs.setdefault(base, {})
        if role in roles:
            raise ValueError(f"NVFP4 requires a single complete gate/up pair per conversion batch; "
                             f"found duplicate {role} tensor for {base}.")
        roles[role] = (name, tensor)

    paired = {}
    for base, roles in pairs.items():
        if set(roles) != {"gate", "up"}:
            present = ", ".join(sorted(roles))
            raise ValueError(f"NVFP4 requires gate/up tensors to be quantized together so they can share "
                             f"one global amax; found only {{{present}}} for {base}.")
        (gate_name, gate), (up_name, up) = roles["gate"], roles["up"]
        paired[gate_name], paired[up_name] = nvfp4_quantize_1d_pair(gate, up)

    out = []
    for (name, tensor), want in zip(converted_named_params, wanted):
        if not want:
            out.append((name, tensor))
            continue
        qweight, block_scale, weight_scale_2 = paired[name] if name in paired else quantize_nvfp4(tensor)
        out.append((name, qweight))
        out.append((name.replace(".weight", ".weight_scale"), block_scale))
        out.append((name.replace(".weight", ".weight_scale_2"), weight_scale_2))
    return out


def _should_quantize_param(name, weight, ignore_rules, literal_rules=None):
    if ignore_rules and _is_ignored(name, ignore_rules, literal_rules):
        return False
    if not name.endswith(".weight"):
        return False
    if weight.dtype not in (torch.float16, torch.bfloat16, torch.float32) or weight.dim() < 2:
        return False
    if weight.shape[-1] % NVFP4_GROUP_SIZE != 0:
        raise ValueError(f"Last dim {weight.shape[-1]} must be divisible by {NVFP4_GROUP_SIZE} for NVFP4 ({name}).")
    return True


def _split_gated_pair_name(name: str):
    for suffix, role in GATED_PAIR_SUFFIXES.items():
        if name.endswith(suffix):
            return name[: -len(suffix)], role
    return None, None


def _quantize_nvfp4_1d(weight: torch.Tensor):
    """1x16 tiles: (uint8 [M, K/2], float8_e4m3fn [M, K/16], float32 [])."""
    weight = weight.contiguous()
    if weight.shape[1] % NVFP4_GROUP_SIZE != 0:
        raise ValueError(f"NVFP4 requires K divisible by {NVFP4_GROUP_SIZE}, got {weight.shape[1]}.")
    return nvfp4_quantize_1d(weight)


def quantize_nvfp4(weight: torch.Tensor):
    if weight.dim() == 2:
        return _quantize_nvfp4_1d(weight)
    if weight.dim() == 3:
        parts = [_quantize_nvfp4_1d(weight[i]) for i in range(weight.shape[0])]
        return tuple(torch.stack([p[k] for p in parts], dim=0) for k in range(3))
    raise ValueError(f"Unsupported weight rank {weight.dim()} for NVFP4 quantization.")
