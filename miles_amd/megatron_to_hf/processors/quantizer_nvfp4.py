"""NVFP4 quantization of routed-expert tensors on the weight-sync path.

Same interface and decisions as the reference's
miles/backends/megatron_utils/megatron_to_hf/processors/quantizer_nvfp4.py: ignore rules (:17-50),
`quantize_params_nvfp4` (:53-98), gate/up pairing in `_quantize_moe_params` (:101-156),
`quantize_nvfp4` for 2-D / 3-D weights (:185-204).
"""

from __future__ import annotations

import re

import torch

from miles_amd.utils.nvfp4 import NVFP4_GROUP_SIZE, nvfp4_quantize_1d, nvfp4_quantize_1d_pair

from ._names import in_bf16_head_or_tail, named_in_extra_high_precision, parse_layer_param

# HF suffix -> role inside a gated MLP; the two roles of one expert share a global amax
GATED_PAIR_SUFFIXES = {".gate_proj.weight": "gate", ".up_proj.weight": "up", ".w1.weight": "gate", ".w3.weight": "up"}
_FLOAT_DTYPES = (torch.float16, torch.bfloat16, torch.float32)

# only the main language decoder: MTP layers and modality towers stay in high precision
_DECODER = r"(?:module\.)*(?:language_model\.)?decoder\.layers\.(\d+)\.(.+)"


class _IgnoreRules:
    """The `ignore` / `exclude_modules` lists of a quantization config.  A plain rule covers the module it names and
    everything below it; a rule starting with `re:` is a regular expression matched at the start of the name."""

    _cache: dict[tuple[str, ...], "_IgnoreRules"] = {}

    def __init__(self, rules: tuple[str, ...]) -> None:
        self.plain = frozenset(r for r in rules if not r.startswith("re:"))
        self.patterns = [re.compile(r[3:]) for r in rules if r.startswith("re:")]

    @classmethod
    def of(cls, quantization_config) -> "_IgnoreRules":
        merged: list[str] = []
        for key in ("ignore", "exclude_modules"):
            value = quantization_config.get(key) or []
            for rule in ([value] if isinstance(value, str) else value):
                if rule not in merged:
                    merged.append(rule)
        key = tuple(merged)
        if key not in cls._cache:
            if len(cls._cache) >= 16:
                cls._cache.clear()
            cls._cache[key] = cls(key)
        return cls._cache[key]

    def __bool__(self) -> bool:
        return bool(self.plain or self.patterns)

    def covers(self, name: str) -> bool:
        if any(p.match(name) for p in self.patterns):
            return True
        node = name                      # walk up the dotted path: a.b.c.weight, a.b.c, a.b, a
        while node:
            if node in self.plain:
                return True
            node = node.rpartition(".")[0]
        return False


def quantize_params_nvfp4(args, megatron_name, converted_named_params, quantization_config):
    assert quantization_config is not None
    assert quantization_config.get("quant_algo") == "NVFP4" or quantization_config.get("quant_method") == "nvfp4"
    if args is not None and (getattr(args, "fp4_param", False) or getattr(args, "fp4_param_gather", False)):
        raise NotImplementedError("fp4-param-gather is unsupported for Miles NVFP4 checkpoint export.")
    if named_in_extra_high_precision(args, megatron_name):
        return converted_named_params
    where = parse_layer_param(megatron_name, decoder=_DECODER, mtp=None, anchored=True)
    if where is None or in_bf16_head_or_tail(args, where.layer_idx):
        return converted_named_params
    if where.routed_expert_linear not in ("linear_fc1", "linear_fc2"):
        return converted_named_params
    return _quantize_moe_params(converted_named_params, _IgnoreRules.of(quantization_config))


def _eligible(name: str, weight: torch.Tensor, rules) -> bool:
    """A floating-point `.weight` matrix that no ignore rule covers; a last dimension that 1x16 blocks do not divide
    is an error, not a reason to skip."""
    if rules and rules.covers(name):
        return False
    if not name.endswith(".weight") or weight.dtype not in _FLOAT_DTYPES or weight.dim() < 2:
        return False
    if weight.shape[-1] % NVFP4_GROUP_SIZE:
        raise ValueError(f"Last dim {weight.shape[-1]} must be divisible by {NVFP4_GROUP_SIZE} for NVFP4 ({name}).")
    return True


def _split_gated_pair_name(name: str):
    """(`<expert prefix>`, "gate" | "up") for a gated-MLP input projection, (None, None) for anything else."""
    for suffix, role in GATED_PAIR_SUFFIXES.items():
        if name.endswith(suffix):
            return name[: -len(suffix)], role
    return None, None


def _quantize_moe_params(converted_named_params, ignore_rules):
    """Quantize every eligible tensor of one conversion batch.  gate / up of an expert go through the paired
    quantizer (one amax over both); a batch that holds only one of the two, or one of them twice, is refused."""
    if not isinstance(ignore_rules, _IgnoreRules):
        ignore_rules = _IgnoreRules(tuple(ignore_rules or ()))
    chosen = {i for i, (name, tensor) in enumerate(converted_named_params) if _eligible(name, tensor, ignore_rules)}

    by_expert: dict[str, dict[str, int]] = {}
    for i in sorted(chosen):
        prefix, role = _split_gated_pair_name(converted_named_params[i][0])
        if prefix is None:
            continue
        slots = by_expert.setdefault(prefix, {})
        if role in slots:
            raise ValueError(f"NVFP4 requires a single complete gate/up pair per conversion batch; "
                             f"found duplicate {role} tensor for {prefix}.")
        slots[role] = i

    results: dict[int, tuple] = {}
    for prefix, slots in by_expert.items():
        if len(slots) != 2:
            raise ValueError(f"NVFP4 requires gate/up tensors to be quantized together so they can share "
                             f"one global amax; found only {{{', '.join(sorted(slots))}}} for {prefix}.")
        gate, up = slots["gate"], slots["up"]
        results[gate], results[up] = nvfp4_quantize_1d_pair(converted_named_params[gate][1], converted_named_params[up][1])

    emitted = []
    for i, (name, tensor) in enumerate(converted_named_params):
        if i not in chosen:
            emitted.append((name, tensor))
            continue
        codes, block_scale, global_scale = results[i] if i in results else quantize_nvfp4(tensor)
        emitted += [(name, codes), (name.replace(".weight", ".weight_scale"), block_scale),
                    (name.replace(".weight", ".weight_scale_2"), global_scale)]
    return emitted


def quantize_nvfp4(weight: torch.Tensor):
    """(uint8 [.., M, K/2], float8_e4m3fn [.., M, K/16], float32 global scale) for a matrix or a stack of matrices,
    each matrix of a stack with its own global scale."""
    if weight.dim() == 3:
        # The stacked results are allocated first and every matrix's job writes its slices: inside a deferred or
        # recorded batch the jobs have not run when this function returns, so nothing may be gathered from
        # per-matrix results here (a torch.stack would copy buffers that are still uninitialised).
        n, rows, cols = weight.shape
        if cols % NVFP4_GROUP_SIZE:
            raise ValueError(f"NVFP4 requires K divisible by {NVFP4_GROUP_SIZE}, got {cols}.")
        codes = torch.empty((n, rows, cols // 2), dtype=torch.uint8, device=weight.device)
        block_scale = torch.empty((n, rows, cols // NVFP4_GROUP_SIZE), dtype=torch.float8_e4m3fn, device=weight.device)
        global_scale = torch.empty((n,), dtype=torch.float32, device=weight.device)
        for i in range(n):
            nvfp4_quantize_1d(weight[i], out=(codes[i], block_scale[i], global_scale[i]))
        return codes, block_scale, global_scale
    if weight.dim() != 2:
        raise ValueError(f"Unsupported weight rank {weight.dim()} for NVFP4 quantization.")
    if weight.shape[1] % NVFP4_GROUP_SIZE:
        raise ValueError(f"NVFP4 requires K divisible by {NVFP4_GROUP_SIZE}, got {weight.shape[1]}.")
    return nvfp4_quantize_1d(weight.contiguous())
