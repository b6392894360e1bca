"""Megatron parameter-name parsing shared by the quantizer processors.

The reference repeats the same regular expressions in every processor
(miles/backends/megatron_utils/megatron_to_hf/processors/quantizer_fp8.py:27-82,
quantizer_mxfp8.py:14-74, quantizer_nvfp4.py:67-92); here they are parsed once into a small record.
"""

from __future__ import annotations

import dataclasses
import re

_ROUTED_EXPERT = re.compile(r"mlp.experts\.(.+)\.weight(\d+)")
_SHARED_EXPERT = re.compile(r"mlp.shared_experts\.(.+)")


@dataclasses.dataclass(frozen=True)
class LayerParam:
    """A parameter inside a decoder (or MTP) layer."""

    layer_idx: int
    rest: str          # name below "layers.<idx>."
    is_mtp: bool

    @property
    def routed_expert_linear(self) -> str | None:
        """'linear_fc1' / 'linear_fc2' for `mlp.experts.<linear>.weight<e>`, else None."""
        m = _ROUTED_EXPERT.match(self.rest)
        return m.group(1) if m else None

    @property
    def shared_expert_rest(self) -> str | None:
        m = _SHARED_EXPERT.match(self.rest)
        return m.group(1) if m else None


def parse_layer_param(megatron_name: str, *, decoder: str, mtp: str | None, anchored: bool) -> LayerParam | None:
    """Split `<decoder>(idx).(rest)`; `anchored` selects re.match (prefix must match) or re.search."""
    find = re.match if anchored else re.search
    m = find(decoder, megatron_name)
    if m:
        return LayerParam(int(m.group(1)), m.group(2), False)
    if mtp is None:
        return None
    m = find(mtp, megatron_name)
    if not m:
        return None
    rest = m.group(2).replace("transformer_layer.", "").replace("mtp_model_layer.", "")
    return LayerParam(int(m.group(1)), rest, True)


def in_bf16_head_or_tail(args, layer_idx: int) -> bool:
    """--first-last-layers-bf16: the first / last N decoder layers stay unquantized."""
    if not getattr(args, "first_last_layers_bf16", False):
        return False
    n = int(args.num_layers)
    head = int(getattr(args, "num_layers_at_start_in_bf16", 0))
    tail = int(getattr(args, "num_layers_at_end_in_bf16", 0))
    return layer_idx < head or layer_idx >= n - tail


def named_in_extra_high_precision(args, megatron_name: str) -> bool:
    layers = getattr(args, "extra_high_precision_layers_megatron", False)
    return bool(layers) and any(layer in megatron_name for layer in layers)
