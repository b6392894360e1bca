"""Atomic grouping and size-bounded packing of HF tensor units for the weight sync.

A unit is the list of (hf_name, tensor) one training-side parameter converted into (a weight, or a weight
plus its quantization scales); units are never split.  Same contracts as the reference's
miles/backends/training_utils/weight_update/hf_weight_iterator/bucketing.py
(`AtomicUpdateGroup` :13-19, `assemble_atomic_update_groups` :22-67, `pack_units_by_size` :70-86) and
atomic_groups.py (`get_hf_atomic_update_groups` :33-57).
"""

from __future__ import annotations

import dataclasses
from collections.abc import Iterable, Iterator

import torch

Unit = list[tuple[str, torch.Tensor]]


@dataclasses.dataclass(frozen=True)
class AtomicUpdateGroup:
    """HF-name suffixes whose tensors must reach the engine in the same load call."""

    key: str
    suffixes: tuple[str, ...]
    optional: bool = False


def _validate(groups: list[AtomicUpdateGroup]) -> None:
    for g in groups:
        assert g.suffixes, f"Atomic update group {g.key} has no suffixes"
        assert all(g.suffixes), f"Atomic update group {g.key} contains empty suffix"
        assert len(set(g.suffixes)) == len(g.suffixes), f"Atomic update group {g.key} contains duplicate suffixes"
    keys = [g.key for g in groups]
    assert len(set(keys)) == len(keys), f"Duplicate atomic update group keys: {keys}"


def assemble_atomic_update_groups(hf_param_units: Iterable[Unit],
                                  atomic_update_groups: list[AtomicUpdateGroup]) -> Iterator[Unit]:
    """Merge the units whose members end in a group's suffixes into one unit per name prefix (members in
    suffix order, each member's other tensors -- its scales -- riding along); pass other units through."""
    _validate(atomic_update_groups)
    waiting: dict[tuple[str, str], list[Unit | None]] = {}
    seen_keys: set[str] = set()
    for unit in hf_param_units:
        if not unit:
            continue
        hits = [(g, idx, name[: -len(suffix)])
                for name, _t in unit
                for g in atomic_update_groups
                for idx, suffix in enumerate(g.suffixes)
                if name.endswith(suffix)]
        assert len(hits) <= 1, f"Unit {[n for n, _ in unit]} matches multiple atomic group suffixes"
        if not hits:
            yield unit
            continue
        group, idx, prefix = hits[0]
        seen_keys.add(group.key)
        slots = waiting.setdefault((prefix, group.key), [None] * len(group.suffixes))
        assert slots[idx] is None, f"Duplicate member in atomic update group: {prefix}{group.suffixes[idx]}"
        slots[idx] = unit
        if all(s is not None for s in slots):
            del waiting[(prefix, group.key)]
            yield [named for member in slots for named in member]
    assert not waiting, f"Incomplete atomic update groups at end of stream: {sorted(waiting)}"
    for g in atomic_update_groups:
        assert g.optional or g.key in seen_keys, \
            f"Atomic update group {g.key} matched no params (suffixes {g.suffixes})"


def pack_units_by_size(hf_param_units: Iterable[Unit], max_bytes: int) -> Iterator[Unit]:
    """Greedy buckets: a bucket closes when adding the next unit would reach `max_bytes`; a unit larger
    than `max_bytes` gets a bucket of its own."""
    bucket: Unit = []
    size = 0
    for unit in hf_param_units:
        unit_bytes = sum(t.nbytes for _n, t in unit)
        if bucket and size + unit_bytes >= max_bytes:
            yield bucket
            bucket, size = [], 0
        bucket.extend(unit)
        size += unit_bytes
    if bucket:
        yield bucket


# ---- per-model atomic groups --------------------------------------------------------------------------
_DEEPSEEK_V4_GROUPS = [
    AtomicUpdateGroup("wqkv_a", (".self_attn.wq_a.weight", ".self_attn.wkv.weight")),
    AtomicUpdateGroup("compressor_wkv_gate", (".self_attn.compressor.wkv.weight", ".self_attn.compressor.wgate.weight")),
    AtomicUpdateGroup("indexer_compressor_wkv_gate",
                      (".self_attn.indexer.compressor.wkv.weight", ".self_attn.indexer.compressor.wgate.weight")),
]
_DEEPSEEK_V41_GROUPS = [AtomicUpdateGroup("wqkv_a", (".attn.wq_a.weight", ".attn.wkv.weight"))]


def get_hf_atomic_update_groups(model_name: str, *, q_lora_rank: int | None = None) -> list[AtomicUpdateGroup]:
    """HF tensors an SGLang loader fuses into one engine parameter must arrive together."""
    normalized = model_name.lower().replace("-", "").replace("_", "")
    if "deepseekv41" in normalized:
        return list(_DEEPSEEK_V41_GROUPS)
    if "deepseekv4" in normalized:
        return list(_DEEPSEEK_V4_GROUPS)
    if "inkling" in normalized:
        return []
    if q_lora_rank is not None:
        # q_a_proj + kv_a_proj_with_mqa are concatenated by the DeepSeek-family loader
        return [AtomicUpdateGroup("q_lora_a_proj",
                                  (".self_attn.q_a_proj.weight", ".self_attn.kv_a_proj_with_mqa.weight"))]
    return []
