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


class _PendingGroups:
    """Members of atomic groups seen so far, keyed by (name prefix, group key), until their group is complete."""

    def __init__(self, groups: list[AtomicUpdateGroup]) -> None:
        self.groups = groups
        self.open: dict[tuple[str, str], list[Unit | None]] = {}
        self.matched: set[str] = set()

    def locate(self, unit: Unit):
        """(group, member index, name prefix) of the one suffix this unit's names end in, or None."""
        found = []
        for name, _tensor in unit:
            for group in self.groups:
                for index, suffix in enumerate(group.suffixes):
                    if name.endswith(suffix):
                        found.append((group, index, name[: len(name) - len(suffix)]))
        assert len(found) <= 1, f"Unit {[n for n, _ in unit]} matches multiple atomic group suffixes"
        return found[0] if found else None

    def place(self, unit: Unit, group: AtomicUpdateGroup, index: int, prefix: str) -> Unit | None:
        """Store the member; the merged unit (members in suffix order) once the last one is in."""
        self.matched.add(group.key)
        key = (prefix, group.key)
        members = self.open.setdefault(key, [None] * len(group.suffixes))
        assert members[index] is None, f"Duplicate member in atomic update group: {prefix}{group.suffixes[index]}"
        members[index] = unit
        if any(m is None for m in members):
            return None
        del self.open[key]
        merged: Unit = []
        for member in members:
            merged.extend(member)
        return merged

    def finish(self) -> None:
        assert not self.open, f"Incomplete atomic update groups at end of stream: {sorted(self.open)}"
        for group in self.groups:
            assert group.optional or group.key in self.matched, \
                f"Atomic update group {group.key} matched no params (suffixes {group.suffixes})"


def assemble_atomic_update_groups(hf_param_units: Iterable[Unit],
                                  atomic_update_groups: list[AtomicUpdateGroup]) -> Iterator[Unit]:
    """Merge the units whose members end in a group's suffixes into one unit per name prefix (members in
    suffix order, each member's other tensors -- its scales -- riding along); pass other units through."""
    _validate(atomic_update_groups)
    pending = _PendingGroups(atomic_update_groups)
    for unit in hf_param_units:
        if not unit:
            continue
        where = pending.locate(unit)
        if where is None:
            yield unit
            continue
        merged = pending.place(unit, *where)
        if merged is not None:
            yield merged
    pending.finish()


def pack_units_by_size(hf_param_units: Iterable[Unit], max_bytes: int) -> Iterator[Unit]:
    """Greedy buckets: a bucket closes when adding the next unit would reach `max_bytes`; a unit larger
    than `max_bytes` gets a bucket of its own."""
    open_bucket: Unit = []
    held = 0
    for unit in hf_param_units:
        incoming = 0
        for _name, tensor in unit:
            incoming += tensor.nbytes
        if open_bucket and held + incoming >= max_bytes:
            yield open_bucket
            open_bucket, held = [], 0
        open_bucket += unit
        held += incoming
    if open_bucket:
        yield open_bucket


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
