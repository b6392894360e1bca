"""Streaming a training model's weights as quantized, HF-named, size-bounded buckets on one GPU.

`HfWeightIteratorBase.iter_hf_weights` keeps the template of the reference's
miles/backends/training_utils/weight_update/hf_weight_iterator/__init__.py:96-122
(units -> atomic groups -> buckets).  `HfWeightIteratorDirect` is the single-GPU form of the reference's
miles/backends/megatron_utils/update_weight/hf_weight_iterator_direct.py:77-146: parameters are taken in name
order, the non-expert ones before the routed experts (:39-43, :85-108), in gather batches of at most
`update_weight_buffer_size` bytes (`_pack_param_infos_by_size`, :246-259), each
parameter goes through `convert_to_hf` (name map + quantizer), and -- unlike the reference, which launches a
chain of kernels per tensor -- all quantizer calls of a batch are recorded and submitted as ONE
`mq_run_jobs` call (grouped kernel launches).  The TP / EP / PP collectives of the reference are outside
this path: the iterator expects full (already gathered) parameters.
"""

from __future__ import annotations

import dataclasses
import re
from abc import ABC, abstractmethod
from argparse import Namespace
from collections.abc import Iterator, Mapping, Sequence

import torch

from miles_amd import launch
from miles_amd.megatron_to_hf import convert_to_hf
from miles_amd.weight_update.bucketing import (AtomicUpdateGroup, Unit, assemble_atomic_update_groups,
                                               get_hf_atomic_update_groups, pack_units_by_size)


@dataclasses.dataclass(frozen=True)
class ParamInfo:
    """Metadata of one training-side parameter (reference: miles/utils/types.py ParamInfo)."""

    name: str
    dtype: torch.dtype
    shape: torch.Size
    size: int          # bytes of the full parameter


class HfWeightIteratorBase(ABC):
    """Yields buckets of (hf_name, tensor); atomic update groups are never split across buckets."""

    def __init__(self, args: Namespace, *, model_name: str, quantization_config: dict | None) -> None:
        self.args = args
        self.model_name = model_name
        self.quantization_config = quantization_config

    def iter_hf_weights(self, weights: Mapping[str, torch.Tensor], *, materialize: bool = True) -> Iterator[Unit]:
        units = self._iter_hf_param_units(weights, materialize=materialize)
        groups = self._hf_atomic_update_groups() if materialize else []
        yield from pack_units_by_size(assemble_atomic_update_groups(units, groups),
                                      self.args.update_weight_buffer_size)

    @abstractmethod
    def _iter_hf_param_units(self, weights: Mapping[str, torch.Tensor], *, materialize: bool) -> Iterator[Unit]:
        """One unit per training-side parameter: every HF tensor it converted into."""

    def _hf_atomic_update_groups(self) -> list[AtomicUpdateGroup]:
        return []


def _pack_param_infos_by_size(args: Namespace, param_infos: Sequence[ParamInfo], *,
                              size_multiplier: int = 1) -> list[list[ParamInfo]]:
    """Greedy gather batches of at most `update_weight_buffer_size` bytes (a larger parameter stands alone)."""
    batches: list[list[ParamInfo]] = [[]]
    used = 0
    for info in param_infos:
        size = info.size * size_multiplier
        if used + size > args.update_weight_buffer_size and batches[-1]:
            batches.append([])
            used = 0
        batches[-1].append(info)
        used += size
    return [b for b in batches if b]


def is_routed_expert_param(name: str) -> bool:
    """A parameter of the routed experts: under `.experts.`, but not an inner list of the shared experts
    (reference: hf_weight_iterator_direct.py `is_routed_expert_param`)."""
    return ".experts." in name and ".shared_experts." not in name


def _split_param_infos(infos: Sequence[ParamInfo]) -> tuple[list[ParamInfo], list[ParamInfo]]:
    """(non-expert infos, routed-expert infos), each sorted by parameter name: the order in which the reference
    streams a model (`_get_megatron_local_param_infos`, hf_weight_iterator_direct.py:293-344 -- every non-expert
    batch is sent before the first expert batch, :85-108)."""
    ordered = sorted(infos, key=lambda info: info.name)
    return ([i for i in ordered if not is_routed_expert_param(i.name)],
            [i for i in ordered if is_routed_expert_param(i.name)])


_GROUPED_EXPERT_WEIGHT = re.compile(r"\.weight(\d+)$")


def _expert_share_of_this_rank(expert_infos: Sequence[ParamInfo]) -> list[ParamInfo]:
    """The routed experts this rank converts.  The reference deals contiguous ranges of local experts to the expert
    data-parallel replicas (`_partition_expert_infos`, :262-278) by the number at the end of a grouped weight's name;
    one GPU is the only replica and takes them all, in name order, but a routed-expert parameter that does not name
    its expert is refused as there."""
    for info in expert_infos:
        if _GROUPED_EXPERT_WEIGHT.search(info.name) is None:
            raise ValueError(f"Cannot identify the routed expert in {info.name!r}")
    return list(expert_infos)


class HfWeightIteratorDirect(HfWeightIteratorBase):
    """Megatron-named full parameters -> quantized HF units, one batched kernel submission per gather batch."""

    def __init__(self, args: Namespace, *, model_name: str, quantization_config: dict | None,
                 packed_weight_basenames: set[str] | None = None) -> None:
        super().__init__(args, model_name=model_name, quantization_config=quantization_config)
        self.packed_weight_basenames = packed_weight_basenames

    def _hf_atomic_update_groups(self):
        return get_hf_atomic_update_groups(self.model_name, q_lora_rank=getattr(self.args, "q_lora_rank", None))

    def _iter_hf_param_units(self, weights, *, materialize):
        infos = [ParamInfo(name, t.dtype, t.shape, t.numel() * t.element_size()) for name, t in weights.items()]
        non_expert_infos, expert_infos = _split_param_infos(infos)
        # every non-expert batch first, then the expert batches, each in name order: what the reference hands its
        # transfer protocol (the bucket composition of a mixture-of-experts sync follows from it)
        batches = _pack_param_infos_by_size(self.args, non_expert_infos)
        if expert_infos:
            batches += _pack_param_infos_by_size(self.args, _expert_share_of_this_rank(expert_infos))
        for batch in batches:
            if not materialize:
                continue
            yield from self._convert_batch([(info.name, weights[info.name]) for info in batch])

    def _convert_batch(self, named_params: Sequence[tuple[str, torch.Tensor]]) -> list[Unit]:
        """Name-map and quantize every parameter of a gather batch; the kernels run when the block ends."""
        with launch.deferred():
            units = [list(convert_to_hf(self.args, self.model_name, name, param, self.quantization_config,
                                        self.packed_weight_basenames))
                     for name, param in named_params]
        return units
