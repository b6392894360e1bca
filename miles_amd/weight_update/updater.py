"""Weight-sync driver: streams quantized HF buckets of a model to a consumer.

Single-process form of the reference's `WeightUpdater.update_weights`
(miles/backends/training_utils/weight_update/updater.py:123-171): the engine session calls, Gloo barriers and
transfer protocols of the reference are outside this path; what remains is the loop
`for bucket in iterator.iter_hf_weights(weights): protocol.send_bucket(bucket)` under the wall-clock span
"update_weights_implementation", followed -- when the caller gives a `finalize` hook, the stand-in for
`protocol.finalize(weight_version)` and the engine calls of :164-170 -- by that hook under the span
"finalize_and_resume_engines" (no hook, no such span: there is nothing to time).  `send_bucket` is any
callable taking a list of (hf_name, tensor); as in the reference, a bucket belongs to the consumer only until
`send_bucket` returns (its memory is reused for a later bucket).  After the first sync the recorded `SyncPlan` is
replayed as long as the parameter set is unchanged.
"""

from __future__ import annotations

import logging
import time
from argparse import Namespace
from collections.abc import Callable, Mapping

import torch

from miles_amd.megatron_to_hf import name_maps
from miles_amd.weight_update.bucketing import Unit
from miles_amd.weight_update.hf_weight_iterator import HfWeightIteratorDirect
from miles_amd.weight_update.packed_bucket import pack_bucket
from miles_amd.weight_update.sync_plan import SyncPlan, weights_signature

_log = logging.getLogger(__name__)


def _fp8_row_block_views_ok(args: Namespace, quantization_config: dict | None) -> bool:
    """q / k / v can be quantized in place when every group's row block is a whole number of 128-row tiles."""
    if not quantization_config or quantization_config.get("quant_method") != "fp8":
        return False
    if list(quantization_config.get("weight_block_size") or []) != [128, 128]:
        return False
    try:
        kv = getattr(args, "kv_channels", None)
        head_dim = kv if kv is not None else args.hidden_size // args.num_attention_heads
        q_per_group = args.num_attention_heads // args.num_query_groups
    except AttributeError:
        return False
    return head_dim % 128 == 0 and (head_dim * q_per_group) % 128 == 0 and args.hidden_size % 8 == 0


class WeightUpdater:
    def __init__(self, args: Namespace, *, weights_getter: Callable[[], Mapping[str, torch.Tensor]], model_name: str,
                 quantization_config: dict | None, send_bucket: Callable[[Unit], None],
                 packed_weight_basenames: set[str] | None = None, use_plan: bool = True,
                 packed_buckets: bool = False, plan_arenas: int | None = 2,
                 finalize: Callable[[int], None] | None = None) -> None:
        self.args = Namespace(**vars(args))
        if _fp8_row_block_views_ok(self.args, quantization_config):
            self.args.qkv_row_block_views = True
        self.weights_getter = weights_getter
        self.send_bucket = send_bucket
        self.finalize = finalize               # called with the new weight version once every bucket has been sent
        self.use_plan = use_plan
        self.packed_buckets = packed_buckets   # hand out PackedBucket payloads (the reference's broadcast_packed mode)
        # output arenas of a recorded sync: bucket k lives in arena k mod plan_arenas and is valid until `send_bucket`
        # returns from it (the reference drops a bucket after sending it); None keeps every bucket in an arena of its own
        self.plan_arenas = plan_arenas
        self.weight_version = 0
        self._iterator = _RowBlockAwareIterator(self.args, model_name=model_name,
                                                quantization_config=quantization_config,
                                                packed_weight_basenames=packed_weight_basenames)
        self._plan: SyncPlan | None = None
        self._refused_signature: tuple | None = None     # the parameter set whose recording could not be replayed
        self.plan_refusal: tuple[str, ...] = ()           # why (see SyncPlan.refusal)
        self._metrics: dict[str, float] = {}

    def pop_metrics(self) -> dict[str, float]:
        """Wall-clock spans of the last sync, in seconds; cleared by the call."""
        out, self._metrics = self._metrics, {}
        return out

    @torch.no_grad()
    def update_weights(self) -> None:
        self.weight_version += 1
        weights = self.weights_getter()
        t0 = time.perf_counter()
        for bucket in self._iter_buckets(weights):
            self.send_bucket(bucket)
        t1 = time.perf_counter()
        self._metrics["update_weights_implementation"] = t1 - t0
        if self.finalize is not None:
            self.finalize(self.weight_version)
            self._metrics["finalize_and_resume_engines"] = time.perf_counter() - t1

    def _iter_buckets(self, weights):
        if self.use_plan and self._plan is not None and self._plan.matches(weights):
            yield from self._plan.replay()
            return
        if self.use_plan and (self._refused_signature is None or weights_signature(weights) != self._refused_signature):
            self._plan = None                      # a plan for another parameter set: let its arenas go first
            plan = SyncPlan.record(self._iterator, weights, packed=self.packed_buckets, ring=self.plan_arenas)
            if plan.replayable:
                self._plan, self._refused_signature = plan, None
                yield from plan.replay()
                return
            # A sync that a replay cannot reproduce (a kernel outside the job list, a tensor some torch op materialised,
            # a bucket that cannot be laid out as a payload) streams through the iterator, this time and for as long as
            # the parameter set stays the one that was refused: recording it again would repeat the per-parameter work
            # of a whole sync for nothing.  Another parameter set (a reloaded model, other dtypes) is recorded afresh.
            self._refused_signature = plan.signature
            self.plan_refusal = plan.refusal
            _log.warning("weight sync is not replayable (%s): every sync of this parameter set runs the full iterator",
                         ", ".join(plan.refusal))
            del plan
        for bucket in self._iterator.iter_hf_weights(weights):
            yield pack_bucket(bucket) if self.packed_buckets else bucket


class _RowBlockAwareIterator(HfWeightIteratorDirect):
    """Flattens row-blocked [groups, rows, hidden] views that ended up unquantized back to 2-D."""

    def _convert_batch(self, named_params):
        units = super()._convert_batch(named_params)
        if getattr(self.args, "qkv_row_block_views", False):
            for unit in units:
                for i, (name, t) in enumerate(unit):
                    if t.dim() == 3 and name.endswith(("q_proj.weight", "k_proj.weight", "v_proj.weight")):
                        unit[i] = (name, name_maps.gather_groups(t, (-1, t.shape[-1])))
        return units
