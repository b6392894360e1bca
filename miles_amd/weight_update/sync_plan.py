"""A recorded weight sync that can be replayed with (almost) no host work.

The shapes, names and addresses of a training model's parameters do not change between RL steps, so the
per-parameter Python work of a sync (name mapping, quantizer dispatch, output allocation, bucketing) only
has to happen once.  `SyncPlan.record` runs the iterator once under `launch.recording()`: every quantizer
call allocates its outputs and records its job; the plan keeps the job list, the output tensors and the
buckets.  `SyncPlan.replay` then re-runs the jobs -- a handful of `mq_run_jobs` calls, each a few grouped
kernel launches -- and hands out the same buckets again, now holding the freshly quantized values.

Replay is only valid when every kernel input aliases live parameter storage (views such as gate/up chunks or
row-blocked q/k/v are fine; a name map that materialises a copy is not): `replayable` says so, and the
updater falls back to the full iterator when it is False.  The plan owns its output tensors: a bucket's
contents are valid until the next replay.
"""

from __future__ import annotations

import bisect
from collections.abc import Iterator, Mapping

import torch

from miles_amd import launch
from miles_amd.weight_update.bucketing import Unit
from miles_amd.weight_update.hf_weight_iterator import HfWeightIteratorBase


def weights_signature(weights: Mapping[str, torch.Tensor]) -> tuple:
    """Identity of a parameter set: addresses, shapes and dtypes in order."""
    return tuple((name, t.data_ptr(), tuple(t.shape), t.dtype) for name, t in weights.items())


class SyncPlan:
    def __init__(self, batch: launch.JobBatch, buckets: list[Unit], jobs_done_at_bucket: list[int],
                 signature: tuple, replayable: bool) -> None:
        self.batch = batch
        self.buckets = buckets
        self.jobs_done_at_bucket = jobs_done_at_bucket
        self.signature = signature
        self.replayable = replayable

    @classmethod
    def record(cls, iterator: HfWeightIteratorBase, weights: Mapping[str, torch.Tensor]) -> "SyncPlan":
        """Run one full sync, keeping everything needed to repeat it."""
        buckets: list[Unit] = []
        marks: list[int] = []
        with launch.recording() as batch:
            for bucket in iterator.iter_hf_weights(weights):
                buckets.append(bucket)
                marks.append(len(batch))   # every job of this bucket (and maybe some of the next) is recorded
        device = next((t.device for t in weights.values() if t.device.type == "cuda"), None)
        batch.device = batch.device or device
        batch.freeze()
        replayable = batch.direct_calls == 0 and cls._inputs_alias(weights, batch)
        plan = cls(batch, buckets, marks, weights_signature(weights), replayable)
        for _ in plan.replay():     # the first execution uses the same launch partition as every replay
            pass
        return plan

    @staticmethod
    def _inputs_alias(weights: Mapping[str, torch.Tensor], batch: launch.JobBatch) -> bool:
        spans = sorted((t.untyped_storage().data_ptr(), t.untyped_storage().data_ptr() + t.untyped_storage().nbytes())
                       for t in weights.values())
        starts = [s for s, _ in spans]
        for ptr in batch.input_pointers():
            i = bisect.bisect_right(starts, ptr) - 1
            if i < 0 or ptr >= spans[i][1]:
                return False
        return True

    def matches(self, weights: Mapping[str, torch.Tensor]) -> bool:
        return self.replayable and weights_signature(weights) == self.signature

    def replay(self) -> Iterator[Unit]:
        """Re-quantize into the plan's output tensors, bucket by bucket, and yield the buckets."""
        done = 0
        for bucket, mark in zip(self.buckets, self.jobs_done_at_bucket):
            self.batch.run_range(done, mark)
            done = max(done, mark)
            yield bucket

    def replay_all(self) -> list[Unit]:
        """Whole model in one submission (fewest launches); returns every bucket."""
        self.batch.run()
        return self.buckets
