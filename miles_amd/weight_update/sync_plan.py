"""A recorded weight sync that can be replayed with (almost) no host work.

The shapes, names and addresses of a training model's parameters do not change between RL steps, so the
per-parameter Python work of a sync (name mapping, quantizer dispatch, output allocation, bucketing) only
has to happen once.  `SyncPlan.record` runs the iterator once under `launch.recording()`: every quantizer
call allocates its outputs and records its job; the plan keeps the job list and the buckets.
`SyncPlan.replay` then runs the jobs -- a handful of `mq_run_jobs` calls, each a few grouped kernel launches --
and hands out the buckets, holding the freshly quantized values.

Memory: the outputs live in a ring of arenas, one bucket per arena (`plan_memory.Placement`), not in one buffer
per tensor, so a plan holds `ring` x the largest bucket (about `update_weight_buffer_size` each) however large the
model is -- the bound the reference keeps by producing, sending and dropping one bucket at a time
(miles/backends/training_utils/weight_update/updater.py:150-160).  A bucket is valid from the moment it is handed
out until the consumer returns from it; work the consumer queued on the launch stream is ordered before the reuse.

Replay is only valid when every kernel input aliases live parameter storage (views such as gate/up chunks or
row-blocked q/k/v are fine; a name map that materialises a copy is not): `replayable` says so, and the
updater falls back to the full iterator when it is False.
"""

from __future__ import annotations

import operator
from collections.abc import Iterator, Mapping

import torch

from miles_amd import _lib, launch
from miles_amd.weight_update.bucketing import Unit
from miles_amd.weight_update.hf_weight_iterator import HfWeightIteratorBase
from miles_amd.weight_update.plan_memory import Placement


_shape_of = operator.attrgetter("shape")


def weights_signature(weights: Mapping[str, torch.Tensor]) -> tuple:
    """Identity of a parameter set: addresses, shapes and dtypes in order."""
    return tuple((name, t.data_ptr(), tuple(t.shape), t.dtype) for name, t in weights.items())


class SyncPlan:
    def __init__(self, batch: launch.JobBatch, buckets: list[Unit], jobs_done_at_bucket: list[int],
                 signature: tuple, replayable: bool, ring: int | None = None, arena_bytes: int = 0) -> None:
        self.batch = batch
        self.buckets = buckets
        self.jobs_done_at_bucket = jobs_done_at_bucket
        self.signature = signature
        self.replayable = replayable
        self.ring = ring or max(len(buckets), 1)     # arenas the buckets rotate through
        self.arena_bytes = arena_bytes              # device memory the plan's outputs occupy
        self._marks: list[int] | None = None
        self._completed = 0         # full replays so far
        self._names: list[str] = []
        self._tensors: list[torch.Tensor] = []
        self._addresses: list[int] = []
        self._shapes: list[torch.Size] = []
        self.refusal: tuple[str, ...] = ()           # why the recording is not replayable (empty when it is)

    def remember(self, weights: Mapping[str, torch.Tensor]) -> None:
        """Keep the parameter objects themselves, for the quick form of `matches`."""
        self._names = list(weights)
        self._tensors = list(weights.values())
        self._addresses = [t.data_ptr() for t in self._tensors]
        self._shapes = [t.shape for t in self._tensors]

    @classmethod
    def record(cls, iterator: HfWeightIteratorBase, weights: Mapping[str, torch.Tensor], *,
               packed: bool = False, ring: int | None = 2) -> "SyncPlan":
        """Run the per-parameter work of one full sync, keeping everything needed to repeat it.  Nothing is
        executed here: `replay()` produces the buckets, the first time as every later time.

        Every tensor a job writes gets its place in one of `ring` output arenas (bucket k in arena k mod ring, None:
        an arena per bucket), so the plan holds `ring` buckets' worth of output memory whatever the size of the model
        (`plan_memory.Placement`).  With `packed`, every bucket becomes a `PackedBucket`: the quantizer jobs are
        pointed at their final place in the bucket's flat payload and pass-through tensors get copy jobs, so a
        replay produces the transport payload with no flattening pass."""
        with launch.recording() as batch:
            batch.device = next((t.device for t in weights.values() if t.device.type == "cuda"), None)
            placement = Placement(batch, weights, packed=packed, ring=ring)
            for bucket in iterator.iter_hf_weights(weights):
                placement.take(bucket)       # every job of this bucket (and maybe some of the next) is recorded
            del bucket
        buckets, marks, ring, arena_bytes = placement.finish()
        batch.freeze()
        # a replay reproduces the sync only if no kernel bypassed the job list, every job input is live parameter
        # storage, a declared constant or made by a job, and every handed-out tensor is one of those too (a tensor
        # that some torch op materialised would go stale)
        refusal = tuple(reason for ok, reason in (
            (batch.direct_calls == 0, f"{batch.direct_calls} kernel launches bypassed the job list"),
            (placement.handed_out_ok, "a handed-out tensor is neither written by a job, nor parameter storage, nor a declared constant"),
            (placement.packable, "a bucket cannot be laid out as one payload"),
            (placement.inputs_alias, "a kernel input does not alias live parameter storage")) if not ok)
        plan = cls(batch, buckets, marks, weights_signature(weights), not refusal, ring, arena_bytes)
        plan.refusal = refusal
        plan.packable = placement.packable
        plan.remember(weights)
        return plan

    def matches(self, weights: Mapping[str, torch.Tensor]) -> bool:
        """True when `weights` is the parameter set the plan was recorded on.  Between RL steps the mapping holds
        the very same tensor objects, so the usual answer costs one identity pass, one address and one shape per tensor
        (about 1 ms for 12 288 expert tensors, against 5 ms for the full signature, which also builds a tuple per
        tensor); a tensor object keeps its dtype for life, so objects, addresses and shapes cover the signature.
        Anything else (other objects, other names, another count) is decided by the full signature."""
        if not self.replayable:
            return False
        if len(weights) == len(self._tensors):
            tensors = list(weights.values())
            if all(map(operator.is_, tensors, self._tensors)) and list(weights) == self._names:
                # (the shapes are compared one by one as they are made: twelve thousand `torch.Size` objects alive at
                # once are twelve thousand container allocations to Python's garbage collector, which then runs its full
                # collection -- 75 ms over the objects of a large plan -- every few syncs)
                return (list(map(torch.Tensor.data_ptr, tensors)) == self._addresses
                        and all(map(operator.eq, map(_shape_of, tensors), self._shapes)))
        return weights_signature(weights) == self.signature

    # a trailing launch smaller than this many elements is topped up with the next bucket's jobs
    SMALL_LAUNCH_ELEMENTS = 64 * 1024 * 1024

    def submission_marks(self) -> list[int]:
        """Where each bucket's submission ends: at least after the bucket's own jobs.  `mq_run_jobs` fuses up to
        `MAX_GROUP` jobs per launch, counted from the start of a submission, so a bucket of 330 small expert tensors
        ends in a launch of ten, which mostly ramps up and down.  When that last launch would cover fewer than
        `SMALL_LAUNCH_ELEMENTS` elements the submission runs on into the next bucket's jobs up to the full group (the
        next bucket's outputs live in another arena, so running ahead by less than `ring` buckets is safe; measured on
        the 18 432-tensor MXFP8 sync: 14.6 -> 14.1 ms).  Buckets of large tensors are submitted as they are -- merging their launches made the
        Qwen3-4B FP8 sync 1 % slower.  A cut never falls between NVFP4 jobs that share an amax record."""
        if self._marks is None:
            records, total, done, marks = self.batch.records, len(self.batch), 0, []
            self.batch.freeze()
            for mark in self.jobs_done_at_bucket:
                if mark > done:
                    group = self.batch.launch_group(mark - 1)     # with a device table a bucket's experts are one launch
                    tail = (mark - done) % group
                    tail_elements = sum(r[7] * r[8] for r in records[mark - tail:mark])
                    if tail and tail_elements < self.SMALL_LAUNCH_ELEMENTS:
                        # bucket k + ring writes the arena of bucket k, which the consumer is about to read
                        ahead = self.jobs_done_at_bucket[min(len(marks) + self.ring - 1, len(self.jobs_done_at_bucket) - 1)]
                        mark = max(mark, min(total, mark + group - tail, ahead))
                        while (0 < mark < total and records[mark][0] == _lib.JOB_NVFP4
                               and records[mark - 1][0] == _lib.JOB_NVFP4 and records[mark][5] == records[mark - 1][5]):
                            mark += 1
                    done = mark
                marks.append(done)
            self._marks = marks
        return self._marks

    def replay(self) -> Iterator[Unit]:
        """Re-quantize into the plan's output tensors, bucket by bucket, and yield the buckets."""
        done = 0
        for bucket, mark in zip(self.buckets, self.submission_marks()):
            self.batch.run_range(done, mark)
            done = max(done, mark)
            yield bucket
        self._completed += 1
        if self._completed == 1:
            # every amax record now holds this model's values: later replays quantize NVFP4 tensors in one pass with
            # them and repeat a tensor only when its amax moved
            self.batch.carry_amax()

