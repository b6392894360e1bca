"""Where the tensors of a recorded sync live: a ring of output arenas instead of one buffer per tensor.

The reference streams a sync through a bounded buffer: a bucket of at most `update_weight_buffer_size` bytes is
produced, sent, and dropped before the next one is made (miles/backends/training_utils/weight_update/updater.py:150-160,
`bucket.clear()` in protocols/broadcast.py:83).  A recorded sync must keep that bound, or it would pin a second,
quantized copy of the whole model next to the trainer.  `Placement` is fed every bucket while the sync is being
recorded (nothing has run yet: the quantizer calls only allocated their outputs and recorded their jobs) and

  * gives every job-written tensor of bucket k a slot in arena k mod n (256-byte aligned, n = `ring`), re-pointing the
    jobs that write or read it, and lets the tensor's first home go at once, so recording never holds more than a
    bucket or two of temporary outputs;
  * with `packed`, lays the bucket out as one flat transport payload instead (tensors back to back, no padding, the
    reference's `_flatten_weight_bucket` layout, protocols/broadcast.py:191-208): quantizer jobs are re-pointed at
    their place in the payload, pass-through tensors get copy jobs, and a quantizer output whose place is not 16-byte
    aligned keeps a buffer of its own behind the payload and is copied in;
  * leaves views of live parameter storage, declared constants and amax records (they carry state from one sync to
    the next) where they are.

`finish()` allocates the arenas (the largest bucket sets their size), resolves every pointer, orders the job list by
bucket and returns the buckets as views into the arenas.  Bucket k is overwritten when the jobs of bucket k + n are
submitted, which the plan never does before the consumer has returned from bucket k: the reference's contract (a
bucket is valid until its own send returns; work the consumer queued on the launch stream stays ordered before the
reuse).
"""

from __future__ import annotations

import bisect
from collections.abc import Mapping

import torch

from miles_amd import _lib, launch
from miles_amd.weight_update.bucketing import Unit
from miles_amd.weight_update.packed_bucket import PackedBucket, layout

_F = launch.JobBatch
_POINTER_FIELDS = (_F.IN, _F.OUT, _F.SCALE, _F.AUX, _F.AUX2)
_SLOT_ALIGN = 256


class NotPackable(Exception):
    """A bucket holds a tensor that can be neither produced in place in a flat payload nor byte-copied into it."""


def _align(n: int, a: int = _SLOT_ALIGN) -> int:
    return (n + a - 1) // a * a


def _written_fields(kind: int) -> tuple[int, ...]:
    if kind == _lib.JOB_INT4_PACK_ASYM:
        return (_F.OUT, _F.SCALE, _F.AUX, _F.AUX2)      # aux: zero points (staging), aux2: packed zero points
    if kind in (_lib.JOB_COPY, _lib.JOB_UE8M0_PACK, _lib.JOB_FP8_DEQUANT):
        return (_F.OUT,)
    return (_F.OUT, _F.SCALE, _F.AUX2)


class _Storage:
    """One torch allocation that jobs of the recorded list touch."""

    __slots__ = ("ptr", "nbytes", "tensors", "written_by", "read_by", "is_record")

    def __init__(self, ptr: int, nbytes: int) -> None:
        self.ptr, self.nbytes = ptr, nbytes
        self.tensors: list[torch.Tensor] = []
        self.written_by: list[tuple[int, int]] = []     # (record index, field)
        self.read_by: list[tuple[int, int]] = []
        self.is_record = False                          # an amax record: state that outlives a sync


class _Arena:
    """A pointer that is resolved when the arenas exist: byte `offset` of the arena of bucket `bucket`."""

    __slots__ = ("bucket", "offset")

    def __init__(self, bucket: int, offset: int) -> None:
        self.bucket, self.offset = bucket, offset


class Placement:
    def __init__(self, batch: launch.JobBatch, weights: Mapping[str, torch.Tensor], *, packed: bool, ring: int | None) -> None:
        self.batch, self.packed, self.ring = batch, packed, ring
        spans = sorted((t.untyped_storage().data_ptr(), t.untyped_storage().data_ptr() + t.untyped_storage().nbytes())
                       for t in weights.values())
        self._span_starts, self._spans = [s for s, _ in spans], spans
        self.records: list[list] = []                   # mutable copies of batch.records, pointers maybe _Arena
        self.rec_bucket: list[int] = []                 # bucket a record is submitted with
        self._storages: dict[int, _Storage] = {}
        self._starts: list[int] | None = None           # sorted storage addresses, rebuilt when stale
        self._rec_storages: list[list[_Storage]] = []   # storages each record touches
        self._kept_done = 0
        self._persistent: list[torch.Tensor] = []       # tensors that stay where they are for the life of the plan
        self.bucket_specs: list[list[tuple]] = []       # per bucket: (name, tensor | (_Arena, dtype, size, stride))
        self.bucket_metas: list = []                    # packed: TensorMeta list and payload size per bucket
        self.bucket_bytes: list[int] = []
        self.copies: list[list[list]] = []              # per bucket: copy records appended behind its jobs
        self.inputs_alias = True                        # every job input is live parameter storage, a constant or job-made
        self.handed_out_ok = True                       # every handed-out tensor is reproduced by a replay
        self.packable = True

    # ---- bookkeeping -----------------------------------------------------------------------------------
    def in_weights(self, ptr: int) -> bool:
        i = bisect.bisect_right(self._span_starts, ptr) - 1
        return i >= 0 and ptr < self._spans[i][1]

    def _storage_at(self, ptr: int) -> _Storage | None:
        s = self._storages.get(ptr)
        if s is not None:
            return s
        if self._starts is None:
            self._starts = sorted(self._storages)
        i = bisect.bisect_right(self._starts, ptr) - 1
        if i >= 0:
            s = self._storages.get(self._starts[i])
            if s is not None and ptr < s.ptr + max(s.nbytes, 1):
                return s
        return None

    def _absorb(self) -> None:
        """Take in what was recorded since the last bucket: the tensors the batch holds and the new job records."""
        kept = self.batch.held
        for t in kept[self._kept_done:]:
            st = t.untyped_storage()
            ptr = st.data_ptr()
            if ptr == 0 or self.in_weights(ptr) or t.device.type != "cuda":
                self._persistent.append(t)
                continue
            s = self._storages.get(ptr)
            if s is None:
                s = self._storages[ptr] = _Storage(ptr, st.nbytes())
                self._starts = None
            s.tensors.append(t)
        del kept[self._kept_done:]       # this object owns them now, and lets a bucket's first homes go once it is placed
        self._kept_done = len(kept)
        bucket = len(self.bucket_specs)
        for rec in self.batch.records[len(self.records):]:
            ri = len(self.records)
            self.records.append(list(rec))
            self.rec_bucket.append(bucket)
            kind, touched = rec[_F.KIND], []
            written = _written_fields(kind)
            for f in _POINTER_FIELDS:
                ptr = rec[f]
                if not ptr or self.in_weights(ptr):
                    continue
                s = self._storage_at(ptr)
                if s is None:
                    if f == _F.IN and ptr not in self.batch.constants:
                        self.inputs_alias = False
                    continue
                if f == _F.AUX and kind in (_lib.JOB_NVFP4, _lib.JOB_FP8_TENSOR):
                    s.is_record = True
                    continue
                (s.written_by if f in written else s.read_by).append((ri, f))
                touched.append(s)
                if f == _F.IN and not s.written_by and ptr not in self.batch.constants:
                    self.inputs_alias = False       # reads something no job of the list made: stale on replay
            self._rec_storages.append(touched)

    def _repoint(self, ri: int, field: int, s: _Storage | None, target: _Arena) -> None:
        self.records[ri][field] = target
        if s is not None:
            for refs in (s.written_by, s.read_by):
                if (ri, field) in refs:
                    refs.remove((ri, field))

    # ---- one bucket -------------------------------------------------------------------------------------
    def _job_made(self, t: torch.Tensor) -> _Storage | None:
        """The storage of a handed-out tensor if some job of the list writes into it."""
        if not t.numel() or self.in_weights(t.data_ptr()):
            return None
        s = self._storage_at(t.data_ptr())
        return s if s is not None and s.written_by and not s.is_record else None

    def take(self, bucket: Unit) -> None:
        self._absorb()
        k = len(self.bucket_specs)
        if not self.packable:                      # the plan will not be kept: nothing to place
            self.bucket_specs.append([(name, t) for name, t in bucket])
            self.copies.append([])
            self.bucket_bytes.append(0)
            return
        specs: list[tuple] = []
        copies: list[list] = []
        jobs: set[int] = set()                     # records that write this bucket's tensors
        touched = [s for s in (self._job_made(t) for _, t in bucket) if s is not None]
        cursor = 0
        if self.packed:
            try:
                cursor = self._lay_out_payload(k, bucket, specs, copies, jobs)
            except NotPackable:
                # the updater flattens such buckets after the fact (one extra copy); the plan is not kept
                self.packable = False
                return self.take(bucket)
        owned: list[_Storage] = []
        seen: set[int] = set()

        def own(s: _Storage) -> None:
            if s.ptr not in seen and not s.is_record and s.written_by and s.ptr in self._storages:
                seen.add(s.ptr)
                owned.append(s)
                jobs.update(ri for ri, _ in s.written_by)

        if not self.packed:
            for s in touched:
                own(s)
        else:
            for rec in copies:                     # sources of payload copies that a job of the list writes
                s = self._storage_at(rec[_F.IN])
                if s is not None:
                    own(s)
        # whatever else this bucket's jobs write (a staging buffer) or read from another job (an intermediate result)
        frontier = list(jobs)
        while frontier:
            ri = frontier.pop()
            for s in self._rec_storages[ri]:
                before = len(jobs)
                own(s)
                if len(jobs) != before:
                    frontier.extend(r for r, _ in s.written_by)
        # place them (behind the payload, if there is one) and re-point every job that touches them
        slots: dict[int, int] = {}
        for s in owned:
            cursor = _align(cursor)
            slots[s.ptr] = cursor
            cursor += s.nbytes
            for ri, f in s.written_by + s.read_by:
                self.records[ri][f] = _Arena(k, slots[s.ptr] + (self.batch.records[ri][f] - s.ptr))
        for ri in jobs:
            self.rec_bucket[ri] = k
        for rec in copies:
            s = self._storage_at(rec[_F.IN])
            if s is not None and s.ptr in slots:
                rec[_F.IN] = _Arena(k, slots[s.ptr] + (rec[_F.IN] - s.ptr))
        if not self.packed:
            for name, t in bucket:
                s = self._job_made(t)
                if s is not None and s.ptr in slots:
                    offset = slots[s.ptr] + (t.data_ptr() - s.ptr)
                    specs.append((name, (_Arena(k, offset), t.dtype, tuple(t.shape), tuple(t.stride()))))
                    continue
                if t.numel() and not self.in_weights(t.data_ptr()) and t.data_ptr() not in self.batch.constants:
                    self.handed_out_ok = False      # some torch op materialised it: stale on replay
                specs.append((name, t))
        # the first homes of this bucket's outputs are free again (nothing was ever written there)
        for s in owned + [s for s in touched if not s.written_by and not s.read_by]:
            self._storages.pop(s.ptr, None)
            s.tensors = []                           # (records still point at the bookkeeping object: drop the memory itself)
        self._starts = None
        self.bucket_specs.append(specs)
        self.copies.append(copies)
        self.bucket_bytes.append(cursor)

    def _lay_out_payload(self, k: int, bucket: Unit, specs: list, copies: list, jobs: set[int]) -> int:
        """Packed form of one bucket: every tensor at its byte offset in the payload.  Returns the payload size."""
        metas, total = layout(bucket)
        recorded = self.batch.records
        # jobs recorded so far that write exactly at a handed-out tensor's address, and byte copies by destination
        writers: dict[int, list[tuple[int, int, _Storage]]] = {}
        gathers: list[tuple[int, int, int, _Storage]] = []
        for _, t in bucket:
            s = self._job_made(t)
            if s is None:
                continue
            for ri, f in s.written_by:
                if recorded[ri][_F.KIND] == _lib.JOB_COPY:
                    rec = recorded[ri]
                    # (a 2-D copy whose destination rows lie apart fills no single run: its tensor is copied afterwards)
                    if rec[_F.ROWS] == 1 or rec[_F.BLOCK_STRIDE] in (0, rec[_F.COLS]):
                        gathers.append((rec[f], ri, rec[_F.ROWS] * rec[_F.COLS], s))
                else:
                    writers.setdefault(recorded[ri][f], []).append((ri, f, s))
        gathers = sorted({g[:3]: g for g in gathers}.values(), key=lambda g: g[0])
        gather_starts = [g[0] for g in gathers]

        def scale_packers(old):
            return [(ri, f, s) for ri, f, s in writers.get(old.data_ptr(), ()) if recorded[ri][_F.KIND] == _lib.JOB_UE8M0_PACK]

        for (name, old), meta in zip(bucket, metas):       # nothing is changed before every tensor is known to fit
            if old.numel() and not old.is_contiguous() and not (scale_packers(old) and meta.start_idx % 4 == 0):
                raise NotPackable(f"{name} is a strided pass-through tensor: it needs a gathering copy")
        for (name, old), meta in zip(bucket, metas):
            place = meta.start_idx
            if not old.numel():
                continue
            if not old.is_contiguous():
                # the transposed view of packed UE8M0 scales: its job writes the contiguous form straight into its place
                for ri, f, s in scale_packers(old):
                    self._repoint(ri, _F.OUT, s, _Arena(k, place))
                    self.records[ri][_F.LD] = 1
                    jobs.add(ri)
                continue
            hits = writers.get(old.data_ptr())
            # codes written by a quantizer need their place on a 16-byte boundary for the tuned kernels (a row-blocked
            # FP8 job has no other kernel at all); a place that follows, say, a 12-byte scale grid is filled by a copy
            if hits and place % 16 and any(f == _F.OUT for _, f, _ in hits):
                hits = None
            if hits:
                for ri, f, s in hits:
                    self._repoint(ri, f, s, _Arena(k, place))
                    jobs.add(ri)
                continue
            # a tensor that copy jobs assemble piece by piece is assembled in its place instead
            lo, nbytes = old.data_ptr(), old.numel() * old.element_size()
            first = bisect.bisect_left(gather_starts, lo)
            pieces, end = [], lo
            for dst, ri, size, s in gathers[first:]:
                if dst != end or dst >= lo + nbytes:
                    break
                pieces.append((ri, s, dst))
                end = dst + size
            if pieces and end == lo + nbytes:
                for ri, s, dst in pieces:
                    self._repoint(ri, _F.OUT, s, _Arena(k, place + dst - lo))
                    jobs.add(ri)
                continue
            copies.append([_lib.JOB_COPY, 0, old.data_ptr(), _Arena(k, place), None, None, None, 1, nbytes, nbytes, 0, 0, 0, 0])
            if self._job_made(old) is None:
                self._persistent.append(old)        # a view of parameter storage or a constant: copied from where it is
                if not self.in_weights(old.data_ptr()) and old.data_ptr() not in self.batch.constants:
                    self.handed_out_ok = False      # some torch op materialised it: stale on replay
        specs.extend((m.name, m) for m in metas)
        self.bucket_metas.append((metas, total))
        return total

    # ---- the end of the recording --------------------------------------------------------------------------
    def finish(self):
        """-> (buckets as views into the arenas, job marks per bucket, bytes of all arenas)."""
        self._absorb()
        n_buckets = len(self.bucket_specs)
        ring = n_buckets if not self.ring else min(self.ring, n_buckets)
        size = _align(max(self.bucket_bytes, default=0), 512)
        device = self.batch.device
        arenas = [torch.empty(size, dtype=torch.uint8, device=device) for _ in range(ring)] if size else []

        def address(p):
            return arenas[p.bucket % ring].data_ptr() + p.offset if isinstance(p, _Arena) else p

        # the job list, bucket by bucket (a stable order: jobs that share an amax record stay neighbours), every bucket's
        # payload copies behind its jobs
        by_bucket: list[list[tuple]] = [[] for _ in range(max(n_buckets, 1))]
        for rec, b in zip(self.records, self.rec_bucket):
            by_bucket[min(b, max(n_buckets - 1, 0))].append(tuple(address(v) for v in rec))
        records: list[tuple] = []
        marks: list[int] = []
        for k in range(n_buckets):
            records.extend(by_bucket[k])
            records.extend(tuple(address(v) for v in rec) for rec in self.copies[k])
            marks.append(len(records))
        if not n_buckets:
            records.extend(by_bucket[0])
        buckets: list[Unit] = []
        payloads = iter(self.bucket_metas)
        for k, specs in enumerate(self.bucket_specs):
            arena = arenas[k % ring] if arenas else None
            if specs and not isinstance(specs[0][1], (torch.Tensor, tuple)):
                metas, total = next(payloads)
                buckets.append(PackedBucket(arena[:total], metas))
                continue
            bucket = []
            for name, spec in specs:
                if isinstance(spec, torch.Tensor):
                    bucket.append((name, spec))
                else:
                    where, dtype, shape, stride = spec
                    itemsize = torch.empty((), dtype=dtype).element_size()
                    assert where.offset % itemsize == 0
                    bucket.append((name, arena.view(dtype).as_strided(shape, stride, where.offset // itemsize)))
            buckets.append(bucket)
        leftovers = [t for s in self._storages.values() for t in s.tensors]
        self.batch.replace_records(records, keep=self._persistent + leftovers + arenas + list(self.batch.held))
        return buckets, marks, ring, ring * size
