"""Submission of quantization jobs to libmiles_quant.so: immediately, or deferred into one batched call.

Outside a `deferred()` block every quantizer wrapper runs its job at once (one `mq_run_jobs` call with a
single job).  Inside the block the wrappers still allocate and return their output tensors, but the jobs
are only recorded; leaving the block submits the whole list with ONE call, which the library turns into
grouped kernel launches (up to 64 tensors per launch).  The returned tensors must not be read before the
block ends.  This is how the weight-sync driver keeps thousands of per-parameter quantizer calls from being
launch-bound without changing the per-tensor call signatures.
"""

from __future__ import annotations

import contextlib
import ctypes
import threading

import torch

from miles_amd import _lib

_state = threading.local()


class _AmaxFeedback:
    """What share of the amax records moved in the syncs the GPU has finished, read without ever waiting for it.

    The folds of a `mq_run_jobs_feedback` call add to two device counters that only grow -- tensors whose record held
    another amax before, and tensors folded -- and every fold launch first mirrors the pair into two pinned words (their
    address travels with every call, as a host argument), so the host reads them with no copy, no event and no wait.  At the start of a submission: when more than half of the tensors
    folded since the last reading had moved, the list is submitted in the plain two-pass form (the carried-over amax
    would cost every such tensor a second pass), until they hold again."""

    # The GPU writes the mirror words whenever a fold runs, possibly after the batch that named them is gone: they come
    # from one pinned block that lives as long as the process and is never handed back to torch's host allocator.  A
    # slot re-used while an old sync still runs can at worst mislead one choice between two forms with equal results.
    _POOL_SLOTS = 1024
    _pool = None
    _pool_free: list[int] = []
    _pool_lock = threading.Lock()

    @classmethod
    def _take_slot(cls):
        with cls._pool_lock:
            if cls._pool is None:
                cls._pool = torch.zeros(cls._POOL_SLOTS, 2, dtype=torch.int32).pin_memory()
                cls._pool_free = list(range(cls._POOL_SLOTS - 1, -1, -1))
            return cls._pool_free.pop() if cls._pool_free else None

    @classmethod
    def create(cls, device):
        """A watcher, or None when every mirror slot is taken (the batch then simply keeps the carried form)."""
        slot = cls._take_slot()
        return None if slot is None else cls(device, slot)

    def __del__(self):
        slot = getattr(self, "_slot", None)
        if slot is not None:
            try:
                with self._pool_lock:
                    self._pool_free.append(slot)
            except Exception:       # interpreter shutdown
                pass

    def __init__(self, device, slot: int) -> None:
        self._slot = slot
        self.mirror = self._pool[slot]
        self.mirror.zero_()
        self.mirror_words = self.mirror.numpy()       # the same pinned words, read without going through torch
        self.mirror_address = self.mirror.data_ptr()
        self.counter = torch.zeros(2, dtype=torch.int32, device=device)
        self.seen = (0, 0)          # the counters as of the last reading that had new folds
        self.plain = False

    def decide(self) -> bool:
        moved_total, folded_total = (int(v) & 0xFFFFFFFF for v in self.mirror_words)
        folded = (folded_total - self.seen[1]) & 0xFFFFFFFF
        if folded:
            moved = (moved_total - self.seen[0]) & 0xFFFFFFFF
            self.seen = (moved_total, folded_total)
            self.plain = moved * 2 > folded
        return self.plain


class JobBatch:
    """An ordered list of mq_job records plus the tensors they reference."""

    def __init__(self) -> None:
        self._records: list[tuple] = []
        self._keep: list[torch.Tensor] = []
        self._array = None
        self._array_plain = None   # the same list without MQ_NVFP4_CARRY_AMAX (see carry_amax)
        self._feedback: _AmaxFeedback | None = None
        self.last_form = None      # "carried" / "plain": the form of the newest submission of a list with carried amax
        self._table = None      # device copy of the launch descriptors (see freeze)
        self.device = None
        self.direct_calls = 0   # kernels launched inside the block without going through the job list
        self.constants: set[int] = set()   # addresses of result tensors whose contents never depend on the weights

    def __len__(self) -> int:
        return len(self._records)

    def add(self, kind, dtype, inp, out, scale, aux, aux2, rows, cols, ld, p0, p1, rows_per_block=0,
            block_stride=0, keep=()) -> None:
        self._records.append((kind, dtype, inp, out, scale, aux, aux2, rows, cols, ld, p0, p1, rows_per_block,
                              block_stride))
        self._keep.extend(keep)
        self._array = None

    # Field positions of a job record (the order of `mq_job` in include/miles_quant.h).
    KIND, DTYPE, IN, OUT, SCALE, AUX, AUX2, ROWS, COLS, LD, P0, P1, ROWS_PER_BLOCK, BLOCK_STRIDE = range(14)

    @property
    def records(self) -> list[tuple]:
        """The recorded jobs, in submission order (read-only view for planners; use `replace_records` to change them)."""
        return self._records

    def replace_records(self, records: list[tuple], keep: list[torch.Tensor] | None = None) -> None:
        """Swap in an edited job list (a planner re-pointing outputs, adding copy jobs); `keep` replaces the tensors
        the batch holds alive."""
        self._records = list(records)
        if keep is not None:
            self._keep = list(keep)
        self._array = None

    def carry_amax(self, adaptive: bool = True) -> int:
        """After this list has run once: let later runs of the same list quantize NVFP4 and per-tensor FP8 tensors in
        one pass with the amax their record kept from the run before (MQ_NVFP4_CARRY_AMAX; the driver checks the amax on
        the way and quantizes a tensor again if it moved, so results do not change).  NVFP4 jobs are only flagged when
        every one of the list is one the packed kernels take (bf16 or fp16, one dtype per record, 16-byte aligned input,
        4-byte aligned codes), so
        that every record goes through the same driver path on every run; per-tensor FP8 jobs always are.
        With `adaptive` the batch also watches how many records moved per sync (`_AmaxFeedback`) and submits the plain
        two-pass form while most of them keep moving.  Returns the number of jobs flagged."""
        nv = [r for r in self._records if r[self.KIND] == _lib.JOB_NVFP4]
        packed_dtypes = (_lib.DTYPE_CODE[torch.bfloat16], _lib.DTYPE_CODE[torch.float16])
        record_dtypes: dict = {}
        for r in nv:
            record_dtypes.setdefault(r[self.AUX], set()).add(r[self.DTYPE])
        nv_fit = (bool(nv) and all(len(d) == 1 for d in record_dtypes.values())
                  and all(r[self.DTYPE] in packed_dtypes and (r[self.IN] or 0) % 16 == 0
                          and (r[self.OUT] or 0) % 4 == 0 and r[self.COLS] % 16 == 0 for r in nv))
        kinds = {_lib.JOB_FP8_TENSOR} | ({_lib.JOB_NVFP4} if nv_fit else set())
        flagged = sum(r[self.KIND] in kinds for r in self._records)
        if flagged:
            self._records = [r[: self.P1] + (r[self.P1] | _lib.NVFP4_CARRY_AMAX,) + r[self.P1 + 1:]
                             if r[self.KIND] in kinds else r for r in self._records]
            self._array = None
            self._array_plain = None
            if adaptive and self.device is not None and self.device.type == "cuda":
                self._feedback = _AmaxFeedback.create(self.device)
        return flagged

    def amax_records(self) -> list[torch.Tensor]:
        """The amax records of the NVFP4 and per-tensor FP8 jobs, one per tensor or gate/up pair, in job order (int32
        tensors; words `_lib.RECORD_AMAX_WORD`, `RECORD_REDO_WORD`, `RECORD_VOLATILE_WORD` hold the folded amax and
        the state of the carried-over amax after a run)."""
        by_address = {t.data_ptr(): t for t in self._keep}
        seen, out = set(), []
        for r in self._records:
            if r[self.KIND] in (_lib.JOB_NVFP4, _lib.JOB_FP8_TENSOR) and r[self.AUX] not in seen:
                seen.add(r[self.AUX])
                out.append(by_address[r[self.AUX]])
        return out

    def hold(self, tensor: torch.Tensor) -> None:
        """Keep a tensor alive for as long as the batch exists."""
        self._keep.append(tensor)

    @property
    def held(self) -> list[torch.Tensor]:
        return self._keep

    # job kinds whose grouped launches can take their descriptors from a device table (mq_run_jobs_tabled)
    _TABLE_KINDS = (_lib.JOB_MXFP8, _lib.JOB_MXFP4, _lib.JOB_INT4_PACK, _lib.JOB_INT4_PACK_ASYM, _lib.JOB_FP8_BLOCK,
                    _lib.JOB_FP8_BLOCKWISE_CAST, _lib.JOB_FP8_BLOCK_POW2, _lib.JOB_NVFP4, _lib.JOB_FP8_TENSOR)

    def freeze(self):
        """Materialise the ctypes job array (done once; `run` can then be repeated).  A list with more jobs of a
        table kind than one launch's kernel arguments hold (MoE experts by the thousand) also gets its descriptors
        copied to device memory, so that `run` is not cut into launches of 64 tensors."""
        if self._array is None:
            arr = (_lib.Job * len(self._records))()
            for i, rec in enumerate(self._records):
                arr[i] = _lib.Job(*rec)
            self._array = arr
            self._array_plain = None
            self._table = None
            if self.device is not None and sum(r[self.KIND] in self._TABLE_KINDS for r in self._records) > _lib.MAX_GROUP:
                host = torch.empty(len(self._records) * _lib.TABLE_ENTRY_BYTES, dtype=torch.uint8)
                _lib.check(_lib.load().mq_job_table_fill(arr, len(self._records), host.data_ptr()))
                self._table = host.to(self.device)
        return self._array

    def launch_group(self, index: int) -> int:
        """How many consecutive jobs one launch can cover at job `index`: `TABLE_GROUP` for a table kind of a frozen
        batch that keeps a device table, `MAX_GROUP` otherwise."""
        tabled = self._table is not None and self._records[index][self.KIND] in self._TABLE_KINDS
        return _lib.TABLE_GROUP if tabled else _lib.MAX_GROUP

    def run(self, stream: int | None = None) -> None:
        self.run_range(0, len(self._records), stream)

    def run_range(self, start: int, stop: int, stream: int | None = None) -> None:
        """Submit jobs [start, stop) of the list (a cut never separates two NVFP4 jobs sharing a record,
        because callers cut at parameter boundaries)."""
        if stop <= start:
            return
        arr = self.freeze()
        if stream is None:
            stream = _lib.stream_ptr(self.device)
        feedback = self._feedback
        if feedback is not None:
            if start == 0:
                self.last_form = "plain" if feedback.decide() else "carried"
            if self.last_form == "plain":
                arr = self._plain_array()
        ptr = ctypes.byref(arr, start * ctypes.sizeof(_lib.Job))
        table = None if self._table is None else self._table.data_ptr() + start * _lib.TABLE_ENTRY_BYTES
        counter, mirror = (None, None) if feedback is None else (feedback.counter.data_ptr(), feedback.mirror_address)
        _lib.check(_lib.load().mq_run_jobs_feedback(ptr, stop - start, table, counter, mirror, stream))

    def _plain_array(self):
        """The job list without the carried-amax flag (same records, same device table)."""
        if self._array_plain is None:
            arr = (_lib.Job * len(self._records))()
            for i, rec in enumerate(self._records):
                if rec[self.KIND] in (_lib.JOB_NVFP4, _lib.JOB_FP8_TENSOR):
                    rec = rec[: self.P1] + (rec[self.P1] & ~_lib.NVFP4_CARRY_AMAX,) + rec[self.P1 + 1:]
                arr[i] = _lib.Job(*rec)
            self._array_plain = arr
        return self._array_plain

    def input_pointers(self) -> list[int]:
        return [rec[2] for rec in self._records]

    def output_pointers(self) -> set[int]:
        """Addresses written by the recorded jobs (codes, scales, NVFP4 global scales, copy destinations)."""
        return {rec[f] for rec in self._records for f in (3, 4, 6) if rec[f] is not None}


def active_batch() -> JobBatch | None:
    return getattr(_state, "batch", None)


@contextlib.contextmanager
def deferred():
    """Record the quantizer calls made inside the block and submit them together on exit.

    Inside an enclosing `deferred()` / `recording()` block this is a pass-through: the jobs join the outer
    batch and run when that one does.
    """
    outer = active_batch()
    if outer is not None:
        yield outer
        return
    batch = JobBatch()
    _state.batch = batch
    try:
        yield batch
    finally:
        _state.batch = None
    batch.run()


@contextlib.contextmanager
def recording():
    """Like `deferred()`, but nothing is submitted on exit: the caller keeps the batch and runs (and re-runs)
    it with `JobBatch.run` / `JobBatch.run_range`."""
    if active_batch() is not None:
        raise _lib.MilesQuantError("recording() cannot start inside another batch")
    batch = JobBatch()
    _state.batch = batch
    try:
        yield batch
    finally:
        _state.batch = None


def note_direct_call() -> None:
    """Called by wrappers whose kernel cannot be expressed as a job and is launched at once; a recorded batch
    that saw one cannot reproduce the whole computation on replay."""
    batch = active_batch()
    if batch is not None:
        batch.direct_calls += 1


def note_constant(t: torch.Tensor) -> None:
    """Called by a processor for a result tensor that is the same on every sync (a shape record, say), so that a
    recorded batch can hand it out again without recomputing it."""
    batch = active_batch()
    if batch is not None:
        batch.constants.add(t.data_ptr())
        batch.hold(t)


def submit(kind, inp: torch.Tensor, out: torch.Tensor, scale, aux, aux2, rows, cols, ld, p0=0, p1=0,
           rows_per_block=0, block_stride=0, dtype=None) -> None:
    """Run (or record) one job.  Tensor arguments may be None where the job kind has no such operand; `dtype` is the
    job's dtype code where that is not the input tensor's (the scales' dtype of an INT4 unpacking job)."""
    rec = (kind, _lib.DTYPE_CODE.get(inp.dtype, 0) if dtype is None else dtype, inp.data_ptr(), out.data_ptr(),
           scale.data_ptr() if scale is not None else None, aux.data_ptr() if aux is not None else None,
           aux2.data_ptr() if aux2 is not None else None, rows, cols, ld, p0, p1, rows_per_block, block_stride)
    keep = [t for t in (inp, out, scale, aux, aux2) if t is not None]
    batch = active_batch()
    if batch is not None:
        if batch.device is None:
            batch.device = inp.device
        batch.add(*rec, keep=keep)
        return
    one = (_lib.Job * 1)(_lib.Job(*rec))
    _lib.check(_lib.load().mq_run_jobs(one, 1, _lib.stream_ptr(inp.device)))
