"""Packed transport buckets: the (name, tensor) list of a bucket laid out back to back in one uint8 buffer.

The reference's `broadcast_packed` transfer mode builds this payload after quantization by concatenating the raw
bytes of every tensor (`_flatten_weight_bucket`, miles/backends/training_utils/weight_update/protocols/
broadcast.py:191-208, through SGLang's `FlattenedTensorBucket`): one more read and write of everything that was
just quantized.  Here the payload is the place the quantizers write to: every tensor of a `PackedBucket` is a view
into `flat` at its final offset, quantizer outputs are produced there directly and only pass-through tensors
(norms, embeddings) are copied in, by grouped copy jobs.

Layout rules are the reference's: tensors in bucket order, no padding, and a tensor whose byte offset is not a
multiple of its element size is rejected with the same ValueError.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from miles_amd import _lib, launch


@dataclass
class TensorMeta:
    """Where one tensor sits in the flat payload (field names follow SGLang's FlattenedTensorMetadata)."""

    name: str
    shape: torch.Size
    dtype: torch.dtype
    start_idx: int
    end_idx: int
    numel: int


def layout(named_tensors) -> tuple[list[TensorMeta], int]:
    """Byte offsets of a bucket's tensors, back to back in order."""
    metas, offset = [], 0
    for name, tensor in named_tensors:
        if offset % tensor.element_size():
            raise ValueError(f"Unaligned flattened weight {name}: byte offset {offset}, dtype {tensor.dtype}")
        nbytes = tensor.numel() * tensor.element_size()
        metas.append(TensorMeta(name, tensor.shape, tensor.dtype, offset, offset + nbytes, tensor.numel()))
        offset += nbytes
    return metas, offset


class PackedBucket(list):
    """A bucket (list of (hf_name, tensor)) whose tensors are views into one flat uint8 payload."""

    def __init__(self, flat: torch.Tensor, metadata: list[TensorMeta]) -> None:
        super().__init__((m.name, self._view(flat, m)) for m in metadata)
        self.flat = flat
        self.metadata = metadata

    @staticmethod
    def _view(flat: torch.Tensor, m: TensorMeta) -> torch.Tensor:
        return flat[m.start_idx:m.end_idx].view(m.dtype).view(m.shape)

    def get_flattened_tensor(self) -> torch.Tensor:
        return self.flat

    def get_metadata(self) -> list[TensorMeta]:
        return self.metadata

    def reconstruct_tensors(self) -> list[tuple[str, torch.Tensor]]:
        return list(self)


def pack_bucket(named_tensors) -> PackedBucket:
    """Copy an already materialised bucket into a fresh flat payload (the path for syncs that cannot be planned)."""
    named_tensors = [(n, t.contiguous()) for n, t in named_tensors]
    metas, total = layout(named_tensors)
    device = named_tensors[0][1].device if named_tensors else torch.device("cpu")
    flat = torch.empty(total, dtype=torch.uint8, device=device)
    packed = PackedBucket(flat, metas)
    with launch.deferred():
        for (_, src), (_, dst) in zip(named_tensors, packed):
            submit_copy(src, dst)
    return packed


def submit_copy(src: torch.Tensor, dst: torch.Tensor) -> None:
    """Record (or run) one verbatim byte copy between two contiguous tensors of equal size."""
    nbytes = src.numel() * src.element_size()
    if nbytes != dst.numel() * dst.element_size():
        raise _lib.MilesQuantError("copy between tensors of different sizes")
    _lib.require_gpu(src, "packed bucket copy")
    if nbytes:
        launch.submit(_lib.JOB_COPY, src, dst, None, None, None, 1, nbytes, nbytes)


def submit_copy_rows(src: torch.Tensor, dst: torch.Tensor) -> None:
    """Record (or run) one 2-D byte copy between two [rows, n] views whose rows are contiguous runs (any row stride of
    at least a row): the strided form of a copy job, one job where `submit_copy` would need one per row."""
    if src.shape != dst.shape or src.dim() != 2 or src.dtype != dst.dtype:
        raise _lib.MilesQuantError("2-D copy between tensors of different shapes")
    rows, n = src.shape
    size = src.element_size()
    if not rows or not n:
        return
    if n > 1 and (src.stride(1) != 1 or dst.stride(1) != 1):
        raise _lib.MilesQuantError("2-D copy needs contiguous rows")
    _lib.require_gpu(src, "packed bucket copy")
    src_pitch = src.stride(0) * size if rows > 1 else n * size
    dst_pitch = dst.stride(0) * size if rows > 1 else n * size
    if src_pitch < n * size or dst_pitch < n * size:
        raise _lib.MilesQuantError("2-D copy with overlapping rows")
    launch.submit(_lib.JOB_COPY, src, dst, None, None, None, rows, n * size, src_pitch, block_stride=dst_pitch)
