"""Segment copy / zero / cast-pack: descriptor tables plus HIP launches.

Host-side counterpart of the reference's ``custom_placements/_copy_kernels.py``
(descriptors :164-246, :366-433; launchers :249-359, :436-484).  A descriptor
is three (or five) int64 device arrays built once per layout and reused; the
kernels behind them are ``fsh_copy_segments`` / ``fsh_zero_segments`` /
``fsh_pack_segments``.
"""

from __future__ import annotations

from collections.abc import Sequence
from dataclasses import dataclass

import torch

from .. import hip_ops

# Split segments are capped at this many so descriptor tables stay small.
_MAX_SEGMENTS = 65535


def _upload_i64(values: Sequence[int], device: torch.device) -> tuple[torch.Tensor, torch.Tensor]:
    """Device int64 tensor of ``values`` plus the pinned host tensor the
    asynchronous copy reads from (the caller keeps it alive)."""
    host = torch.tensor(list(values), dtype=torch.int64, pin_memory=True)
    dev = torch.empty(host.shape, dtype=torch.int64, device=device)
    if host.numel():
        dev.copy_(host, non_blocking=True)
    return dev, host


@dataclass
class SegmentCopyDescriptor:
    """Segments ``(src_offset, numel, dst_offset)`` of one source tensor, in
    elements, on the device.  Long segments are cut into pieces of at most
    ``max_chunks_per_segment * block_size`` elements so a launch sized by the
    longest piece wastes few workgroups."""

    src_offsets: torch.Tensor
    numels: torch.Tensor
    dst_offsets: torch.Tensor
    max_segment_numel: int
    nsegments: int
    block_size: int
    _staged_hosts: tuple[torch.Tensor, ...]

    @classmethod
    def create(
        cls,
        *,
        src_offsets: Sequence[int],
        numels: Sequence[int],
        dst_offsets: Sequence[int],
        device: torch.device,
        block_size: int = 4096,
        max_chunks_per_segment: int = 8,
    ) -> "SegmentCopyDescriptor":
        if not (len(src_offsets) == len(numels) == len(dst_offsets)):
            raise ValueError("Segment descriptor lists must have the same length.")
        if len(numels) > _MAX_SEGMENTS:
            raise ValueError(f"At most {_MAX_SEGMENTS} segments are supported, got {len(numels)}.")
        piece = max_chunks_per_segment * block_size
        while sum(-(-n // piece) for n in numels) > _MAX_SEGMENTS:
            piece *= 2
        src, cnt, dst = [], [], []
        for s, n, d in zip(src_offsets, numels, dst_offsets, strict=True):
            done = 0
            while done < n:
                step = min(piece, n - done)
                src.append(s + done)
                cnt.append(step)
                dst.append(d + done)
                done += step
        src_t, src_h = _upload_i64(src, device)
        cnt_t, cnt_h = _upload_i64(cnt, device)
        dst_t, dst_h = _upload_i64(dst, device)
        return cls(
            src_offsets=src_t,
            numels=cnt_t,
            dst_offsets=dst_t,
            max_segment_numel=max(cnt, default=0),
            nsegments=len(cnt),
            block_size=block_size,
            _staged_hosts=(src_h, cnt_h, dst_h),
        )


def copy_segments(source: torch.Tensor, output: torch.Tensor, descriptor: SegmentCopyDescriptor) -> None:
    """Copy every segment of ``descriptor`` from ``source`` to ``output`` in
    one launch.  Offsets count elements from each tensor's first element."""
    if descriptor.nsegments == 0 or descriptor.max_segment_numel == 0:
        return
    hip_ops.copy_segments(
        source, output, descriptor.src_offsets, descriptor.numels, descriptor.dst_offsets,
        descriptor.max_segment_numel,
    )


def zero_segments(output: torch.Tensor, descriptor: SegmentCopyDescriptor) -> None:
    """Zero the destination segments of ``descriptor`` in one launch."""
    if descriptor.nsegments == 0 or descriptor.max_segment_numel == 0:
        return
    hip_ops.zero_segments(output, descriptor.numels, descriptor.dst_offsets, descriptor.max_segment_numel)


@dataclass
class SegmentPackDescriptor:
    """Segments gathered from several flat inputs: input index, source offset,
    length, destination offset (elements), plus the inputs' device addresses."""

    input_ptrs: torch.Tensor
    tensor_indices: torch.Tensor
    src_offsets: torch.Tensor
    numels: torch.Tensor
    dst_offsets: torch.Tensor
    max_segment_numel: int
    nsegments: int
    _staged_hosts: tuple[torch.Tensor, ...]
    _input_ptr_values: tuple[int, ...] = ()

    @classmethod
    def create(
        cls,
        *,
        ninputs: int,
        tensor_indices: Sequence[int],
        src_offsets: Sequence[int],
        numels: Sequence[int],
        dst_offsets: Sequence[int],
        device: torch.device,
        max_piece_numel: int = 32768,
    ) -> "SegmentPackDescriptor":
        if not (len(tensor_indices) == len(src_offsets) == len(numels) == len(dst_offsets)):
            raise ValueError("Segment descriptor lists must have the same length.")
        # Long segments are cut so that a launch sized by the longest piece
        # does not idle on the short ones.  A negative tensor index is a
        # zero-fill segment.
        piece = max_piece_numel
        while sum(-(-n // piece) for n in numels) > _MAX_SEGMENTS:
            piece *= 2
        idx, src, cnt, dst = [], [], [], []
        for t, s, n, d in zip(tensor_indices, src_offsets, numels, dst_offsets, strict=True):
            done = 0
            while done < n:
                step = min(piece, n - done)
                idx.append(t)
                src.append(s + done)
                cnt.append(step)
                dst.append(d + done)
                done += step
        idx_t, idx_h = _upload_i64(idx, device)
        src_t, src_h = _upload_i64(src, device)
        cnt_t, cnt_h = _upload_i64(cnt, device)
        dst_t, dst_h = _upload_i64(dst, device)
        return cls(
            input_ptrs=torch.empty((ninputs,), dtype=torch.int64, device=device),
            tensor_indices=idx_t,
            src_offsets=src_t,
            numels=cnt_t,
            dst_offsets=dst_t,
            max_segment_numel=max(cnt, default=0),
            nsegments=len(idx),
            _staged_hosts=(idx_h, src_h, cnt_h, dst_h),
        )

    def update_input_ptrs(self, inputs: list[torch.Tensor]) -> list[torch.Tensor]:
        """Refresh the device address table when the inputs moved; returns the
        pinned staging tensor to keep alive (empty when nothing changed)."""
        values = tuple(t.data_ptr() for t in inputs)
        if values == self._input_ptr_values:
            return []
        host = torch.tensor(values, dtype=torch.int64, pin_memory=True)
        if host.numel():
            self.input_ptrs.copy_(host, non_blocking=True)
        self._input_ptr_values = values
        return [host]

    @property
    def tensors(self) -> list[torch.Tensor]:
        return [self.input_ptrs, self.tensor_indices, self.src_offsets, self.numels, self.dst_offsets]


def pack_segments_into_flat_buffer(
    inputs: list[torch.Tensor],
    tensor_indices: Sequence[int],
    src_offsets: Sequence[int],
    numels: Sequence[int],
    dst_offsets: Sequence[int],
    output: torch.Tensor,
    *,
    descriptor: SegmentPackDescriptor | None = None,
) -> list[torch.Tensor] | None:
    """Gather flat source segments into ``output`` with a cast (fp32/bf16 in
    either direction) in one launch.  With a prebuilt ``descriptor`` the four
    segment lists are ignored.  Returns the tensors the caller must keep
    alive until the launch has run, or None when the inputs are not supported
    (the same conditions the reference's packer declines)."""
    if torch.compiler.is_compiling():
        return None
    if output.dim() != 1 or output.device.type != "cuda" or not output.is_contiguous():
        return None
    if not (len(tensor_indices) == len(src_offsets) == len(numels) == len(dst_offsets)):
        raise ValueError("Segment descriptor lists must have the same length.")
    if not inputs:
        return [] if len(tensor_indices) == 0 else None
    in_dtype = inputs[0].dtype
    supported = (torch.float32, torch.bfloat16)
    if in_dtype not in supported or output.dtype not in supported:
        return None
    for t in inputs:
        if t.device != output.device or t.dtype != in_dtype or t.dim() != 1 or not t.is_contiguous():
            return None
    if descriptor is None:
        descriptor = SegmentPackDescriptor.create(
            ninputs=len(inputs), tensor_indices=tensor_indices, src_offsets=src_offsets, numels=numels,
            dst_offsets=dst_offsets, device=output.device,
        )
    elif descriptor.input_ptrs.device != output.device or descriptor.input_ptrs.numel() != len(inputs):
        return None
    staged = descriptor.update_input_ptrs(inputs)
    keep = [*descriptor.tensors, *staged, *inputs]
    if output.numel() == 0 or descriptor.nsegments == 0 or descriptor.max_segment_numel == 0:
        return keep
    hip_ops.pack_segments(
        descriptor.input_ptrs, descriptor.tensor_indices, descriptor.src_offsets, descriptor.numels,
        descriptor.dst_offsets, descriptor.max_segment_numel, in_dtype, output,
    )
    return keep


__all__ = [
    "SegmentCopyDescriptor",
    "SegmentPackDescriptor",
    "copy_segments",
    "pack_segments_into_flat_buffer",
    "zero_segments",
]
