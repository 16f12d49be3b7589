"""Copy helpers and gradient-reduction semantics shared by the placements.

Mirrors the helper surface of the reference's ``custom_placements/utils.py``:
``foreach_copy_`` and the flat-buffer packers (:20-105), the reduce-op /
divide-factor table (:116-144), ``reduce_grads_on_one_rank`` (:147-154) and
``reduce_scatter_grads`` (:157-172).  On one GPU the reduce-scatter is served by
:class:`LocalReduceGroup`: every simulated rank deposits its send buffer in one
device allocation and the owning rank's range is folded in fixed rank order by
the ``fsh_reduce_rows_f32`` kernel.
"""

from __future__ import annotations

from typing import TYPE_CHECKING, Any

import torch
import torch.distributed as dist

from .. import hip_ops
from ._copy_kernels import (
    SegmentCopyDescriptor,
    SegmentPackDescriptor,
    copy_segments,
    pack_segments_into_flat_buffer,
)

if TYPE_CHECKING:
    from ..placement_contract import GradientReduction


def foreach_copy_(dst_tensors: list[torch.Tensor], src_tensors: list[torch.Tensor]) -> None:
    """Pairwise ``dst.copy_(src)`` with one runtime boundary in eager mode."""
    if len(dst_tensors) != len(src_tensors):
        raise AssertionError(
            f"Expected {len(dst_tensors)} destination tensors to match {len(src_tensors)} source tensors."
        )
    if not dst_tensors:
        return
    if torch.compiler.is_compiling():
        for dst, src in zip(dst_tensors, src_tensors, strict=True):
            dst.copy_(src)
    else:
        torch._foreach_copy_(dst_tensors, src_tensors)


def _hip_castable(tensor: torch.Tensor, dtype: torch.dtype) -> bool:
    floats = (torch.float32, torch.bfloat16)
    return (
        not torch.compiler.is_compiling()
        and tensor.device.type == "cuda"
        and tensor.is_contiguous()
        and tensor.dtype in floats
        and dtype in floats
    )


def copy_tensor_to_dtype(tensor: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """``tensor`` itself when it is already contiguous in ``dtype``; otherwise
    a fresh contiguous cast (one HIP cast-pack launch for fp32/bf16)."""
    if tensor.is_contiguous() and tensor.dtype == dtype:
        return tensor
    out = torch.empty(tensor.shape, dtype=dtype, device=tensor.device)
    if tensor.numel() == 0:
        return out
    if _hip_castable(tensor, dtype):
        copy_tensors_into_flat_buffer([tensor], out.view(-1))
    else:
        foreach_copy_([out], [tensor])
    return out


def pack_tensors_into_flat_buffer(tensors: list[torch.Tensor], dtype: torch.dtype) -> torch.Tensor:
    """Concatenate ``tensors`` (flattened) into one new flat buffer of ``dtype``."""
    if not tensors:
        raise AssertionError("Expected at least one tensor to pack.")
    out = torch.empty(sum(t.numel() for t in tensors), dtype=dtype, device=tensors[0].device)
    copy_tensors_into_flat_buffer(tensors, out)
    return out


def pack_tensors_into_flat_buffer_with_scratch(
    tensors: list[torch.Tensor], dtype: torch.dtype
) -> tuple[torch.Tensor, list[torch.Tensor]]:
    """As above, also returning tensors the caller must keep alive until the
    queued copy has run (descriptor tables of the HIP launch)."""
    if not tensors:
        raise AssertionError("Expected at least one tensor to pack.")
    out = torch.empty(sum(t.numel() for t in tensors), dtype=dtype, device=tensors[0].device)
    return out, copy_tensors_into_flat_buffer(tensors, out)


def copy_tensors_into_flat_buffer(tensors: list[torch.Tensor], out: torch.Tensor) -> list[torch.Tensor]:
    """Copy/cast ``tensors`` back to back into the preallocated flat ``out``."""
    offsets, total = [], 0
    for t in tensors:
        offsets.append(total)
        total += t.numel()
    if total != out.numel():
        raise AssertionError(f"Packed tensor numel {total} does not match output numel {out.numel()}.")
    live = [(t, o) for t, o in zip(tensors, offsets) if t.numel() > 0]
    if not live:
        return []
    if all(_hip_castable(t, out.dtype) and t.dtype == live[0][0].dtype for t, _ in live) and out.is_contiguous():
        flats = [t.view(-1) for t, _ in live]
        keep = pack_segments_into_flat_buffer(
            flats,
            tensor_indices=list(range(len(flats))),
            src_offsets=[0] * len(flats),
            numels=[t.numel() for t in flats],
            dst_offsets=[o for _, o in live],
            output=out,
        )
        if keep is not None:
            return keep
    foreach_copy_([out.narrow(0, o, t.numel()).view(t.shape) for t, o in live], [t for t, _ in live])
    return []


# ----------------------------------------------------------------- reductions
def _to_dist_reduce_op(op: Any) -> Any:
    if op == "avg" or op == dist.ReduceOp.AVG:
        return dist.ReduceOp.AVG
    if op == "sum" or op == dist.ReduceOp.SUM:
        return dist.ReduceOp.SUM
    raise ValueError(f"Unsupported gradient reduce op: {op!r}")


def gradient_reduce_plan(
    reduction: "GradientReduction", group_size: int, dtype: torch.dtype
) -> tuple[str, float | None, float | None]:
    """How one reduce-scatter realizes ``reduction``:
    ``(kind, pre_divide, post_divide)`` with kind ``"sum"``, ``"avg"`` or
    ``"premul_sum"`` (each input multiplied by ``1/factor`` before summing; the
    factor is then returned as ``pre_divide`` for reference, not applied
    twice).  Follows the table of the reference's
    ``_gradient_reduce_scatter_op`` (custom_placements/utils.py:116-144)."""
    if _to_dist_reduce_op(reduction.op) == dist.ReduceOp.SUM:
        return "sum", None, None
    factor = group_size if reduction.divide_factor is None else reduction.divide_factor
    if group_size == 1:
        return "sum", None, (None if factor == 1 else factor)
    if factor == group_size:
        return "avg", None, None
    if dtype in (torch.float32, torch.bfloat16):
        return "premul_sum", factor, None
    pre = 1
    while factor % pre == 0 and factor / pre > pre:
        pre *= 2
    return "sum", (None if pre == 1 else pre), factor / pre


def _gradient_reduce_scatter_op(
    reduction: "GradientReduction", group_size: int, dtype: torch.dtype
) -> tuple[Any, float | None, float | None]:
    """The same table expressed as a ``torch.distributed`` reduce op plus
    pre/post divide factors, for callers that run a real collective."""
    kind, pre, post = gradient_reduce_plan(reduction, group_size, dtype)
    if kind == "sum":
        return dist.ReduceOp.SUM, pre, post
    if kind == "avg":
        return dist.ReduceOp.AVG, None, None
    return dist._make_nccl_premul_sum(1.0 / pre), None, None


def reduce_grads_on_one_rank(grads: torch.Tensor, reduction: "GradientReduction") -> None:
    """Apply ``reduction`` in place to packed gradients of a 1-rank group."""
    _, pre, post = gradient_reduce_plan(reduction, 1, grads.dtype)
    if pre is not None:
        raise AssertionError("A 1-rank gradient reduction has no pre-divide factor.")
    if post is not None:
        grads.div_(post)


class LocalReduceGroup:
    """One-GPU stand-in for the process group of ``world_size`` ranks: serves
    the reduce-scatter of the gradient path and the all-gather of the unshard.

    ``contributions`` is a [world_size, world_size * segment] tensor: row r is
    the reduce-scatter input rank r would send (``world_size`` padded rank
    segments back to back).  ``reduce_scatter_grads`` on this group writes
    ``rank``'s segment of the fixed-order sum over rows 0..W-1.
    """

    def __init__(self, world_size: int, rank: int, *, local_row_only: bool = False) -> None:
        """``local_row_only``: the all-gather writes this rank's row and leaves
        the other rows of the output as they are (no ``gather_rows`` needed).
        For timing the local steps of an unshard; the output is then not a
        gathered layout that can be unpacked."""
        if not 0 <= rank < world_size:
            raise ValueError(f"rank must be in [0, {world_size}), got {rank}")
        self._world_size = world_size
        self._rank = rank
        self.local_row_only = local_row_only
        self.contributions: torch.Tensor | None = None
        self.deposited: set[int] = set()
        #: all-gather rows of the other ranks, by rank (see ``all_gather_rows``)
        self.gather_rows: dict[int, torch.Tensor] = {}
        self._gather_descriptors: dict = {}

    def size(self) -> int:
        return self._world_size

    def rank(self) -> int:
        return self._rank

    def allocate(self, send_numel: int, dtype: torch.dtype, device: torch.device) -> torch.Tensor:
        """Allocate the contribution rows; a harness may fill row r directly
        (then call ``mark_deposited(r)``) instead of copying through ``deposit``."""
        self.contributions = torch.empty((self._world_size, send_numel), dtype=dtype, device=device)
        self.deposited.clear()
        return self.contributions

    def mark_deposited(self, *ranks: int) -> None:
        self.deposited.update(ranks)

    def deposit(self, rank: int, send_buf: torch.Tensor) -> None:
        """Store rank ``rank``'s reduce-scatter input (one device copy)."""
        if self.contributions is None:
            self.allocate(send_buf.numel(), send_buf.dtype, send_buf.device)
        assert self.contributions is not None
        self.contributions[rank].copy_(send_buf.reshape(-1))
        self.deposited.add(rank)


def group_size(group: Any) -> int:
    """Ranks of a process group or of its one-GPU stand-in."""
    if isinstance(group, LocalReduceGroup):
        return group.size()
    return dist.get_world_size(group)


def all_gather_rows(output: torch.Tensor, input: torch.Tensor, group: Any, *, async_op: bool = False) -> Any | None:
    """All-gather equal rows into ``output`` (``world_size`` rows back to back).

    With a :class:`LocalReduceGroup` the exchange is local: this rank's
    ``input`` lands in its row and every other rank's row is copied from
    ``group.gather_rows`` (which the harness fills with what those ranks would
    send; a one-rank group needs none).  With a ``torch.distributed`` group it
    is one collective, as in the reference."""
    if isinstance(group, LocalReduceGroup):
        world, rank = group.size(), group.rank()
        if output.numel() != world * input.numel():
            raise ValueError(f"all-gather output has {output.numel()} elements, expected {world} x {input.numel()}")
        rows = output.view(world, input.numel())
        if group.local_row_only:
            rows[rank].copy_(input.reshape(-1))
            return None
        missing = sorted(set(range(world)) - {rank} - set(group.gather_rows))
        if missing:
            raise ValueError(f"LocalReduceGroup is missing the all-gather rows of ranks {missing}.")
        if _gather_rows_in_one_launch(group, rows, input, rank):
            return None
        rows[rank].copy_(input.reshape(-1))
        for other, row in group.gather_rows.items():
            if other != rank:
                rows[other].copy_(row.reshape(-1))
        return None
    if group is None:
        raise ValueError("all_gather_rows needs a process group (or a LocalReduceGroup on one GPU); got None.")
    return dist.all_gather_into_tensor(output, input, group=group, async_op=async_op)


def _gather_rows_in_one_launch(group: LocalReduceGroup, rows: torch.Tensor, input: torch.Tensor, rank: int) -> bool:
    """The local all-gather as one segment-copy launch (a device copy per row
    through the runtime's copy engine path runs at a sixth of the memory
    rate): every row is a segment whose source offset counts from this rank's
    ``input``.  The descriptor tables are kept per set of addresses, which
    repeat from step to step.  False when the rows do not qualify."""
    if torch.compiler.is_compiling() or rows.device.type != "cuda" or not rows.is_contiguous():
        return False
    world, n = rows.shape
    size = rows.element_size()
    sources = {rank: input.reshape(-1), **{r: row.reshape(-1) for r, row in group.gather_rows.items() if r != rank}}
    base = sources[rank].data_ptr()
    for r in range(world):
        src = sources[r]
        if src.device != rows.device or src.dtype != rows.dtype or src.numel() != n or not src.is_contiguous():
            return False
        if (src.data_ptr() - base) % size:
            return False
    key = (rows.data_ptr(), tuple(sources[r].data_ptr() for r in range(world)), n, size)
    descriptor = group._gather_descriptors.get(key)
    if descriptor is None:
        if len(group._gather_descriptors) >= 64:
            group._gather_descriptors.clear()
        descriptor = group._gather_descriptors[key] = SegmentCopyDescriptor.create(
            src_offsets=[(sources[r].data_ptr() - base) // size for r in range(world)],
            numels=[n] * world,
            dst_offsets=[r * n for r in range(world)],
            device=rows.device,
        )
    copy_segments(sources[rank], rows.view(-1), descriptor)
    return True


def _local_reduce(output: torch.Tensor, group: LocalReduceGroup, reduction: "GradientReduction") -> None:
    contributions = group.contributions
    if contributions is None:
        raise ValueError("LocalReduceGroup has no contributions; deposit every rank's send buffer first.")
    world = group.size()
    segment = output.numel()
    if contributions.shape != (world, world * segment):
        raise ValueError(
            f"Expected contributions of shape {(world, world * segment)}, got {tuple(contributions.shape)}."
        )
    kind, pre, post = gradient_reduce_plan(reduction, world, contributions.dtype)
    if kind == "avg":
        # ncclAvg on floating-point data is a pre-multiplied sum by 1/nranks.
        mode, factor = hip_ops.REDUCE_PREMUL, 1.0 / world
    elif kind == "premul_sum":
        mode, factor = hip_ops.REDUCE_PREMUL, 1.0 / pre
    elif pre is not None:
        mode, factor = hip_ops.REDUCE_PREMUL, 1.0 / pre
    else:
        mode, factor = hip_ops.REDUCE_SUM, 1.0
    hip_ops.reduce_rows(output, contributions, group.rank() * segment, mode=mode, factor=factor)
    if post is not None:
        output.div_(post)


def reduce_scatter_grads(output: torch.Tensor, input: torch.Tensor, reduction: "GradientReduction", group: Any) -> None:
    """Reduce-scatter packed gradients into ``output`` as ``reduction`` asks.

    With a :class:`LocalReduceGroup` the reduction runs on this GPU (``input``
    is deposited as this rank's contribution unless already present) and
    consumes the deposits; with a
    ``torch.distributed`` group it is one collective, as in the reference."""
    if isinstance(group, LocalReduceGroup):
        if group.rank() not in group.deposited:
            group.deposit(group.rank(), input)
        missing = sorted(set(range(group.size())) - group.deposited)
        if missing:
            raise ValueError(f"LocalReduceGroup is missing the contributions of ranks {missing}.")
        _local_reduce(output, group, reduction)
        group.deposited.clear()  # consumed: the next reduction needs fresh contributions
        return
    if group is None:
        raise ValueError(
            "reduce_scatter_grads needs a process group (or a LocalReduceGroup on one GPU); got None."
        )
    op, pre, post = _gradient_reduce_scatter_op(reduction, group.size(), input.dtype)
    if pre is not None:
        input = input / pre
    dist.reduce_scatter_tensor(output=output, input=input, op=op, group=group)
    if post is not None:
        output.div_(post)


def make_segment_pack_descriptor_if_supported(
    *, ninputs: int, tensor_indices, src_offsets, numels, dst_offsets, device: torch.device
) -> SegmentPackDescriptor | None:
    if torch.compiler.is_compiling():
        return None
    return SegmentPackDescriptor.create(
        ninputs=ninputs, tensor_indices=tensor_indices, src_offsets=src_offsets, numels=numels,
        dst_offsets=dst_offsets, device=device,
    )


def pack_segments_into_flat_buffer_if_supported(
    inputs, tensor_indices, src_offsets, numels, dst_offsets, out, descriptor=None
) -> list[torch.Tensor] | None:
    """HIP descriptor packing when the inputs qualify, else None (caller falls
    back to ``foreach_copy_``)."""
    if torch.compiler.is_compiling():
        return None
    return pack_segments_into_flat_buffer(
        inputs, tensor_indices, src_offsets, numels, dst_offsets, out, descriptor=descriptor
    )


__all__ = [
    "LocalReduceGroup",
    "all_gather_rows",
    "copy_tensor_to_dtype",
    "copy_tensors_into_flat_buffer",
    "foreach_copy_",
    "gradient_reduce_plan",
    "group_size",
    "make_segment_pack_descriptor_if_supported",
    "pack_segments_into_flat_buffer_if_supported",
    "pack_tensors_into_flat_buffer",
    "pack_tensors_into_flat_buffer_with_scratch",
    "reduce_grads_on_one_rank",
    "reduce_scatter_grads",
    "_gradient_reduce_scatter_op",
    "_to_dist_reduce_op",
]
