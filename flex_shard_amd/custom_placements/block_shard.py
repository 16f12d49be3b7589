"""``BlockShard`` (layout back-end of ``BucketedOwned``) and ``BucketedBlockShard``.

``BucketedBlockShard`` keeps the reference's public surface
(custom_placements/block_shard.py:537-1404): a param-major flat bucket cut into
per-rank ranges, view-in unshard, a one-pass reduce-scatter copy-in and
copy-out views.  The device work goes through the HIP segment kernels; the
one-pass copy-in here is a *single* launch for every gradient and every zero
gap (the reference launches one kernel per gradient plus one for the zeros).

``BlockShard`` carries only the per-parameter layout math the owner placement
lowers to (custom_placements/block_shard.py:89-284); its collective lifecycle
belongs to the multi-rank mixed bucket, which is outside this package.
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import TYPE_CHECKING, Any

import torch
import torch.nn as nn

from ..placement_contract import (
    BucketParamStorageLayout,
    BucketStorageLayout,
    GlobalLayout,
    Placement,
    PlacementPreparedReduceGrad,
    PlacementPreparedUnshard,
    PlacementReduceGradResult,
    PlacementUnshardResult,
)
from .. import hip_ops
from ..profiling import record_comm, record_copy_in, record_copy_out, record_range
from ._copy_kernels import SegmentCopyDescriptor, SegmentPackDescriptor, copy_segments, pack_segments_into_flat_buffer
from .utils import (
    all_gather_rows,
    copy_tensor_to_dtype,
    foreach_copy_,
    group_size,
    pack_segments_into_flat_buffer_if_supported,
    pack_tensors_into_flat_buffer_with_scratch,
    reduce_scatter_grads,
)

if TYPE_CHECKING:
    from ..bucket_storage import BucketLayout, BucketParamLayout, ParamInfo
    from ..placement_contract import GradientReduction


def _unsharded_dtype(info: "ParamInfo") -> torch.dtype:
    return getattr(info, "unsharded_dtype", info.dtype)


def _grad_reduce_dtype(info: "ParamInfo") -> torch.dtype:
    return getattr(info, "grad_reduce_dtype", info.dtype)


def _align_up(value: int, alignment: int) -> int:
    if alignment <= 0:
        raise ValueError(f"Expected positive alignment, got {alignment}.")
    return -(-value // alignment) * alignment


def _rank_range_views(
    bucket: torch.Tensor,
    padded_segments: torch.Tensor,
    rank_offsets: tuple[int, ...],
    rank_numels: tuple[int, ...],
) -> tuple[list[torch.Tensor], list[torch.Tensor]]:
    """Pairs (range of ``bucket``, head of that rank's padded row) for every
    rank with a non-empty range."""
    in_bucket, in_rows = [], []
    for rank, (start, count) in enumerate(zip(rank_offsets, rank_numels, strict=True)):
        if count:
            in_bucket.append(bucket[start : start + count])
            in_rows.append(padded_segments[rank, :count])
    return in_bucket, in_rows


class BlockShard(Placement):
    """Contiguous whole blocks of one parameter per rank along ``dim``."""

    def __init__(self, blocks_per_rank: tuple[int, ...], dim: int = 0) -> None:
        if isinstance(dim, bool) or not isinstance(dim, int):
            raise ValueError(f"BlockShard dim must be an integer, got {dim!r}.")
        if any(isinstance(c, bool) or not isinstance(c, int) or c < 0 for c in blocks_per_rank):
            raise ValueError("BlockShard blocks_per_rank must contain non-negative integers.")
        if sum(blocks_per_rank) == 0:
            raise ValueError("BlockShard blocks_per_rank must contain at least one positive count.")
        self.dim = dim
        self.blocks_per_rank = blocks_per_rank

    def __eq__(self, other: object) -> bool:
        return isinstance(other, BlockShard) and (self.dim, self.blocks_per_rank) == (other.dim, other.blocks_per_rank)

    def __hash__(self) -> int:
        return hash((type(self), self.dim, self.blocks_per_rank))

    def __repr__(self) -> str:
        suffix = "" if self.dim == 0 else f", dim={self.dim}"
        return f"BlockShard(blocks_per_rank={self.blocks_per_rank}{suffix})"

    def _validate_world_size(self, world_size: int) -> None:
        if len(self.blocks_per_rank) != world_size:
            raise ValueError(
                "BlockShard blocks_per_rank length must match world size: "
                f"got {len(self.blocks_per_rank)} counts for world size {world_size}."
            )

    def _normalize_dim(self, global_shape: torch.Size) -> int:
        if not global_shape:
            raise ValueError("BlockShard requires a parameter with at least one dimension.")
        dim = self.dim + len(global_shape) if self.dim < 0 else self.dim
        if not 0 <= dim < len(global_shape):
            raise ValueError(f"BlockShard dim {self.dim} is invalid for parameter shape {tuple(global_shape)}.")
        return dim

    def _block_dim_size(self, global_shape: torch.Size) -> int:
        dim = self._normalize_dim(global_shape)
        blocks = sum(self.blocks_per_rank)
        if global_shape[dim] % blocks:
            raise ValueError(
                f"BlockShard requires global_shape[{dim}] to be divisible by sum(blocks_per_rank): "
                f"got size {global_shape[dim]} and blocks_per_rank {self.blocks_per_rank}."
            )
        return global_shape[dim] // blocks

    def _block_numel(self, global_shape: torch.Size) -> int:
        dim = self._normalize_dim(global_shape)
        return math.prod(global_shape[:dim]) * self._block_dim_size(global_shape) * math.prod(global_shape[dim + 1 :])

    def _shard_bounds_for_rank(self, global_shape: torch.Size, rank: int, world_size: int) -> tuple[int, int]:
        self._validate_world_size(world_size)
        if not 0 <= rank < world_size:
            raise ValueError(f"BlockShard rank must be in [0, {world_size}), got {rank}.")
        size = self._block_dim_size(global_shape)
        start = sum(self.blocks_per_rank[:rank]) * size
        return start, start + self.blocks_per_rank[rank] * size

    def compute_local_shape(self, global_shape: torch.Size, rank: int, world_size: int) -> torch.Size:
        dim = self._normalize_dim(global_shape)
        start, end = self._shard_bounds_for_rank(global_shape, rank, world_size)
        shape = list(global_shape)
        shape[dim] = end - start
        return torch.Size(shape)

    def extract_local_shard(self, param: torch.Tensor, rank: int, world_size: int) -> torch.Tensor:
        dim = self._normalize_dim(param.shape)
        start, end = self._shard_bounds_for_rank(param.shape, rank, world_size)
        return param.narrow(dim, start, end - start)

    def global_layout(self, info: "ParamInfo", rank: int, world_size: int) -> GlobalLayout:
        dim = self._normalize_dim(info.global_shape)
        start, _ = self._shard_bounds_for_rank(info.global_shape, rank, world_size)
        if info.local_numel == 0:
            return GlobalLayout(tuple(info.global_shape), (), (), ())
        offset = [0] * len(info.global_shape)
        offset[dim] = start
        return GlobalLayout(
            global_shape=tuple(info.global_shape),
            global_offsets=(tuple(offset),),
            local_offsets=((0,) * len(info.local_shape),),
            local_sizes=(tuple(info.local_shape),),
        )


class BucketedBlockShard(Placement):
    """Block-shard one bucket-global, param-major flat buffer.

    ``dims`` names the prefix dimensions whose rows stay whole (``(0,)``,
    ``(0, 1)``, ...); ``blocks_per_rank`` gives each rank a number of equal
    bucket-global blocks.  Each parameter starts at a multiple of the lcm of
    the row widths and the bucket is padded so every block holds whole rows;
    gaps and the tail are zeros.  With equal ranges the bucket itself is the
    all-gather output and the reduce-scatter input.
    """

    @dataclass(frozen=True)
    class _UnshardState:
        infos: list
        pg: Any
        debug_fqn: str | None

    @dataclass(frozen=True)
    class _ReduceGradState:
        infos: list
        rank: int
        pg: Any
        debug_fqn: str | None
        padded_segment_numel: int

    @dataclass(frozen=True)
    class _ReduceCopyInPlan:
        """Where a bucket's grads land in the reduce-scatter input rows for one
        row stride, in elements from the first row's start: per param its
        segments (offset in the grad, length, destination offset) and the
        segments to zero (destination offset, length).  ``alignment`` is the
        gcd of every number above; ``descriptors`` caches device tables per
        (device, source dtype)."""

        bucket_layout: Any
        param_segments: tuple[tuple[tuple[int, int, int], ...], ...]
        zero_segments: tuple[tuple[int, int], ...]
        alignment: int
        descriptors: dict

    def __init__(self, dims: tuple[int, ...] = (0,), blocks_per_rank: tuple[int, ...] = (1,)) -> None:
        if not dims:
            raise ValueError("BucketedBlockShard dims must be non-empty.")
        wanted = tuple(range(len(dims)))
        if dims != wanted:
            raise ValueError(f"BucketedBlockShard currently requires prefix dims {wanted}, but got {dims}.")
        if any(count < 0 for count in blocks_per_rank):
            raise ValueError("BucketedBlockShard blocks_per_rank must be non-negative.")
        if sum(blocks_per_rank) == 0:
            raise ValueError("BucketedBlockShard blocks_per_rank must contain at least one positive count.")
        self.dims = dims
        self.blocks_per_rank = blocks_per_rank
        self._reduce_copy_in_plans: dict = {}
        self._send_row_descriptors: dict = {}
        self._scatter_descriptors: dict = {}

    def __eq__(self, other: object) -> bool:
        if not isinstance(other, BucketedBlockShard):
            return False
        return (self.dims, self.blocks_per_rank) == (other.dims, other.blocks_per_rank)

    def __hash__(self) -> int:
        return hash((type(self), self.dims, self.blocks_per_rank))

    def __repr__(self) -> str:
        return f"BucketedBlockShard(dims={self.dims}, blocks_per_rank={self.blocks_per_rank})"

    # ------------------------------------------------------------ layout math
    def _validate_world_size(self, world_size: int) -> None:
        if len(self.blocks_per_rank) != world_size:
            raise ValueError(
                "BucketedBlockShard blocks_per_rank length must match world size: "
                f"got {len(self.blocks_per_rank)} block counts for world size {world_size}."
            )

    def _prefix_numel(self, global_shape: torch.Size) -> int:
        if len(global_shape) < len(self.dims):
            raise ValueError(
                f"BucketedBlockShard dims {self.dims} are invalid for parameter shape {tuple(global_shape)}."
            )
        return math.prod(global_shape[: len(self.dims)])

    def _suffix_shape(self, global_shape: torch.Size) -> torch.Size:
        return torch.Size(global_shape[len(self.dims) :])

    def _suffix_numel(self, global_shape: torch.Size) -> int:
        return math.prod(self._suffix_shape(global_shape))

    def _bucket_layout(self, info: "ParamInfo") -> "BucketLayout":
        if info.bucket_layout is None:
            raise AssertionError("Expected BucketedBlockShard ParamInfo to carry a bucket layout.")
        return info.bucket_layout

    def _param_layout(self, info: "ParamInfo") -> "BucketParamLayout":
        return self._bucket_layout(info).param_layouts[info.fqn]

    def compute_local_shape(self, global_shape: torch.Size, rank: int, world_size: int) -> torch.Size:
        raise NotImplementedError(
            "BucketedBlockShard computes local shapes from the whole bucket. Use bucket_storage_layout() instead."
        )

    def extract_local_shard(self, param: torch.Tensor, rank: int, world_size: int) -> torch.Tensor:
        raise NotImplementedError(
            "BucketedBlockShard extracts local shards from bucket-global ranges. Use bucket storage views instead."
        )

    def global_layout(self, info: "ParamInfo", rank: int, world_size: int) -> GlobalLayout:
        if self.dims != (0,):
            raise NotImplementedError("BucketedBlockShard distributed checkpointing supports only dims=(0,).")
        shape = tuple(info.global_shape)
        if info.local_numel == 0:
            return GlobalLayout(shape, (), (), ())
        layout = self._param_layout(info)
        within = layout.local_global_offset - layout.param_offset
        row = self._suffix_numel(info.global_shape)
        if within % row:
            raise AssertionError(f"BucketedBlockShard local range for {info.fqn!r} is not row-aligned.")
        return GlobalLayout(
            global_shape=shape,
            global_offsets=((within // row, *([0] * (len(shape) - 1))),),
            local_offsets=((0,) * len(info.local_shape),),
            local_sizes=(tuple(info.local_shape),),
        )

    def _param_alignment_numel(self, named_params: list[tuple[str, nn.Parameter]]) -> int:
        alignment = 1
        for _, param in named_params:
            self._prefix_numel(param.shape)
            alignment = math.lcm(alignment, self._suffix_numel(param.shape))
        return alignment

    def _bucket_param_offsets(
        self, named_params: list[tuple[str, nn.Parameter]], alignment_numel: int
    ) -> tuple[dict[str, int], int]:
        starts: dict[str, int] = {}
        cursor = 0
        for fqn, param in named_params:
            cursor = _align_up(cursor, alignment_numel)
            starts[fqn] = cursor
            cursor += param.numel()
        return starts, cursor

    def _bucket_rank_layout(
        self, unpadded_global_numel: int, alignment_numel: int
    ) -> tuple[int, tuple[int, ...], tuple[int, ...]]:
        blocks = sum(self.blocks_per_rank)
        padded = _align_up(unpadded_global_numel, alignment_numel * blocks)
        per_block = padded // blocks
        numels = tuple(count * per_block for count in self.blocks_per_rank)
        offsets = tuple(sum(numels[:rank]) for rank in range(len(numels)))
        return padded, offsets, numels

    def _local_shape_from_numel(self, global_shape: torch.Size, local_numel: int) -> torch.Size:
        suffix = self._suffix_shape(global_shape)
        width = math.prod(suffix)
        if local_numel % width:
            raise ValueError(
                "BucketedBlockShard bucket split produced a shard that is not aligned to "
                f"flattened prefix rows for shape {tuple(global_shape)}."
            )
        return torch.Size([local_numel // width, *suffix])

    def bucket_storage_layout(
        self,
        named_params: list[tuple[str, nn.Parameter]],
        param_placements: dict[str, tuple[Placement, ...]],
        mesh: Any,
    ) -> BucketStorageLayout:
        from ..bucket_storage import BucketLayout, BucketParamLayout

        if not named_params:
            return BucketStorageLayout(param_layouts={}, total_bytes=0)
        self._validate_world_size(mesh.size())
        rank = mesh.get_local_rank()
        first_fqn, first = named_params[0]
        dtype = first.dtype
        alignment = self._param_alignment_numel(named_params)
        starts, unpadded = self._bucket_param_offsets(named_params, alignment)
        padded, rank_offsets, rank_numels = self._bucket_rank_layout(unpadded, alignment)
        lo, hi = rank_offsets[rank], rank_offsets[rank] + rank_numels[rank]

        bucket_params: dict[str, BucketParamLayout] = {}
        local: dict[str, tuple[torch.Size, int, int]] = {}
        for fqn, param in named_params:
            if param.dtype != dtype:
                raise ValueError(
                    f"BucketedBlockShard requires one dtype per bucket: {first_fqn!r} uses {dtype} "
                    f"but {fqn!r} uses {param.dtype}."
                )
            if param_placements[fqn] != (self,):
                raise ValueError(
                    "BucketedBlockShard requires the same placement instance for every parameter in a "
                    f"bucket; {fqn!r} uses {param_placements[fqn]!r}."
                )
            begin = max(lo, starts[fqn])
            end = min(hi, starts[fqn] + param.numel())
            count = max(0, end - begin)
            local[fqn] = (self._local_shape_from_numel(param.shape, count), count, (begin - lo) * dtype.itemsize)
            bucket_params[fqn] = BucketParamLayout(param_offset=starts[fqn], local_global_offset=begin)

        bucket_layout = BucketLayout(
            global_numel=padded,
            local_numel=rank_numels[rank],
            rank_offsets=rank_offsets,
            rank_numels=rank_numels,
            param_layouts=bucket_params,
        )
        if rank_numels[rank] > 0 and not any(count for _, count, _ in local.values()):
            raise ValueError(
                "BucketedBlockShard planned a rank-local bucket range that contains only padding. "
                "Split the bucket or choose blocks_per_rank that assign parameter data to every non-empty rank."
            )
        return BucketStorageLayout(
            param_layouts={
                fqn: BucketParamStorageLayout(
                    local_shape=shape,
                    local_numel=count,
                    byte_offset=byte_offset,
                    storage_nbytes=count * dtype.itemsize,
                    bucket_layout=bucket_layout,
                )
                for fqn, (shape, count, byte_offset) in local.items()
            },
            total_bytes=rank_numels[rank] * dtype.itemsize,
        )

    def copy_param_to_storage(
        self, byte_storage: torch.Tensor, info: "ParamInfo", param: torch.Tensor, rank: int, world_size: int
    ) -> None:
        data = param.detach()
        if data.device.type == "meta" or info.local_numel == 0:
            return
        layout = self._param_layout(info)
        begin = layout.local_global_offset - layout.param_offset
        piece = data.contiguous().view(-1)[begin : begin + info.local_numel]
        nbytes = piece.numel() * piece.element_size()
        byte_storage[info.byte_offset : info.byte_offset + nbytes].copy_(piece.view(torch.uint8))

    def _make_local_bucket_view(self, tensors: list[torch.Tensor], infos: list["ParamInfo"]) -> torch.Tensor:
        """This rank's whole range as one flat view of the storage the local
        params live in (they are views of one allocation at their byte
        offsets), so the all-gather input needs no copy."""
        local_numel = self._bucket_layout(infos[0]).local_numel
        if local_numel == 0:
            return tensors[0].new_empty(0)
        anchor: torch.Tensor | None = None
        base_ptr = 0
        for tensor, info in zip(tensors, infos, strict=True):
            if tensor.numel() == 0:
                continue
            start_ptr = tensor.data_ptr() - info.byte_offset
            storage_ptr = tensor.untyped_storage().data_ptr()
            if anchor is None:
                anchor, base_ptr = tensor, start_ptr
            elif storage_ptr != anchor.untyped_storage().data_ptr() or start_ptr != base_ptr:
                raise ValueError("BucketedBlockShard expected local tensors to share one bucket storage allocation.")
            if (start_ptr - storage_ptr) % tensor.element_size():
                raise AssertionError("BucketedBlockShard local bucket storage is not dtype-aligned.")
        if anchor is None:
            raise ValueError(
                "BucketedBlockShard cannot create a view-in send buffer because this rank has no "
                "parameter tensor covering its non-empty bucket range."
            )
        storage = anchor.untyped_storage()
        offset = (base_ptr - storage.data_ptr()) // anchor.element_size()
        return anchor.new_empty(0).set_(storage, offset, (local_numel,), (1,))

    # ---------------------------------------------------------------- unshard
    def prepare_unshard_bucket(
        self, tensors: list[torch.Tensor], infos: list["ParamInfo"], mesh: Any, debug_fqn: str | None
    ) -> PlacementPreparedUnshard:
        dtype = _unsharded_dtype(infos[0])
        if any(_unsharded_dtype(info) != dtype for info in infos):
            raise ValueError("BucketedBlockShard requires one unsharded dtype per bucket.")
        with record_copy_in():
            send = self._make_local_bucket_view(tensors, infos)
            send, scratch = self._send_row(send, dtype, max(self._bucket_layout(infos[0]).rank_numels))
        return PlacementPreparedUnshard(
            placement=self,
            buffers=[send, *scratch],
            placement_state=BucketedBlockShard._UnshardState(infos=infos, pg=mesh.get_group(), debug_fqn=debug_fqn),
        )

    def _send_row(self, local: torch.Tensor, dtype: torch.dtype, widest: int) -> tuple[torch.Tensor, list[torch.Tensor]]:
        """The all-gather input of this rank: its flat range in the unsharded
        dtype, zero-padded to the longest rank range.  A range that already
        has that dtype and length is sent as it lies (no copy); anything else
        is one cast-pack launch that writes the cast elements and the zero pad
        together (the reference casts with a foreach copy and then pads with
        ``F.pad``, custom_placements/block_shard.py:948-958).  Returns the row
        and the tensors to keep alive until the launch has run."""
        short_by = widest - local.numel()
        if local.dtype == dtype and short_by <= 0:
            return local, []
        floats = (torch.float32, torch.bfloat16)
        if (
            torch.compiler.is_compiling()
            or local.device.type != "cuda"
            or local.dtype not in floats
            or dtype not in floats
            or local.numel() == 0
        ):
            send, scratch = local, []
            if send.dtype != dtype:
                send, scratch = pack_tensors_into_flat_buffer_with_scratch([send], dtype)
            else:
                send = copy_tensor_to_dtype(send, dtype)
            if short_by > 0:
                send = nn.functional.pad(send, (0, short_by))
            return send, scratch
        # One descriptor per source range and stream: its device table holds
        # the source address and is refreshed by a copy queued on the current
        # stream, so equally sized buckets (the layers of a model) or two
        # streams sharing one table could overwrite it before the other's
        # launch has read it.
        key = (local.data_ptr(), local.numel(), widest, local.device, hip_ops.stream_ptr(local.device))
        descriptor = self._send_row_descriptors.get(key)
        if descriptor is None:
            pad = [(-1, 0, short_by, local.numel())] if short_by > 0 else []
            segments = [(0, 0, local.numel(), 0), *pad]
            descriptor = SegmentPackDescriptor.create(
                ninputs=1,
                tensor_indices=[seg[0] for seg in segments],
                src_offsets=[seg[1] for seg in segments],
                numels=[seg[2] for seg in segments],
                dst_offsets=[seg[3] for seg in segments],
                device=local.device,
            )
            if len(self._send_row_descriptors) >= 256:
                self._send_row_descriptors.clear()
            self._send_row_descriptors[key] = descriptor
        row = torch.empty(max(widest, local.numel()), dtype=dtype, device=local.device)
        keep = pack_segments_into_flat_buffer([local], (), (), (), (), row, descriptor=descriptor)
        if keep is None:
            raise AssertionError("BucketedBlockShard send-row pack was declined for a contiguous float range.")
        return row, keep

    def run_prepared_unshard(self, prepared: PlacementPreparedUnshard, *, async_op: bool = False) -> Any | None:
        state = prepared.placement_state
        if not isinstance(state, BucketedBlockShard._UnshardState):
            raise AssertionError(f"Expected BucketedBlockShard._UnshardState, got {type(state).__name__}")
        send = prepared.buffers[0]
        layout = self._bucket_layout(state.infos[0])
        if prepared.persistent_buffers is not None:
            bucket = prepared.persistent_buffers[0]  # a refill gathers straight into it
        else:
            bucket = send.new_empty(layout.global_numel)
            prepared.buffers.insert(1, bucket)
        world_size = group_size(state.pg)
        target = bucket if world_size * send.numel() == bucket.numel() else bucket.new_empty(world_size * send.numel())
        with record_comm("FlexShard::all_gather", state.debug_fqn):
            work = all_gather_rows(target, send, state.pg, async_op=async_op)
        if target is not bucket:
            if work is not None:
                work.wait()
                work = None
            self._scatter_padded_rows_into_bucket(bucket, target.view(world_size, -1), layout)
        return work

    def _scatter_padded_rows_into_bucket(self, bucket: torch.Tensor, rows: torch.Tensor, layout: "BucketLayout") -> None:
        """Copy each rank's valid prefix of its padded gathered row into its
        range of ``bucket`` (uneven ranges only): one segment-copy launch for
        all ranks (the reference issues a foreach copy over per-rank views,
        custom_placements/block_shard.py:998-1011)."""
        with record_copy_out():
            if torch.compiler.is_compiling() or bucket.device.type != "cuda" or not rows.is_contiguous():
                in_bucket, in_rows = _rank_range_views(bucket, rows, layout.rank_offsets, layout.rank_numels)
                foreach_copy_(in_bucket, in_rows)
                return
            key = (id(layout), rows.shape[1], bucket.device)
            cached = self._scatter_descriptors.get(key)
            if cached is None or cached[0] is not layout:
                live = [
                    (rank * rows.shape[1], count, start)
                    for rank, (start, count) in enumerate(zip(layout.rank_offsets, layout.rank_numels, strict=True))
                    if count
                ]
                descriptor = SegmentCopyDescriptor.create(
                    src_offsets=[seg[0] for seg in live],
                    numels=[seg[1] for seg in live],
                    dst_offsets=[seg[2] for seg in live],
                    device=bucket.device,
                )
                if len(self._scatter_descriptors) >= 16:
                    self._scatter_descriptors.clear()
                self._scatter_descriptors[key] = cached = (layout, descriptor)
            copy_segments(rows, bucket, cached[1])

    def finish_prepared_unshard(self, prepared: PlacementPreparedUnshard) -> PlacementUnshardResult:
        state = prepared.placement_state
        if not isinstance(state, BucketedBlockShard._UnshardState):
            raise AssertionError(f"Expected BucketedBlockShard._UnshardState, got {type(state).__name__}")
        if prepared.persistent_buffers is not None:
            return PlacementUnshardResult(full_params=[], persistent_buffers=list(prepared.persistent_buffers))
        gathered = prepared.buffers[1]
        if prepared.persistent:
            # First unshard: the gathered bucket was produced on the unshard
            # stream; persistent storage belongs to the current stream.
            bucket = torch.empty_like(gathered)
            with record_copy_out():
                bucket.copy_(gathered)
        else:
            bucket = gathered
        full = []
        for info in state.infos:
            start = self._param_layout(info).param_offset
            full.append(bucket[start : start + info.global_numel].view(info.global_shape))
        return PlacementUnshardResult(full_params=full, persistent_buffers=[bucket] if prepared.persistent else [])

    # --------------------------------------------------------- gradient path
    def _gradient_bucket_of(
        self, tensors: list[torch.Tensor], infos: list["ParamInfo"], global_numel: int, dtype: torch.dtype
    ) -> torch.Tensor | None:
        """The flat gradient bucket every grad views at its layout offset, if
        there is one (then the reduction reads it without a copy-in)."""
        bucket = tensors[0]._base
        if bucket is None or bucket.dtype != dtype or bucket.shape != (global_numel,) or not bucket.is_contiguous():
            return None
        origin = bucket.storage_offset()
        for tensor, info in zip(tensors, infos, strict=True):
            at_offset = tensor.storage_offset() - origin == self._param_layout(info).param_offset
            if tensor._base is not bucket or tensor.shape != info.global_shape or not tensor.is_contiguous() or not at_offset:
                return None
        return bucket

    def _reduce_copy_in_plan(self, infos: list["ParamInfo"], row_stride: int) -> "BucketedBlockShard._ReduceCopyInPlan":
        layout = self._bucket_layout(infos[0])
        key = (id(layout), tuple(info.fqn for info in infos), row_stride)
        cached = self._reduce_copy_in_plans.get(key)
        if cached is not None and cached.bucket_layout is layout:
            return cached
        widest = max(layout.rank_numels)
        spans = [(self._param_layout(info).param_offset, info.global_numel) for info in infos]
        per_param: list[list[tuple[int, int, int]]] = [[] for _ in infos]
        zeros: list[tuple[int, int]] = []
        for rank, (r_start, r_count) in enumerate(zip(layout.rank_offsets, layout.rank_numels, strict=True)):
            row0 = rank * row_stride
            taken: list[tuple[int, int]] = []
            for segments, (p_start, p_count) in zip(per_param, spans, strict=True):
                lo = max(p_start, r_start)
                hi = min(p_start + p_count, r_start + r_count)
                if lo < hi:
                    segments.append((lo - p_start, hi - lo, row0 + lo - r_start))
                    taken.append((lo - r_start, hi - r_start))
            # Everything not covered by a param is zero: gaps between params,
            # the bucket's tail padding, the pad up to the longest range.
            col = 0
            for lo, hi in sorted(taken):
                if lo > col:
                    zeros.append((row0 + col, lo - col))
                col = max(col, hi)
            if col < widest:
                zeros.append((row0 + col, widest - col))
        numbers = [v for segments in per_param for seg in segments for v in seg]
        numbers += [v for seg in zeros for v in seg]
        plan = BucketedBlockShard._ReduceCopyInPlan(
            bucket_layout=layout,
            param_segments=tuple(tuple(s) for s in per_param),
            zero_segments=tuple(zeros),
            alignment=math.gcd(*numbers) or 1,
            descriptors={},
        )
        self._reduce_copy_in_plans[key] = plan
        return plan

    def _packs_reduce_scatter_grad_in_one_pass(self, tensors: list[torch.Tensor], dtype: torch.dtype) -> bool:
        """Whether the single-launch copy-in can write these grads: eager mode,
        contiguous GPU grads of one dtype, fp32/bf16 on both sides (a cast to
        the reduce dtype is fused into the copy)."""
        if torch.compiler.is_compiling():
            return False
        floats = (torch.float32, torch.bfloat16)
        first = tensors[0].dtype
        return dtype in floats and all(
            t.device.type == "cuda" and t.dtype == first and t.dtype in floats and t.is_contiguous() for t in tensors
        )

    def _pack_reduce_scatter_grad(
        self, tensors: list[torch.Tensor], infos: list["ParamInfo"], world_size: int, send_rows: torch.Tensor
    ) -> list[torch.Tensor]:
        """Write the reduce-scatter input into ``send_rows`` ([world size, the
        longest rank range], possibly a view of wider rows): each rank's range
        of the param-major grads, zeros elsewhere.  One launch writes every
        element once.  Returns tensors to keep alive until the launch ran."""
        if send_rows.shape != (world_size, max(self._bucket_layout(infos[0]).rank_numels)):
            raise AssertionError(
                "BucketedBlockShard send rows must be world size by the longest rank range, "
                f"got {tuple(send_rows.shape)}."
            )
        if send_rows.stride(1) != 1 or not self._packs_reduce_scatter_grad_in_one_pass(tensors, send_rows.dtype):
            raise AssertionError("BucketedBlockShard can't pack these grads in one pass.")
        row_stride = send_rows.stride(0)
        plan = self._reduce_copy_in_plan(infos, row_stride)
        out = send_rows.as_strided(((send_rows.size(0) - 1) * row_stride + send_rows.size(1),), (1,))
        sources = [t.view(-1) for t in tensors]
        key = (out.device, sources[0].dtype)
        descriptor = plan.descriptors.get(key)
        if descriptor is None:
            index, src, cnt, dst = [], [], [], []
            for which, segments in enumerate(plan.param_segments):
                for s, n, d in segments:
                    index.append(which)
                    src.append(s)
                    cnt.append(n)
                    dst.append(d)
            for d, n in plan.zero_segments:
                index.append(-1)
                src.append(0)
                cnt.append(n)
                dst.append(d)
            descriptor = SegmentPackDescriptor.create(
                ninputs=len(sources), tensor_indices=index, src_offsets=src, numels=cnt, dst_offsets=dst,
                device=out.device,
            )
            plan.descriptors[key] = descriptor
        keep = pack_segments_into_flat_buffer_if_supported(sources, [], [], [], [], out, descriptor=descriptor)
        if keep is None:
            raise AssertionError("BucketedBlockShard one-pass copy-in was declined by the HIP packer.")
        return keep

    def prepare_reduce_grad(
        self, tensors: list[torch.Tensor], infos: list["ParamInfo"], mesh: Any, debug_fqn: str | None
    ) -> PlacementPreparedReduceGrad:
        world_size = mesh.size()
        dtype = _grad_reduce_dtype(infos[0])
        device = tensors[0].device
        layout = self._bucket_layout(infos[0])
        widest = max(layout.rank_numels)
        state = BucketedBlockShard._ReduceGradState(
            infos=infos, rank=mesh.get_local_rank(), pg=mesh.get_group(), debug_fqn=debug_fqn,
            padded_segment_numel=widest,
        )
        even = world_size * widest == layout.global_numel
        if even:
            bucket = self._gradient_bucket_of(tensors, infos, layout.global_numel, dtype)
            if bucket is not None:
                return PlacementPreparedReduceGrad(placement=self, buffers=[bucket], placement_state=state)
        if self._packs_reduce_scatter_grad_in_one_pass(tensors, dtype):
            with record_range("FlexShard::reduce_scatter_copy_in", debug_fqn):
                send = torch.empty(world_size * widest, dtype=dtype, device=device)
                keep = self._pack_reduce_scatter_grad(tensors, infos, world_size, send.view(world_size, widest))
            return PlacementPreparedReduceGrad(placement=self, buffers=[send, *keep], placement_state=state)
        # Compiling, off the GPU, or unusual dtypes: copy through a zeroed
        # gradient bucket with ATen.
        with record_range("FlexShard::reduce_scatter_copy_in", debug_fqn):
            bucket = torch.zeros(layout.global_numel, dtype=dtype, device=device)
            dsts = []
            for info in infos:
                start = self._param_layout(info).param_offset
                dsts.append(bucket[start : start + info.global_numel])
            foreach_copy_(dsts, [t.reshape(-1) for t in tensors])
            send = bucket
            if not even:
                send = torch.zeros(world_size * widest, dtype=dtype, device=device)
                in_bucket, in_rows = _rank_range_views(
                    bucket, send.view(world_size, widest), layout.rank_offsets, layout.rank_numels
                )
                foreach_copy_(in_rows, in_bucket)
        return PlacementPreparedReduceGrad(placement=self, buffers=[send], placement_state=state)

    def reduce_prepared_grad(
        self, prepared: PlacementPreparedReduceGrad, reduction: "GradientReduction"
    ) -> PlacementReduceGradResult:
        state = prepared.placement_state
        if not isinstance(state, BucketedBlockShard._ReduceGradState):
            raise AssertionError(f"Expected BucketedBlockShard._ReduceGradState, got {type(state).__name__}")
        send = prepared.buffers[0]
        recv = torch.empty(state.padded_segment_numel, dtype=send.dtype, device=send.device)
        with record_comm("FlexShard::post_backward_reduce", state.debug_fqn):
            reduce_scatter_grads(recv, send, reduction, state.pg)
        with record_range("FlexShard::reduce_scatter_copy_out", state.debug_fqn):
            shards = []
            for info in state.infos:
                start = info.byte_offset // info.dtype.itemsize
                shards.append(recv[start : start + info.local_numel].view(info.local_shape))
        return PlacementReduceGradResult(shards, [recv])


def make_bucketed_block_placement_fn(*, dims: tuple[int, ...], blocks_per_rank: tuple[int, ...]):
    """A placement function assigning one ``BucketedBlockShard`` per bucket."""

    def bucketed_block_placements(named_params: list[tuple[str, nn.Parameter]], mesh: Any) -> dict:
        if len(blocks_per_rank) != mesh.size():
            raise ValueError(
                "BucketedBlockShard blocks_per_rank length must match mesh size: "
                f"got {len(blocks_per_rank)} block counts for mesh size {mesh.size()}."
            )
        placement = BucketedBlockShard(dims=dims, blocks_per_rank=blocks_per_rank)
        return {fqn: (placement,) for fqn, _ in named_params}

    return bucketed_block_placements


__all__ = ["BlockShard", "BucketedBlockShard", "make_bucketed_block_placement_fn"]
