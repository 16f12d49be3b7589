"""Quantized all-gather on bucketed block sharding with blockwise scales.

``BlockwiseQuantBucketedBlockShard`` keeps the reference's surface
(custom_placements/blockwise_quant_bucketed_block_shard.py:154-1511): a bucket
is cut into contiguous runs of ``shard_block_rows``-row units over the dense
parameters, every rank owns whole block rows and quantizes its own shard with
no cross-rank amax, and the gathered weight is bit-identical to "all-gather
the dense weights, then quantize".

What differs is the device work.  The local send payload is produced by *one*
HIP launch (tile quantize fused with packing and pad zeroing) instead of one
quantizer launch per chunk plus two foreach copies, and the gathered rank rows
are compacted by one segment-copy launch, optionally fused with dequantization
(``finish_prepared_unshard_with_dequant``).  There is no CPU compute path:
tensors off the GPU raise.
"""

from __future__ import annotations

import sys
from collections.abc import Sequence
from dataclasses import dataclass
from typing import TYPE_CHECKING, Any

import torch
import torch.nn as nn

from .. import hip_ops
from ..placement_contract import (
    BucketParamStorageLayout,
    BucketStorageLayout,
    GlobalLayout,
    PlacementPreparedUnshard,
    PlacementUnshardResult,
)
from ..profiling import record_comm, record_copy_in, record_copy_out
from . import quant_plan
from ._copy_kernels import SegmentCopyDescriptor, copy_segments
from .block_shard import BucketedBlockShard
from .quant_plan import ScaleRegion as _ScaleRegion
from .quant_plan import align_up as _align_up
from .quant_plan import ceil_div as _ceil_div
from .quant_plan import matrix_shape as _matrix_shape
from .utils import all_gather_rows

if TYPE_CHECKING:
    from ..bucket_storage import ParamInfo
    from ..placement_contract import Placement

_VEC_COPY_DTYPE = torch.int32
_VEC_COPY_NBYTES = _VEC_COPY_DTYPE.itemsize
_VEC_ALIGN_BYTES = quant_plan.VEC_ALIGN_BYTES


def _validate_block_size(block_size: int) -> None:
    if not isinstance(block_size, int):
        raise TypeError(f"block_size must be an int, got {type(block_size).__name__}")
    if block_size <= 0:
        raise ValueError(f"block_size must be positive, got {block_size}")


def _validate_2d_non_empty(shape: Sequence[int], what: str) -> tuple[int, int]:
    if len(shape) != 2:
        raise ValueError(f"{what} expects 2D, got {tuple(shape)}")
    rows, cols = shape
    if rows <= 0 or cols <= 0:
        raise ValueError(f"{what} requires non-empty 2D shape, got {tuple(shape)}")
    return rows, cols


def _unravel_index(index: int, shape: Sequence[int]) -> tuple[int, ...]:
    coords = []
    for size in reversed(shape):
        index, coord = divmod(index, size)
        coords.append(coord)
    return tuple(reversed(coords))


def _scale_shape(shape: Sequence[int], block_size: int) -> tuple[int, int]:
    _validate_block_size(block_size)
    rows, cols = _validate_2d_non_empty(shape, "blockwise scale")
    return _ceil_div(rows, block_size), _ceil_div(cols, block_size)


def _padded_shape(shape: Sequence[int], block_size: int) -> tuple[int, int]:
    tiles_r, tiles_c = _scale_shape(shape, block_size)
    return tiles_r * block_size, tiles_c * block_size


def _callable_name(value: Any) -> str:
    return getattr(value, "__qualname__", type(value).__qualname__)


def _is_vec_copy_viewable(tensor: torch.Tensor) -> bool:
    """Whether a uint8 tensor can be viewed as int32 (torch's dtype-view rules)."""
    if torch.compiler.is_compiling():
        return False
    return (
        tensor.dtype == torch.uint8
        and tensor.ndim > 0
        and tensor.stride(-1) == 1
        and tensor.size(-1) % _VEC_COPY_NBYTES == 0
        and tensor.storage_offset() % _VEC_COPY_NBYTES == 0
        and all(stride % _VEC_COPY_NBYTES == 0 for stride in tensor.stride()[:-1])
    )


def _is_backward_graph_task() -> bool:
    return torch._C._current_graph_task_id() >= 0


def _require_gpu_rows(tensor: torch.Tensor, what: str) -> None:
    if tensor.device.type != "cuda":
        raise RuntimeError(
            f"{what} runs on the GPU through libflexshard_hip.so; got a tensor on {tensor.device}. "
            "This package has no CPU compute path."
        )


_getrefcount = sys.getrefcount
_profiler = torch.autograd.profiler
_storage_use_count = torch._C._storage_Use_Count
_raw_stream = torch._C._cuda_getCurrentRawStream

PAYLOAD_RING_SLOTS = 4
GATHER_RING_SLOTS = 3


class _QuantUnshardState:
    """The placement's private state of one prepared unshard."""

    __slots__ = ("infos", "pg", "debug_fqn", "metadata", "copied_out")

    def __init__(self, infos: list, pg: Any, debug_fqn: str | None, metadata: quant_plan.QuantBucketMetadata) -> None:
        self.infos, self.pg, self.debug_fqn, self.metadata = infos, pg, debug_fqn, metadata
        #: the persistent buffers were refilled behind the exchange, in ``run_prepared_unshard``
        self.copied_out = False


# A forward pack that a backward re-gather may take once is remembered as a
# plain tuple (the cheapest object to build on every forward unshard):
#   (signature, versions, stream, metadata, infos, sources, packed)
# signature: address, dtype, shape, strides, negative bit and quantization
# dtype of every shard that holds rows; versions: their version counters at
# pack time; stream: the raw stream the pack was queued on; sources keeps the
# shards' storage alive, so that an equal address still means the same memory;
# infos pins the ParamInfo objects by identity.
_E_SIGNATURE, _E_VERSIONS, _E_STREAM, _E_METADATA, _E_INFOS, _E_SOURCES, _E_PACKED = range(7)


class _BufferRing:
    """A few recycled uint8 buffers of one size, allocated under one stream.

    ``take`` hands out a buffer that nobody else refers to any more: the
    tensor object has no other Python holder and no C++ holder (a collective's
    work object keeps its operands), and its storage is shared by no view or
    alias.  That makes reuse *on the ring's stream* safe under the ownership
    rule of ``PlacementPreparedUnshard.buffers``: the runtime drops its
    references only after every other stream that read a buffer has been
    ordered before the stream that allocated it, which is what the caching
    allocator needs as well.  When every slot is held, the buffer comes from
    the allocator and is not kept, so the ring never holds more than ``slots``
    buffers and a caller that keeps payloads (the backward cache does, one per
    bucket) simply gets fresh ones."""

    __slots__ = ("nbytes", "device", "capacity", "_slots", "_next")

    def __init__(self, nbytes: int, device: torch.device, capacity: int) -> None:
        self.nbytes, self.device, self.capacity = nbytes, device, capacity
        self._slots: list[list] = []
        self._next = 0

    def take(self) -> tuple[torch.Tensor, int]:
        """A free buffer and its device address."""
        # The slot behind the one handed out last: with buffers released in the
        # order they were taken, it is the one released longest ago.
        slots = self._slots
        index = self._next
        if index < len(slots):
            slot = slots[index]
            if _getrefcount(slot[0]) == slot[3] and slot[0]._use_count() == 1 and _storage_use_count(slot[2]) == slot[4]:
                self._next = index + 1 if index + 1 < len(slots) else 0
                return slot[0], slot[1]
        return self._take_any()

    def _take_any(self) -> tuple[torch.Tensor, int]:
        slots = self._slots
        for index, slot in enumerate(slots):
            if _getrefcount(slot[0]) == slot[3] and slot[0]._use_count() == 1 and _storage_use_count(slot[2]) == slot[4]:
                self._next = index + 1 if index + 1 < len(slots) else 0
                return slot[0], slot[1]
        tensor = torch.empty(self.nbytes, dtype=torch.uint8, device=self.device)
        address = tensor.data_ptr()
        if len(slots) < self.capacity:
            storage = tensor.untyped_storage()
            slot = [tensor, address, storage._cdata, 0, 0, storage]
            # the counts of a free slot: what they read now, minus this frame's own reference
            slot[3] = _getrefcount(slot[0]) - 1
            slot[4] = _storage_use_count(slot[2])
            slots.append(slot)
            self._next = 0
        return tensor, address


class _SteadyPack:
    """The stored launch of one rank's quantize + pack for shards that stay
    where they are, with the rings its payloads and gather outputs come from
    (one pair per stream the bucket is prepared on)."""

    __slots__ = (
        "layout", "metadata", "rank", "ntensors", "infos", "live", "signature", "launch", "device", "device_index",
        "cache_key", "payload_nbytes", "gathered_nbytes", "rings", "launch_fn", "launch_handle",
    )

    def __init__(self, *, layout, metadata, rank, ntensors, infos, live, signature, launch, device, world_size) -> None:
        self.layout, self.metadata, self.rank, self.ntensors = layout, metadata, rank, ntensors
        self.infos, self.live, self.signature, self.launch, self.device = infos, live, signature, launch, device
        self.device_index = torch.cuda.current_device() if device.index is None else device.index
        self.cache_key = (rank, id(metadata))
        self.launch_fn, self.launch_handle = launch.raw_launch()
        self.payload_nbytes = metadata.packed_send_nbytes_per_rank
        self.gathered_nbytes = world_size * self.payload_nbytes
        self.rings: dict[int, tuple[_BufferRing, _BufferRing]] = {}

    def rings_for(self, stream: int, shared: dict) -> tuple[_BufferRing, _BufferRing]:
        """This bucket's payload and gather-output rings on ``stream``, taken
        from (or added to) ``shared``, the placement's rings by (device,
        stream, size): buckets of one size, like the layers of a model, share
        them, so the recycled memory does not grow with the number of buckets."""
        if len(self.rings) >= 4:  # a bucket is prepared on one or two streams; do not grow without bound
            self.rings.clear()
        pair = []
        for nbytes, slots in ((self.payload_nbytes, PAYLOAD_RING_SLOTS), (self.gathered_nbytes, GATHER_RING_SLOTS)):
            key = (self.device, stream, nbytes, slots)
            ring = shared.get(key)
            if ring is None:
                ring = shared[key] = _BufferRing(nbytes, self.device, slots)
            pair.append(ring)
        rings = self.rings[stream] = (pair[0], pair[1])
        return rings


class BlockwiseQuantBucketedBlockShard(BucketedBlockShard):
    """Bucketed block shard that all-gathers blockwise-quantized weights.

    Subclasses define the format: ``_chunk_scale_numels``, ``_param_scale_view``,
    ``_make_quantized_weight`` and the device hooks ``_quantize_pack_source_kind``
    / ``_make_quantize_pack_launch``; ``_scale_regions`` may be overridden for scale
    tensors whose per-rank chunks do not concatenate flat.
    """

    qdata_dtype: torch.dtype
    scale_dtype: torch.dtype
    num_scale_tensors: int = 1
    #: refill persistent buffers in ``run_prepared_unshard`` (behind a synchronous
    #: exchange, on its stream) rather than in ``finish_prepared_unshard``
    refill_behind_exchange: bool = True

    _BlockRowParam = quant_plan.BlockRowParam
    _BlockRowUnit = quant_plan.BlockRowUnit
    _QuantChunk = quant_plan.QuantChunk
    _QuantPackChunk = quant_plan.QuantPackChunk
    _QuantRankPackPlan = quant_plan.QuantRankPackPlan
    _QuantBucketMetadata = quant_plan.QuantBucketMetadata

    @dataclass(frozen=True)
    class _QuantMetadataPlan:
        bucket_layout: Any
        metadata: quant_plan.QuantBucketMetadata

    _QuantUnshardState = _QuantUnshardState

    @dataclass(frozen=True)
    class _CopyOutPlan:
        """Payload regions ``(rank, row byte offset, nbytes, out byte offset)``
        of one bucket, with device descriptors keyed by (device, row stride,
        copy unit) in bytes."""

        metadata: quant_plan.QuantBucketMetadata
        regions: tuple[tuple[int, int, int, int], ...]
        vec_aligned: bool
        descriptors: dict

    def __init__(self, *, world_size: int, shard_block_rows: int, qdata_dtype: torch.dtype) -> None:
        if world_size <= 0:
            raise ValueError(f"{type(self).__name__} world_size must be positive, got {world_size}.")
        super().__init__(blocks_per_rank=(1,) * world_size)
        _validate_block_size(shard_block_rows)
        if qdata_dtype.itemsize != 1:
            raise ValueError(f"{type(self).__name__} requires a one-byte qdata_dtype, got {qdata_dtype}.")
        self.qdata_dtype = qdata_dtype
        self.shard_block_rows = shard_block_rows
        self._metadata_plans: dict[int, BlockwiseQuantBucketedBlockShard._QuantMetadataPlan] = {}
        self._local_packed_cache: dict = {}
        self._copy_out_plans: dict = {}
        self._unpack_tables: dict = {}
        self._steady_packs: dict = {}
        self._buffer_rings: dict = {}

    @property
    def world_size(self) -> int:
        return len(self.blocks_per_rank)

    @property
    def _scale_itemsize(self) -> int:
        return self.scale_dtype.itemsize

    # ------------------------------------------------------------ format hooks
    def _chunk_scale_numels(self, rows: int, in_dim: int) -> tuple[int, ...]:
        """Element count of each scale tensor of a chunk starting on a unit edge."""
        raise NotImplementedError

    def _scale_regions(
        self, scale_index: int, rank_pack_plans: tuple[quant_plan.QuantRankPackPlan, ...]
    ) -> tuple[_ScaleRegion, ...]:
        """Regions whose concatenation yields scale tensor ``scale_index`` of
        every parameter in parameter order."""
        return quant_plan.default_scale_regions(scale_index, rank_pack_plans, self._scale_itemsize)

    def _param_scale_view(self, scale_index: int, scale: torch.Tensor, matrix_shape: torch.Size) -> torch.Tensor:
        raise NotImplementedError

    def _make_quantized_weight(
        self, qdata: torch.Tensor, scales: tuple[torch.Tensor, ...], *, orig_dtype: torch.dtype, requires_grad: bool
    ) -> torch.Tensor:
        raise NotImplementedError

    def _quantize_pack_source_kind(self, tensor_dtype: torch.dtype, quant_dtype: torch.dtype) -> int | None:
        """The kernel's source kind for a shard stored in ``tensor_dtype`` and
        quantized as ``quant_dtype``; None when the shard must be cast first."""
        raise NotImplementedError

    def _make_quantize_pack_launch(
        self,
        specs: list[hip_ops.QuantChunkSpec],
        payload_nbytes: int,
        zero_ranges: tuple[tuple[int, int], tuple[int, int]],
        device: torch.device,
    ) -> hip_ops.QuantPackPlan:
        """A reusable launch of the format's fused quantize + pack kernel."""
        raise NotImplementedError

    # ----------------------------------------------------------------- planner
    _can_partition_units = staticmethod(quant_plan.can_partition_units)
    _min_partition_capacity = staticmethod(quant_plan.min_partition_capacity)
    _rank_unit_cuts = staticmethod(quant_plan.rank_unit_cuts)

    def _validate_param_shape(self, fqn: str, shape: Sequence[int]) -> None:
        if len(shape) < 2:
            raise ValueError(
                f"{type(self).__name__} only supports 2D or stacked 2D weights, "
                f"but {fqn!r} has shape {tuple(shape)}."
            )
        if 0 in shape:
            raise ValueError(
                f"{type(self).__name__} requires non-empty weights, but {fqn!r} has shape {tuple(shape)}."
            )

    def _build_block_row_units(self, params: Sequence[quant_plan.BlockRowParam]) -> list[quant_plan.BlockRowUnit]:
        return quant_plan.build_block_row_units(
            params, self.shard_block_rows, self.qdata_dtype.itemsize, self._scale_itemsize, self._chunk_scale_numels
        )

    def _block_row_params_from_named(
        self,
        named_params: list[tuple[str, nn.Parameter]],
        param_placements: dict[str, tuple["Placement", ...]],
    ) -> tuple[list[quant_plan.BlockRowParam], list[quant_plan.BlockRowUnit]]:
        first_fqn, first = named_params[0]
        params = []
        offset = 0
        for fqn, param in named_params:
            if param.dtype != first.dtype:
                raise ValueError(
                    f"{type(self).__name__} requires one dtype per bucket: {first_fqn!r} uses {first.dtype} "
                    f"but {fqn!r} uses {param.dtype}."
                )
            if param_placements[fqn] != (self,):
                raise ValueError(
                    f"{type(self).__name__} requires the same placement instance for every parameter "
                    f"in a bucket; {fqn!r} uses {param_placements[fqn]!r}."
                )
            self._validate_param_shape(fqn, param.shape)
            params.append(quant_plan.BlockRowParam(fqn=fqn, global_shape=param.shape, param_offset=offset))
            offset += param.numel()
        return params, self._build_block_row_units(params)

    def _block_row_params_from_infos(
        self, infos: list["ParamInfo"]
    ) -> tuple[list[quant_plan.BlockRowParam], list[quant_plan.BlockRowUnit]]:
        layout = self._bucket_layout(infos[0])
        params = []
        for info in infos:
            self._validate_param_shape(info.fqn, info.global_shape)
            params.append(
                quant_plan.BlockRowParam(
                    fqn=info.fqn,
                    global_shape=info.global_shape,
                    param_offset=layout.param_layouts[info.fqn].param_offset,
                )
            )
        return params, self._build_block_row_units(params)

    def _build_quant_metadata(
        self,
        params: Sequence[quant_plan.BlockRowParam],
        units: Sequence[quant_plan.BlockRowUnit],
        unit_cuts: Sequence[int],
    ) -> quant_plan.QuantBucketMetadata:
        return quant_plan.build_quant_metadata(
            params,
            units,
            unit_cuts,
            scale_itemsize=self._scale_itemsize,
            num_scale_tensors=self.num_scale_tensors,
            chunk_scale_numels=self._chunk_scale_numels,
            scale_regions=self._scale_regions,
        )

    def _unit_cuts_from_rank_layout(
        self, units: Sequence[quant_plan.BlockRowUnit], rank_offsets: Sequence[int], rank_numels: Sequence[int]
    ) -> tuple[int, ...]:
        return quant_plan.unit_cuts_from_rank_layout(units, rank_offsets, rank_numels)

    def _quant_metadata_from_infos(self, infos: list["ParamInfo"]) -> quant_plan.QuantBucketMetadata:
        layout = self._bucket_layout(infos[0])
        plan = self._metadata_plans.get(id(layout))
        if plan is not None and plan.bucket_layout is layout:
            return plan.metadata
        params, units = self._block_row_params_from_infos(infos)
        cuts = self._unit_cuts_from_rank_layout(units, layout.rank_offsets, layout.rank_numels)
        metadata = self._build_quant_metadata(params, units, cuts)
        self._metadata_plans[id(layout)] = self._QuantMetadataPlan(bucket_layout=layout, metadata=metadata)
        return metadata

    def _chunk_numel(self, chunk: quant_plan.QuantChunk, in_dim: int) -> int:
        return (chunk.row_end - chunk.row_start) * in_dim

    # ---------------------------------------------------- storage / checkpoint
    def bucket_storage_layout(
        self,
        named_params: list[tuple[str, nn.Parameter]],
        param_placements: dict[str, tuple["Placement", ...]],
        mesh: Any,
    ) -> BucketStorageLayout:
        from ..bucket_storage import BucketLayout, BucketParamLayout

        if not named_params:
            return BucketStorageLayout(param_layouts={}, total_bytes=0)
        world_size = mesh.size()
        self._validate_world_size(world_size)
        rank = mesh.get_local_rank()
        dtype = named_params[0][1].dtype
        params, units = self._block_row_params_from_named(named_params, param_placements)
        costs = [u.cost_bytes for u in units]
        cuts = self._rank_unit_cuts(costs, world_size, self._min_partition_capacity(costs, world_size))
        edges = [0]
        for unit in units:
            edges.append(edges[-1] + unit.dense_numel)
        rank_offsets = tuple(edges[c] for c in cuts[:-1])
        rank_numels = tuple(edges[hi] - edges[lo] for lo, hi in zip(cuts[:-1], cuts[1:], strict=True))
        metadata = self._build_quant_metadata(params, units, cuts)
        mine = {chunk.fqn: chunk for chunk in metadata.chunks if chunk.rank == rank}

        bucket_params: dict[str, BucketParamLayout] = {}
        shard_layouts: dict[str, tuple[torch.Size, int, int]] = {}
        for param in params:
            # A local shard is a row range of the flattened matrix; stacked
            # dims stay as size-1 dims so the shard keeps the parameter's rank.
            lead = (1,) * (len(param.global_shape) - 2)
            in_dim = param.global_shape[-1]
            chunk = mine.get(param.fqn)
            if chunk is None:
                shard_layouts[param.fqn] = (torch.Size([*lead, 0, in_dim]), 0, 0)
                local_start = param.param_offset
            else:
                rows = chunk.row_end - chunk.row_start
                shard_layouts[param.fqn] = (
                    torch.Size([*lead, rows, in_dim]),
                    rows * in_dim,
                    chunk.rank_dense_offset * dtype.itemsize,
                )
                local_start = chunk.global_dense_offset
            bucket_params[param.fqn] = BucketParamLayout(param_offset=param.param_offset, local_global_offset=local_start)

        bucket_layout = BucketLayout(
            global_numel=edges[-1],
            local_numel=rank_numels[rank],
            rank_offsets=rank_offsets,
            rank_numels=rank_numels,
            param_layouts=bucket_params,
        )
        self._metadata_plans[id(bucket_layout)] = self._QuantMetadataPlan(bucket_layout=bucket_layout, metadata=metadata)
        return BucketStorageLayout(
            param_layouts={
                fqn: BucketParamStorageLayout(
                    local_shape=shape,
                    local_numel=numel,
                    byte_offset=byte_offset,
                    storage_nbytes=numel * dtype.itemsize,
                    bucket_layout=bucket_layout,
                )
                for fqn, (shape, numel, byte_offset) in shard_layouts.items()
            },
            total_bytes=rank_numels[rank] * dtype.itemsize,
        )

    def global_layout(self, info: "ParamInfo", rank: int, world_size: int) -> GlobalLayout:
        """One box per stacked matrix this rank's row range touches."""
        shape = tuple(info.global_shape)
        if info.local_numel == 0:
            return GlobalLayout(shape, (), (), ())
        *stack, out_dim, in_dim = shape
        layout = self._param_layout(info)
        row_lo = (layout.local_global_offset - layout.param_offset) // in_dim
        row_hi = row_lo + info.local_numel // in_dim
        zeros, ones = (0,) * len(stack), (1,) * len(stack)
        g_off, l_off, sizes = [], [], []
        for matrix in range(row_lo // out_dim, _ceil_div(row_hi, out_dim)):
            base = matrix * out_dim
            lo, hi = max(row_lo, base), min(row_hi, base + out_dim)
            g_off.append((*_unravel_index(matrix, stack), lo - base, 0))
            l_off.append((*zeros, lo - row_lo, 0))
            sizes.append((*ones, hi - lo, in_dim))
        return GlobalLayout(shape, tuple(g_off), tuple(l_off), tuple(sizes))

    # ------------------------------------------------ local quantize + pack
    def _shard_signature(self, tensors: list[torch.Tensor], infos: list["ParamInfo"], live: tuple[int, ...]):
        """What a stored launch and a cached payload depend on besides the
        shards' contents, for the shards that hold rows (``live``): which
        memory each is (address, dtype, shape, strides, negative bit; bf16 and
        fp32 shards have no conjugate bit) and the dtype it is quantized in.
        Also returns the shards' version counters."""
        signature, versions = [], []
        for index in live:
            t = tensors[index]
            info = infos[index]  # param_dtype or dtype: ParamInfo.unsharded_dtype, read without the property call
            signature.append((t.data_ptr(), t.dtype, t.shape, t.stride(), t.is_neg(), info.param_dtype or info.dtype))
            versions.append(t._version)
        return signature, versions

    def _steady_pack_for(
        self, tensors: list[torch.Tensor], infos: list["ParamInfo"], rank: int
    ) -> "tuple[_SteadyPack | None, list | None, list | None]":
        """The stored launch of these very shards, with their signature and
        version counters; (None, None, None) when there is none (first call,
        shards that moved, staged shards)."""
        group = self._steady_packs.get((id(infos[0].bucket_layout), rank))
        if group is None:
            return None, None, None
        live, by_first_address = group
        steady = by_first_address.get(tensors[live[0]].data_ptr() if live else 0)
        if steady is None or steady.layout is not infos[0].bucket_layout or len(tensors) != steady.ntensors:
            return None, None, None
        if live and tensors[live[0]].get_device() != steady.device_index:  # an address means something on one device only
            return None, None, None
        # (the loop of _shard_signature, with the identity check of the infos folded in)
        steady_infos = steady.infos
        signature, versions = [], []
        for index in live:
            info = infos[index]
            if info is not steady_infos[index]:
                return None, None, None
            t = tensors[index]
            signature.append((t.data_ptr(), t.dtype, t.shape, t.stride(), t.is_neg(), info.param_dtype or info.dtype))
            versions.append(t._version)
        if signature != steady.signature:
            return None, None, None
        return steady, signature, versions

    def _build_pack_launch(
        self, tensors: list[torch.Tensor], infos: list["ParamInfo"], rank: int, metadata: quant_plan.QuantBucketMetadata
    ) -> tuple[hip_ops.QuantPackPlan, list[torch.Tensor], torch.device]:
        """Validate the shards against the rank's pack plan and build the
        launch.  Returns it with the staged copies it reads (empty in the
        normal case: every shard is read where it lies) and the device."""
        if len(tensors) != len(infos):
            raise ValueError(
                f"Quantized copy-in requires one tensor per ParamInfo, got {len(tensors)} tensors and {len(infos)} infos."
            )
        plan = metadata.rank_pack_plans[rank]
        device = next((t.device for t in tensors if t.numel() > 0), tensors[0].device)
        if device.type != "cuda":
            raise RuntimeError(
                "Quantized copy-in runs on the GPU through libflexshard_hip.so; got tensors on "
                f"{device}. This package has no CPU compute path."
            )
        specs: list[hip_ops.QuantChunkSpec] = []
        staged: list[torch.Tensor] = []
        qdata_cursor = 0
        scale_cursor = plan.scale_byte_offset
        for chunk in plan.chunks:
            info = infos[chunk.param_index]
            if info.fqn != chunk.fqn:
                raise AssertionError(
                    f"Quantized pack plan parameter order changed: expected {chunk.fqn!r} at index "
                    f"{chunk.param_index}, got {info.fqn!r}."
                )
            source = tensors[chunk.param_index]
            _require_gpu_rows(source, "Quantized copy-in")
            shard = source.reshape(chunk.local_shape)
            if shard.untyped_storage().data_ptr() != source.untyped_storage().data_ptr():
                # The shard could not be viewed as [rows, in_dim] (e.g. a strided
                # slice of a stacked parameter), so reshape made a temporary
                # copy.  Its address must not outlive this call in a stored
                # launch.
                staged.append(shard)
            if shard.numel() != chunk.qdata_numel:
                raise AssertionError(
                    f"Quantized local dense shard does not match planned chunk for {chunk.fqn!r}: "
                    f"expected {chunk.qdata_numel} elements, got {shard.numel()}."
                )
            if len(chunk.scale_numels) != 1:
                raise NotImplementedError("the fused quantize+pack kernel handles one scale tensor per chunk")
            quant_dtype = info.unsharded_dtype
            kind = self._quantize_pack_source_kind(shard.dtype, quant_dtype)
            if kind is None or shard.stride(-1) != 1 or shard.is_neg():
                # Unusual dtype pair, a transposed view or a lazily negated one:
                # stage a contiguous copy in the quantization dtype (the
                # reference stages every non-contiguous or differently typed
                # shard this way).
                shard = shard.to(quant_dtype).contiguous().resolve_neg()
                staged.append(shard)
                kind = self._quantize_pack_source_kind(quant_dtype, quant_dtype)
                if kind is None:
                    raise NotImplementedError(f"{type(self).__name__} cannot quantize {quant_dtype} shards")
            specs.append(hip_ops.QuantChunkSpec(shard, qdata_cursor, scale_cursor, kind))
            qdata_cursor += chunk.qdata_numel
            scale_cursor += chunk.scale_numels[0] * self._scale_itemsize
        if qdata_cursor != plan.qdata_numel or scale_cursor != plan.packed_nbytes:
            raise AssertionError("Quantized pack plan sizes are inconsistent with its chunks.")
        nbytes = metadata.packed_send_nbytes_per_rank
        zero_ranges = ((plan.qdata_numel, plan.scale_byte_offset), (plan.packed_nbytes, nbytes))
        return self._make_quantize_pack_launch(specs, nbytes, zero_ranges, device), staged, device

    def _remember_steady_pack(
        self,
        launch: hip_ops.QuantPackPlan,
        tensors: list[torch.Tensor],
        infos: list["ParamInfo"],
        rank: int,
        metadata: quant_plan.QuantBucketMetadata,
        device: torch.device,
    ) -> "_SteadyPack":
        layout = infos[0].bucket_layout
        live = tuple(chunk.param_index for chunk in metadata.rank_pack_plans[rank].chunks)
        key = (id(layout), rank)
        group = self._steady_packs.get(key)
        if group is None or group[0] != live or len(group[1]) >= 64:
            group = self._steady_packs[key] = (live, {})
        signature, _ = self._shard_signature(tensors, infos, live)
        steady = _SteadyPack(
            layout=layout, metadata=metadata, rank=rank, ntensors=len(tensors), infos=tuple(infos), live=live,
            signature=signature, launch=launch, device=device, world_size=len(metadata.rank_qdata_numels),
        )
        group[1][tensors[live[0]].data_ptr() if live else 0] = steady
        return steady

    def _pack_local_quantized_chunks(
        self,
        tensors: list[torch.Tensor],
        infos: list["ParamInfo"],
        rank: int,
        metadata: quant_plan.QuantBucketMetadata,
    ) -> torch.Tensor:
        """Quantize this rank's dense shards and pack them, in one launch, into
        a fresh payload ``[data | pad | scales | pad]`` of the common row size."""
        if len(tensors) != len(infos):
            raise ValueError(
                f"Quantized copy-in requires one tensor per ParamInfo, got {len(tensors)} tensors and {len(infos)} infos."
            )
        nbytes = metadata.packed_send_nbytes_per_rank
        steady = None
        if tensors and not torch.compiler.is_compiling():
            steady, _, _ = self._steady_pack_for(tensors, infos, rank)
        if steady is not None and steady.metadata is metadata:
            payload = torch.empty(nbytes, dtype=torch.uint8, device=steady.device)
            steady.launch.launch_raw(payload.data_ptr(), _raw_stream(steady.device_index))
            return payload
        launch, staged, device = self._build_pack_launch(tensors, infos, rank, metadata)
        payload = torch.empty(nbytes, dtype=torch.uint8, device=device)
        launch.launch(payload)
        if not staged and not torch.compiler.is_compiling():
            self._remember_steady_pack(launch, tensors, infos, rank, metadata, device)
        # Staged copies were allocated and are consumed on the current stream,
        # so the caching allocator may recycle them as soon as they go out of
        # scope.
        del staged
        return payload

    def _cached_local_quantized_chunks(
        self, tensors: list[torch.Tensor], infos: list["ParamInfo"], rank: int
    ) -> tuple[torch.Tensor, quant_plan.QuantBucketMetadata]:
        """Forward always packs and remembers the payload; a backward re-gather
        may take it back once if nothing about its sources changed.  This is
        the path of a bucket's first unshard, of shards that moved and of
        staged shards; the steady-state branch of ``_prepare_unshard`` serves every later call."""
        if len(tensors) != len(infos):
            raise ValueError(
                f"Quantized copy-in requires one tensor per ParamInfo, got {len(tensors)} tensors and {len(infos)} infos."
            )
        metadata = self._quant_metadata_from_infos(infos)
        if torch.compiler.is_compiling():
            return self._pack_local_quantized_chunks(tensors, infos, rank, metadata), metadata
        live = tuple(chunk.param_index for chunk in metadata.rank_pack_plans[rank].chunks)
        for index in live:
            _require_gpu_rows(tensors[index], "Quantized copy-in")
        device = tensors[live[0]].device if live else tensors[0].device
        stream = hip_ops.stream_ptr(device) if device.type == "cuda" else 0
        signature, versions = self._shard_signature(tensors, infos, live)
        key = (rank, id(metadata))
        if _is_backward_graph_task():
            entry = self._local_packed_cache.pop(key, None)
            if self._cache_entry_matches(entry, metadata, signature, versions, stream, infos):
                return entry[_E_PACKED], metadata
            return self._pack_local_quantized_chunks(tensors, infos, rank, metadata), metadata
        packed = self._pack_local_quantized_chunks(tensors, infos, rank, metadata)
        self._local_packed_cache[key] = (signature, versions, stream, metadata, tuple(infos), tuple(tensors), packed)
        return packed, metadata

    @staticmethod
    def _cache_entry_matches(entry, metadata, signature, versions, stream: int, infos) -> bool:
        """A cached payload may be taken back when it was packed from the same
        memory (signature), unchanged since (version counters), for the same
        bucket and ParamInfo objects, on the stream the consumer is ordered
        after."""
        return (
            entry is not None
            and entry[_E_METADATA] is metadata
            and entry[_E_STREAM] == stream
            and entry[_E_SIGNATURE] == signature
            and entry[_E_VERSIONS] == versions
            and len(entry[_E_INFOS]) == len(infos)
            and all(a is b for a, b in zip(infos, entry[_E_INFOS]))
        )

    def release_buffer_rings(self) -> None:
        """Drop the recycled payload and gather buffers (they are otherwise
        held until the placement goes away)."""
        self._buffer_rings.clear()
        for _, by_first_address in self._steady_packs.values():
            for steady in by_first_address.values():
                steady.rings.clear()

    # -------------------------------------------------------- unshard lifecycle
    def prepare_unshard_bucket(
        self, tensors: list[torch.Tensor], infos: list["ParamInfo"], mesh: Any, debug_fqn: str | None
    ) -> PlacementPreparedUnshard:
        """Quantize + pack the local shards and allocate the gather output."""
        return self._prepare_unshard(tensors, infos, mesh, debug_fqn, True)

    def _prepare_local_unshard_payload(
        self, tensors: list[torch.Tensor], infos: list["ParamInfo"], mesh: Any, debug_fqn: str | None
    ) -> PlacementPreparedUnshard:
        """The same without the gather output (a mixed bucket gathers its
        members' payloads in one buffer of its own)."""
        return self._prepare_unshard(tensors, infos, mesh, debug_fqn, False)

    def _prepare_unshard(
        self, tensors: list[torch.Tensor], infos: list["ParamInfo"], mesh: Any, debug_fqn: str | None, with_gathered: bool
    ) -> PlacementPreparedUnshard:
        rank = mesh.get_local_rank()
        if tensors and len(tensors) == len(infos) and not _profiler._is_profiler_enabled and not torch.compiler.is_compiling():
            # Steady state (every unshard of a bucket after its first): the
            # launch is stored, so this is one pass over the shards that hold
            # rows to see that they are the memory the launch reads, a payload
            # and a gather output from this stream's recycled buffers, and one
            # C call.  Written out in one piece: at a few microseconds per
            # call, every Python call and temporary counts.
            layout = infos[0].bucket_layout
            group = self._steady_packs.get((id(layout), rank))
            if group is not None:
                live, by_first_address = group
                steady = by_first_address.get(tensors[live[0]].data_ptr() if live else 0)
                if (
                    steady is not None
                    and steady.layout is layout
                    and len(tensors) == steady.ntensors
                    # an address means something on one device only (-1: not on a GPU)
                    and (not live or tensors[live[0]].get_device() == steady.device_index)
                ):
                    versions = []
                    for index, want in zip(live, steady.signature):
                        info, t = infos[index], tensors[index]
                        if (
                            info is not steady.infos[index]
                            or t.data_ptr() != want[0]
                            or t.dtype != want[1]
                            or t.shape != want[2]
                            or t.stride() != want[3]
                            or t.is_neg() != want[4]
                            or (info.param_dtype or info.dtype) != want[5]
                        ):
                            break
                        versions.append(t._version)
                    else:
                        signature = steady.signature  # equal to these shards', entry by entry
                        stream = _raw_stream(steady.device_index)
                        rings = steady.rings.get(stream)
                        if rings is None:
                            rings = steady.rings_for(stream, self._buffer_rings)
                        cache = self._local_packed_cache
                        payload = None
                        if _is_backward_graph_task():
                            # a backward re-gather may take the forward's payload back, once
                            entry = cache.pop(steady.cache_key, None)
                            if self._cache_entry_matches(entry, steady.metadata, signature, versions, stream, infos):
                                payload = entry[_E_PACKED]
                            else:
                                payload, address = rings[0].take()
                                steady.launch.launch_raw(address, stream)
                        else:
                            payload, address = rings[0].take()
                            if steady.launch_fn(steady.launch_handle, address, stream) != 0:
                                steady.launch.launch_raw(address, stream)  # raises with the library's message
                            cache[steady.cache_key] = (
                                signature, versions, stream, steady.metadata, tuple(infos), tuple(tensors), payload
                            )
                        return PlacementPreparedUnshard(
                            self,
                            [payload, rings[1].take()[0]] if with_gathered else [payload],
                            _QuantUnshardState(infos, mesh.get_group(), debug_fqn, steady.metadata),
                        )
        with record_copy_in():
            local, metadata = self._cached_local_quantized_chunks(tensors, infos, rank)
        buffers = [local]
        if with_gathered:
            buffers.append(torch.empty(mesh.size() * local.numel(), dtype=local.dtype, device=local.device))
        return PlacementPreparedUnshard(
            placement=self,
            buffers=buffers,
            placement_state=_QuantUnshardState(infos, mesh.get_group(), debug_fqn, metadata),
        )

    def _unshard_state(self, prepared: PlacementPreparedUnshard) -> "_QuantUnshardState":
        state = prepared.placement_state
        if not isinstance(state, BlockwiseQuantBucketedBlockShard._QuantUnshardState):
            raise AssertionError(f"Expected {type(self).__name__}._QuantUnshardState, got {type(state).__name__}")
        return state

    def run_prepared_unshard(self, prepared: PlacementPreparedUnshard, *, async_op: bool = False) -> Any | None:
        """One uint8 all-gather of the equally sized payload rows.  A refill of
        persistent buffers (their storage is allocated before the unshard
        begins: ``refills_persistent_buffers_in_finish`` is False) is written
        here, right behind a synchronous exchange and on its stream, so a
        prefetched bucket arrives unpacked and the consumer stream's finish is
        views only; the gathered rows are then dead when run returns.  A first
        unshard, an asynchronous exchange and a traced graph leave the
        copy-out to finish."""
        state = self._unshard_state(prepared)
        local, gathered = prepared.buffers
        with record_comm("FlexShard::all_gather", state.debug_fqn):
            work = all_gather_rows(gathered, local, state.pg, async_op=async_op)
        if (
            self.refill_behind_exchange
            and work is None
            and prepared.persistent_buffers is not None
            and not torch.compiler.is_compiling()
        ):
            rows = gathered.view(len(state.metadata.rank_qdata_numels), local.numel())
            self._check_rank_rows(state, rows)
            with record_copy_out():
                state.copied_out = self._copy_out_rank_rows_fused(state.metadata, rows, prepared.persistent_buffers[0])
        return work

    def finish_prepared_unshard(self, prepared: PlacementPreparedUnshard) -> PlacementUnshardResult:
        state = self._unshard_state(prepared)
        rows = prepared.buffers[1].view(len(state.metadata.rank_qdata_numels), prepared.buffers[0].numel())
        return self._finish_unshard_from_rank_rows(prepared, rows)

    def _check_rank_rows(self, state: "_QuantUnshardState", rank_rows: torch.Tensor) -> None:
        expected = (len(state.metadata.rank_qdata_numels), state.metadata.packed_send_nbytes_per_rank)
        if tuple(rank_rows.shape) != expected:
            raise ValueError(f"Expected gathered rank rows with shape {expected}, got {tuple(rank_rows.shape)}.")
        if rank_rows.dtype != torch.uint8:
            raise ValueError(f"Packed quantized gathered rank rows must use uint8 transport, got {rank_rows.dtype}.")

    def _finish_unshard_from_rank_rows(
        self, prepared: PlacementPreparedUnshard, rank_rows: torch.Tensor
    ) -> PlacementUnshardResult:
        """Unpack from rank-major rows (possibly strided, at odd byte offsets)."""
        state = self._unshard_state(prepared)
        self._check_rank_rows(state, rank_rows)
        return self._finish_quant_unshard_from_rank_rows(prepared, rank_rows, state)

    def _compact_sizes(self, metadata: quant_plan.QuantBucketMetadata) -> tuple[int, int, list[int]]:
        """(data bytes, aligned scale start, bytes of each scale tensor group)."""
        data = sum(metadata.rank_qdata_numels)
        groups = [sum(r.nbytes for r in regions) for regions in metadata.scale_regions_by_index]
        return data, _align_up(data, _VEC_ALIGN_BYTES), groups

    def _compact_buffer(
        self, prepared: PlacementPreparedUnshard, metadata: quant_plan.QuantBucketMetadata, device: torch.device
    ) -> torch.Tensor:
        if prepared.persistent_buffers is not None:
            return prepared.persistent_buffers[0]
        _, scale_start, groups = self._compact_sizes(metadata)
        return torch.empty(scale_start + sum(groups), dtype=torch.uint8, device=device)

    def _full_params_from_compact(self, state: "_QuantUnshardState", compact: torch.Tensor) -> list[torch.Tensor]:
        """Per-parameter views of the compact buffer handed to the weight factory."""
        data_nbytes, scale_start, groups = self._compact_sizes(state.metadata)
        qdata_flat = compact[:data_nbytes].view(self.qdata_dtype)
        flat_scales = [g.view(self.scale_dtype) for g in torch.split(compact[scale_start:], groups)]
        shapes = [_matrix_shape(info.global_shape) for info in state.infos]
        per_param_counts = [self._chunk_scale_numels(*shape) for shape in shapes]
        # torch.split raises unless the parameters tile each buffer exactly.
        qdata_params = torch.split(qdata_flat, [info.global_numel for info in state.infos])
        scales_by_index = [
            torch.split(flat, [counts[k] for counts in per_param_counts]) for k, flat in enumerate(flat_scales)
        ]
        full = []
        for p, (info, qdata, shape) in enumerate(zip(state.infos, qdata_params, shapes, strict=True)):
            scales = tuple(self._param_scale_view(k, per_param[p], shape) for k, per_param in enumerate(scales_by_index))
            full.append(
                self._make_quantized_weight_checked(
                    qdata.view(info.global_shape), scales, orig_dtype=info.unsharded_dtype, requires_grad=info.requires_grad
                )
            )
        return full

    def _finish_quant_unshard_from_rank_rows(
        self, prepared: PlacementPreparedUnshard, rank_rows: torch.Tensor, state: "_QuantUnshardState"
    ) -> PlacementUnshardResult:
        compact = self._compact_buffer(prepared, state.metadata, rank_rows.device)
        if state.copied_out and prepared.persistent_buffers is not None:
            return PlacementUnshardResult(
                full_params=self._full_params_from_compact(state, compact), persistent_buffers=[compact]
            )
        with record_copy_out():
            # Rank cuts partition one globally ordered stream of block rows, so
            # joining each rank's valid region restores parameter order.
            if not self._copy_out_rank_rows_fused(state.metadata, rank_rows, compact):
                data_nbytes, scale_start, _ = self._compact_sizes(state.metadata)
                self._copy_out_rank_rows_cat(
                    state.metadata, rank_rows, compact, qdata_nbytes=data_nbytes, scale_byte_offset=scale_start
                )
        return PlacementUnshardResult(
            full_params=self._full_params_from_compact(state, compact),
            persistent_buffers=[compact] if prepared.persistent else [],
        )

    def _copy_out_plan(
        self, metadata: quant_plan.QuantBucketMetadata, *, data_elem_nbytes: int, with_scales: bool
    ) -> "_CopyOutPlan":
        key = (id(metadata), data_elem_nbytes, with_scales)
        plan = self._copy_out_plans.get(key)
        if plan is not None and plan.metadata is metadata:
            return plan
        regions: list[tuple[int, int, int, int]] = []
        cursor = 0
        for rank, numel in enumerate(metadata.rank_qdata_numels):
            regions.append((rank, 0, numel * data_elem_nbytes, cursor))
            cursor += numel * data_elem_nbytes
        if with_scales:
            cursor = _align_up(cursor, _VEC_ALIGN_BYTES)
            for group in metadata.scale_regions_by_index:
                for region in group:
                    regions.append((region.rank, region.offset, region.nbytes, cursor))
                    cursor += region.nbytes
        live = tuple(r for r in regions if r[2] > 0)
        plan = BlockwiseQuantBucketedBlockShard._CopyOutPlan(
            metadata=metadata,
            regions=live,
            vec_aligned=all(v % _VEC_COPY_NBYTES == 0 for r in live for v in r[1:]),
            descriptors={},
        )
        self._copy_out_plans[key] = plan
        return plan

    def _copy_out_rank_rows_fused(
        self,
        metadata: quant_plan.QuantBucketMetadata,
        rank_rows: torch.Tensor,
        out: torch.Tensor,
        *,
        data_elem_nbytes: int = 1,
        with_scales: bool = True,
    ) -> bool:
        """Join every rank's payload regions into ``out`` with one HIP launch.
        ``rank_rows`` and ``out`` are uint8; data regions land in rank order,
        the scale regions follow from the 16-byte aligned offset.  Returns
        False only while compiling (the caller then uses ``torch.cat``)."""
        if torch.compiler.is_compiling():
            return False
        _require_gpu_rows(rank_rows, "The rank-row copy-out")
        plan = self._copy_out_plan(metadata, data_elem_nbytes=data_elem_nbytes, with_scales=with_scales)
        row_stride = rank_rows.stride(0) if rank_rows.size(0) > 1 else rank_rows.size(1)
        # The physical rows including any padding between them: plan offsets
        # count from the first row's first byte.
        source = rank_rows.as_strided(((rank_rows.size(0) - 1) * row_stride + rank_rows.size(1),), (1,))
        if plan.vec_aligned and _is_vec_copy_viewable(rank_rows) and _is_vec_copy_viewable(out):
            source = source.view(_VEC_COPY_DTYPE)
            out = out.view(_VEC_COPY_DTYPE)
        unit = source.element_size()
        key = (rank_rows.device, row_stride, unit)
        descriptor = plan.descriptors.get(key)
        if descriptor is None:
            descriptor = SegmentCopyDescriptor.create(
                src_offsets=[(rank * row_stride + offset) // unit for rank, offset, _, _ in plan.regions],
                numels=[nbytes // unit for _, _, nbytes, _ in plan.regions],
                dst_offsets=[dst // unit for _, _, _, dst in plan.regions],
                device=rank_rows.device,
            )
            plan.descriptors[key] = descriptor
        copy_segments(source, out, descriptor)
        return True

    def _copy_out_rank_rows_cat(
        self,
        metadata: quant_plan.QuantBucketMetadata,
        rank_rows: torch.Tensor,
        compact: torch.Tensor,
        *,
        qdata_nbytes: int,
        scale_byte_offset: int,
    ) -> None:
        """``torch.cat`` form of the copy-out, used only under ``torch.compile``
        (a traced graph cannot call the HIP library)."""
        data = [rank_rows[rank, :numel] for rank, numel in enumerate(metadata.rank_qdata_numels) if numel]
        scales = [
            rank_rows[region.rank, region.offset : region.offset + region.nbytes]
            for group in metadata.scale_regions_by_index
            for region in group
            if region.nbytes
        ]
        if data:
            torch.cat(data, out=compact[:qdata_nbytes])
        if scales:
            torch.cat(scales, out=compact[scale_byte_offset:])

    def _make_quantized_weight_checked(
        self, qdata: torch.Tensor, scales: tuple[torch.Tensor, ...], *, orig_dtype: torch.dtype, requires_grad: bool
    ) -> torch.Tensor:
        weight = self._make_quantized_weight(qdata, scales, orig_dtype=orig_dtype, requires_grad=requires_grad)
        if not isinstance(weight, torch.Tensor):
            raise TypeError(f"_make_quantized_weight must return a torch.Tensor, got {type(weight).__name__}.")
        return weight


_merge_adjacent_regions = quant_plan.merge_adjacent_regions

__all__ = ["BlockwiseQuantBucketedBlockShard"]
