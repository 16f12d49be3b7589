"""One exchange for a bucket that mixes small dense parameters with a
blockwise-quantized member.

Mirror of the reference's ``custom_placements/mixed_bucket.py`` for the two
member kinds that sit on the FP8 hot path: ``shard0`` (``Shard(0)``: norms and
biases, gathered in their own dtype) and the blockwise-quantized member
(:304-334, the optimizer-visible ``Fp8BucketedBlockShard``).  Every member
group prepares its own send buffer; the mixed bucket lays the groups out in
one rank row (:1407-1474, ``_plan_group_offsets`` :1603-1657: quantized
payloads on 16-byte boundaries, bytes when the groups' dtypes differ), gathers
the rows in one exchange (:663-684) and hands each group its columns of the
gathered rows: the quantized member unpacks straight from those strided rank
rows (:722-732), a dense member from a contiguous copy.  Gradients mirror it
(:1094-1366): one ``[world, row]`` reduce-scatter input in which the quantized
member's gradients are packed in one pass into wider rows, one reduction, and
per-group views of the result.

Not built: ``BlockShard`` / ``BucketedOwned`` members and the owner-rows
transports that go with them (:108-170, :781-1092); their factories raise.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import TYPE_CHECKING, Any

import torch
import torch.nn as nn

from ..placement_contract import (
    BucketParamStorageLayout,
    BucketStorageLayout,
    Placement,
    PlacementPreparedReduceGrad,
    PlacementPreparedUnshard,
    PlacementReduceGradResult,
    PlacementUnshardResult,
)
from ..profiling import record_comm, record_copy_in, record_copy_out, record_range
from .block_shard import BucketedBlockShard, _grad_reduce_dtype
from .blockwise_quant_bucketed_block_shard import BlockwiseQuantBucketedBlockShard
from .fp8_bucketed_block_shard import Fp8BucketedBlockShard
from .quant_plan import VEC_ALIGN_BYTES, align_up
from .shard import Shard
from .utils import all_gather_rows, reduce_scatter_grads

if TYPE_CHECKING:
    from ..bucket_storage import ParamInfo
    from ..placement_contract import GradientReduction


@dataclass(frozen=True)
class _PlacementGroup:
    placement: Placement
    key: object
    indices: list[int]
    tensors: list[torch.Tensor]
    infos: list["ParamInfo"]


@dataclass(frozen=True)
class _MixedUnshardGroupState:
    prepared: PlacementPreparedUnshard
    indices: tuple[int, ...]
    offset: int
    numel: int


@dataclass(frozen=True)
class _MixedUnshardState:
    groups: list[_MixedUnshardGroupState]
    world_size: int
    row_numel: int
    requires_dtype_reinterpretation: bool
    pg: Any
    debug_fqn: str | None


@dataclass(frozen=True)
class _MixedReduceGradGroupState:
    prepared: PlacementPreparedReduceGrad
    indices: list[int]
    offset: int
    numel: int


@dataclass(frozen=True)
class _MixedReduceGradState:
    groups: list[_MixedReduceGradGroupState]
    world_size: int
    row_numel: int
    pg: Any
    debug_fqn: str | None


class _MixedBucketMember:
    """What the optimizer and the bucket runtime see per parameter: a member
    equal to its collective placement whose bucket hooks are the mixed
    bucket's."""

    _mixed_bucket: "MixedBucketPlacement"
    _collective_placement: Placement

    def __eq__(self, other: object) -> bool:
        if isinstance(other, _MixedBucketMember):
            other = other._collective_placement
        return self._collective_placement == other

    def __hash__(self) -> int:
        return hash(self._collective_placement)

    def bucket_compatibility_key(self) -> object:
        return self._mixed_bucket

    def bucket_storage_layout(self, named_params, param_placements, mesh):
        return self._mixed_bucket.bucket_storage_layout(named_params, param_placements, mesh)

    def prepare_unshard_bucket(self, tensors, infos, mesh, debug_fqn):
        return self._mixed_bucket.prepare_unshard_bucket(tensors, infos, mesh, debug_fqn)

    def run_prepared_unshard(self, prepared, *, async_op: bool = False):
        return self._mixed_bucket.run_prepared_unshard(prepared, async_op=async_op)

    def finish_prepared_unshard(self, prepared):
        return self._mixed_bucket.finish_prepared_unshard(prepared)

    def prepare_reduce_grad(self, tensors, infos, mesh, debug_fqn):
        return self._mixed_bucket.prepare_reduce_grad(tensors, infos, mesh, debug_fqn)

    def reduce_prepared_grad(self, prepared, reduction):
        return self._mixed_bucket.reduce_prepared_grad(prepared, reduction)


class _MixedShard0(_MixedBucketMember, Shard):
    __eq__ = _MixedBucketMember.__eq__
    __hash__ = _MixedBucketMember.__hash__

    def __init__(self, mixed_bucket: "MixedBucketPlacement") -> None:
        Shard.__init__(self, 0)
        self._mixed_bucket = mixed_bucket
        self._collective_placement = mixed_bucket._shard


class _MixedFp8BucketedBlockShard(_MixedBucketMember, Fp8BucketedBlockShard):
    """Optimizer-visible blockwise FP8 member of one mixed bucket placement."""

    __eq__ = _MixedBucketMember.__eq__
    __hash__ = _MixedBucketMember.__hash__

    def __init__(self, mixed_bucket: "MixedBucketPlacement", placement: Fp8BucketedBlockShard) -> None:
        Fp8BucketedBlockShard.__init__(
            self, world_size=placement.world_size, weight_factory=placement.weight_factory,
            block_size=placement.block_size, fp8_dtype=placement.qdata_dtype,
        )
        self._mixed_bucket = mixed_bucket
        self._collective_placement = placement


def _collective_placement(placement: Placement) -> Placement:
    return placement._collective_placement if isinstance(placement, _MixedBucketMember) else placement


def _group_tensors_by_placement(tensors, infos, key_fn=None) -> list[_PlacementGroup]:
    groups: list[_PlacementGroup] = []
    for index, (tensor, info) in enumerate(zip(tensors, infos, strict=True)):
        placement = _collective_placement(info.placement)
        # Quantized pack plans span the whole member and index infos by
        # position, and quantization reads each param in its own dtype, so a
        # quantized member is never split.
        key = None if key_fn is None or isinstance(placement, BlockwiseQuantBucketedBlockShard) else key_fn(info)
        for group in groups:
            if placement == group.placement and key == group.key:
                group.indices.append(index)
                group.tensors.append(tensor)
                group.infos.append(info)
                break
        else:
            groups.append(_PlacementGroup(placement, key, [index], [tensor], [info]))
    return groups


def _plan_group_offsets(group_numels: list[int], group_alignments: list[int], row_alignment: int) -> tuple[list[int], int]:
    """Offsets of the groups in a rank row, each on its alignment, and the row
    length rounded up to ``row_alignment``."""
    offsets, cursor = [], 0
    for numel, alignment in zip(group_numels, group_alignments, strict=True):
        cursor = align_up(cursor, alignment)
        offsets.append(cursor)
        cursor += numel
    return offsets, align_up(cursor, row_alignment)


def _num_persistent_buffers(placement: Placement, num_params: int) -> int:
    # A quantized group backs all its params with one compact buffer; a Shard
    # group backs each param with its own buffer.
    return 1 if isinstance(placement, BlockwiseQuantBucketedBlockShard) else num_params


class MixedBucketPlacement(Placement):
    """One exchange for the member groups of a mixed bucket."""

    # Shard members write a refill's persistent buffers in finish.
    refills_persistent_buffers_in_finish = True

    def __init__(self, segments_by_fqn: dict[str, list[Any]] | None = None) -> None:
        if segments_by_fqn:
            raise NotImplementedError("BucketedOwned members of a mixed bucket are not built")
        self._shard = Shard(0)
        self.shard0 = _MixedShard0(self)
        self._blockwise_quant_member: _MixedFp8BucketedBlockShard | None = None

    def block_shard(self, **kwargs):
        raise NotImplementedError("BlockShard members of a mixed bucket are not built")

    def blockwise_quant_bucketed_block_shard(self, placement: BlockwiseQuantBucketedBlockShard):
        member = self._blockwise_quant_member
        if member is None:
            if type(placement) is not Fp8BucketedBlockShard:
                raise TypeError(
                    f"Mixed FlexShard buckets do not support blockwise quantized placement {type(placement).__name__}."
                )
            member = _MixedFp8BucketedBlockShard(self, placement)
            self._blockwise_quant_member = member
        elif member._collective_placement is not placement:
            raise NotImplementedError("A mixed bucket supports one blockwise quantized placement instance.")
        return member

    def __eq__(self, other: object) -> bool:
        return self is other

    def __hash__(self) -> int:
        return hash(id(self))

    def compute_local_shape(self, global_shape, rank, world_size):
        raise NotImplementedError("Mixed bucket placement is bucket-scoped.")

    def extract_local_shard(self, param, rank, world_size):
        raise NotImplementedError("Mixed bucket placement is bucket-scoped.")

    # ------------------------------------------------------------------ layout
    def bucket_storage_layout(
        self,
        named_params: list[tuple[str, nn.Parameter]],
        param_placements: dict[str, tuple[Placement, ...]],
        mesh: Any,
    ) -> BucketStorageLayout:
        """The member groups' own bucket layouts back to back in the local
        storage, in the order the groups first appear."""
        groups: list[list[tuple[str, nn.Parameter, Placement]]] = []
        for fqn, param in named_params:
            (placement,) = param_placements[fqn]
            if not isinstance(placement, _MixedBucketMember):
                raise TypeError(
                    f"MixedBucketPlacement requires mixed member placements, but {fqn!r} uses {type(placement).__name__}."
                )
            if placement._mixed_bucket is not self:
                raise ValueError("MixedBucketPlacement cannot mix member placements from different bucket instances.")
            collective = placement._collective_placement
            for group in groups:
                if group[0][2] == collective:
                    group.append((fqn, param, collective))
                    break
            else:
                groups.append([(fqn, param, collective)])
        layouts: dict[str, BucketParamStorageLayout] = {}
        byte_offset = 0
        for group in groups:
            collective = group[0][2]
            named = [(fqn, param) for fqn, param, _ in group]
            layout = collective.bucket_storage_layout(named, {fqn: (collective,) for fqn, _ in named}, mesh)
            for fqn, p in layout.param_layouts.items():
                layouts[fqn] = BucketParamStorageLayout(
                    local_shape=p.local_shape, local_numel=p.local_numel, byte_offset=byte_offset + p.byte_offset,
                    storage_nbytes=p.storage_nbytes, bucket_layout=p.bucket_layout,
                )
            byte_offset += layout.total_bytes
        return BucketStorageLayout(param_layouts=layouts, total_bytes=byte_offset)

    # ----------------------------------------------------------------- unshard
    def prepare_unshard_bucket(
        self, tensors: list[torch.Tensor], infos: list["ParamInfo"], mesh: Any, debug_fqn: str | None
    ) -> PlacementPreparedUnshard:
        world_size = mesh.size()
        groups = _group_tensors_by_placement(tensors, infos, lambda info: info.unsharded_dtype)
        prepared_groups: list[tuple[PlacementPreparedUnshard, tuple[int, ...]]] = []
        group_buffers: list[torch.Tensor] = []
        with record_copy_in():
            for group in groups:
                if isinstance(group.placement, BlockwiseQuantBucketedBlockShard):
                    prepared = group.placement._prepare_local_unshard_payload(group.tensors, group.infos, mesh, debug_fqn)
                elif isinstance(group.placement, Shard):
                    # The mixed exchange fills the group's gather buffer, also
                    # on a 1-rank mesh where Shard alone skips its all-gather.
                    prepared = group.placement._prepare_unshard_bucket(
                        group.tensors, group.infos, mesh, debug_fqn, skip_single_rank_all_gather=False
                    )
                else:
                    raise TypeError(f"Mixed FlexShard unshard does not support {type(group.placement).__name__}.")
                prepared_groups.append((prepared, tuple(group.indices)))
                group_buffers.extend(prepared.buffers)
            sends = [prepared.buffers[0] for prepared, _ in prepared_groups]
            device = sends[0].device
            if any(send.device != device for send in sends):
                raise ValueError("Mixed FlexShard unshard requires one device per bucket.")
            reinterpret = len({send.dtype for send in sends}) > 1
            dtype = torch.uint8 if reinterpret else sends[0].dtype
            numels = [send.numel() * send.element_size() if reinterpret else send.numel() for send in sends]
            quant_transport = [
                isinstance(prepared.placement, BlockwiseQuantBucketedBlockShard) and prepared.buffers[0].dtype == torch.uint8
                for prepared, _ in prepared_groups
            ]
            alignments = [VEC_ALIGN_BYTES if quant else 1 for quant in quant_transport]
            offsets, row_numel = _plan_group_offsets(numels, alignments, VEC_ALIGN_BYTES if any(quant_transport) else 1)
            group_states = [
                _MixedUnshardGroupState(prepared=prepared, indices=indices, offset=offset, numel=numel)
                for (prepared, indices), offset, numel in zip(prepared_groups, offsets, numels, strict=True)
            ]
            send = torch.empty(row_numel, dtype=dtype, device=device)
            cursor = 0
            for state in group_states:  # the gaps in front of aligned groups and the row's tail
                if cursor < state.offset:
                    send[cursor : state.offset].zero_()
                cursor = state.offset + state.numel
            if cursor < row_numel:
                send[cursor:].zero_()
            for state in group_states:
                group_send = state.prepared.buffers[0]
                send.narrow(0, state.offset, state.numel).copy_(
                    group_send.contiguous().view(torch.uint8).reshape(-1) if reinterpret else group_send
                )
            gathered = torch.empty(world_size * row_numel, dtype=dtype, device=device)
        return PlacementPreparedUnshard(
            placement=self,
            buffers=[send, gathered, *group_buffers],
            placement_state=_MixedUnshardState(
                groups=group_states, world_size=world_size, row_numel=row_numel,
                requires_dtype_reinterpretation=reinterpret, pg=mesh.get_group(), debug_fqn=debug_fqn,
            ),
        )

    @staticmethod
    def _unshard_state(prepared: PlacementPreparedUnshard) -> _MixedUnshardState:
        state = prepared.placement_state
        if not isinstance(state, _MixedUnshardState):
            raise AssertionError(f"Expected _MixedUnshardState, got {type(state).__name__}")
        return state

    def run_prepared_unshard(self, prepared: PlacementPreparedUnshard, *, async_op: bool = False) -> Any | None:
        state = self._unshard_state(prepared)
        with record_comm("FlexShard::mixed_all_gather", state.debug_fqn):
            return all_gather_rows(prepared.buffers[1], prepared.buffers[0], state.pg, async_op=async_op)

    def finish_prepared_unshard(self, prepared: PlacementPreparedUnshard) -> PlacementUnshardResult:
        state = self._unshard_state(prepared)
        refill = prepared.persistent_buffers is not None  # a refill returns no full params
        gathered_by_rank = prepared.buffers[1].view(state.world_size, state.row_numel)
        full_params: list[torch.Tensor | None] = [None] * sum(len(group.indices) for group in state.groups)
        buffers: list[torch.Tensor] = []
        persistent_buffers: list[torch.Tensor] = []
        buffer_offset = 0
        with record_copy_out():
            for group in state.groups:
                placement = group.prepared.placement
                count = _num_persistent_buffers(placement, len(group.indices))
                group_persistent = (
                    prepared.persistent_buffers[buffer_offset : buffer_offset + count] if refill else None
                )
                buffer_offset += count
                columns = gathered_by_rank[:, group.offset : group.offset + group.numel]
                if isinstance(placement, BlockwiseQuantBucketedBlockShard):
                    # unpacked straight from the strided rank rows
                    gathered = columns
                    group.prepared.persistent = prepared.persistent
                    group.prepared.persistent_buffers = group_persistent
                    result = placement._finish_unshard_from_rank_rows(group.prepared, gathered)
                else:
                    if state.requires_dtype_reinterpretation:
                        gathered = group.prepared.buffers[1]
                        gathered.view(torch.uint8).view_as(columns).copy_(columns)
                    else:
                        gathered = columns.contiguous().view(-1)
                    group_prepared = PlacementPreparedUnshard(
                        placement=placement,
                        buffers=[group.prepared.buffers[0], gathered, *group.prepared.buffers[2:]],
                        placement_state=group.prepared.placement_state,
                        persistent=prepared.persistent,
                        persistent_buffers=group_persistent,
                    )
                    result = placement.finish_prepared_unshard(group_prepared)
                buffers.append(gathered)
                if not refill:
                    for index, full_param in zip(group.indices, result.full_params, strict=True):
                        full_params[index] = full_param
                buffers.extend(result.buffers)
                persistent_buffers.extend(result.persistent_buffers)
        if refill:
            return PlacementUnshardResult(full_params=[], buffers=buffers, persistent_buffers=persistent_buffers)
        if any(full_param is None for full_param in full_params):
            raise AssertionError("Mixed unshard did not produce every param.")
        return PlacementUnshardResult(full_params=full_params, buffers=buffers, persistent_buffers=persistent_buffers)

    # --------------------------------------------------------------- gradients
    def prepare_reduce_grad(
        self, tensors: list[torch.Tensor], infos: list["ParamInfo"], mesh: Any, debug_fqn: str | None
    ) -> PlacementPreparedReduceGrad:
        world_size = mesh.size()
        groups = _group_tensors_by_placement(tensors, infos)
        prepared_groups: list[tuple[PlacementPreparedReduceGrad, list[int], int]] = []
        group_buffers: list[torch.Tensor] = []
        dtype: torch.dtype | None = None
        device: torch.device | None = None
        with record_range("FlexShard::mixed_reduce_scatter_copy_in", debug_fqn):
            for group in groups:
                reduce_dtype = _grad_reduce_dtype(group.infos[0])
                if isinstance(
                    group.placement, BlockwiseQuantBucketedBlockShard
                ) and group.placement._packs_reduce_scatter_grad_in_one_pass(group.tensors, reduce_dtype):
                    # The grads are packed straight into the bucket's send
                    # buffer below, in one pass, rather than into a world-size
                    # buffer of the group's own first.
                    group_numel = max(group.placement._bucket_layout(group.infos[0]).rank_numels)
                    prepared = PlacementPreparedReduceGrad(
                        placement=group.placement,
                        buffers=[],
                        placement_state=BucketedBlockShard._ReduceGradState(
                            infos=group.infos, rank=mesh.get_local_rank(), pg=mesh.get_group(), debug_fqn=debug_fqn,
                            padded_segment_numel=group_numel,
                        ),
                    )
                    group_dtype, group_device = reduce_dtype, group.tensors[0].device
                else:
                    prepared = group.placement.prepare_reduce_grad(group.tensors, group.infos, mesh, debug_fqn)
                    send = prepared.buffers[0]
                    if send.numel() % world_size:
                        raise AssertionError(
                            f"Mixed reduce-scatter subgroup send size must be divisible by world size {world_size}, "
                            f"got {send.numel()}."
                        )
                    group_numel, group_dtype, group_device = send.numel() // world_size, send.dtype, send.device
                if dtype is None:
                    dtype, device = group_dtype, group_device
                elif (group_dtype, group_device) != (dtype, device):
                    raise ValueError(
                        "Mixed FlexShard reduce-grad requires one send dtype and device per bucket, but got "
                        f"{dtype}/{device} and {group_dtype}/{group_device}."
                    )
                prepared_groups.append((prepared, group.indices, group_numel))
                group_buffers.extend(prepared.buffers)
            offsets, row_numel = _plan_group_offsets(
                [numel for _, _, numel in prepared_groups], [1] * len(prepared_groups), 1
            )
            group_states = [
                _MixedReduceGradGroupState(prepared=prepared, indices=indices, offset=offset, numel=numel)
                for (prepared, indices, numel), offset in zip(prepared_groups, offsets, strict=True)
            ]
            send = torch.empty(world_size * row_numel, dtype=dtype, device=device)
            send_rows = send.view(world_size, row_numel)
            for group, state in zip(groups, group_states, strict=True):
                columns = send_rows[:, state.offset : state.offset + state.numel]
                if not state.prepared.buffers:
                    group_buffers.extend(
                        group.placement._pack_reduce_scatter_grad(group.tensors, group.infos, world_size, columns)
                    )
                else:
                    columns.copy_(state.prepared.buffers[0].view(world_size, state.numel))
        return PlacementPreparedReduceGrad(
            placement=self,
            buffers=[send, *group_buffers],
            placement_state=_MixedReduceGradState(
                groups=group_states, world_size=world_size, row_numel=row_numel, pg=mesh.get_group(),
                debug_fqn=debug_fqn,
            ),
        )

    def reduce_prepared_grad(
        self, prepared: PlacementPreparedReduceGrad, reduction: "GradientReduction"
    ) -> PlacementReduceGradResult:
        state = prepared.placement_state
        if not isinstance(state, _MixedReduceGradState):
            raise AssertionError(f"Expected _MixedReduceGradState, got {type(state).__name__}")
        send = prepared.buffers[0]
        recv = torch.empty(state.row_numel, dtype=send.dtype, device=send.device)
        with record_comm("FlexShard::mixed_reduce_scatter", state.debug_fqn):
            reduce_scatter_grads(recv, send, reduction, state.pg)
        sharded: list[torch.Tensor | None] = [None] * sum(len(group.indices) for group in state.groups)
        with record_range("FlexShard::mixed_reduce_scatter_copy_out", state.debug_fqn):
            for group in state.groups:
                group_recv = recv.narrow(0, group.offset, group.numel)
                for index, grad in zip(group.indices, _finish_mixed_reduce_group(group.prepared, group_recv), strict=True):
                    sharded[index] = grad
        if any(grad is None for grad in sharded):
            raise AssertionError("Mixed reduce-grad did not produce every grad.")
        return PlacementReduceGradResult(sharded, [recv])


def _finish_mixed_reduce_group(prepared: PlacementPreparedReduceGrad, recv: torch.Tensor) -> list[torch.Tensor]:
    placement, state = prepared.placement, prepared.placement_state
    if isinstance(placement, Shard):
        return placement._unpack_reduce_scatter_grad(recv, state)
    if isinstance(placement, BlockwiseQuantBucketedBlockShard):
        rank_offset = placement._bucket_layout(state.infos[0]).rank_offsets[state.rank]
        shards = []
        for info in state.infos:
            start = placement._param_layout(info).local_global_offset - rank_offset
            shards.append(recv[start : start + info.local_numel].view(info.local_shape))
        return shards
    raise TypeError(
        "Mixed FlexShard reduce-grad supports only Shard(0) and blockwise quantized placements, "
        f"but got {type(placement).__name__}."
    )


__all__ = ["MixedBucketPlacement"]
