"""``Shard(0)``: a parameter split in equal row chunks over the ranks.

Mirror of the reference's ``custom_placements/shard.py`` for the dim-0 case,
which is what a mixed bucket uses for the small dense parameters (norms,
biases) that travel next to its FP8 payload: ``compute_local_shape`` /
``extract_local_shard`` (:118-143), ``global_layout`` (:145-160), the padded
per-parameter storage of ``bucket_storage_layout`` (:162-195), the all-gather
unshard with persistent refills in finish (:217-428) and the reduce-scatter
gradient path (:430-572).  The reference copies between parameter layouts and
collective buffers with ``torch.ops.fsdp`` kernels of a newer PyTorch; the
parameters here are small, so strided tensor copies do it.  ``Shard(i)`` for
``i > 0`` is not built and raises.
"""

from __future__ import annotations

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
from ..profiling import record_comm, record_copy_in, record_copy_out, record_range
from .utils import all_gather_rows, foreach_copy_, reduce_grads_on_one_rank, reduce_scatter_grads

if TYPE_CHECKING:
    from ..bucket_storage import ParamInfo
    from ..placement_contract import GradientReduction


class Shard(Placement):
    """Symmetric sharding: dim 0 split in ``ceil(rows / world)`` chunks, the
    last ranks' chunks short or empty; storage reserves rank 0's chunk on every
    rank so that the all-gather rows are equal."""

    # Finish copies the gathered values into a refill's persistent buffers;
    # run gathers into a separate buffer.
    refills_persistent_buffers_in_finish = True

    @dataclass(frozen=True)
    class _UnshardState:
        infos: list["ParamInfo"]
        world_size: int
        pg: Any
        debug_fqn: str | None
        padded_local_numels: tuple[int, ...]
        local_copy_out: bool = False  # 1-rank unshard without all-gather

    @dataclass(frozen=True)
    class _ReduceGradState:
        infos: list["ParamInfo"]
        padded_local_numels: tuple[int, ...]
        rank: int
        world_size: int
        pg: Any
        debug_fqn: str | None

    def __init__(self, dim: int = 0) -> None:
        if dim != 0:
            raise NotImplementedError(f"Shard({dim}): only dim 0 is built")
        self.dim = dim

    def __eq__(self, other: object) -> bool:
        return isinstance(other, Shard) and self.dim == other.dim

    def __hash__(self) -> int:
        return hash((Shard, self.dim))

    def __repr__(self) -> str:
        return f"Shard({self.dim})"

    def bucket_compatibility_key(self) -> object:
        return Shard

    # ------------------------------------------------------------------ layout
    @staticmethod
    def _chunk(rows: int, world_size: int) -> int:
        return -(-rows // world_size)

    def compute_local_shape(self, global_shape: torch.Size, rank: int, world_size: int) -> torch.Size:
        if len(global_shape) == 0:
            raise ValueError("Shard(0) needs a parameter with at least one dimension.")
        rows = global_shape[0]
        chunk = self._chunk(rows, world_size)
        start = chunk * rank
        return torch.Size([min(rows, start + chunk) - min(rows, start), *global_shape[1:]])

    def extract_local_shard(self, param: torch.Tensor, rank: int, world_size: int) -> torch.Tensor:
        chunk = self._chunk(param.shape[0], world_size)
        return param[min(param.shape[0], chunk * rank) : min(param.shape[0], chunk * (rank + 1))]

    def global_layout(self, info: "ParamInfo", rank: int, world_size: int) -> GlobalLayout:
        chunk = self._chunk(info.global_shape[0], world_size)
        offset = [0] * len(info.global_shape)
        offset[0] = min(chunk * rank, info.global_shape[0])
        has_data = info.local_numel > 0
        return GlobalLayout(
            global_shape=tuple(info.global_shape),
            global_offsets=(tuple(offset),) if has_data else (),
            local_offsets=((0,) * len(info.local_shape),) if has_data else (),
            local_sizes=(tuple(info.local_shape),) if has_data else (),
        )

    def bucket_storage_layout(
        self,
        named_params: list[tuple[str, nn.Parameter]],
        param_placements: dict[str, tuple[Placement, ...]],
        mesh: Any,
    ) -> BucketStorageLayout:
        rank, world_size = mesh.get_local_rank(), mesh.size()
        layouts: dict[str, BucketParamStorageLayout] = {}
        byte_offset = 0
        for fqn, param in named_params:
            (placement,) = param_placements[fqn]
            if not isinstance(placement, Shard):
                raise AssertionError(f"Expected Shard for {fqn!r}, got {placement!r}")
            local_shape = placement.compute_local_shape(param.shape, rank, world_size)
            # Rank 0 has the largest chunk; its capacity is reserved on every rank.
            storage_nbytes = placement.compute_local_numel(param.shape, 0, world_size) * param.dtype.itemsize
            layouts[fqn] = BucketParamStorageLayout(
                local_shape=local_shape, local_numel=local_shape.numel(), byte_offset=byte_offset,
                storage_nbytes=storage_nbytes,
            )
            byte_offset += storage_nbytes
        return BucketStorageLayout(param_layouts=layouts, total_bytes=byte_offset)

    def copy_param_to_storage(
        self, byte_storage: torch.Tensor, info: "ParamInfo", param: torch.Tensor, rank: int, world_size: int
    ) -> None:
        if param.device.type != "meta":
            data_nbytes = info.local_numel * info.dtype.itemsize
            if info.storage_nbytes > data_nbytes:  # the pad travels with the all-gather: keep it zero
                byte_storage[info.byte_offset + data_nbytes : info.byte_offset + info.storage_nbytes].zero_()
        super().copy_param_to_storage(byte_storage, info, param, rank, world_size)

    @staticmethod
    def _padded_local_numels(infos: list["ParamInfo"]) -> tuple[int, ...]:
        return tuple(info.storage_nbytes // info.dtype.itemsize for info in infos)

    # ----------------------------------------------------------------- unshard
    def _padded_send(self, tensors: list[torch.Tensor], infos: list["ParamInfo"], dtype: torch.dtype) -> torch.Tensor:
        """This rank's chunks back to back in ``dtype``, each zero-padded to
        rank 0's chunk size."""
        padded = self._padded_local_numels(infos)
        send = torch.zeros(sum(padded), dtype=dtype, device=tensors[0].device)
        pieces = torch.split(send, list(padded))
        pairs = [(p[: t.numel()], t.reshape(-1)) for p, t in zip(pieces, tensors, strict=True) if t.numel()]
        if pairs:
            foreach_copy_([dst for dst, _ in pairs], [src for _, src in pairs])
        return send

    def prepare_unshard_bucket(
        self, tensors: list[torch.Tensor], infos: list["ParamInfo"], mesh: Any, debug_fqn: str | None
    ) -> PlacementPreparedUnshard:
        return self._prepare_unshard_bucket(tensors, infos, mesh, debug_fqn, skip_single_rank_all_gather=True)

    def _prepare_unshard_bucket(
        self, tensors: list[torch.Tensor], infos: list["ParamInfo"], mesh: Any, debug_fqn: str | None, *,
        skip_single_rank_all_gather: bool,
    ) -> PlacementPreparedUnshard:
        """Prepare the send and gather buffers or, on a 1-rank mesh with
        ``skip_single_rank_all_gather``, only the local storage.  A mixed
        bucket, which gathers every group in one exchange, needs the buffers."""
        world_size = mesh.size()
        dtype = infos[0].unsharded_dtype
        if any(info.unsharded_dtype != dtype for info in infos):
            raise ValueError("Shard requires one unsharded dtype per bucket.")
        with record_copy_in():
            send = self._padded_send(tensors, infos, dtype)
        local_only = world_size == 1 and skip_single_rank_all_gather
        buffers = [send] if local_only else [send, send.new_empty(world_size * send.numel())]
        return PlacementPreparedUnshard(
            placement=self,
            buffers=buffers,
            placement_state=Shard._UnshardState(
                infos=infos, world_size=world_size, pg=mesh.get_group(), debug_fqn=debug_fqn,
                padded_local_numels=self._padded_local_numels(infos), local_copy_out=local_only,
            ),
        )

    @staticmethod
    def _unshard_state(prepared: PlacementPreparedUnshard) -> "Shard._UnshardState":
        state = prepared.placement_state
        if not isinstance(state, Shard._UnshardState):
            raise AssertionError(f"Expected Shard._UnshardState, got {type(state).__name__}")
        return state

    def run_prepared_unshard(self, prepared: PlacementPreparedUnshard, *, async_op: bool = False) -> Any | None:
        state = self._unshard_state(prepared)
        if state.local_copy_out:
            return None
        with record_comm("FlexShard::all_gather", state.debug_fqn):
            return all_gather_rows(prepared.buffers[1], prepared.buffers[0], state.pg, async_op=async_op)

    def _copy_out_unshard(
        self, gathered: torch.Tensor, state: "Shard._UnshardState", persistent_buffers: list[torch.Tensor] | None
    ) -> tuple[list[torch.Tensor], list[torch.Tensor]]:
        """Full params and the padded buffers backing them.  A refill writes
        the given buffers and returns no full params: the caller keeps the ones
        of the first unshard, which view these buffers."""
        world = state.world_size
        rows = gathered.view(world, -1)
        full_params, padded_params, srcs, dsts = [], [], [], []
        offset = 0
        for index, (info, padded) in enumerate(zip(state.infos, state.padded_local_numels, strict=True)):
            buffer = (
                persistent_buffers[index] if persistent_buffers is not None
                else torch.empty(world * padded, dtype=info.unsharded_dtype, device=gathered.device)
            )
            padded_params.append(buffer)
            if persistent_buffers is None:
                full_params.append(buffer[: info.global_numel].view(info.global_shape))
            # every rank's chunk lands in its place: the padded param is a [world, chunk] matrix
            dsts.append(buffer.view(world, padded))
            srcs.append(rows[:, offset : offset + padded])
            offset += padded
        foreach_copy_(dsts, srcs)
        return full_params, padded_params

    def finish_prepared_unshard(self, prepared: PlacementPreparedUnshard) -> PlacementUnshardResult:
        state = self._unshard_state(prepared)
        with record_copy_out():
            full, padded = self._copy_out_unshard(
                prepared.buffers[0 if state.local_copy_out else 1], state, prepared.persistent_buffers
            )
        return PlacementUnshardResult(full_params=full, persistent_buffers=padded if prepared.persistent else [])

    # --------------------------------------------------------------- gradients
    def _pack_reduce_scatter_grad(
        self, tensors: list[torch.Tensor], infos: list["ParamInfo"], world_size: int, out_rows: torch.Tensor | None = None
    ) -> tuple[torch.Tensor, tuple[int, ...]]:
        """Full gradients -> ``[world, row]`` reduce-scatter input in the reduce
        dtype: rank r's row holds chunk r of every gradient, short chunks
        zero-padded.  ``out_rows`` ([world, >= row], possibly strided) receives
        the rows in place of a new buffer."""
        dtype = infos[0].grad_reduce_dtype
        padded = tuple(
            self._chunk(info.global_shape[0], world_size) * (info.global_numel // max(info.global_shape[0], 1))
            for info in infos
        )
        row = sum(padded)
        if out_rows is None:
            send = torch.zeros(world_size * row, dtype=dtype, device=tensors[0].device)
            rows = send.view(world_size, row)
        else:
            send, rows = out_rows, out_rows
            rows[:, :row].zero_()
        offset = 0
        for grad, info, width in zip(tensors, infos, padded, strict=True):
            flat = grad.reshape(-1)
            whole = flat.numel() // width if width else 0  # ranks with a full chunk
            if whole:
                rows[:whole, offset : offset + width].copy_(flat[: whole * width].view(whole, width))
            rest = flat.numel() - whole * width
            if rest:
                rows[whole, offset : offset + rest].copy_(flat[whole * width :])
            offset += width
        return send, padded

    def prepare_reduce_grad(
        self, tensors: list[torch.Tensor], infos: list["ParamInfo"], mesh: Any, debug_fqn: str | None
    ) -> PlacementPreparedReduceGrad:
        world_size = mesh.size()
        with record_range("FlexShard::reduce_scatter_copy_in", debug_fqn):
            send, padded = self._pack_reduce_scatter_grad(tensors, infos, world_size)
        return PlacementPreparedReduceGrad(
            placement=self,
            buffers=[send],
            placement_state=Shard._ReduceGradState(
                infos=infos, padded_local_numels=padded, rank=mesh.get_local_rank(), world_size=world_size,
                pg=mesh.get_group(), debug_fqn=debug_fqn,
            ),
        )

    def _unpack_reduce_scatter_grad(self, recv: torch.Tensor, state: "Shard._ReduceGradState") -> list[torch.Tensor]:
        shards, offset = [], 0
        for info, width in zip(state.infos, state.padded_local_numels, strict=True):
            shape = self.compute_local_shape(info.global_shape, state.rank, state.world_size)
            shards.append(recv.narrow(0, offset, shape.numel()).view(shape))
            offset += width
        return shards

    def reduce_prepared_grad(
        self, prepared: PlacementPreparedReduceGrad, reduction: "GradientReduction"
    ) -> PlacementReduceGradResult:
        state = prepared.placement_state
        if not isinstance(state, Shard._ReduceGradState):
            raise AssertionError(f"Expected Shard._ReduceGradState, got {type(state).__name__}")
        send = prepared.buffers[0]
        if state.world_size == 1:
            # no exchange: the packed gradients are this rank's shards
            reduce_grads_on_one_rank(send, reduction)
            recv, buffers = send, []
        else:
            recv = torch.empty(send.numel() // state.world_size, dtype=send.dtype, device=send.device)
            with record_comm("FlexShard::post_backward_reduce", state.debug_fqn):
                reduce_scatter_grads(recv, send, reduction, state.pg)
            buffers = [recv]
        with record_range("FlexShard::reduce_scatter_copy_out", state.debug_fqn):
            shards = self._unpack_reduce_scatter_grad(recv, state)
        return PlacementReduceGradResult(shards, buffers)


def make_shard_placement_fn(dim: int = 0):
    """A placement function assigning ``Shard(dim)`` to every parameter."""

    def placement_fn(named_params: list[tuple[str, nn.Parameter]], mesh: Any) -> dict:
        return {fqn: (Shard(dim),) for fqn, _ in named_params}

    return placement_fn


__all__ = ["Shard", "make_shard_placement_fn"]
