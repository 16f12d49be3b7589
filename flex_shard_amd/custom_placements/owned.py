"""``BucketedOwned``: whole parameters (or whole dim-0 slabs) live on owner ranks.

Keeps the reference's public surface (custom_placements/owned.py:39-583): the
segment spec, the placement's constructor / equality / repr, the lowering of an
ownership map to per-parameter one-hot ``BlockShard`` layouts, LPT owner
assignment and the four segment / placement-function factories.  The owner's
local storage layout ("its row of the gathered buffer": groups of same-owner
parameters back to back) follows the owner-rows layout the reference's mixed
bucket derives for such buckets (custom_placements/mixed_bucket.py:522-562,
:1603-1675).

The multi-rank collectives of an owned bucket (broadcast of owner rows,
reduce to owner) belong to the mixed-bucket runtime and are not part of this
single-GPU package; the lifecycle hooks raise ``NotImplementedError``.  What an
owner does locally with its whole matrices -- the Muon step -- is in
:mod:`flex_shard_amd.dist_muon`.
"""

from __future__ import annotations

import math
from collections.abc import Mapping, Sequence
from dataclasses import dataclass
from typing import TYPE_CHECKING, Any, Literal

import torch
import torch.nn as nn

from ..placement_contract import (
    BucketParamStorageLayout,
    BucketStorageLayout,
    GlobalLayout,
    Placement,
)
from .block_shard import BlockShard
from .owner_balance import assign_to_hosts_then_ranks, lpt_owners, mesh_rank_hosts

if TYPE_CHECKING:
    from ..bucket_storage import ParamInfo


@dataclass(frozen=True)
class BucketedOwnedSegmentSpec:
    """A flat slice of one parameter owned by one rank."""

    name: str
    fqn: str
    param_offset: int
    numel: int
    owner_rank: int
    storage_order: int = 0


BucketedOwnedViewKind = Literal["full_param", "expert_block"]

_OUT_OF_SCOPE = (
    "BucketedOwned's bucket collectives run in the multi-rank mixed-bucket runtime, which this "
    "single-GPU package does not include."
)


class BucketedOwned(Placement):
    """Bucket-global owner-partition placement."""

    def __init__(
        self,
        segments_by_fqn: dict[str, list[BucketedOwnedSegmentSpec]],
        *,
        view_kind: BucketedOwnedViewKind = "full_param",
    ) -> None:
        if view_kind not in ("full_param", "expert_block"):
            raise ValueError(
                f"BucketedOwned view_kind must be 'full_param' or 'expert_block', but got {view_kind!r}."
            )
        ordered: dict[str, tuple[BucketedOwnedSegmentSpec, ...]] = {}
        for fqn, segments in segments_by_fqn.items():
            if not segments:
                raise ValueError(f"BucketedOwned requires at least one segment for {fqn!r}.")
            by_offset = tuple(sorted(segments, key=lambda s: s.param_offset))
            for segment in by_offset:
                if segment.fqn != fqn:
                    raise ValueError(
                        f"BucketedOwned segment {segment.name!r} is under key {fqn!r} but names FQN {segment.fqn!r}."
                    )
                if segment.numel <= 0:
                    raise ValueError(f"BucketedOwned segment {segment.name!r} has invalid numel {segment.numel}.")
            ordered[fqn] = by_offset
        self.segments_by_fqn = ordered
        self.view_kind = view_kind
        self._hash_key = tuple(sorted(ordered.items()))

    def __eq__(self, other: object) -> bool:
        return (
            isinstance(other, BucketedOwned)
            and self.view_kind == other.view_kind
            and self._hash_key == other._hash_key
        )

    def __hash__(self) -> int:
        return hash((type(self), self.view_kind, self._hash_key))

    def __repr__(self) -> str:
        return f"BucketedOwned(num_params={len(self.segments_by_fqn)}, view_kind={self.view_kind!r})"

    # ---------------------------------------------------------------- lowering
    @staticmethod
    def _validate_shape(fqn: str, shape: Sequence[int]) -> tuple[int, ...]:
        shape_t = tuple(shape)
        if not shape_t:
            raise ValueError(f"BucketedOwned cannot lower scalar parameter {fqn!r} to BlockShard.")
        if any(size < 0 for size in shape_t):
            raise ValueError(f"BucketedOwned shape for {fqn!r} must be non-negative, but got {shape}.")
        return shape_t

    @staticmethod
    def _validate_segment(fqn: str, segment: BucketedOwnedSegmentSpec, world_size: int) -> None:
        if segment.fqn != fqn:
            raise ValueError(
                f"BucketedOwned segment {segment.name!r} is under key {fqn!r} but names FQN {segment.fqn!r}."
            )
        if segment.param_offset < 0:
            raise ValueError("BucketedOwned param_offset must be non-negative.")
        if segment.numel <= 0:
            raise ValueError("BucketedOwned numel must be positive.")
        if not 0 <= segment.owner_rank < world_size:
            raise ValueError(
                f"BucketedOwned owner for segment {segment.name!r} must be in [0, {world_size}), "
                f"but got {segment.owner_rank}."
            )

    @staticmethod
    def _one_hot_blocks(owner_rank: int, world_size: int) -> tuple[int, ...]:
        return tuple(int(rank == owner_rank) for rank in range(world_size))

    @staticmethod
    def _blocks_per_rank_from_dim0_slices(
        fqn: str, shape: tuple[int, ...], segments: tuple[BucketedOwnedSegmentSpec, ...], world_size: int
    ) -> tuple[int, ...]:
        slab = math.prod(shape[1:])
        if slab <= 0 or len(segments) != shape[0]:
            raise NotImplementedError(f"BucketedOwned {fqn!r} must contain one complete dim-0 slab per segment.")
        owners = []
        for index, segment in enumerate(segments):
            if segment.param_offset != index * slab or segment.numel != slab:
                raise NotImplementedError(
                    f"BucketedOwned {fqn!r} must contain equal complete dim-0 slabs; "
                    "partial segments cannot lower to BlockShard."
                )
            owners.append(segment.owner_rank)
        if any(a > b for a, b in zip(owners, owners[1:])):
            raise NotImplementedError(
                f"BucketedOwned {fqn!r} requires contiguous, nondecreasing dim-0 slab owners to lower to BlockShard."
            )
        return tuple(owners.count(rank) for rank in range(world_size))

    def _lower_to_block_shards(
        self, logical_shapes_by_fqn: Mapping[str, Sequence[int]], world_size: int
    ) -> dict[str, BlockShard]:
        """Per-FQN ``BlockShard`` for whole-tensor and whole-slab ownership."""
        if world_size <= 0:
            raise ValueError(f"world_size must be positive, but got {world_size}.")
        lowered: dict[str, BlockShard] = {}
        for fqn, raw_shape in logical_shapes_by_fqn.items():
            if fqn not in self.segments_by_fqn:
                raise ValueError(f"BucketedOwned missing segments for {fqn!r}.")
            shape = self._validate_shape(fqn, raw_shape)
            segments = self.segments_by_fqn[fqn]
            for segment in segments:
                self._validate_segment(fqn, segment, world_size)
            whole = len(segments) == 1 and segments[0].param_offset == 0 and segments[0].numel == math.prod(shape)
            blocks = (
                self._one_hot_blocks(segments[0].owner_rank, world_size)
                if whole
                else self._blocks_per_rank_from_dim0_slices(fqn, shape, segments, world_size)
            )
            lowered[fqn] = BlockShard(blocks_per_rank=blocks, dim=0)
        return lowered

    def owned_fqns(self, rank: int) -> list[str]:
        """FQNs with at least one segment owned by ``rank``, in map order."""
        return [fqn for fqn, segs in self.segments_by_fqn.items() if any(s.owner_rank == rank for s in segs)]

    # ------------------------------------------------------------------ layout
    def compute_local_shape(self, global_shape: torch.Size, rank: int, world_size: int) -> torch.Size:
        raise NotImplementedError("BucketedOwned local shape is FQN-dependent; use bucket_storage_layout().")

    def extract_local_shard(self, param: torch.Tensor, rank: int, world_size: int) -> torch.Tensor:
        raise NotImplementedError("BucketedOwned local shard is FQN-dependent; use copy_param_to_storage().")

    def global_layout(self, info: "ParamInfo", rank: int, world_size: int) -> GlobalLayout:
        shard = self._lower_to_block_shards({info.fqn: tuple(info.global_shape)}, world_size)[info.fqn]
        return shard.global_layout(info, rank, world_size)

    def bucket_storage_layout(
        self,
        named_params: list[tuple[str, nn.Parameter]],
        param_placements: dict[str, tuple[Placement, ...]],
        mesh: Any,
    ) -> BucketStorageLayout | None:
        """Each rank stores its owned parameters: parameters with the same
        lowered layout form a group, groups of one owner lie back to back in
        that owner's row in first-appearance order, and a parameter sits in its
        group at the running offset of the group's earlier parameters."""
        wanted = {fqn for fqn, _ in named_params}
        have = set(self.segments_by_fqn)
        if wanted != have:
            raise ValueError(
                "BucketedOwned segment map must match the bucket FQNs exactly: "
                f"missing={sorted(wanted - have)} extra={sorted(have - wanted)}"
            )
        for fqn, _ in named_params:
            if param_placements[fqn] != (self,):
                raise ValueError(
                    "BucketedOwned requires the same placement instance for every parameter in a bucket; "
                    f"{fqn!r} uses {param_placements[fqn]!r}."
                )
        if not named_params:
            return BucketStorageLayout(param_layouts={}, total_bytes=0)
        rank, world_size = mesh.get_local_rank(), mesh.size()
        lowered = self._lower_to_block_shards({fqn: tuple(p.shape) for fqn, p in named_params}, world_size)
        dtype = named_params[0][1].dtype
        one_owner = all(
            sorted(lowered[fqn].blocks_per_rank) == [0] * (world_size - 1) + [1] and p.dtype == dtype
            for fqn, p in named_params
        )
        layouts: dict[str, BucketParamStorageLayout] = {}
        if one_owner:
            groups: list[list[tuple[str, nn.Parameter]]] = []
            for fqn, param in named_params:
                for group in groups:
                    if lowered[group[0][0]] == lowered[fqn]:
                        group.append((fqn, param))
                        break
                else:
                    groups.append([(fqn, param)])
            row_numels = [0] * world_size
            for group in groups:
                owner = lowered[group[0][0]].blocks_per_rank.index(1)
                cursor = row_numels[owner]
                for fqn, param in group:
                    local = lowered[fqn].local_storage_layout(param.shape, param.dtype, rank, world_size)
                    layouts[fqn] = BucketParamStorageLayout(
                        local_shape=local.local_shape,
                        local_numel=local.local_numel,
                        byte_offset=cursor * dtype.itemsize if owner == rank else 0,
                        storage_nbytes=local.storage_nbytes,
                    )
                    cursor += param.numel()
                row_numels[owner] = cursor
            return BucketStorageLayout(param_layouts=layouts, total_bytes=row_numels[rank] * dtype.itemsize)
        # Slab ownership or mixed dtypes: sequential per-parameter layout.
        cursor = 0
        for fqn, param in named_params:
            local = lowered[fqn].local_storage_layout(param.shape, param.dtype, rank, world_size)
            layouts[fqn] = BucketParamStorageLayout(
                local_shape=local.local_shape,
                local_numel=local.local_numel,
                byte_offset=cursor if local.storage_nbytes > 0 else 0,
                storage_nbytes=local.storage_nbytes,
            )
            cursor += local.storage_nbytes
        return BucketStorageLayout(param_layouts=layouts, total_bytes=cursor)

    def copy_param_to_storage(
        self, byte_storage: torch.Tensor, info: "ParamInfo", param: torch.Tensor, rank: int, world_size: int
    ) -> None:
        shard = self._lower_to_block_shards({info.fqn: tuple(info.global_shape)}, world_size)[info.fqn]
        shard.copy_param_to_storage(byte_storage, info, param, rank, world_size)

    # ------------------------------------------------ collectives (not built)
    def prepare_unshard_bucket(self, tensors, infos, mesh, debug_fqn):
        raise NotImplementedError(_OUT_OF_SCOPE)

    def run_prepared_unshard(self, prepared, *, async_op: bool = False):
        raise NotImplementedError(_OUT_OF_SCOPE)

    def finish_prepared_unshard(self, prepared):
        raise NotImplementedError(_OUT_OF_SCOPE)

    def prepare_reduce_grad(self, tensors, infos, mesh, debug_fqn):
        raise NotImplementedError(_OUT_OF_SCOPE)

    def reduce_prepared_grad(self, prepared, reduction):
        raise NotImplementedError(_OUT_OF_SCOPE)


def _assign_params_to_ranks(
    named_params: list[tuple[str, nn.Parameter]],
    world_size: int,
    hosts: Sequence[int] | None = None,
    carried_loads: Sequence[int] | None = None,
) -> dict[str, int]:
    """Owner of each whole parameter, largest first: hosts first when ``hosts``
    is given, else the least-loaded rank."""
    numels = [param.numel() for _, param in named_params]
    if hosts is not None:
        owners = assign_to_hosts_then_ranks(numels, hosts, carried_loads=carried_loads)
    else:
        owners = lpt_owners(numels, world_size, carried_loads)
    return {fqn: owner for (fqn, _), owner in zip(named_params, owners)}


def make_bucketed_owned_full_param_segments(
    named_params: list[tuple[str, nn.Parameter]],
    world_size: int,
    *,
    hosts: Sequence[int] | None = None,
    carried_loads: Sequence[int] | None = None,
) -> dict[str, list[BucketedOwnedSegmentSpec]]:
    """One whole-parameter segment per parameter, owners balanced by numel."""
    if world_size <= 0:
        raise ValueError(f"world_size must be positive, but got {world_size}.")
    if hosts is not None and len(hosts) != world_size:
        raise ValueError(f"hosts must give each of {world_size} ranks a host.")
    if carried_loads is not None and len(carried_loads) != world_size:
        raise ValueError(f"carried_loads must give each of {world_size} ranks a load.")
    owners = _assign_params_to_ranks(named_params, world_size, hosts, carried_loads)
    return {
        fqn: [
            BucketedOwnedSegmentSpec(
                name=f"{fqn}#full", fqn=fqn, param_offset=0, numel=param.numel(), owner_rank=owners[fqn],
                storage_order=order,
            )
        ]
        for order, (fqn, param) in enumerate(named_params)
    }


def make_bucketed_owned_full_param_placement_fn(*, carry_loads: bool = False):
    """A whole-parameter ``BucketedOwned`` placement function; with
    ``carry_loads`` later buckets balance against the owners of earlier ones."""
    carried: dict[tuple[int, ...], list[int]] = {}

    def placement_fn(named_params: list[tuple[str, nn.Parameter]], mesh: Any) -> dict:
        mesh_ranks = tuple(mesh.mesh.flatten().tolist())
        loads = carried.setdefault(mesh_ranks, [0] * mesh.size())
        segments = make_bucketed_owned_full_param_segments(
            named_params,
            mesh.size(),
            hosts=mesh_rank_hosts(list(mesh_ranks)),
            carried_loads=loads if carry_loads else None,
        )
        if carry_loads:
            for specs in segments.values():
                for spec in specs:
                    loads[spec.owner_rank] += spec.numel
        placement = BucketedOwned(segments, view_kind="full_param")
        return {fqn: (placement,) for fqn, _ in named_params}

    return placement_fn


def _expert_block_order_key(fqn: str, suffix_order: tuple[str, ...]) -> int:
    for index, suffix in enumerate(suffix_order):
        if fqn.endswith(suffix):
            return index
    raise ValueError(f"Unexpected grouped expert weight FQN: {fqn}")


def make_bucketed_owned_expert_block_segments(
    named_params: list[tuple[str, nn.Parameter]],
    world_size: int,
    *,
    suffix_order: tuple[str, ...] = (".w1", ".w3", ".w2"),
) -> dict[str, list[BucketedOwnedSegmentSpec]]:
    """Per-expert segments of packed ``[experts, ...]`` weights, experts
    assigned to contiguous owner ranges."""
    if world_size <= 0:
        raise ValueError(f"world_size must be positive, but got {world_size}.")
    if not suffix_order:
        raise ValueError("suffix_order must contain at least one suffix.")
    if not named_params:
        return {}
    bad = [(fqn, tuple(p.shape)) for fqn, p in named_params if p.dim() < 3 or not fqn.endswith(suffix_order)]
    if bad:
        raise ValueError(
            f"BucketedOwned expert block expects packed weights with at least 3 dims and a suffix in "
            f"{suffix_order}: {bad}"
        )
    experts = named_params[0][1].shape[0]
    if any(p.shape[0] != experts for _, p in named_params):
        raise ValueError("BucketedOwned expert block requires matching expert counts.")
    ordered = sorted(named_params, key=lambda item: _expert_block_order_key(item[0], suffix_order))
    per_owner = max(1, -(-experts // world_size))
    out: dict[str, list[BucketedOwnedSegmentSpec]] = {fqn: [] for fqn, _ in ordered}
    for expert in range(experts):
        owner = min(expert // per_owner, world_size - 1)
        for order, (fqn, param) in enumerate(ordered):
            slab = math.prod(param.shape[1:])
            out[fqn].append(
                BucketedOwnedSegmentSpec(
                    name=f"{fqn}#expert{expert}", fqn=fqn, param_offset=expert * slab, numel=slab,
                    owner_rank=owner, storage_order=expert * len(ordered) + order,
                )
            )
    return out


def make_bucketed_owned_expert_block_placement_fn(*, suffix_order: tuple[str, ...] = (".w1", ".w3", ".w2")):
    """A placement function for one packed expert-weight bucket."""

    def placement_fn(named_params: list[tuple[str, nn.Parameter]], mesh: Any) -> dict:
        segments = make_bucketed_owned_expert_block_segments(named_params, mesh.size(), suffix_order=suffix_order)
        placement = BucketedOwned(segments, view_kind="expert_block")
        return {fqn: (placement,) for fqn, _ in named_params}

    return placement_fn


__all__ = [
    "BucketedOwned",
    "BucketedOwnedSegmentSpec",
    "make_bucketed_owned_expert_block_placement_fn",
    "make_bucketed_owned_expert_block_segments",
    "make_bucketed_owned_full_param_placement_fn",
    "make_bucketed_owned_full_param_segments",
]
