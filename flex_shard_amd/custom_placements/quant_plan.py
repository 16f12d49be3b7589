"""Block-row planner and payload metadata of the quantized bucket placements.

Pure integer host math, shared by every format built on
``BlockwiseQuantBucketedBlockShard``.  Restates, with the same results, the
reference's planner (custom_placements/blockwise_quant_bucketed_block_shard.py
:411-519), payload metadata (:196-245, :572-681) and region helpers (:146-151,
:363-385, :1514-1528).

Vocabulary: a *unit* is a run of up to ``shard_block_rows`` rows of one
parameter's flattened ``[prod(shape[:-1]), shape[-1]]`` matrix, never split
between ranks; a *chunk* is one rank's run of consecutive units of one
parameter; a rank's *payload* is ``[FP8 bytes of its chunks | pad to 16 |
scales of its chunks | pad to the common row size]``.
"""

from __future__ import annotations

import math
from bisect import bisect_right
from collections.abc import Callable, Sequence
from dataclasses import dataclass
from typing import NamedTuple

import torch

VEC_ALIGN_BYTES = 16  # pad between data and scales, and of every payload row


def ceil_div(numerator: int, denominator: int) -> int:
    return -(-numerator // denominator)


def align_up(value: int, alignment: int) -> int:
    return ceil_div(value, alignment) * alignment


def matrix_shape(shape: Sequence[int]) -> torch.Size:
    """The matrix a (possibly stacked) weight is planned and quantized as."""
    return torch.Size((math.prod(shape[:-1]), shape[-1]))


class ScaleRegion(NamedTuple):
    """Bytes ``[offset, offset + nbytes)`` of one rank's payload row."""

    rank: int
    offset: int
    nbytes: int


@dataclass(frozen=True)
class BlockRowParam:
    fqn: str
    global_shape: torch.Size
    param_offset: int

    @property
    def matrix_shape(self) -> torch.Size:
        return matrix_shape(self.global_shape)


@dataclass(frozen=True)
class BlockRowUnit:
    fqn: str
    row_start: int
    row_end: int
    dense_numel: int
    cost_bytes: int


@dataclass(frozen=True)
class QuantChunk:
    """One rank-owned contiguous row range of one parameter."""

    rank: int
    fqn: str
    row_start: int
    row_end: int
    global_dense_offset: int
    rank_dense_offset: int
    qdata_offset: int


@dataclass(frozen=True)
class QuantPackChunk:
    """Copy-in plan of one rank-local chunk."""

    param_index: int
    fqn: str
    local_shape: torch.Size
    qdata_numel: int
    scale_numels: tuple[int, ...]


@dataclass(frozen=True)
class QuantRankPackPlan:
    """Copy-in plan of one rank: chunks in parameter order; scales follow the
    aligned data grouped by scale tensor index."""

    chunks: tuple[QuantPackChunk, ...]
    qdata_numel: int
    scale_byte_offset: int
    packed_nbytes: int
    qdata_chunk_numels: tuple[int, ...]
    scale_chunk_nbytes: tuple[int, ...]


@dataclass(frozen=True)
class QuantBucketMetadata:
    """The quantized communication layout of a bucket."""

    chunks: tuple[QuantChunk, ...]
    rank_pack_plans: tuple[QuantRankPackPlan, ...]
    rank_qdata_numels: tuple[int, ...]
    rank_scale_numels: tuple[int, ...]
    rank_scale_byte_offsets: tuple[int, ...]
    rank_packed_nbytes: tuple[int, ...]
    packed_send_nbytes_per_rank: int
    scale_regions_by_index: tuple[tuple[ScaleRegion, ...], ...]


# ------------------------------------------------------------------ planner
def can_partition_units(unit_costs: Sequence[int], num_partitions: int, capacity: int) -> bool:
    """Whether a greedy left-to-right fill puts the units into at most
    ``num_partitions`` contiguous ranges of at most ``capacity`` bytes."""
    used, load = 1, 0
    for cost in unit_costs:
        if cost > capacity:
            return False
        if load + cost > capacity:
            used, load = used + 1, 0
        load += cost
    return used <= num_partitions


def min_partition_capacity(unit_costs: Sequence[int], num_partitions: int) -> int:
    """The smallest per-range capacity of any contiguous partition into at
    most ``num_partitions`` ranges (binary search over the greedy test)."""
    if num_partitions <= 0:
        raise ValueError(f"num_partitions must be positive, got {num_partitions}.")
    if not unit_costs:
        return 0
    total = sum(unit_costs)
    lo, hi = max(max(unit_costs), ceil_div(total, num_partitions)), total
    while lo < hi:
        mid = (lo + hi) // 2
        if can_partition_units(unit_costs, num_partitions, mid):
            hi = mid
        else:
            lo = mid + 1
    return lo


def rank_unit_cuts(unit_costs: Sequence[int], world_size: int, capacity: int) -> tuple[int, ...]:
    """``world_size + 1`` unit indices delimiting each rank's range: greedy
    fill to ``capacity``; while ranks are left over, peel the first unit off
    the first range that has more than one; ranks that still cannot be served
    get empty ranges at the end."""
    cuts = [0]
    load = 0
    for index, cost in enumerate(unit_costs):
        if load and load + cost > capacity:
            cuts.append(index)
            load = 0
        load += cost
    cuts.append(len(unit_costs))
    while len(cuts) - 1 < world_size:
        splittable = next((i for i in range(len(cuts) - 1) if cuts[i + 1] - cuts[i] > 1), None)
        if splittable is None:
            cuts.append(cuts[-1])
        else:
            cuts.insert(splittable + 1, cuts[splittable] + 1)
    if len(cuts) - 1 > world_size:
        raise AssertionError("Quantized block-row planner produced more rank intervals than ranks.")
    return tuple(cuts)


def build_block_row_units(
    params: Sequence[BlockRowParam],
    shard_block_rows: int,
    qdata_itemsize: int,
    scale_itemsize: int,
    chunk_scale_numels: Callable[[int, int], tuple[int, ...]],
) -> list[BlockRowUnit]:
    units: list[BlockRowUnit] = []
    for param in params:
        rows, in_dim = param.matrix_shape
        for start in range(0, rows, shard_block_rows):
            end = min(rows, start + shard_block_rows)
            dense = (end - start) * in_dim
            scales = sum(chunk_scale_numels(end - start, in_dim))
            units.append(
                BlockRowUnit(
                    fqn=param.fqn,
                    row_start=start,
                    row_end=end,
                    dense_numel=dense,
                    cost_bytes=dense * qdata_itemsize + scales * scale_itemsize,
                )
            )
    return units


def unit_cuts_from_rank_layout(
    units: Sequence[BlockRowUnit], rank_offsets: Sequence[int], rank_numels: Sequence[int]
) -> tuple[int, ...]:
    """Recover the unit cuts from a bucket layout's dense rank ranges."""
    edges = [0]
    for unit in units:
        edges.append(edges[-1] + unit.dense_numel)
    # Units are non-empty, so every edge is distinct; an empty rank's offset
    # equals its successor's and maps to the same unit index.
    index_of_edge = {edge: index for index, edge in enumerate(edges)}
    bounds = (*rank_offsets, rank_offsets[-1] + rank_numels[-1])
    if any(b not in index_of_edge for b in bounds):
        raise AssertionError("Quantized block-row rank layout is not aligned to row-block units.")
    return tuple(index_of_edge[b] for b in bounds)


def merge_adjacent_regions(regions: Sequence[ScaleRegion]) -> tuple[ScaleRegion, ...]:
    """Drop empty regions and join each region that continues the previous one
    in the same rank."""
    merged: list[ScaleRegion] = []
    for region in regions:
        if region.nbytes == 0:
            continue
        last = merged[-1] if merged else None
        if last is not None and last.rank == region.rank and last.offset + last.nbytes == region.offset:
            merged[-1] = last._replace(nbytes=last.nbytes + region.nbytes)
        else:
            merged.append(region)
    return tuple(merged)


def build_quant_metadata(
    params: Sequence[BlockRowParam],
    units: Sequence[BlockRowUnit],
    unit_cuts: Sequence[int],
    *,
    scale_itemsize: int,
    num_scale_tensors: int,
    chunk_scale_numels: Callable[[int, int], tuple[int, ...]],
    scale_regions: Callable[[int, tuple[QuantRankPackPlan, ...]], tuple[ScaleRegion, ...]],
) -> QuantBucketMetadata:
    by_fqn = {p.fqn: (index, p) for index, p in enumerate(params)}
    chunks: list[QuantChunk] = []
    plans: list[QuantRankPackPlan] = []
    for rank, (lo, hi) in enumerate(zip(unit_cuts[:-1], unit_cuts[1:], strict=True)):
        cursor = 0  # dense elements (= FP8 bytes) of this rank placed so far
        pack_chunks: list[QuantPackChunk] = []
        position = lo
        while position < hi:
            first = units[position]
            last = first
            position += 1
            while position < hi and units[position].fqn == first.fqn:
                last = units[position]
                position += 1
            index, param = by_fqn[first.fqn]
            in_dim = param.matrix_shape[1]
            rows = last.row_end - first.row_start
            chunks.append(
                QuantChunk(
                    rank=rank,
                    fqn=param.fqn,
                    row_start=first.row_start,
                    row_end=last.row_end,
                    global_dense_offset=param.param_offset + first.row_start * in_dim,
                    rank_dense_offset=cursor,
                    qdata_offset=cursor,
                )
            )
            pack_chunks.append(
                QuantPackChunk(
                    param_index=index,
                    fqn=param.fqn,
                    local_shape=torch.Size((rows, in_dim)),
                    qdata_numel=rows * in_dim,
                    scale_numels=chunk_scale_numels(rows, in_dim),
                )
            )
            cursor += rows * in_dim
        scale_total = sum(sum(c.scale_numels) for c in pack_chunks)
        scale_start = align_up(cursor, VEC_ALIGN_BYTES)
        plans.append(
            QuantRankPackPlan(
                chunks=tuple(pack_chunks),
                qdata_numel=cursor,
                scale_byte_offset=scale_start,
                packed_nbytes=scale_start + scale_total * scale_itemsize,
                qdata_chunk_numels=tuple(c.qdata_numel for c in pack_chunks),
                scale_chunk_nbytes=tuple(
                    c.scale_numels[k] * scale_itemsize for k in range(num_scale_tensors) for c in pack_chunks
                ),
            )
        )
    plans_t = tuple(plans)
    packed = tuple(p.packed_nbytes for p in plans_t)
    return QuantBucketMetadata(
        chunks=tuple(chunks),
        rank_pack_plans=plans_t,
        rank_qdata_numels=tuple(p.qdata_numel for p in plans_t),
        rank_scale_numels=tuple(sum(sum(c.scale_numels) for c in p.chunks) for p in plans_t),
        rank_scale_byte_offsets=tuple(p.scale_byte_offset for p in plans_t),
        rank_packed_nbytes=packed,
        packed_send_nbytes_per_rank=align_up(max(packed, default=0), VEC_ALIGN_BYTES),
        scale_regions_by_index=tuple(
            merge_adjacent_regions(scale_regions(k, plans_t)) for k in range(num_scale_tensors)
        ),
    )


def default_scale_regions(
    scale_index: int, rank_pack_plans: Sequence[QuantRankPackPlan], scale_itemsize: int
) -> tuple[ScaleRegion, ...]:
    """Every rank contributes its whole ``scale_index`` group, so rank chunks
    concatenate flat into each parameter's scale tensor."""
    regions = []
    for rank, plan in enumerate(rank_pack_plans):
        before = sum(sum(c.scale_numels[:scale_index]) for c in plan.chunks)
        count = sum(c.scale_numels[scale_index] for c in plan.chunks)
        regions.append(ScaleRegion(rank, plan.scale_byte_offset + scale_itemsize * before, scale_itemsize * count))
    return tuple(regions)


def owner_of_unit(unit_cuts: Sequence[int], unit_index: int) -> int:
    """The rank whose range holds unit ``unit_index``."""
    return bisect_right(list(unit_cuts[1:]), unit_index)
