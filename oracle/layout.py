"""Integer host math of the hot path, enumerated naively.  TEST INFRASTRUCTURE ONLY.

The package's host code derives everything from cached metadata objects; this
module recomputes the same facts by walking every 128-row unit (or every
element range) in order, so agreement between the two is a real check.
Citations are paths under the reference checkout (``src/flex_shard/...``).
"""

from __future__ import annotations

import math
from dataclasses import dataclass

import torch

ALIGN = 16  # custom_placements/blockwise_quant_bucketed_block_shard.py:73


def ceil_div(a: int, b: int) -> int:
    return -(-a // b)


def align_up(value: int, alignment: int) -> int:
    return ceil_div(value, alignment) * alignment


def matrix_shape(shape) -> tuple[int, int]:
    """Stacked weights are planned as their flattened matrix (:100-102)."""
    return math.prod(shape[:-1]), shape[-1]


@dataclass(frozen=True)
class Unit:
    """One indivisible run of up to ``block`` rows of one parameter."""

    param: int
    row_start: int
    row_end: int
    in_dim: int
    dense_numel: int
    scale_numel: int
    cost_bytes: int


def block_row_units(shapes, block: int, scale_itemsize: int = 4) -> list[Unit]:
    """custom_placements/blockwise_quant_bucketed_block_shard.py:497-519."""
    units = []
    for index, shape in enumerate(shapes):
        rows, in_dim = matrix_shape(shape)
        for row_start in range(0, rows, block):
            row_end = min(rows, row_start + block)
            dense = (row_end - row_start) * in_dim
            scales = ceil_div(row_end - row_start, block) * ceil_div(in_dim, block)
            units.append(Unit(index, row_start, row_end, in_dim, dense, scales, dense + scales * scale_itemsize))
    return units


def fits(costs: list[int], parts: int, capacity: int) -> bool:
    """Greedy feasibility test (:411-427)."""
    used, current = 1, 0
    for cost in costs:
        if cost > capacity:
            return False
        if current + cost > capacity:
            used += 1
            current = 0
        current += cost
    return used <= parts


def min_capacity(costs: list[int], parts: int) -> int:
    """Smallest capacity for which ``fits`` holds (:429-453)."""
    if not costs:
        return 0
    lo = max(max(costs), ceil_div(sum(costs), parts))
    hi = sum(costs)
    while lo < hi:
        mid = (lo + hi) // 2
        if fits(costs, parts, mid):
            hi = mid
        else:
            lo = mid + 1
    return lo


def rank_cuts(costs: list[int], world_size: int) -> tuple[int, ...]:
    """Contiguous min-max partition of units into ``world_size`` ranges
    (:455-483, :1000-1005): greedy fill to the minimal capacity, then split
    the first multi-unit range until every rank has a range; when no range can
    be split the trailing ranks stay empty."""
    capacity = min_capacity(costs, world_size)
    cuts = [0]
    load = 0
    for index, cost in enumerate(costs):
        if load > 0 and load + cost > capacity:
            cuts.append(index)
            load = 0
        load += cost
    cuts.append(len(costs))
    while len(cuts) - 1 < world_size:
        for position in range(len(cuts) - 1):
            if cuts[position + 1] - cuts[position] > 1:
                cuts.insert(position + 1, cuts[position] + 1)
                break
        else:
            cuts.append(cuts[-1])
    return tuple(cuts)


def brute_force_min_capacity(costs: list[int], parts: int) -> int:
    """Exhaustive optimum over every placement of ``parts - 1`` cut points
    (empty ranges allowed).  Only for a handful of units."""
    from itertools import combinations_with_replacement

    best = None
    n = len(costs)
    for cut_points in combinations_with_replacement(range(n + 1), parts - 1):
        bounds = (0, *cut_points, n)
        worst = max(sum(costs[a:b]) for a, b in zip(bounds, bounds[1:]))
        best = worst if best is None else min(best, worst)
    return best


@dataclass(frozen=True)
class QuantLayout:
    """Everything the FP8 bucket derives from its unit cuts."""

    units: tuple[Unit, ...]
    cuts: tuple[int, ...]
    rank_offsets: tuple[int, ...]
    rank_numels: tuple[int, ...]
    rank_scale_numels: tuple[int, ...]
    rank_scale_byte_offsets: tuple[int, ...]
    rank_packed_nbytes: tuple[int, ...]
    row_nbytes: int


def quant_layout(shapes, block: int, world_size: int) -> QuantLayout:
    """Rank ranges and payload sizes (:572-681, :1006-1014)."""
    units = block_row_units(shapes, block)
    cuts = rank_cuts([u.cost_bytes for u in units], world_size)
    offsets, numels, scales = [], [], []
    start = 0
    for lo, hi in zip(cuts, cuts[1:]):
        dense = sum(u.dense_numel for u in units[lo:hi])
        offsets.append(start)
        numels.append(dense)
        scales.append(sum(u.scale_numel for u in units[lo:hi]))
        start += dense
    scale_offsets = tuple(align_up(n, ALIGN) for n in numels)
    packed = tuple(o + 4 * s for o, s in zip(scale_offsets, scales))
    return QuantLayout(
        units=tuple(units),
        cuts=cuts,
        rank_offsets=tuple(offsets),
        rank_numels=tuple(numels),
        rank_scale_numels=tuple(scales),
        rank_scale_byte_offsets=scale_offsets,
        rank_packed_nbytes=packed,
        row_nbytes=align_up(max(packed, default=0), ALIGN),
    )


def local_row_ranges(layout: QuantLayout, rank: int, num_params: int) -> list[tuple[int, int]]:
    """Per parameter, the (row_start, row_end) this rank owns; (0, 0) if none."""
    ranges = [(0, 0)] * num_params
    for unit in layout.units[layout.cuts[rank] : layout.cuts[rank + 1]]:
        lo, hi = ranges[unit.param]
        ranges[unit.param] = (unit.row_start, unit.row_end) if hi == 0 else (lo, unit.row_end)
    return ranges


def pack_rank_payload(
    layout: QuantLayout,
    rank: int,
    qdata: list[torch.Tensor],
    scales: list[torch.Tensor],
    block: int,
    fill: int = 0,
) -> torch.Tensor:
    """One rank's send payload (:792-897): the FP8 bytes of its units in unit
    order, zero pad to 16 bytes, the fp32 scale rows of the same units, zero
    pad to the common row size.  ``qdata[p]`` is the whole parameter's
    [rows, in_dim] FP8 bytes and ``scales[p]`` its whole scale matrix: because
    cuts fall on tile-row boundaries the per-rank quantization is a slice of
    the whole-matrix one."""
    data_parts, scale_parts = [], []
    for unit in layout.units[layout.cuts[rank] : layout.cuts[rank + 1]]:
        data_parts.append(qdata[unit.param].view(torch.uint8)[unit.row_start : unit.row_end].reshape(-1))
        scale_row = unit.row_start // block
        scale_parts.append(scales[unit.param][scale_row : scale_row + 1].reshape(-1).view(torch.uint8))
    payload = torch.full((layout.row_nbytes,), fill, dtype=torch.uint8)
    data = torch.cat(data_parts) if data_parts else torch.empty(0, dtype=torch.uint8)
    scale_bytes = torch.cat(scale_parts) if scale_parts else torch.empty(0, dtype=torch.uint8)
    start = layout.rank_scale_byte_offsets[rank]
    payload[: data.numel()] = data
    payload[data.numel() : start] = 0
    payload[start : start + scale_bytes.numel()] = scale_bytes
    payload[start + scale_bytes.numel() :] = 0
    return payload


def compact_from_full(qdata: list[torch.Tensor], scales: list[torch.Tensor]) -> torch.Tensor:
    """The compact unshard buffer (:1237-1264) built directly from whole-matrix
    quantization: every parameter's FP8 bytes in bucket order, pad to 16
    bytes, every parameter's scales in bucket order."""
    data = torch.cat([q.view(torch.uint8).reshape(-1) for q in qdata])
    scale_bytes = torch.cat([s.reshape(-1).view(torch.uint8) for s in scales])
    out = torch.zeros(align_up(data.numel(), ALIGN) + scale_bytes.numel(), dtype=torch.uint8)
    out[: data.numel()] = data
    out[align_up(data.numel(), ALIGN) :] = scale_bytes
    return out


def compact_from_rank_rows(layout: QuantLayout, rank_rows: torch.Tensor, fill: int = 0) -> torch.Tensor:
    """Join gathered rank rows ([W, row_nbytes], possibly strided) into the
    compact buffer (:1320-1358, :1424-1490): data of rank 0..W-1, then from
    the aligned offset the scale bytes of rank 0..W-1.  Bytes of the alignment
    gap keep ``fill`` (the reference leaves them unwritten)."""
    data_total = sum(layout.rank_numels)
    scale_start = align_up(data_total, ALIGN)
    out = torch.full((scale_start + 4 * sum(layout.rank_scale_numels),), fill, dtype=torch.uint8)
    cursor = 0
    for rank, numel in enumerate(layout.rank_numels):
        out[cursor : cursor + numel] = rank_rows[rank, :numel]
        cursor += numel
    cursor = scale_start
    for rank, count in enumerate(layout.rank_scale_numels):
        lo = layout.rank_scale_byte_offsets[rank]
        out[cursor : cursor + 4 * count] = rank_rows[rank, lo : lo + 4 * count]
        cursor += 4 * count
    return out


@dataclass(frozen=True)
class DenseBucketLayout:
    """custom_placements/block_shard.py:711-754."""

    alignment: int
    param_offsets: tuple[int, ...]
    global_numel: int
    rank_offsets: tuple[int, ...]
    rank_numels: tuple[int, ...]


def dense_bucket_layout(shapes, blocks_per_rank, num_prefix_dims: int = 1) -> DenseBucketLayout:
    """Param-major flat bucket: each start aligned to the lcm of the row
    widths, the total padded to ``alignment * sum(blocks)``, rank r taking
    ``blocks_per_rank[r]`` equal blocks."""
    alignment = 1
    for shape in shapes:
        alignment = math.lcm(alignment, math.prod(shape[num_prefix_dims:]))
    offsets, cursor = [], 0
    for shape in shapes:
        cursor = align_up(cursor, alignment)
        offsets.append(cursor)
        cursor += math.prod(shape)
    total_blocks = sum(blocks_per_rank)
    padded = align_up(cursor, alignment * total_blocks)
    block_numel = padded // total_blocks
    rank_offsets, rank_numels, start = [], [], 0
    for count in blocks_per_rank:
        rank_offsets.append(start)
        rank_numels.append(count * block_numel)
        start += count * block_numel
    return DenseBucketLayout(alignment, tuple(offsets), padded, tuple(rank_offsets), tuple(rank_numels))


def reduce_scatter_input(
    grads: list[torch.Tensor],
    param_offsets,
    global_numel: int,
    rank_offsets,
    rank_numels,
    dtype: torch.dtype,
) -> torch.Tensor:
    """tests/test_flex_shard_fp8_allgather.py:1039-1064 -- scatter the grads
    into a zeroed bucket, then give each rank its range zero-padded to the
    longest range: a [W, max(rank_numels)] matrix."""
    bucket = torch.zeros(global_numel, dtype=dtype)
    for grad, offset in zip(grads, param_offsets):
        bucket[offset : offset + grad.numel()] = grad.reshape(-1).to(dtype)
    rows = torch.zeros(len(rank_numels), max(rank_numels), dtype=dtype)
    for rank, (offset, numel) in enumerate(zip(rank_offsets, rank_numels)):
        rows[rank, :numel] = bucket[offset : offset + numel]
    return rows


def lpt_owners(numels: list[int], world_size: int, carried=None) -> list[int]:
    """custom_placements/owned.py:410-422 -- largest first onto the least
    loaded rank; ties go to the lower rank, equal sizes keep bucket order."""
    loads = [0] * world_size if carried is None else list(carried)
    owners = [0] * len(numels)
    for index in sorted(range(len(numels)), key=lambda i: -numels[i]):
        rank = min(range(world_size), key=lambda r: (loads[r], r))
        owners[index] = rank
        loads[rank] += numels[index]
    return owners
