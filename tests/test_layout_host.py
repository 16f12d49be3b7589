"""Integer host math (CPU only): the oracle's naive layout routines and the
package's placement classes, both pinned by the reference's known answers
(tests/golden), by exhaustive optimality checks, and against each other."""

import itertools
import random

import pytest
import torch
import torch.nn as nn

from flex_shard_amd import (
    BucketedBlockShard,
    Fp8BucketedBlockShard,
    GlobalLayout,
    make_bucketed_block_placement_fn,
    make_fp8_bucketed_block_placement_fn,
)
from flex_shard_amd.custom_placements import quant_plan
from flex_shard_amd.testing import LLAMA3_8B_LAYER, FakeMesh, local_rows, make_param_infos
from oracle import layout as olayout


def _factory(fp8_data, recip_scale, block_size, *, orig_dtype, requires_grad):
    return fp8_data


def _meta_params(shapes, dtype=torch.float32):
    return [(f"w{i}", nn.Parameter(torch.empty(tuple(s), device="meta", dtype=dtype))) for i, s in enumerate(shapes)]


def _fp8(world_size, block):
    return Fp8BucketedBlockShard(world_size=world_size, weight_factory=_factory, block_size=block)


# --------------------------------------------------------------- the planner
def test_planner_is_optimal_on_every_small_instance():
    """The binary-searched capacity equals the exhaustive optimum, and the
    cuts respect it, for every cost vector up to 6 units over a small alphabet
    and a random sample of longer ones."""
    rng = random.Random(0)
    instances = [list(c) for n in range(1, 6) for c in itertools.product((1, 2, 5), repeat=n)]
    instances += [[rng.randint(1, 40) for _ in range(rng.randint(6, 9))] for _ in range(60)]
    for costs in instances:
        for parts in (1, 2, 3, 4):
            best = olayout.brute_force_min_capacity(costs, parts)
            assert olayout.min_capacity(costs, parts) == best
            assert quant_plan.min_partition_capacity(costs, parts) == best
            cuts = olayout.rank_cuts(costs, parts)
            assert cuts == quant_plan.rank_unit_cuts(costs, parts, best)
            assert len(cuts) == parts + 1 and cuts[0] == 0 and cuts[-1] == len(costs)
            assert list(cuts) == sorted(cuts)
            assert max(sum(costs[a:b]) for a, b in zip(cuts, cuts[1:])) == best


def test_planner_gives_every_rank_a_unit_when_it_can():
    # 5 equal units over 4 ranks: greedy fills 2+2+1, the split step must give
    # the 4th rank a unit rather than leave it empty.
    assert olayout.rank_cuts([1] * 5, 4) == (0, 1, 2, 4, 5)
    assert olayout.rank_cuts([7], 4) == (0, 1, 1, 1, 1)  # nothing to split: trailing ranks empty


def test_reference_layout_known_answers(golden):
    g = golden["fp8_layout_two_params"]
    named = _meta_params(g["shapes"])
    pl = _fp8(g["world_size"], g["block"])
    for rank in range(g["world_size"]):
        layout = pl.bucket_storage_layout(named, {f: (pl,) for f, _ in named}, FakeMesh(g["world_size"], rank))
        got = [list(layout.param_layouts[f].local_shape) for f, _ in named]
        assert got == g["local_shapes_by_rank"][rank]
        bucket = layout.param_layouts["w0"].bucket_layout
        assert list(bucket.rank_offsets) == g["rank_offsets"] and list(bucket.rank_numels) == g["rank_numels"]
    ol = olayout.quant_layout(g["shapes"], g["block"], g["world_size"])
    assert list(ol.rank_offsets) == g["rank_offsets"] and list(ol.rank_numels) == g["rank_numels"]

    g = golden["fp8_layout_partial_rows"]
    named = _meta_params(g["shapes"])
    pl = _fp8(g["world_size"], g["block"])
    for rank in range(g["world_size"]):
        layout = pl.bucket_storage_layout(named, {"w0": (pl,)}, FakeMesh(g["world_size"], rank))
        assert [list(layout.param_layouts["w0"].local_shape)] == g["local_shapes_by_rank"][rank]

    g = golden["fp8_layout_empty_rank"]
    named = _meta_params(g["shapes"])
    pl = _fp8(g["world_size"], g["block"])
    layout = pl.bucket_storage_layout(named, {"w0": (pl,)}, FakeMesh(g["world_size"], g["rank"]))
    assert layout.total_bytes == g["total_bytes"]
    assert layout.param_layouts["w0"].local_numel == g["local_numel"]
    assert layout.param_layouts["w0"].storage_nbytes == g["storage_nbytes"]


def test_local_row_ranges_fall_on_block_boundaries(golden):
    g = golden["fp8_layout_two_params"]
    named = _meta_params(g["shapes"])
    pl = _fp8(g["world_size"], g["block"])
    for rank in range(g["world_size"]):
        infos = make_param_infos(named, pl, FakeMesh(g["world_size"], rank))
        for (_, param), info in zip(named, infos):
            layout = info.bucket_layout.param_layouts[info.fqn]
            start = (layout.local_global_offset - layout.param_offset) // param.shape[1]
            end = start + info.local_shape[0]
            edges = {min(r, param.shape[0]) for r in range(0, param.shape[0] + g["block"], g["block"])}
            assert start in edges and end in edges


def test_stacked_weight_global_layouts(golden):
    g = golden["fp8_stacked_global_layouts"]
    param = nn.Parameter(torch.arange(96, dtype=torch.float32).reshape(g["shape"]))
    pl = _fp8(g["world_size"], g["block"])
    infos = [make_param_infos([("w13", param)], pl, FakeMesh(g["world_size"], r))[0] for r in range(g["world_size"])]
    assert [list(i.local_shape) for i in infos] == [g["local_shape"]] * g["world_size"]
    rebuilt = torch.zeros_like(param)
    for rank, info in enumerate(infos):
        layout = pl.global_layout(info, rank, g["world_size"])
        want = g["layouts"][rank]
        assert layout == GlobalLayout(
            tuple(g["shape"]),
            tuple(map(tuple, want["global_offsets"])),
            tuple(map(tuple, want["local_offsets"])),
            tuple(map(tuple, want["local_sizes"])),
        )
        shard = local_rows(param, info)
        for go, lo, sz in zip(layout.global_offsets, layout.local_offsets, layout.local_sizes):
            dst = tuple(slice(a, a + n) for a, n in zip(go, sz))
            src = tuple(slice(a, a + n) for a, n in zip(lo, sz))
            rebuilt[dst] = shard[src]
    assert torch.equal(rebuilt, param.detach())


def test_llama_layer_plan(golden):
    """The benchmark bucket: unit cuts, rank 0's share and the payload row size."""
    g = golden["llama3_8b_layer_plan"]
    shapes = [shape for _, shape in LLAMA3_8B_LAYER]
    ol = olayout.quant_layout(shapes, g["block"], g["world_size"])
    assert list(ol.cuts) == g["unit_cuts"]
    assert ol.rank_numels[0] == g["rank0_numel"] and ol.rank_scale_numels[0] == g["rank0_scales"]
    assert ol.row_nbytes == g["row_nbytes"] and sum(ol.rank_numels) == g["global_numel"]
    named = _meta_params(shapes, torch.bfloat16)
    pl = _fp8(g["world_size"], g["block"])
    infos = make_param_infos(named, pl, FakeMesh(g["world_size"], 0))
    md = pl._quant_metadata_from_infos(infos)
    assert md.packed_send_nbytes_per_rank == g["row_nbytes"]
    assert md.rank_qdata_numels == ol.rank_numels and md.rank_scale_numels == ol.rank_scale_numels
    assert [c.fqn for c in md.chunks if c.rank == 0] == ["w0", "w1", "w2", "w3"]
    assert [(c.row_start, c.row_end) for c in md.chunks if c.rank == 0] == [(0, 4096), (0, 1024), (0, 1024), (0, 512)]


def test_metadata_matches_naive_enumeration_on_random_buckets():
    rng = random.Random(7)
    for _ in range(40):
        block = rng.choice((2, 4, 8))
        world = rng.choice((1, 2, 3, 4, 8))
        shapes = []
        for _ in range(rng.randint(1, 4)):
            if rng.random() < 0.25:
                shapes.append((rng.randint(1, 3), rng.randint(1, 9), rng.randint(1, 12)))
            else:
                shapes.append((rng.randint(1, 20), rng.randint(1, 12)))
        ol = olayout.quant_layout(shapes, block, world)
        named = _meta_params(shapes)
        pl = _fp8(world, block)
        for rank in range(world):
            infos = make_param_infos(named, pl, FakeMesh(world, rank))
            md = pl._quant_metadata_from_infos(infos)
            assert md.rank_qdata_numels == ol.rank_numels
            assert md.rank_scale_numels == ol.rank_scale_numels
            assert md.rank_scale_byte_offsets == ol.rank_scale_byte_offsets
            assert md.rank_packed_nbytes == ol.rank_packed_nbytes
            assert md.packed_send_nbytes_per_rank == ol.row_nbytes
            bucket = infos[0].bucket_layout
            assert bucket.rank_offsets == ol.rank_offsets and bucket.rank_numels == ol.rank_numels
            ranges = olayout.local_row_ranges(ol, rank, len(shapes))
            for info, (lo, hi), shape in zip(infos, ranges, shapes):
                assert info.local_numel == (hi - lo) * shape[-1]
            # byte offsets of local shards are the running sum of earlier shards
            running = 0
            for info in infos:
                if info.local_numel:
                    assert info.byte_offset == running * 4
                    running += info.local_numel
        # the scale regions concatenate every rank's scales in rank order
        regions = md.scale_regions_by_index[0]
        assert sum(r.nbytes for r in regions) == 4 * sum(ol.rank_scale_numels)
        assert [r.rank for r in regions] == sorted(r.rank for r in regions)


def test_validation_errors():
    pl = _fp8(2, 4)
    with pytest.raises(ValueError, match="2D weights"):
        pl.bucket_storage_layout([("w", nn.Parameter(torch.zeros(16)))], {"w": (pl,)}, FakeMesh(2))
    with pytest.raises(ValueError, match="non-empty"):
        pl.bucket_storage_layout([("w", nn.Parameter(torch.zeros(0, 8)))], {"w": (pl,)}, FakeMesh(2))
    with pytest.raises(ValueError, match="one-byte"):
        Fp8BucketedBlockShard(world_size=2, weight_factory=_factory, block_size=4, fp8_dtype=torch.float16)
    with pytest.raises(TypeError, match="callable"):
        Fp8BucketedBlockShard(world_size=2, weight_factory=None)
    with pytest.raises(ValueError, match="positive"):
        Fp8BucketedBlockShard(world_size=0, weight_factory=_factory)
    with pytest.raises(ValueError, match="world size"):
        pl.bucket_storage_layout(_meta_params([(8, 8)]), {"w0": (pl,)}, FakeMesh(3))
    other = _fp8(2, 4)
    with pytest.raises(ValueError, match="same placement instance"):
        named = _meta_params([(8, 8)])
        pl.bucket_storage_layout(named, {"w0": (pl, other)}, FakeMesh(2))
    with pytest.raises(ValueError, match="one dtype per bucket"):
        named = [("a", nn.Parameter(torch.zeros(4, 4))), ("b", nn.Parameter(torch.zeros(4, 4, dtype=torch.bfloat16)))]
        pl.bucket_storage_layout(named, {"a": (pl,), "b": (pl,)}, FakeMesh(2))


def test_fp8_placement_value_semantics():
    a, b = _fp8(2, 4), _fp8(2, 4)
    assert a == b and hash(a) == hash(b)
    assert a != _fp8(4, 4) and a != _fp8(2, 8)
    assert a != Fp8BucketedBlockShard(world_size=2, weight_factory=lambda *x, **k: None, block_size=4)
    assert repr(a) == "Fp8BucketedBlockShard(world_size=2, block_size=4, weight_factory=_factory)"
    fn = make_fp8_bucketed_block_placement_fn(weight_factory=_factory, block_size=4)
    placements = fn(_meta_params([(8, 8), (4, 4)]), FakeMesh(4))
    assert placements["w0"][0] is placements["w1"][0] and placements["w0"][0].world_size == 4


# --------------------------------------------------------- BucketedBlockShard
def test_bucketed_block_shard_config_errors():
    with pytest.raises(ValueError, match="prefix dims"):
        BucketedBlockShard(dims=(1,), blocks_per_rank=(1, 1))
    with pytest.raises(ValueError, match="non-negative"):
        BucketedBlockShard(dims=(0,), blocks_per_rank=(1, -1))
    with pytest.raises(ValueError, match="at least one positive"):
        BucketedBlockShard(dims=(0,), blocks_per_rank=(0, 0))
    pl = BucketedBlockShard(dims=(0, 1), blocks_per_rank=(1,))
    with pytest.raises(ValueError, match="invalid for parameter shape"):
        pl.bucket_storage_layout([("w", nn.Parameter(torch.empty(2)))], {"w": (pl,)}, FakeMesh(1))
    pl = BucketedBlockShard(dims=(0,), blocks_per_rank=(1, 1))
    with pytest.raises(ValueError, match="world size"):
        pl.bucket_storage_layout([("w", nn.Parameter(torch.empty(2, 2)))], {"w": (pl,)}, FakeMesh(1))
    with pytest.raises(ValueError, match="mesh size"):
        make_bucketed_block_placement_fn(dims=(0,), blocks_per_rank=(1, 1))([], FakeMesh(3))
    a = BucketedBlockShard((0,), (1, 2))
    assert a == BucketedBlockShard((0,), (1, 2)) and hash(a) == hash(BucketedBlockShard((0,), (1, 2)))
    assert repr(a) == "BucketedBlockShard(dims=(0,), blocks_per_rank=(1, 2))"


def test_bucketed_block_shard_local_views(golden):
    """weight [4,2] + bias [4] with blocks (1,3): every rank's local params are
    the bucket-global ranges of the flattened params (reference:
    tests/test_flex_shard_block_shard.py:156-201)."""
    g = golden["dense_bucket_case"]
    weight = nn.Parameter(torch.arange(8, dtype=torch.float32).view(4, 2))
    bias = nn.Parameter(torch.arange(4, dtype=torch.float32))
    named = [("weight", weight), ("bias", bias)]
    pl = BucketedBlockShard(dims=(0,), blocks_per_rank=tuple(g["blocks_per_rank"]))
    ol = olayout.dense_bucket_layout(g["shapes"], g["blocks_per_rank"])
    for rank in range(2):
        infos = make_param_infos(named, pl, FakeMesh(2, rank))
        bucket = infos[0].bucket_layout
        assert bucket.global_numel == ol.global_numel
        assert bucket.rank_offsets == ol.rank_offsets and bucket.rank_numels == ol.rank_numels
        storage = torch.zeros(bucket.local_numel * 4, dtype=torch.uint8)
        for (fqn, param), info in zip(named, infos):
            pl.copy_param_to_storage(storage, info, param, rank, 2)
        for (fqn, param), info, offset in zip(named, infos, ol.param_offsets):
            lo = max(ol.rank_offsets[rank], offset)
            hi = min(ol.rank_offsets[rank] + ol.rank_numels[rank], offset + param.numel())
            want = param.detach().view(-1)[max(0, lo - offset) : max(0, hi - offset)]
            got = pl.make_local_storage_view(storage, info)
            assert torch.equal(got.reshape(-1), want)
            layout = pl.global_layout(info, rank, 2)
            if info.local_numel:
                assert layout.global_offsets[0][0] == (lo - offset) // max(1, param[0].numel())


def test_padding_only_rank_is_rejected():
    pl = BucketedBlockShard(dims=(0,), blocks_per_rank=(1, 1))
    named = [("weight", nn.Parameter(torch.arange(4, dtype=torch.float32).view(1, 4)))]
    layout = pl.bucket_storage_layout(named, {"weight": (pl,)}, FakeMesh(2, 0))
    assert layout.total_bytes == 16
    with pytest.raises(ValueError, match="contains only padding"):
        pl.bucket_storage_layout(named, {"weight": (pl,)}, FakeMesh(2, 1))


def test_llama_dense_bucket_layout(golden):
    g = golden["llama3_8b_dense_bucket"]
    shapes = [shape for _, shape in LLAMA3_8B_LAYER]
    ol = olayout.dense_bucket_layout(shapes, (1,) * 8)
    assert ol.alignment == g["alignment"] and list(ol.param_offsets) == g["param_offsets"]
    assert ol.global_numel == g["global_numel"] and set(ol.rank_numels) == {g["rank_numel"]}
    pl = BucketedBlockShard(dims=(0,), blocks_per_rank=(1,) * 8)
    infos = make_param_infos(_meta_params(shapes, torch.bfloat16), pl, FakeMesh(8, 0))
    bucket = infos[0].bucket_layout
    assert bucket.global_numel == g["global_numel"]
    assert [bucket.param_layouts[i.fqn].param_offset for i in infos] == g["param_offsets"]


def test_reduce_copy_in_plan_covers_every_row_element_once(golden):
    """The one-pass plan's copy and zero segments tile the [W, longest range]
    send rows exactly (no gaps, no overlaps), for the reference's cases and
    for rows wider than the group."""
    cases = []
    for case in golden["reduce_copy_in_cases"]["fp8_layout_cases"].values():
        cases.append((_fp8(case["world_size"], 4), case["shapes"], case["world_size"]))
    dense = golden["reduce_copy_in_cases"]["dense_case"]
    cases.append((BucketedBlockShard(dims=(0,), blocks_per_rank=tuple(dense["blocks_per_rank"])), dense["shapes"], 4))
    for pl, shapes, world in cases:
        infos = make_param_infos(_meta_params(shapes, torch.bfloat16), pl, FakeMesh(world))
        widest = max(infos[0].bucket_layout.rank_numels)
        for extra in (0, 5):
            stride = widest + extra
            plan = pl._reduce_copy_in_plan(infos, stride)
            cover = torch.zeros(world * stride, dtype=torch.int32)
            for segments in plan.param_segments:
                for _, n, dst in segments:
                    cover[dst : dst + n] += 1
            for dst, n in plan.zero_segments:
                cover[dst : dst + n] += 1
            rows = cover.view(world, stride)
            assert (rows[:, :widest] == 1).all() and (rows[:, widest:] == 0).all()
        assert pl._reduce_copy_in_plan(infos, widest) is pl._reduce_copy_in_plan(infos, widest)
    (plan,) = [p for k, p in cases[-1][0]._reduce_copy_in_plans.items() if k[2] == max(infos[0].bucket_layout.rank_numels)]
    assert len(plan.zero_segments) > 4  # gaps between params plus every row's tail


def test_copy_out_plan_regions(golden):
    g = golden["fused_copy_out_cases"]
    for case in g["cases"].values():
        pl = _fp8(g["world_size"], g["block"])
        infos = make_param_infos(_meta_params(case["shapes"]), pl, FakeMesh(g["world_size"]))
        md = pl._quant_metadata_from_infos(infos)
        assert 0 in md.rank_qdata_numels
        plan = pl._copy_out_plan(md, data_elem_nbytes=1, with_scales=True)
        assert plan.vec_aligned == (case["aligned_unit"] == 4)
        data_total = sum(md.rank_qdata_numels)
        cursor = 0
        for rank, offset, nbytes, dst in plan.regions:
            if offset == 0 and dst < data_total:
                assert dst == cursor and nbytes == md.rank_qdata_numels[rank]
                cursor += nbytes
        assert cursor == data_total
        scale_regions = [r for r in plan.regions if r[3] >= data_total]
        assert scale_regions[0][3] == -(-data_total // 16) * 16
        assert pl._copy_out_plan(md, data_elem_nbytes=1, with_scales=True) is plan
