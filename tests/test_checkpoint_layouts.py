"""Checkpoint layouts: the known answers of the reference's own layout tests
(src/flex_shard/tests/test_flex_shard_checkpoint.py:119-190, 247-255, 274-292,
331-339, 354-372), the property that every rank's boxes tile the full
parameter exactly once for every placement, re-sharding between mesh sizes
through the layouts alone, and the optimizer-state hook.  All on the CPU."""

from types import SimpleNamespace

import pytest
import torch
import torch.nn as nn

from flex_shard_amd import (
    BlockShard,
    BucketedBlockShard,
    BucketedOwned,
    Fp8BucketedBlockShard,
    GlobalLayout,
    Shard,
    compose_global_layouts,
    get_global_layout,
    set_global_layout,
)
from flex_shard_amd.custom_placements.owned import BucketedOwnedSegmentSpec
from flex_shard_amd.flex_shard import (
    copy_full_into_shard,
    copy_shard_into_full,
    get_flex_shard_global_layouts,
    register_optimizer_checkpoint_hook,
    set_state_dict_global_layouts,
)
from flex_shard_amd.testing import FakeMesh, make_param_infos


def _factory(fp8_data, recip_scale, block_size, *, orig_dtype, requires_grad):
    return fp8_data


def _infos(named, placement, rank, world_size):
    """Bucket placements lay the bucket out; per-parameter ones (BlockShard)
    get one parameter after the other."""
    return make_param_infos(named, placement, FakeMesh(world_size, rank))


def _layouts(named, placement, rank, world_size):
    infos = _infos(named, placement, rank, world_size)
    return {i.fqn: placement.global_layout(i, rank, world_size) for i in infos}


def _one(placement, shape, rank, world_size):
    return _layouts([("weight", nn.Parameter(torch.empty(shape)))], placement, rank, world_size)["weight"]


# ------------------------------------------------------------------ known answers of the reference's tests
def test_shard_uneven_and_empty_ranks():
    assert _one(Shard(0), (5, 4), 1, 2) == GlobalLayout((5, 4), ((3, 0),), ((0, 0),), ((2, 4),))
    assert _one(Shard(0), (1, 4), 2, 3) == GlobalLayout((1, 4), (), (), ())


def test_block_shard_along_columns():
    placement = BlockShard(blocks_per_rank=(2, 0, 1), dim=1)
    assert _one(placement, (2, 6), 2, 3) == GlobalLayout((2, 6), ((0, 4),), ((0, 0),), ((2, 2),))


def test_bucketed_owned_row_segments():
    placement = BucketedOwned(
        {"slabs": [BucketedOwnedSegmentSpec(f"slabs#{row}", "slabs", 4 * row, 4, owner) for row, owner in enumerate((0, 0, 1))]}
    )
    named = [("slabs", nn.Parameter(torch.empty(3, 4)))]
    assert _layouts(named, placement, 1, 2)["slabs"] == GlobalLayout((3, 4), ((2, 0),), ((0, 0),), ((1, 4),))


def test_bucketed_block_shard_second_parameter():
    placement = BucketedBlockShard(dims=(0,), blocks_per_rank=(1, 1))
    named = [("prefix", nn.Parameter(torch.empty(2, 3))), ("weight", nn.Parameter(torch.empty(4, 3)))]
    assert _layouts(named, placement, 1, 2)["weight"] == GlobalLayout((4, 3), ((1, 0),), ((0, 0),), ((3, 3),))


def test_compose_multi_chunk():
    # the intermediate tensor stacks global rows [1, 3) and [5, 7); the local
    # tensor holds intermediate row 1 and a column slab of rows 2-3
    outer = GlobalLayout((8, 6), ((1, 0), (5, 0)), ((0, 0), (2, 0)), ((2, 6), (2, 6)))
    inner = GlobalLayout((4, 6), ((1, 0), (2, 2)), ((0, 0), (1, 2)), ((1, 6), (2, 4)))
    assert compose_global_layouts(outer, inner) == GlobalLayout(
        (8, 6), ((2, 0), (5, 2)), ((0, 0), (1, 2)), ((1, 6), (2, 4))
    )


def test_prefix_dims_beyond_rows_are_not_checkpointable():
    placement = BucketedBlockShard(dims=(0, 1))
    named = [("weight", nn.Parameter(torch.arange(24.0).view(2, 3, 4)))]
    info = make_param_infos(named, placement, FakeMesh(1, 0))[0]
    with pytest.raises(NotImplementedError, match="distributed checkpointing supports only dims"):
        placement.global_layout(info, 0, 1)


# ------------------------------------------------------------------ every element exactly once; re-sharding
def _cases():
    torch.manual_seed(0)
    dense = [("a", nn.Parameter(torch.randn(5, 4))), ("b", nn.Parameter(torch.randn(7))), ("c", nn.Parameter(torch.randn(3, 2, 4)))]
    rows = [("q", nn.Parameter(torch.randn(12, 8))), ("k", nn.Parameter(torch.randn(20, 8)))]
    yield "shard0", dense, lambda w: Shard(0), (1, 2, 3, 4)
    yield "block_shard_cols", [("w", nn.Parameter(torch.randn(3, 12)))], lambda w: BlockShard((2, 0, 1)[:w] if w == 3 else (1,) * w, dim=1), (2, 3)
    yield "bucketed_block_shard", [dense[0], dense[1]], lambda w: BucketedBlockShard(dims=(0,), blocks_per_rank=(1,) * w), (1, 2, 3)
    yield "fp8_bucketed_block_shard", rows, lambda w: Fp8BucketedBlockShard(world_size=w, weight_factory=_factory, block_size=4), (1, 2, 3, 5)


@pytest.mark.parametrize("name,named,make_placement,world_sizes", list(_cases()), ids=[c[0] for c in _cases()])
def test_rank_boxes_tile_the_full_parameter(name, named, make_placement, world_sizes):
    fulls = {fqn: p.detach().clone() for fqn, p in named}
    previous = None
    for world_size in world_sizes:
        placement = make_placement(world_size)
        cover = {fqn: torch.zeros_like(t) for fqn, t in fulls.items()}
        rebuilt = {fqn: torch.full_like(t, float("nan")) for fqn, t in fulls.items()}
        shards = []
        for rank in range(world_size):
            infos = _infos(named, placement, rank, world_size)
            mine = {}
            for info in infos:
                layout = placement.global_layout(info, rank, world_size)
                assert layout.global_shape == tuple(fulls[info.fqn].shape)
                local = torch.full(tuple(info.local_shape), float("nan"))
                # load: the rank's shard out of the full tensor (or out of the previous mesh's shards)
                copy_full_into_shard(local, previous[info.fqn] if previous else fulls[info.fqn], layout)
                assert not torch.isnan(local).any(), "a layout must name every local element"
                _count_boxes(cover[info.fqn], layout)
                copy_shard_into_full(rebuilt[info.fqn], local, layout)
                mine[info.fqn] = local
            shards.append(mine)
        for fqn, full in fulls.items():
            assert torch.equal(cover[fqn], torch.ones_like(full)), f"{name} W={world_size}: {fqn} not covered exactly once"
            assert torch.equal(rebuilt[fqn], full)
        previous = rebuilt  # the next mesh size loads from what this one saved


def _count_boxes(cover, layout):
    for offsets, sizes in zip(layout.global_offsets, layout.local_sizes, strict=True):
        cover[tuple(slice(o, o + n) for o, n in zip(offsets, sizes, strict=True))] += 1


def test_shard0_shards_match_the_placements_own_cut():
    full = torch.arange(35.0).view(7, 5)
    for world_size in (2, 3, 4):
        for rank in range(world_size):
            want = Shard(0).extract_local_shard(full, rank, world_size)
            layout = _layouts([("w", nn.Parameter(full.clone()))], Shard(0), rank, world_size)["w"]
            got = torch.empty(want.shape)
            copy_full_into_shard(got, full, layout)
            assert torch.equal(got, want)


def test_copy_checks_the_full_shape():
    layout = GlobalLayout((4, 3), ((0, 0),), ((0, 0),), ((2, 3),))
    with pytest.raises(ValueError, match=r"shape \(4, 3\)"):
        copy_shard_into_full(torch.zeros(5, 3), torch.zeros(2, 3), layout)
    with pytest.raises(ValueError, match=r"shape \(4, 3\)"):
        copy_full_into_shard(torch.zeros(2, 3), torch.zeros(5, 3), layout)


# ------------------------------------------------------------------ state dicts and optimizer states
def _runtime(model, placement, rank=0, world_size=1):
    """What the checkpoint helpers read of a bucket runtime, built on the CPU."""
    named = list(model.named_parameters())
    mesh = FakeMesh(world_size, rank)
    infos = make_param_infos(named, placement, mesh)
    bucket_params = []
    for (fqn, param), info in zip(named, infos, strict=True):
        info.outer_layout = get_global_layout(param)
        sharded = nn.Parameter(placement.extract_local_shard(param.detach(), rank, world_size).clone())
        module_path, _, leaf = fqn.rpartition(".")
        (model.get_submodule(module_path) if module_path else model)._parameters[leaf] = sharded
        bucket_params.append(SimpleNamespace(info=info, sharded_param=sharded))
    return SimpleNamespace(infos=infos, mesh=mesh, bucket_params=bucket_params)


def _adam_step(model, optimizer):
    for param in model.parameters():
        param.grad = torch.ones_like(param)
    optimizer.step()


def test_state_dict_composes_declared_outer_layout():
    model = nn.Module()
    model.weight = nn.Parameter(torch.empty(4, 3))
    layout = GlobalLayout((8, 3), ((4, 0),), ((0, 0),), ((4, 3),))
    set_global_layout(model.weight, layout)
    runtime = _runtime(model, Shard(0))
    state_dict = model.state_dict()
    set_state_dict_global_layouts([runtime], state_dict)
    assert get_global_layout(state_dict["weight"]) == layout
    # rank 1 of 2 holds rows [2, 4) of the intermediate tensor = global rows [6, 8)
    model2 = nn.Module()
    model2.weight = nn.Parameter(torch.empty(4, 3))
    set_global_layout(model2.weight, layout)
    got = get_flex_shard_global_layouts([_runtime(model2, Shard(0), 1, 2)])["weight"]
    assert got == GlobalLayout((8, 3), ((6, 0),), ((0, 0),), ((2, 3),))


def test_states_take_their_parameters_layouts():
    model = nn.Module()
    model.weight = nn.Parameter(torch.arange(12.0).view(4, 3))
    model.bias = nn.Parameter(torch.arange(4.0))
    weight_layout = GlobalLayout((8, 3), ((4, 0),), ((0, 0),), ((4, 3),))
    set_global_layout(model.weight, weight_layout)
    runtime = _runtime(model, Shard(0))
    optimizer = torch.optim.Adam(model.parameters(), amsgrad=True)
    register_optimizer_checkpoint_hook(optimizer, [runtime])
    _adam_step(model, optimizer)
    state = optimizer.state_dict()["state"]
    bias_layout = GlobalLayout((4,), ((0,),), ((0,),), ((4,),))
    for param_id, layout in ((0, weight_layout), (1, bias_layout)):
        for state_name in ("exp_avg", "exp_avg_sq", "max_exp_avg_sq"):
            assert get_global_layout(state[param_id][state_name]) == layout
        assert get_global_layout(state[param_id]["step"]) is None


def test_unsupported_optimizer_raises():
    model = nn.Linear(4, 5)
    runtime = _runtime(model, Shard(0))
    optimizer = torch.optim.SGD(model.parameters(), lr=0.1, momentum=0.9)
    with pytest.raises(NotImplementedError, match="supports Adam and AdamW, got SGD"):
        register_optimizer_checkpoint_hook(optimizer, [runtime])


def test_state_shape_mismatch_raises():
    model = nn.Linear(4, 5)
    runtime = _runtime(model, Shard(0))
    optimizer = torch.optim.Adam(model.parameters())
    register_optimizer_checkpoint_hook(optimizer, [runtime])
    _adam_step(model, optimizer)
    optimizer.state[model.weight]["exp_avg"] = torch.zeros(1)
    with pytest.raises(NotImplementedError, match=r"'exp_avg' of FlexShard parameter 'weight' has shape \(1,\)"):
        optimizer.state_dict()


def test_registering_again_replaces_the_hook():
    model = nn.Linear(4, 5)
    runtime = _runtime(model, Shard(0))
    optimizer = torch.optim.Adam(model.parameters())
    register_optimizer_checkpoint_hook(optimizer, [runtime])
    register_optimizer_checkpoint_hook(optimizer, [runtime])
    assert len(optimizer._optimizer_state_dict_post_hooks) == 1
