"""Host logic of the runtime slice that needs no GPU: the one-GPU group's
local all-gather and the bucket placement compatibility check."""

import pytest
import torch
import torch.nn as nn

from flex_shard_amd import Fp8BucketedBlockShard, LocalReduceGroup, MixedBucketPlacement, Shard
from flex_shard_amd.custom_placements.utils import all_gather_rows, group_size
from flex_shard_amd.flex_shard.bucket_comm import _get_bucket_placement
from flex_shard_amd.testing import FakeMesh, make_param_infos


def _factory(fp8_data, recip_scale, block_size, *, orig_dtype, requires_grad):
    return fp8_data


def test_local_all_gather_places_every_rank_row():
    group = LocalReduceGroup(3, 1)
    assert group_size(group) == 3
    mine = torch.arange(4, dtype=torch.uint8) + 10
    out = torch.zeros(12, dtype=torch.uint8)
    with pytest.raises(ValueError, match=r"rows of ranks \[0, 2\]"):
        all_gather_rows(out, mine, group)
    group.gather_rows[0] = torch.arange(4, dtype=torch.uint8)
    group.gather_rows[2] = torch.arange(4, dtype=torch.uint8) + 20
    assert all_gather_rows(out, mine, group) is None
    assert out.tolist() == [0, 1, 2, 3, 10, 11, 12, 13, 20, 21, 22, 23]
    with pytest.raises(ValueError, match="expected 3 x 4"):
        all_gather_rows(torch.zeros(8, dtype=torch.uint8), mine, group)
    with pytest.raises(ValueError, match="process group"):
        all_gather_rows(out, mine, None)
    solo = torch.zeros(4, dtype=torch.uint8)
    all_gather_rows(solo, mine, LocalReduceGroup(1, 0))
    assert torch.equal(solo, mine)


def test_bucket_placement_must_be_compatible():
    a = Fp8BucketedBlockShard(world_size=2, weight_factory=_factory)
    b = Fp8BucketedBlockShard(world_size=2, weight_factory=_factory, block_size=64)
    named = [("w", nn.Parameter(torch.empty(256, 128, device="meta", dtype=torch.bfloat16)))]
    info_a = make_param_infos(named, a, FakeMesh(2, 0))[0]
    info_b = make_param_infos(named, b, FakeMesh(2, 0))[0]
    assert _get_bucket_placement([info_a, info_a], "unshard") is a
    with pytest.raises(ValueError, match="compatible placements"):
        _get_bucket_placement([info_a, info_b], "unshard")


def test_member_and_factory_errors():
    mixed, other = MixedBucketPlacement({}), MixedBucketPlacement({})
    raw = Fp8BucketedBlockShard(world_size=2, weight_factory=_factory, block_size=4)
    member = mixed.blockwise_quant_bucketed_block_shard(raw)
    assert mixed.blockwise_quant_bucketed_block_shard(raw) is member
    with pytest.raises(NotImplementedError, match="one blockwise quantized placement instance"):
        mixed.blockwise_quant_bucketed_block_shard(
            Fp8BucketedBlockShard(world_size=2, weight_factory=_factory, block_size=4)
        )
    with pytest.raises(NotImplementedError, match="BlockShard members"):
        mixed.block_shard(blocks_per_rank=(1, 1))
    named = [("n", nn.Parameter(torch.zeros(8, dtype=torch.bfloat16)))]
    with pytest.raises(ValueError, match="different bucket instances"):
        mixed.bucket_storage_layout(named, {"n": (other.shard0,)}, FakeMesh(2, 0))
    with pytest.raises(TypeError, match="mixed member placements"):
        mixed.bucket_storage_layout(named, {"n": (Shard(0),)}, FakeMesh(2, 0))
    with pytest.raises(NotImplementedError, match="only dim 0"):
        Shard(1)


def test_shard0_round_trip_on_three_ranks():
    """Uneven chunks (5 rows and 4 elements over 3 ranks): every rank's
    unshard returns the full parameters; layouts report the chunk boxes."""
    placement = Shard(0)
    named = [("a", nn.Parameter(torch.arange(10.0).view(5, 2))), ("b", nn.Parameter(torch.arange(4.0)))]
    prepared = []
    for rank in range(3):
        group = LocalReduceGroup(3, rank)
        mesh = FakeMesh(3, rank, group)
        infos = make_param_infos(named, placement, mesh)
        shards = [placement.extract_local_shard(p.detach(), rank, 3) for _, p in named]
        assert [tuple(i.local_shape) for i in infos] == [tuple(s.shape) for s in shards]
        layout = placement.global_layout(infos[0], rank, 3)
        assert layout.global_offsets == (((2 * rank, 0),) if rank < 3 and infos[0].local_numel else ())
        prepared.append((placement.prepare_unshard_bucket(shards, infos, mesh, None), group))
    assert [p.buffers[0].numel() for p, _ in prepared] == [6, 6, 6]  # rank 0's capacity on every rank
    for rank, (mine, group) in enumerate(prepared):
        for other, (theirs, _) in enumerate(prepared):
            if other != rank:
                group.gather_rows[other] = theirs.buffers[0]
        placement.run_prepared_unshard(mine)
        full = placement.finish_prepared_unshard(mine).full_params
        assert torch.equal(full[0], named[0][1].detach()) and torch.equal(full[1], named[1][1].detach())
    # one rank: no exchange buffers, the reduction divides in place
    mesh = FakeMesh(1, 0, LocalReduceGroup(1, 0))
    infos = make_param_infos(named, placement, mesh)
    solo = placement.prepare_unshard_bucket([p.detach() for _, p in named], infos, mesh, None)
    assert len(solo.buffers) == 1 and placement.run_prepared_unshard(solo) is None
    assert torch.equal(placement.finish_prepared_unshard(solo).full_params[0], named[0][1].detach())
    from flex_shard_amd import GradientReduction

    grads = [torch.ones(5, 2), torch.full((4,), 2.0)]
    reduced = placement.reduce_prepared_grad(placement.prepare_reduce_grad(grads, infos, mesh, None), GradientReduction())
    assert torch.equal(reduced.sharded_grads[0], grads[0]) and torch.equal(reduced.sharded_grads[1], grads[1])
