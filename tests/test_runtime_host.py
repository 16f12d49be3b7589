"""Host logic of the runtime slice that needs no GPU: the one-GPU group's
local all-gather and the bucket placement compatibility check."""

import pytest
import torch
import torch.nn as nn

from flex_shard_amd import Fp8BucketedBlockShard, LocalReduceGroup
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
