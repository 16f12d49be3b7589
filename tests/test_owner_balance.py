"""Owner assignment of whole-parameter placements against the known answers
of the reference's own tests (src/flex_shard/tests/test_matrix_assignment.py
:266-275 hosts of mesh ranks, :276-318 the second bucket's carried loads,
:349-359 hosts before ranks, :361-404 loads carried across buckets).  Host
math only."""

import os
from unittest import mock
from unittest.mock import MagicMock

import torch
import torch.nn as nn

from flex_shard_amd import make_bucketed_owned_full_param_placement_fn
from flex_shard_amd.custom_placements.owned import make_bucketed_owned_full_param_segments
from flex_shard_amd.custom_placements.owner_balance import assign_to_hosts_then_ranks, mesh_rank_hosts

# One MoE layer's whole Muon matrices of DeepSeek V3 671B: attention wo and
# wq_a, the shared experts' gate and up, down, router.
_MOE_LAYER = (7168 * 16384, 1536 * 7168, 2048 * 7168, 2048 * 7168, 7168 * 2048, 256 * 7168)


def test_mesh_rank_hosts():
    assert mesh_rank_hosts(range(8), 4) == (0, 0, 0, 0, 1, 1, 1, 1)
    # a mesh of global ranks (one pipeline stage's data-parallel ranks): hosts are numbered in mesh order
    assert mesh_rank_hosts((64, 65, 72, 73), 8) == (0, 0, 1, 1)
    assert mesh_rank_hosts(range(4), 1) == (0, 1, 2, 3)
    with mock.patch.dict(os.environ, {"LOCAL_WORLD_SIZE": "2"}):
        assert mesh_rank_hosts(range(4)) == (0, 0, 1, 1)


def test_heavy_and_light_hosts_alternate():
    """Four MoE layers on 64 ranks of 8 hosts: each wo exceeds a host's share
    (117.4M against 87.2M), so the hosts holding one alternate with the others,
    and a second bucket balanced against the carried loads flips them."""
    hosts = mesh_rank_hosts(range(64), 8)
    numels = [numel for _ in range(4) for numel in _MOE_LAYER]
    first = assign_to_hosts_then_ranks(numels, hosts, one_per_rank=True)
    assert sorted(hosts[first[6 * layer]] for layer in range(4)) == [0, 2, 4, 6]
    loads = [0] * 8
    for numel, rank in zip(numels, first):
        loads[hosts[rank]] += numel
    assert loads[0::2] == [_MOE_LAYER[0]] * 4
    assert loads[1::2] == [sum(_MOE_LAYER) - _MOE_LAYER[0]] * 4
    carried = [0] * 64
    for numel, rank in zip(numels, first):
        carried[rank] += numel
    second = assign_to_hosts_then_ranks(numels, hosts, carried_loads=carried, one_per_rank=True)
    assert sorted(hosts[second[6 * layer]] for layer in range(4)) == [1, 3, 5, 7]


def test_one_host_alternates_ranks():
    owners = assign_to_hosts_then_ranks((100, 100, 100, 100, 10, 10, 10, 10), (0,) * 8, one_per_rank=True)
    assert sorted(owners[:4]) == [0, 2, 4, 6]


def test_bucketed_owned_segments_place_hosts_first():
    named = [(f"p{i}", nn.Parameter(torch.empty(n))) for i, n in enumerate((100, 100, 10, 10))]
    two_level = make_bucketed_owned_full_param_segments(named, 8, hosts=mesh_rank_hosts(range(8), 4))
    rank_order = make_bucketed_owned_full_param_segments(named, 8)
    assert {two_level[p][0].owner_rank for p in ("p0", "p1")} == {0, 4}
    assert {rank_order[p][0].owner_rank for p in ("p0", "p1")} == {0, 1}


def test_placement_fn_carries_loads_across_buckets():
    """16 identical buckets of a DeepSeek V3 MoE block's owned matrices on 64
    ranks of 8 hosts: placed one at a time every bucket gets the same 6 owners;
    carrying the loads spreads them over the ranks."""
    shapes = ((7168, 16384), (1536, 7168), (576, 7168), (256, 7168), (2, 2048, 7168), (7168, 2048))
    mesh = MagicMock()
    mesh.mesh = torch.arange(64)
    mesh.size.return_value = 64

    def owned_numel(placement_fn):
        loads = [0] * 64
        for block in range(16):
            named = [(f"layers.{block}.m{i}", nn.Parameter(torch.empty(s, device="meta"))) for i, s in enumerate(shapes)]
            for fqn, (placement,) in placement_fn(named, mesh).items():
                for segment in placement.segments_by_fqn[fqn]:
                    loads[segment.owner_rank] += segment.numel
        return loads

    with mock.patch.dict(os.environ, {"LOCAL_WORLD_SIZE": "8"}):
        per_bucket = owned_numel(make_bucketed_owned_full_param_placement_fn())
        carried = owned_numel(make_bucketed_owned_full_param_placement_fn(carry_loads=True))
    assert sum(load > 0 for load in per_bucket) == 6
    assert max(per_bucket) == 16 * 7168 * 16384
    # each rank owns at most one wo and about a fair share in all
    assert sum(load > 0 for load in carried) >= 60
    assert max(carried) <= 7168 * 16384 + sum(carried) // 64
