"""GPU parity of the dense ``BucketedBlockShard`` unshard at several ranks with
uneven rank ranges: cast copy-in, zero-padded send row, uneven-range copy-out,
first persistent copy and in-place refill
(custom_placements/block_shard.py:932-1051).

Every rank of the mesh is run on the one GPU through ``LocalReduceGroup``:
prepare on each rank, exchange the send rows locally, run + finish on each
rank.  The expected result is the originals themselves: the unshard is a
permutation-free copy, so full parameters must equal the originals (cast to
the unsharded dtype) bit for bit, on every rank.
"""

import pytest
import torch
import torch.nn as nn

from flex_shard_amd import BucketedBlockShard, LocalReduceGroup
from flex_shard_amd.testing import FakeMesh, make_param_infos

pytestmark = pytest.mark.gpu


def _rank_state(named, blocks_per_rank, rank, device, param_dtype):
    world = len(blocks_per_rank)
    placement = BucketedBlockShard(dims=(0,), blocks_per_rank=tuple(blocks_per_rank))
    group = LocalReduceGroup(world, rank)
    mesh = FakeMesh(world, rank, group)
    infos = make_param_infos(named, placement, mesh)
    for info in infos:
        info.param_dtype = param_dtype
    layout = infos[0].bucket_layout
    storage = torch.zeros(layout.local_numel * named[0][1].dtype.itemsize, dtype=torch.uint8, device=device)
    for (_, param), info in zip(named, infos):
        placement.copy_param_to_storage(storage, info, param, rank, world)
    shards = [placement.make_local_storage_view(storage, info) for info in infos]
    return placement, group, mesh, infos, storage, shards


def _unshard_every_rank(named, blocks_per_rank, device, param_dtype, *, persistent_by_rank=None):
    """prepare on every rank -> local exchange -> run + finish on every rank."""
    world = len(blocks_per_rank)
    states = [_rank_state(named, blocks_per_rank, r, device, param_dtype) for r in range(world)]
    prepared = [
        st[0].prepare_unshard_bucket(st[5], st[3], st[2], None) for st in states
    ]
    results = []
    for rank, (st, prep) in enumerate(zip(states, prepared)):
        placement, group = st[0], st[1]
        group.gather_rows = {other: prepared[other].buffers[0] for other in range(world) if other != rank}
        if persistent_by_rank is not None:
            prep.persistent = True
            prep.persistent_buffers = persistent_by_rank[rank]
        placement.run_prepared_unshard(prep)
        results.append(placement.finish_prepared_unshard(prep))
    return states, prepared, results


CASES = [
    # (shapes, blocks_per_rank): the reference's known-answer bucket, then uneven three- and four-rank meshes
    ([(4, 2), (4,)], (1, 3)),
    ([(7, 3), (5, 4), (9, 3)], (2, 1, 0, 3)),
    ([(130, 24), (64, 24), (17, 8)], (3, 1, 2)),
    ([(256, 512), (384, 512), (512,)], (1, 3)),
    ([(96, 128), (128, 128)], (1, 1, 1, 1)),  # equal ranges: the gather lands in the bucket, no copy-out
]


@pytest.mark.parametrize("shapes,blocks", CASES)
@pytest.mark.parametrize("master,unsharded", [(torch.float32, torch.bfloat16), (torch.float32, None), (torch.bfloat16, None)])
def test_dense_unshard_restores_every_parameter(device, shapes, blocks, master, unsharded):
    gen = torch.Generator().manual_seed(len(shapes) * 17 + len(blocks))
    named = [(f"p{i}", nn.Parameter(torch.randn(s, generator=gen).to(master).to(device))) for i, s in enumerate(shapes)]
    want_dtype = unsharded or master
    states, prepared, results = _unshard_every_rank(named, blocks, device, unsharded)
    layout = states[0][3][0].bucket_layout
    widest = max(layout.rank_numels)
    for rank, (st, prep, result) in enumerate(zip(states, prepared, results)):
        assert len(result.full_params) == len(named) and not result.persistent_buffers
        for (_, param), full in zip(named, result.full_params):
            assert full.dtype == want_dtype and full.shape == param.shape
            assert torch.equal(full, param.detach().to(want_dtype))
    # the send row of a short rank is its range followed by zeros up to the longest range
    for rank, (st, prep) in enumerate(zip(states, prepared)):
        count = layout.rank_numels[rank]
        # prepared.buffers[0] is the send row (run inserted the bucket after it)
        send = prep.buffers[0]
        if count == 0:
            continue
        flat_local = st[4].view(master)[:count].to(want_dtype)
        if uneven := len(set(layout.rank_numels)) > 1:
            assert send.numel() == widest
            assert torch.equal(send[:count], flat_local) and not send[count:].any()
        else:
            assert send.numel() == count and torch.equal(send, flat_local)
        if not uneven and want_dtype == master:
            assert send.data_ptr() == st[4].data_ptr()  # view-in: the storage itself is the send row


def test_reference_known_answer_blocks_1_3(device, golden):
    """tests/test_flex_shard_block_shard.py:156-201: weight arange(8).view(4, 2)
    and bias arange(4) in fp32 on blocks_per_rank (1, 3): the local views of the
    two ranks, and the unshard restores both parameters on both ranks."""
    case = golden["dense_bucket_case"]
    assert case["blocks_per_rank"] == [1, 3]
    weight = nn.Parameter(torch.arange(8, dtype=torch.float32, device=device).view(4, 2))
    bias = nn.Parameter(torch.arange(4, dtype=torch.float32, device=device))
    named = [("weight", weight), ("bias", bias)]
    states, prepared, results = _unshard_every_rank(named, (1, 3), device, None)
    layout = states[0][3][0].bucket_layout
    # alignment lcm(2, 1) = 2, offsets 0 and 8, 12 elements padded to 2 * 4 blocks -> 16; ranges 4 and 12
    assert layout.global_numel == 16 and layout.rank_offsets == (0, 4) and layout.rank_numels == (4, 12)
    rank0, rank1 = states[0][5], states[1][5]
    assert torch.equal(rank0[0], weight.detach()[:2]) and rank0[1].numel() == 0
    assert torch.equal(rank1[0], weight.detach()[2:]) and torch.equal(rank1[1], bias.detach())
    for result in results:
        assert torch.equal(result.full_params[0], weight.detach()) and torch.equal(result.full_params[1], bias.detach())


@pytest.mark.parametrize("shapes,blocks", [([(7, 3), (5, 4), (9, 3)], (2, 1, 0, 3)), ([(256, 512), (384, 512), (512,)], (1, 3)),
                                           ([(96, 128), (128, 128)], (1, 1))])
def test_persistent_unshard_and_in_place_refill(device, shapes, blocks):
    """First persistent unshard: full parameters view a buffer finish
    allocates on the current stream (bucket.copy_(gathered)).  A refill gets
    the buffer back and writes it in place: same storage, same views, new
    values; finish then returns no new full parameters."""
    gen = torch.Generator().manual_seed(23)
    named = [(f"p{i}", nn.Parameter(torch.randn(s, generator=gen).to(device))) for i, s in enumerate(shapes)]
    world = len(blocks)
    states, prepared, first = _unshard_every_rank(
        named, blocks, device, torch.bfloat16, persistent_by_rank=[None] * world
    )
    buffers = [r.persistent_buffers for r in first]
    for result, prep in zip(first, prepared):
        (bucket,) = result.persistent_buffers
        assert bucket.data_ptr() != prep.buffers[1].data_ptr()  # its own allocation, not the gathered temporary
        for (_, param), full in zip(named, result.full_params):
            assert torch.equal(full, param.detach().bfloat16())
            assert full.untyped_storage().data_ptr() == bucket.untyped_storage().data_ptr()
    with torch.no_grad():
        for _, param in named:
            param.mul_(-1.5).add_(0.25)
    pointers = [b[0].data_ptr() for b in buffers]
    _, _, refill = _unshard_every_rank(named, blocks, device, torch.bfloat16, persistent_by_rank=buffers)
    for rank, (result, earlier) in enumerate(zip(refill, first)):
        assert not result.full_params and result.persistent_buffers[0] is buffers[rank][0]
        assert buffers[rank][0].data_ptr() == pointers[rank]
        for (_, param), full in zip(named, earlier.full_params):
            assert torch.equal(full, param.detach().bfloat16())  # the views of the first unshard see the new values
