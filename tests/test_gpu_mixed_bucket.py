"""A mixed bucket (Shard(0) members next to a blockwise FP8 member): one
exchange row per rank, the FP8 member unpacked from strided rank rows at odd
byte offsets, one reduce-scatter input.  Mirrors the reference's
``test_mixed_fp8_bucket_uses_one_collective_and_matches_reference`` and
``test_mixed_fp8_member_with_param_dtype_overrides_is_one_group``
(tests/test_flex_shard_fp8_allgather.py:391-441, :1284-1400) on one GPU, the
other ranks' rows being deposited in the one-GPU group."""

import pytest
import torch
import torch.nn as nn

from flex_shard_amd import (
    Fp8BucketedBlockShard,
    GradientReduction,
    LocalReduceGroup,
    MixedBucketPlacement,
    Shard,
)
from flex_shard_amd.custom_placements import utils as placement_utils
from flex_shard_amd.testing import FakeMesh, local_rows, make_mixed_param_infos, make_param_infos
from oracle import eager

pytestmark = pytest.mark.gpu


class _RecordingFactory:
    def __init__(self):
        self.calls = []

    def __call__(self, fp8_data, recip_scale, block_size, *, orig_dtype, requires_grad):
        self.calls.append((fp8_data, recip_scale, orig_dtype, requires_grad))
        return fp8_data


def _local_shards(named, infos, rank, world):
    shards = []
    for (_, param), info in zip(named, infos, strict=True):
        placement = info.placement
        if isinstance(placement, Shard):
            shards.append(placement.extract_local_shard(param.detach(), rank, world).clone())
        else:
            shards.append(local_rows(param, info).clone())
    return shards


def _bucket(device, world, block, shapes, reduce_dtype=torch.float32):
    gen = torch.Generator().manual_seed(sum(sum(s) for _, s, _ in shapes) + world)
    factory = _RecordingFactory()
    raw = Fp8BucketedBlockShard(world_size=world, weight_factory=factory, block_size=block)
    mixed = MixedBucketPlacement({})
    member = mixed.blockwise_quant_bucketed_block_shard(raw)
    named, placements = [], {}
    for fqn, shape, kind in shapes:
        named.append((fqn, nn.Parameter((torch.randn(shape, generator=gen) * 0.5).bfloat16().to(device))))
        placements[fqn] = (mixed.shard0 if kind == "shard0" else member,)
    ranks = []
    for rank in range(world):
        group = LocalReduceGroup(world, rank)
        mesh = FakeMesh(world, rank, group)
        infos = make_mixed_param_infos(named, placements, mesh)
        for info in infos:
            info.reduce_dtype = reduce_dtype
        ranks.append((mesh, group, infos, _local_shards(named, infos, rank, world)))
    return mixed, raw, member, factory, named, ranks


def _unshard_as(mixed, ranks, rank, persistent=False, persistent_buffers=None):
    """Prepare on every rank, deposit the others' rows in `rank`'s group, run and finish on `rank`."""
    prepared = [mixed.prepare_unshard_bucket(shards, infos, mesh, None) for mesh, _, infos, shards in ranks]
    mine = prepared[rank]
    group = ranks[rank][1]
    for other, p in enumerate(prepared):
        if other != rank:
            group.gather_rows[other] = p.buffers[0]
    mine.persistent = persistent
    mine.persistent_buffers = persistent_buffers
    calls = []
    original = placement_utils.all_gather_rows

    def counting(*args, **kwargs):
        calls.append(1)
        return original(*args, **kwargs)

    import flex_shard_amd.custom_placements.mixed_bucket as mixed_module

    mixed_module.all_gather_rows = counting
    try:
        mixed.run_prepared_unshard(mine)
    finally:
        mixed_module.all_gather_rows = original
    assert len(calls) == 1  # one exchange for all groups
    return mine, mixed.finish_prepared_unshard(mine)


def test_small_mixed_bucket_matches_the_reference_quantizer(device):
    block, world = 4, 2
    mixed, raw, member, factory, named, ranks = _bucket(
        device, world, block, [("norm", (8,), "shard0"), ("weight", (16, 8), "fp8")]
    )
    assert member == raw and mixed.shard0 == Shard(0) and member.bucket_compatibility_key() is mixed
    originals = {fqn: p.detach().clone() for fqn, p in named}
    for rank in range(world):
        factory.calls.clear()
        prepared, result = _unshard_as(mixed, ranks, rank)
        assert prepared.buffers[0].dtype == torch.uint8  # bf16 norm bytes next to the FP8 payload
        norm, weight = result.full_params
        assert torch.equal(norm, originals["norm"])
        ((fp8, scale, orig_dtype, requires_grad),) = factory.calls
        assert weight is fp8 and orig_dtype == torch.bfloat16 and requires_grad
        want_q, want_s = eager.quantize_blockwise(originals["weight"].cpu(), block)
        assert torch.equal(fp8.view(torch.uint8).cpu(), want_q.view(torch.uint8))
        assert torch.equal(scale.cpu().view(torch.int32), want_s.view(torch.int32))

    # gradients: every rank contributes the parameters themselves, so the average is the parameters
    reduce_inputs = []
    for mesh, group, infos, _ in ranks:
        grads = [originals[info.fqn].float() for info in infos]
        reduce_inputs.append(mixed.prepare_reduce_grad(grads, infos, mesh, None))
    for rank, (mesh, group, infos, shards) in enumerate(ranks):
        for other, p in enumerate(reduce_inputs):
            if other != rank:
                group.deposit(other, p.buffers[0])
        reduced = mixed.reduce_prepared_grad(reduce_inputs[rank], GradientReduction())
        for grad, shard in zip(reduced.sharded_grads, shards, strict=True):
            assert grad.dtype == torch.float32 and torch.equal(grad, shard.float())

    # a persistent unshard, then a refill after the local shards changed
    prepared, first = _unshard_as(mixed, ranks, 0, persistent=True)
    assert len(first.persistent_buffers) == 2  # one per Shard param, one compact buffer for the FP8 member
    norm, weight = first.full_params
    with torch.no_grad():
        for _, _, _, shards in ranks:
            for shard in shards:
                shard.add_(1.0)
    for buffer in first.persistent_buffers:
        nbytes = buffer.untyped_storage().size()
        buffer.untyped_storage().resize_(0)
        buffer.untyped_storage().resize_(nbytes)
    _, refill = _unshard_as(mixed, ranks, 0, persistent=True, persistent_buffers=first.persistent_buffers)
    assert refill.full_params == [] and all(a is b for a, b in zip(refill.persistent_buffers, first.persistent_buffers))
    assert torch.equal(norm, originals["norm"] + 1.0)
    want_q, _ = eager.quantize_blockwise((originals["weight"] + 1.0).cpu(), block)
    assert torch.equal(weight.view(torch.uint8).cpu(), want_q.view(torch.uint8))


def test_mixed_bucket_equals_the_members_alone(device):
    """Block 128, four ranks, two norms (one with a short last chunk), a bias
    and two weights: the FP8 member's results equal the same placement used
    alone, bit for bit, although its payload sits at an offset inside wider
    rank rows; gradients reduce through one buffer."""
    world = 4
    shapes = [("norm1", (4099,), "shard0"), ("w1", (512, 256), "fp8"), ("bias", (512,), "shard0"),
              ("w2", (256, 384), "fp8"), ("norm2", (256,), "shard0")]
    mixed, raw, member, factory, named, ranks = _bucket(device, world, 128, shapes)
    originals = {fqn: p.detach().clone() for fqn, p in named}
    rank = 2
    prepared, result = _unshard_as(mixed, ranks, rank)
    state = prepared.placement_state
    assert [[ranks[rank][2][i].fqn for i in g.indices] for g in state.groups] == [["norm1", "bias", "norm2"], ["w1", "w2"]]
    assert state.groups[1].offset % 16 == 0 and state.row_numel % 16 == 0
    by_name = dict(zip([fqn for fqn, _, _ in shapes], result.full_params))
    for fqn in ("norm1", "bias", "norm2"):
        assert torch.equal(by_name[fqn], originals[fqn])
    # the FP8 member alone
    alone_factory = _RecordingFactory()
    alone = Fp8BucketedBlockShard(world_size=world, weight_factory=alone_factory, block_size=128)
    weights = [(fqn, p) for fqn, p in named if fqn.startswith("w")]
    alone_prepared = []
    for r in range(world):
        mesh = FakeMesh(world, r)
        infos = make_param_infos(weights, alone, mesh)
        alone_prepared.append(alone.prepare_unshard_bucket([local_rows(p, i) for (_, p), i in zip(weights, infos)], infos, mesh, None))
    rows = torch.stack([p.buffers[0] for p in alone_prepared])
    alone_result = alone._finish_unshard_from_rank_rows(alone_prepared[rank], rows)
    for (fp8, scale, _, _), (fp8_alone, scale_alone, _, _) in zip(factory.calls, alone_factory.calls, strict=True):
        assert torch.equal(fp8.view(torch.uint8), fp8_alone.view(torch.uint8)) and torch.equal(scale, scale_alone)
    assert len(alone_result.full_params) == 2

    # gradients: rank r contributes (r + 1) * g; AVG over 4 ranks = 2.5 * g
    gen = torch.Generator().manual_seed(9)
    grads = {fqn: torch.randn(p.shape, generator=gen).to(device) for fqn, p in named}
    inputs = []
    for r, (mesh, group, infos, _) in enumerate(ranks):
        inputs.append(mixed.prepare_reduce_grad([grads[i.fqn] * float(r + 1) for i in infos], infos, mesh, None))
    mesh, group, infos, shards = ranks[rank]
    for other, p in enumerate(inputs):
        if other != rank:
            group.deposit(other, p.buffers[0])
    reduced = mixed.reduce_prepared_grad(inputs[rank], GradientReduction())
    for grad, info, (fqn, param) in zip(reduced.sharded_grads, infos, named, strict=True):
        full = sum((grads[fqn] * float(r + 1)) * 0.25 for r in range(world))  # pre-multiplied sum in rank order
        if isinstance(info.placement, Shard):
            want = info.placement.extract_local_shard(full, rank, world)
        else:
            want = local_rows(nn.Parameter(full), info)
        assert grad.shape == want.shape and torch.equal(grad, want), fqn


def test_fp8_member_quantizes_each_param_from_its_own_dtype(device):
    """One FP8 group although the params' unsharded dtypes differ."""
    factory = _RecordingFactory()
    mixed = MixedBucketPlacement({})
    member = mixed.blockwise_quant_bucketed_block_shard(
        Fp8BucketedBlockShard(world_size=1, weight_factory=factory, block_size=4)
    )
    gen = torch.Generator().manual_seed(4)
    named = [(f"w{i}", nn.Parameter(torch.randn(rows, 8, generator=gen).to(device))) for i, rows in enumerate((8, 6, 4))]
    mesh = FakeMesh(1, 0, LocalReduceGroup(1, 0))
    infos = make_mixed_param_infos(named, {fqn: (member,) for fqn, _ in named}, mesh)
    for info in infos:
        info.param_dtype = torch.float32 if info.fqn == "w1" else torch.bfloat16
    prepared = mixed.prepare_unshard_bucket([p.detach() for _, p in named], infos, mesh, None)
    assert [[infos[i].fqn for i in g.indices] for g in prepared.placement_state.groups] == [["w0", "w1", "w2"]]
    mixed.run_prepared_unshard(prepared)
    mixed.finish_prepared_unshard(prepared)
    assert [call[2] for call in factory.calls] == [torch.bfloat16, torch.float32, torch.bfloat16]
    for (fp8, scale, _, _), (fqn, param) in zip(factory.calls, named):
        source = param.detach().cpu() if fqn == "w1" else param.detach().cpu().bfloat16()
        want_q, want_s = eager.quantize_blockwise(source, 4)
        assert torch.equal(fp8.view(torch.uint8).cpu(), want_q.view(torch.uint8)), fqn
        assert torch.equal(scale.cpu().view(torch.int32), want_s.view(torch.int32)), fqn
