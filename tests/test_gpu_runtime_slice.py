"""The placements under a real forward and backward on one GPU: the stream
hand-off (side-stream unshard and gradient reduction, event ordering, buffer
release), persistent unsharded parameters and their refill, reshard, and the
accumulation of the reduced shards -- checked bit for bit against the same
kernels called directly on the current stream."""

import pytest
import torch
import torch.nn as nn

from flex_shard_amd import Fp8BucketedBlockShard, GradientReduction, LocalReduceGroup
from flex_shard_amd.blockwise_fp8 import (
    BlockwiseFp8Weight,
    Fp8BlockwiseGemms,
    convert_to_flex_shard_float8_blockwise_linear,
    make_blockwise_fp8_weight,
    prequantized_linear,
)
from flex_shard_amd.custom_placements.fp8_bucketed_block_shard import _quantize_dense_weight_to_blockwise_fp8
from flex_shard_amd.flex_shard import BucketCommContext, BucketRuntime, StreamHandoff, begin_bucket_unshard
from flex_shard_amd.testing import FakeMesh, local_rows, make_param_infos

pytestmark = pytest.mark.gpu


def _mlp(device, gen):
    model = nn.Sequential(nn.Linear(256, 384, bias=False), nn.Linear(384, 256, bias=False))
    with torch.no_grad():
        for p in model.parameters():
            p.copy_(torch.randn(p.shape, generator=gen) * 0.05)
    return model.to(device=device, dtype=torch.bfloat16)


def _direct(weights, x, grad_out):
    """Forward and backward of the two-layer MLP with the kernels called
    directly: returns (out, grad_x, [grad_w0, grad_w1]) in bf16."""
    gemms = Fp8BlockwiseGemms(128)
    quantized = []
    for w in weights:
        q, s = _quantize_dense_weight_to_blockwise_fp8(w, 128, torch.float8_e4m3fn)
        quantized.append(BlockwiseFp8Weight(q, s, 128))
    hidden = gemms.forward(x, quantized[0])
    out = gemms.forward(hidden, quantized[1])
    grad_hidden, grad_w1 = gemms.backward(grad_out, hidden, quantized[1], True, True)
    grad_x, grad_w0 = gemms.backward(grad_hidden, x, quantized[0], True, True)
    return out, grad_x, [grad_w0, grad_w1]


def test_one_rank_bucket_under_hooks(device):
    gen = torch.Generator().manual_seed(0)
    model = _mlp(device, gen)
    full = [p.detach().clone() for p in model.parameters()]
    convert_to_flex_shard_float8_blockwise_linear(model)
    group = LocalReduceGroup(1, 0)
    mesh = FakeMesh(1, 0, group)
    placement = Fp8BucketedBlockShard(world_size=1, weight_factory=make_blockwise_fp8_weight)
    context = BucketCommContext.create(device)
    runtime = BucketRuntime.shard_module_params(model, ["0.weight", "1.weight"], placement, mesh, context)
    runtime.install_hooks(model)
    assert all(torch.equal(s.view(w.shape), w) for s, w in zip(runtime.sharded_params, full))

    x = torch.randn(96, 256, generator=gen).bfloat16().to(device).requires_grad_()
    grad_out = (torch.randn(96, 256, generator=gen) * 0.01).bfloat16().to(device)
    for step in range(3):
        if step:  # an "optimizer step" on the local shards: the next unshard must refill from them
            with torch.no_grad():
                for p in runtime.sharded_params:
                    p.mul_(0.5)
                    p.grad = None
                x.grad = None
        out = model(x)
        # between forward and backward the modules hold the shards and the full weights' storage is freed
        assert model[0]._parameters["weight"] is runtime.sharded_params[0]
        assert all(b.untyped_storage().size() == 0 for b in runtime.persistent_buffers)
        buffers, unsharded = list(runtime.persistent_buffers), list(runtime.unsharded_params)
        out.backward(grad_out)
        context.wait_and_clear_reduce_grad_states()
        assert not context.reduce_grad_states and not runtime.is_unsharded
        assert all(a is b for a, b in zip(buffers, runtime.persistent_buffers))
        assert all(a is b for a, b in zip(unsharded, runtime.unsharded_params))
        weights = [w * (0.5**step) for w in full]
        want_out, want_gx, want_gw = _direct(weights, x.detach(), grad_out)
        assert torch.equal(out.detach(), want_out)
        assert torch.equal(x.grad, want_gx)
        for p, g in zip(runtime.sharded_params, want_gw):
            # reduced in fp32, stored in the sharded parameter's own dtype
            assert p.grad.dtype == torch.bfloat16 and torch.equal(p.grad.view(g.shape), g)
    torch.cuda.synchronize()


def test_rank_zero_of_two_driven_by_hand(device):
    """Rank 0 of a 2-rank mesh: the other rank's all-gather row and its
    reduce-scatter contribution are deposited in the one-GPU group; the unshard
    runs on the side stream, the reduction on the reduce stream."""
    gen = torch.Generator().manual_seed(1)
    model = _mlp(device, gen)
    full = [p.detach().clone() for p in model.parameters()]
    named = [("0.weight", nn.Parameter(full[0])), ("1.weight", nn.Parameter(full[1]))]
    convert_to_flex_shard_float8_blockwise_linear(model)
    placement = Fp8BucketedBlockShard(world_size=2, weight_factory=make_blockwise_fp8_weight)
    group = LocalReduceGroup(2, 0)
    mesh0, mesh1 = FakeMesh(2, 0, group), FakeMesh(2, 1, None)
    # what rank 1 would send: its quantized, packed payload
    infos1 = make_param_infos(named, placement, mesh1)
    for info in infos1:
        info.reduce_dtype = torch.float32  # the runtime's default mixed-precision policy
    prepared1 = placement.prepare_unshard_bucket([local_rows(p, i) for (_, p), i in zip(named, infos1)], infos1, mesh1, None)
    group.gather_rows[1] = prepared1.buffers[0]

    context = BucketCommContext.create(device)
    runtime = BucketRuntime.shard_module_params(
        model, ["0.weight", "1.weight"], placement, mesh0, context, GradientReduction()
    )
    assert sum(p.numel() for p in runtime.sharded_params) < sum(w.numel() for w in full)
    handle = runtime.begin_unshard()
    runtime.finish_unshard(handle)
    with pytest.raises(RuntimeError, match="only be finished once"):
        handle.finish()
    runtime._swap_in_params(runtime.unsharded_params)
    x = torch.randn(64, 256, generator=gen).bfloat16().to(device)
    grad_out = (torch.randn(64, 256, generator=gen) * 0.01).bfloat16().to(device)
    out = model(x)
    want_out, _, want_gw = _direct(full, x, grad_out)
    assert torch.equal(out.detach(), want_out)
    out.backward(grad_out)
    grads0 = [p.grad for p in runtime.unsharded_params]
    assert all(g.dtype == torch.float32 for g in grads0)
    assert all(torch.equal(g, w.float()) for g, w in zip(grads0, want_gw))
    # rank 1's contribution: other gradients, laid out as its reduce-scatter input
    grads1 = [torch.randn(g.shape, generator=gen).to(device) for g in grads0]
    send1 = placement.prepare_reduce_grad(grads1, infos1, mesh1, None).buffers[0]
    group.deposit(1, send1)
    runtime.reduce_grads()
    runtime.reshard()
    context.wait_and_clear_reduce_grad_states()
    for param, info, g0, g1 in zip(runtime.sharded_params, runtime.infos, grads0, grads1):
        # pre-multiplied sum in rank order in fp32, stored in the sharded parameter's dtype
        want = local_rows(nn.Parameter((g0 * 0.5 + g1 * 0.5).bfloat16()), info)
        assert param.grad.shape == info.local_shape and torch.equal(param.grad, want)
    torch.cuda.synchronize()


def test_unshard_buffers_are_released_through_both_streams(device):
    gen = torch.Generator().manual_seed(2)
    weight = nn.Parameter((torch.randn(256, 256, generator=gen) * 0.05).bfloat16().to(device))
    placement = Fp8BucketedBlockShard(world_size=1, weight_factory=make_blockwise_fp8_weight)
    mesh = FakeMesh(1, 0, LocalReduceGroup(1, 0))
    infos = make_param_infos([("w", weight)], placement, mesh)
    side = torch.cuda.Stream(device)
    handle = begin_bucket_unshard([weight.detach()], infos, mesh, side)
    assert handle.prepared.buffers  # payload and gathered rows, allocated on the side stream
    handle.release_buffers()
    assert not handle.prepared.buffers
    handle = begin_bucket_unshard([weight.detach()], infos, mesh, side)
    result = handle.finish()
    assert not handle.prepared.buffers and not result.buffers and len(result.persistent_buffers) == 1
    q, s = _quantize_dense_weight_to_blockwise_fp8(weight.detach(), 128, torch.float8_e4m3fn)
    got = result.full_params[0]
    assert torch.equal(got.fp8_data.view(torch.uint8), q.view(torch.uint8)) and torch.equal(got.recip_scale, s)
    kept = [torch.ones(4, device=device)]
    handoff = StreamHandoff(kept, (side, torch.cuda.current_stream(device)))
    handoff.release_after_current_stream()
    handoff.release_after_current_stream()  # idempotent
    assert not kept
    torch.cuda.synchronize()


def test_two_dense_buckets_share_the_streams(device):
    """Two BucketedBlockShard buckets (one per layer) under hooks on one
    context that allows a single reduction in flight: the second bucket's
    reduction retires the first.  Forward, input gradient and shard gradients
    equal the unsharded model's, bit for bit (bf16 weights are gathered as they
    are, gradients reduced in fp32 over one rank)."""
    from flex_shard_amd import BucketedBlockShard

    gen = torch.Generator().manual_seed(3)
    model = _mlp(device, gen)
    plain = _mlp(device, torch.Generator().manual_seed(3))
    context = BucketCommContext.create(device, max_pending_reduce_grads=1)
    mesh = FakeMesh(1, 0, LocalReduceGroup(1, 0))
    runtimes = []
    for index, layer in enumerate(model):
        placement = BucketedBlockShard(dims=(0,), blocks_per_rank=(1,))
        runtime = BucketRuntime.shard_module_params(model, [f"{index}.weight"], placement, mesh, context)
        runtime.install_hooks(layer)
        runtimes.append(runtime)
    x = torch.randn(32, 256, generator=gen).bfloat16().to(device)
    grad_out = torch.randn(32, 256, generator=gen).bfloat16().to(device)
    for step in range(2):
        x_run, x_ref = x.clone().requires_grad_(), x.clone().requires_grad_()
        out = model(x_run)
        assert all(not r.is_unsharded for r in runtimes)
        out.backward(grad_out)
        context.wait_and_clear_reduce_grad_states()
        ref = plain(x_ref)
        ref.backward(grad_out)
        assert torch.equal(out.detach(), ref.detach()) and torch.equal(x_run.grad, x_ref.grad)
        for runtime, layer in zip(runtimes, plain):
            (shard,) = runtime.sharded_params
            assert torch.equal(shard.grad.view(layer.weight.shape), layer.weight.grad)
            shard.grad = None
            layer.weight.grad = None
    torch.cuda.synchronize()


def test_mixed_bucket_under_hooks(device):
    """Biases as Shard(0) members next to the FP8 weights in one mixed bucket
    of a one-rank mesh, driven by the forward/backward hooks: outputs and all
    gradients equal the same autograd graph on directly built FP8 weights."""
    from flex_shard_amd import MixedBucketPlacement

    gen = torch.Generator().manual_seed(5)
    model = nn.Sequential(nn.Linear(256, 384), nn.Linear(384, 256))
    with torch.no_grad():
        for p in model.parameters():
            p.copy_(torch.randn(p.shape, generator=gen) * 0.05)
    model = model.to(device=device, dtype=torch.bfloat16)
    full = {fqn: p.detach().clone() for fqn, p in model.named_parameters()}
    convert_to_flex_shard_float8_blockwise_linear(model)
    mixed = MixedBucketPlacement({})
    member = mixed.blockwise_quant_bucketed_block_shard(
        Fp8BucketedBlockShard(world_size=1, weight_factory=make_blockwise_fp8_weight)
    )
    fqns = ["0.weight", "0.bias", "1.weight", "1.bias"]
    placements = {fqn: (member if fqn.endswith("weight") else mixed.shard0) for fqn in fqns}
    context = BucketCommContext.create(device)
    runtime = BucketRuntime.shard_module_params(
        model, fqns, placements, FakeMesh(1, 0, LocalReduceGroup(1, 0)), context
    )
    runtime.install_hooks(model)
    x = torch.randn(64, 256, generator=gen).bfloat16().to(device)
    grad_out = (torch.randn(64, 256, generator=gen) * 0.01).bfloat16().to(device)
    for step in range(2):
        x_run = x.clone().requires_grad_()
        out = model(x_run)
        assert all(b.untyped_storage().size() == 0 for b in runtime.persistent_buffers)
        out.backward(grad_out)
        context.wait_and_clear_reduce_grad_states()
        # the same graph on weights quantized directly
        leaves = {}
        for fqn, value in full.items():
            if fqn.endswith("weight"):
                q, s = _quantize_dense_weight_to_blockwise_fp8(value, 128, torch.float8_e4m3fn)
                leaves[fqn] = BlockwiseFp8Weight(q, s, 128, requires_grad=True)
            else:
                leaves[fqn] = value.clone().requires_grad_()
        x_ref = x.clone().requires_grad_()
        hidden = prequantized_linear(x_ref, leaves["0.weight"], leaves["0.bias"])
        ref = prequantized_linear(hidden, leaves["1.weight"], leaves["1.bias"])
        ref.backward(grad_out)
        assert torch.equal(out.detach(), ref.detach()) and torch.equal(x_run.grad, x_ref.grad)
        for bucket_param in runtime.bucket_params:
            shard, want = bucket_param.sharded_param, leaves[bucket_param.info.fqn].grad
            assert shard.grad.dtype == torch.bfloat16
            assert torch.equal(shard.grad.view(want.shape), want.to(torch.bfloat16)), bucket_param.info.fqn
            shard.grad = None
    torch.cuda.synchronize()


def test_prefetched_unshard_is_taken_by_the_next_unshard(device):
    """The second layer's bucket is prefetched before the first layer runs (its
    quantize + pack goes to the unshard stream under the first layer's GEMMs);
    results equal the run without prefetch, and a prefetch that is not used
    can be released."""
    gen = torch.Generator().manual_seed(6)
    model = _mlp(device, gen)
    convert_to_flex_shard_float8_blockwise_linear(model)
    context = BucketCommContext.create(device)
    mesh = FakeMesh(1, 0, LocalReduceGroup(1, 0))
    runtimes = []
    for index, layer in enumerate(model):
        placement = Fp8BucketedBlockShard(world_size=1, weight_factory=make_blockwise_fp8_weight)
        runtime = BucketRuntime.shard_module_params(model, [f"{index}.weight"], placement, mesh, context)
        runtime.install_hooks(layer)
        runtimes.append(runtime)
    x = torch.randn(64, 256, generator=gen).bfloat16().to(device)
    grad_out = (torch.randn(64, 256, generator=gen) * 0.01).bfloat16().to(device)

    def run(prefetch: bool):
        for runtime in runtimes:
            for shard in runtime.sharded_params:
                shard.grad = None
        x_run = x.clone().requires_grad_()
        if prefetch:
            runtimes[1].prefetch()
            assert runtimes[1]._pending_unshard is not None
        out = model(x_run)
        assert runtimes[1]._pending_unshard is None
        if prefetch:  # backward runs layer 1 first, then layer 0
            runtimes[0].prefetch()
        out.backward(grad_out)
        context.wait_and_clear_reduce_grad_states()
        return out.detach(), x_run.grad, [r.sharded_params[0].grad.clone() for r in runtimes]

    plain = run(False)  # also the first unshard, which creates the persistent buffers
    for _ in range(2):
        fetched = run(True)
        assert torch.equal(plain[0], fetched[0]) and torch.equal(plain[1], fetched[1])
        assert all(torch.equal(a, b) for a, b in zip(plain[2], fetched[2]))
    runtimes[0].prefetch()
    runtimes[0].release_prefetch()
    assert runtimes[0]._pending_unshard is None
    assert all(b.untyped_storage().size() == 0 for b in runtimes[0].persistent_buffers)
    again = run(False)
    assert torch.equal(plain[0], again[0])
    torch.cuda.synchronize()


def test_checkpoint_layouts_of_sharded_buckets(device):
    """Two ranks shard the same model; their state dicts, saved box by box
    through the declared layouts, rebuild the full weights, and a one-rank
    runtime loads them back.  Adam's states carry the same layouts."""
    from flex_shard_amd import get_global_layout
    from flex_shard_amd.flex_shard import (
        copy_full_into_shard,
        copy_shard_into_full,
        register_optimizer_checkpoint_hook,
        set_state_dict_global_layouts,
    )

    gen = torch.Generator().manual_seed(5)
    reference = _mlp(device, gen)
    full = {name: p.detach().clone() for name, p in reference.named_parameters()}
    saved = {name: torch.full_like(p, float("nan")) for name, p in full.items()}
    context = BucketCommContext.create(device)
    for rank in range(2):
        model = _mlp(device, torch.Generator().manual_seed(5))
        placement = Fp8BucketedBlockShard(world_size=2, weight_factory=make_blockwise_fp8_weight)
        runtime = BucketRuntime.shard_module_params(
            model, ["0.weight", "1.weight"], placement, FakeMesh(2, rank, LocalReduceGroup(2, rank)), context
        )
        state_dict = model.state_dict()
        set_state_dict_global_layouts([runtime], state_dict)
        for name, tensor in state_dict.items():
            layout = get_global_layout(tensor)
            assert layout.global_shape == tuple(full[name].shape)
            assert sum(s[0] for s in layout.local_sizes) == tensor.shape[0]  # whole 128-row blocks of this rank
            copy_shard_into_full(saved[name], tensor, layout)
        optimizer = torch.optim.AdamW(model.parameters(), lr=1e-3)
        register_optimizer_checkpoint_hook(optimizer, [runtime])
        for p in model.parameters():
            p.grad = torch.ones_like(p)
        optimizer.step()
        states = optimizer.state_dict()["state"]
        for param_id, name in enumerate(("0.weight", "1.weight")):
            assert get_global_layout(states[param_id]["exp_avg"]) == get_global_layout(state_dict[name])
            assert get_global_layout(states[param_id]["step"]) is None
    assert all(torch.equal(saved[name], full[name]) for name in full)

    model = _mlp(device, torch.Generator().manual_seed(6))  # different weights, overwritten by the load
    placement = Fp8BucketedBlockShard(world_size=1, weight_factory=make_blockwise_fp8_weight)
    runtime = BucketRuntime.shard_module_params(
        model, ["0.weight", "1.weight"], placement, FakeMesh(1, 0, LocalReduceGroup(1, 0)), context
    )
    state_dict = model.state_dict()
    set_state_dict_global_layouts([runtime], state_dict)
    for name, tensor in state_dict.items():
        copy_full_into_shard(tensor, saved[name], get_global_layout(tensor))
    assert all(torch.equal(p.view(full[name].shape), full[name]) for name, p in model.named_parameters())
    torch.cuda.synchronize()


def test_microbatches_without_sync_accumulate_in_fp32_and_the_upcast_is_deferred(device):
    """Two microbatches: the first backward runs without gradient sync and
    keeps its full-parameter gradients upcast to fp32; the second one syncs,
    its bf16 gradients are added in place to the kept fp32 ones (no separate
    cast), and the reduction's copy-in reads them.  A single syncing backward
    hands autograd's bf16 gradients straight to the copy-in.  Both against the
    kernels called directly."""
    gen = torch.Generator().manual_seed(5)
    model = _mlp(device, gen)
    full = [p.detach().clone() for p in model.parameters()]
    convert_to_flex_shard_float8_blockwise_linear(model)
    mesh = FakeMesh(1, 0, LocalReduceGroup(1, 0))
    placement = Fp8BucketedBlockShard(world_size=1, weight_factory=make_blockwise_fp8_weight)
    context = BucketCommContext.create(device)
    runtime = BucketRuntime.shard_module_params(model, ["0.weight", "1.weight"], placement, mesh, context)
    runtime.install_hooks(model)
    xs = [torch.randn(64, 256, generator=gen).bfloat16().to(device) for _ in range(2)]
    gos = [(torch.randn(64, 256, generator=gen) * 0.01).bfloat16().to(device) for _ in range(2)]
    wants = [_direct(full, x, go)[2] for x, go in zip(xs, gos)]

    seen_dtypes = []
    runtime.set_requires_gradient_sync(False)
    model(xs[0]).backward(gos[0])
    assert runtime.needs_sync and not runtime.is_unsharded
    kept = [p.grad for p in runtime.unsharded_params]
    assert all(g.dtype == torch.float32 for g in kept)  # a backward that starts a gradient keeps the upcast
    assert all(torch.equal(g, w.float()) for g, w in zip(kept, wants[0]))
    runtime.set_requires_gradient_sync(True)
    for p in runtime.unsharded_params:
        p.register_hook(lambda g: seen_dtypes.append(g.dtype))
    model(xs[1]).backward(gos[1])
    context.wait_and_clear_reduce_grad_states()
    assert seen_dtypes and all(d == torch.bfloat16 for d in seen_dtypes)  # the upcast was deferred
    assert not runtime.needs_sync and all(p.grad is None for p in runtime.unsharded_params)
    assert all(p.grad_dtype == torch.float32 for p in runtime.unsharded_params)  # restored for the next backward
    for shard, w0, w1 in zip(runtime.sharded_params, wants[0], wants[1]):
        want = (w0.float() + w1.float()).bfloat16()  # summed in fp32, stored in the shard's dtype
        assert torch.equal(shard.grad.view(want.shape), want)

    # one syncing backward: bf16 gradients reach the copy-in as they are
    for p in runtime.sharded_params:
        p.grad = None
    seen_dtypes.clear()
    model(xs[0]).backward(gos[0])
    context.wait_and_clear_reduce_grad_states()
    assert seen_dtypes and all(d == torch.bfloat16 for d in seen_dtypes)
    for shard, w0 in zip(runtime.sharded_params, wants[0]):
        assert torch.equal(shard.grad.view(w0.shape), w0)
    torch.cuda.synchronize()


def test_two_fp8_buckets_with_prefetch_on_alternating_unshard_streams(device):
    """Two FP8 buckets (one per layer) under hooks that prefetch the bucket used
    next, in the forward and in the backward: the prefetched unshards are begun
    on the context's two unshard streams in turn, while the other layer
    computes, and taken by the next unshard.  Rank 0 of 2 (the other rank's
    rows and contributions deposited), three steps with an update of the
    shards in between; everything against the kernels called directly."""
    gen = torch.Generator().manual_seed(11)
    model = _mlp(device, gen)
    full = [p.detach().clone() for p in model.parameters()]
    convert_to_flex_shard_float8_blockwise_linear(model)
    context = BucketCommContext.create(device)
    assert len(context.unshard_streams) == 2
    world = 2
    runtimes, groups, others = [], [], []
    for index, layer in enumerate(model):
        fqn = f"{index}.weight"
        named = [(fqn, nn.Parameter(full[index].clone()))]
        placement = Fp8BucketedBlockShard(world_size=world, weight_factory=make_blockwise_fp8_weight)
        group = LocalReduceGroup(world, 0)
        mesh1 = FakeMesh(world, 1)
        infos1 = make_param_infos(named, placement, mesh1)
        for info in infos1:
            info.reduce_dtype = torch.float32
        others.append((placement, named, infos1, mesh1))
        runtime = BucketRuntime.shard_module_params(model, [fqn], placement, FakeMesh(world, 0, group), context)
        runtimes.append(runtime)
        groups.append(group)
    used_streams = []
    for index, (layer, runtime) in enumerate(zip(model, runtimes)):
        runtime.install_hooks(
            layer,
            forward_prefetch=runtimes[index + 1] if index + 1 < len(runtimes) else None,
            backward_prefetch=runtimes[index - 1] if index > 0 else None,
        )
        inner = runtime.begin_unshard

        def recording(*args, _inner=inner, **kwargs):
            handle = _inner(*args, **kwargs)
            used_streams.append(handle._side_stream.cuda_stream if handle._side_stream is not None else None)
            return handle

        runtime.begin_unshard = recording
    prefetched = {"forward": 0, "backward": 0}
    for name, runtime in (("forward", runtimes[1]), ("backward", runtimes[0])):
        inner = runtime.prefetch

        def counting(_inner=inner, _name=name):
            prefetched[_name] += 1
            return _inner()

        runtime.prefetch = counting

    x = torch.randn(96, 256, generator=gen).bfloat16().to(device).requires_grad_()
    grad_out = (torch.randn(96, 256, generator=gen) * 0.01).bfloat16().to(device)
    scale = 1.0
    for step in range(3):
        if step:
            scale *= 0.5
            with torch.no_grad():
                for runtime in runtimes:
                    for p in runtime.sharded_params:
                        p.mul_(0.5)
                        p.grad = None
                x.grad = None
        weights = [w * scale for w in full]
        want_out, want_gx, want_gw = _direct(weights, x.detach(), grad_out)
        # what rank 1 sends: its payload of the current weights, and a gradient contribution
        contributions = []
        for index, (placement, named, infos1, mesh1) in enumerate(others):
            named[0][1].data.copy_(weights[index])
            shards1 = [local_rows(p, i) for (_, p), i in zip(named, infos1)]
            groups[index].gather_rows[1] = placement.prepare_unshard_bucket(shards1, infos1, mesh1, None).buffers[0].clone()
            other_grad = torch.randn(full[index].shape, generator=gen).to(device)
            groups[index].deposit(1, placement.prepare_reduce_grad([other_grad], infos1, mesh1, None).buffers[0])
            contributions.append(other_grad)
        out = model(x)
        assert all(not r.is_unsharded for r in runtimes)
        out.backward(grad_out)
        context.wait_and_clear_reduce_grad_states()
        assert torch.equal(out.detach(), want_out) and torch.equal(x.grad, want_gx)
        for runtime, gw, other_grad in zip(runtimes, want_gw, contributions):
            (info,) = runtime.infos
            want = local_rows(nn.Parameter((gw.float() * 0.5 + other_grad * 0.5).bfloat16()), info)
            assert torch.equal(runtime.sharded_params[0].grad, want)
    assert prefetched == {"forward": 3, "backward": 3}
    side = [s for s in used_streams if s is not None]
    assert len(side) == len(used_streams) == 12  # 2 buckets x (forward + backward) x 3 steps, all on side streams
    assert set(side) == {s.cuda_stream for s in context.unshard_streams}
    assert all(a != b for a, b in zip(side, side[1:]))  # the two streams take turns
    torch.cuda.synchronize()
