"""Seeded random buckets through the whole FP8 unshard path on the GPU
(quantize + pack on every rank, rank rows gathered contiguous or strided at an
odd byte offset, unpack with and without dequantization) against the CPU
oracle: payload bytes, FP8 bytes, scale bits and dequantized bf16 bits."""

import numpy as np
import pytest
import torch
import torch.nn as nn

from flex_shard_amd import Fp8BucketedBlockShard
from flex_shard_amd.testing import (
    FakeMesh,
    gather_rank_rows,
    local_rows,
    make_param_infos,
)
from oracle import cport
from oracle import layout as olayout

pytestmark = pytest.mark.gpu


class _RecordingFactory:
    def __init__(self):
        self.calls = []

    def __call__(self, fp8_data, recip_scale, block_size, *, orig_dtype, requires_grad):
        self.calls.append((fp8_data, recip_scale))
        return fp8_data


def _bits(t):
    return t.contiguous().view(torch.int32)


def _random_bucket(rng, block):
    """1-6 parameters: matrices around multiples of the tile size (whole and
    partial tiles in both directions, single rows, widths below one tile), some
    stacked, with outliers, zero tiles, a subnormal tile and huge values."""
    shapes = []
    for _ in range(int(rng.integers(1, 7))):
        rows = int(rng.integers(0, 4)) * block + int(rng.integers(0, block + 1))
        cols = int(rng.integers(0, 4)) * block + int(rng.integers(0, block + 1))
        rows, cols = max(rows, 1), max(cols, 1)
        if rng.random() < 0.25:
            shapes.append((int(rng.integers(2, 4)), rows, cols))
        else:
            shapes.append((rows, cols))
    params = []
    for shape in shapes:
        w = torch.from_numpy(rng.standard_normal(shape).astype(np.float32)) * float(10.0 ** rng.integers(-4, 3))
        flat = w.view(-1, shape[-1])
        r, c = flat.shape
        for _ in range(int(rng.integers(0, 3))):  # zero tiles
            r0, c0 = int(rng.integers(0, r)) // block * block, int(rng.integers(0, c)) // block * block
            flat[r0 : r0 + block, c0 : c0 + block] = 0
        for _ in range(int(rng.integers(0, 3))):  # outliers
            flat[int(rng.integers(0, r)), int(rng.integers(0, c))] = float(rng.choice([448.0, -3.0e4, 1.0e30, 7.5e-3]))
        if rng.random() < 0.3:  # a tile whose amax is below the floor
            r0, c0 = int(rng.integers(0, r)) // block * block, int(rng.integers(0, c)) // block * block
            flat[r0 : r0 + block, c0 : c0 + block] = 1.0e-20
        params.append(w)
    return shapes, params


@pytest.mark.parametrize("seed", range(160))
def test_random_bucket_round_trip_matches_oracle(device, seed):
    rng = np.random.default_rng(1000 + seed)
    block = int(rng.choice([2, 4, 8, 16, 32, 128]))
    world = int(rng.choice([1, 2, 3, 4, 5, 8]))
    fp32_master = bool(rng.random() < 0.3)
    shapes, params = _random_bucket(rng, block)
    dtype = torch.float32 if fp32_master else torch.bfloat16
    named = [(f"w{i}", nn.Parameter(p.to(dtype).to(device), requires_grad=False)) for i, p in enumerate(params)]
    factory = _RecordingFactory()
    pl = Fp8BucketedBlockShard(world_size=world, weight_factory=factory, block_size=block)

    prepared = []
    for rank in range(world):
        mesh = FakeMesh(world, rank)
        infos = make_param_infos(named, pl, mesh)
        for info in infos:
            info.param_dtype = torch.bfloat16  # an fp32 master is quantized as its bf16 rounding
        shards = [local_rows(p, i) for (_, p), i in zip(named, infos, strict=True)]
        prepared.append(pl.prepare_unshard_bucket(shards, infos, mesh, None))

    # every rank's payload: the naive pack of whole-matrix quantization, pads zero
    matrix_shapes = [olayout.matrix_shape(s) for s in shapes]
    lay = olayout.quant_layout(matrix_shapes, block, world)
    quantized = [cport.quantize_blockwise(p.view(-1, p.shape[-1]), block, cast_to_bf16=True) for p in params]
    qs, ss = [q for q, _ in quantized], [s for _, s in quantized]
    for rank in range(world):
        want = olayout.pack_rank_payload(lay, rank, qs, ss, block)
        assert torch.equal(prepared[rank].buffers[0].cpu(), want), f"payload of rank {rank}"

    # gathered rows, contiguous or strided from an odd byte; unpack on a random rank
    rows = gather_rank_rows(prepared)
    if rng.random() < 0.5:
        shift = int(rng.choice([1, 3, 5, 7]))
        parent = torch.full((world, rows.shape[1] + 9), 0xEE, dtype=torch.uint8, device=device)
        parent[:, shift : shift + rows.shape[1]] = rows
        rows = parent[:, shift : shift + rows.shape[1]]
    on_rank = int(rng.integers(0, world))
    result, dequant = pl.finish_prepared_unshard_with_dequant(prepared[on_rank], rows)
    assert len(factory.calls) == len(shapes) == len(dequant)
    for (fp8, recip), deq, shape, (oq, osc) in zip(factory.calls, dequant, shapes, quantized, strict=True):
        assert tuple(fp8.shape) == tuple(shape)
        assert torch.equal(fp8.reshape(-1, shape[-1]).view(torch.uint8).cpu(), oq)
        assert torch.equal(_bits(recip.cpu()).view(-1), _bits(osc).view(-1))
        want = cport.dequant_blockwise(oq, osc, block)
        assert deq.dtype == torch.bfloat16 and tuple(deq.shape) == tuple(shape)
        got = deq.reshape(-1, shape[-1]).cpu()
        nan = want.isnan()
        assert torch.equal(got.isnan(), nan)
        assert torch.equal(got.view(torch.int16)[~nan], want.view(torch.int16)[~nan])
    factory.calls.clear()
    plain = pl._finish_unshard_from_rank_rows(prepared[on_rank], rows)
    for weight, (oq, _), shape in zip(plain.full_params, quantized, shapes, strict=True):
        assert torch.equal(weight.reshape(-1, shape[-1]).view(torch.uint8).cpu(), oq)


# ------------------------------------------------------------ dense unshard
def _dense_shapes(rng, nblocks):
    """1-5 parameters whose sharded dimension divides into ``nblocks`` blocks,
    vectors among them."""
    shapes = []
    for _ in range(int(rng.integers(1, 6))):
        rows = nblocks * int(rng.integers(1, 6))
        if rng.random() < 0.25:
            shapes.append((rows,))
        else:
            shapes.append((rows, int(rng.integers(1, 40))))
    return shapes


def _dense_case(rng, worlds, most_blocks):
    """Random uneven blocks per rank and parameter shapes that the planner
    accepts (it refuses a bucket in which some rank's range is only padding)."""
    from flex_shard_amd import BucketedBlockShard

    for _ in range(50):
        world = int(rng.choice(worlds))
        blocks = [int(rng.integers(0, most_blocks + 1)) for _ in range(world)]
        if sum(blocks) == 0:
            blocks[int(rng.integers(0, world))] = 1
        shapes = _dense_shapes(rng, sum(blocks))
        pl = BucketedBlockShard(dims=(0,), blocks_per_rank=tuple(blocks))
        named = [(f"p{i}", nn.Parameter(torch.empty(s, device="meta"))) for i, s in enumerate(shapes)]
        try:
            for rank in range(world):
                make_param_infos(named, pl, FakeMesh(world, rank))
        except ValueError as exc:
            assert "only padding" in str(exc)
            continue
        return world, blocks, shapes
    raise AssertionError("no accepted bucket in 50 draws")


@pytest.mark.parametrize("seed", range(40))
def test_random_dense_unshard_restores_every_parameter(device, seed):
    """BucketedBlockShard with random uneven blocks per rank (empty ranks
    among them): prepare on every rank, local exchange, run + finish on every
    rank; the full parameters are the originals in the unsharded dtype."""
    from tests.test_gpu_dense_unshard import _unshard_every_rank

    rng = np.random.default_rng(5000 + seed)
    world, blocks, shapes = _dense_case(rng, [2, 3, 4, 5], 3)
    master, unsharded = [(torch.float32, torch.bfloat16), (torch.float32, None), (torch.bfloat16, None)][int(rng.integers(0, 3))]
    gen = torch.Generator().manual_seed(seed)
    named = [(f"p{i}", nn.Parameter(torch.randn(s, generator=gen).to(master).to(device))) for i, s in enumerate(shapes)]
    want_dtype = unsharded or master
    _, _, results = _unshard_every_rank(named, tuple(blocks), device, unsharded)
    for result in results:
        for (_, param), full in zip(named, result.full_params, strict=True):
            assert full.dtype == want_dtype and full.shape == param.shape
            assert torch.equal(full, param.detach().to(want_dtype))


# ------------------------------------------------------------ gradient path
@pytest.mark.parametrize("seed", range(40))
def test_random_gradient_bucket_copy_in_and_reduce(device, seed):
    """Random dense buckets: every rank's one-pass copy-in equals the oracle's
    reduce-scatter input rows, and the fixed-order reduction on a random rank
    equals the oracle's left fold of the rank contributions, for SUM, AVG and a
    custom divide factor, with fp32 or bf16 gradients reduced in fp32."""
    import torch.distributed as dist

    from flex_shard_amd import BucketedBlockShard, GradientReduction, LocalReduceGroup

    rng = np.random.default_rng(9000 + seed)
    world, blocks, shapes = _dense_case(rng, [2, 3, 4, 8], 2)
    grad_dtype = torch.bfloat16 if rng.random() < 0.5 else torch.float32
    rank = int(rng.integers(0, world))
    reduction, post = [(GradientReduction(op=dist.ReduceOp.SUM), 1.0), (GradientReduction(), float(world)),
                       (GradientReduction(divide_factor=16.0), 16.0)][int(rng.integers(0, 3))]
    pl = BucketedBlockShard(dims=(0,), blocks_per_rank=tuple(blocks))
    group = LocalReduceGroup(world, rank)
    named = [(f"w{i}", nn.Parameter(torch.empty(s, device="meta", dtype=torch.bfloat16))) for i, s in enumerate(shapes)]
    infos = make_param_infos(named, pl, FakeMesh(world, rank, group))
    for info in infos:
        info.reduce_dtype = torch.float32
    layout = infos[0].bucket_layout
    per_rank, mine = [], None
    for r in range(world):
        gen = torch.Generator().manual_seed(seed * 100 + r)
        grads = [torch.randn(s, generator=gen).to(grad_dtype).to(device) for s in shapes]
        per_rank.append(grads)
        prepared = pl.prepare_reduce_grad(grads, infos, FakeMesh(world, rank, group), None)
        want_rows = olayout.reduce_scatter_input(
            [g.cpu() for g in grads], [layout.param_layouts[i.fqn].param_offset for i in infos],
            layout.global_numel, layout.rank_offsets, layout.rank_numels, torch.float32,
        )
        assert torch.equal(prepared.buffers[0].view(want_rows.shape).cpu(), want_rows), f"copy-in of rank {r}"
        group.deposit(r, prepared.buffers[0])
        if r == rank:
            mine = prepared
    result = pl.reduce_prepared_grad(mine, reduction)
    for i, (info, shard) in enumerate(zip(infos, result.sharded_grads, strict=True)):
        total = None
        for r in range(world):  # the left fold in rank order, each term scaled as the reduction scales it
            term = per_rank[r][i].cpu().float()
            if post != 1.0:
                term = term * (1.0 / post)
            total = term.clone() if total is None else total + term
        lo = layout.param_layouts[info.fqn].local_global_offset - layout.param_layouts[info.fqn].param_offset
        want = total.reshape(-1)[lo : lo + info.local_numel].view(info.local_shape)
        assert shard.dtype == torch.float32 and torch.equal(shard.cpu(), want), (rank, i)


# ------------------------------------------------------------ FP8 products
def _small_int_fp8(shape, gen, high):
    return torch.randint(-high, high + 1, shape, generator=gen).to(torch.float32).to(torch.float8_e4m3fn)


@pytest.mark.parametrize("seed", range(36))
def test_random_shapes_of_the_three_fp8_products_are_integer_exact(device, seed):
    """Random m, n (any size) and k (multiples of 128), small-integer operands
    and power-of-two scales: forward, input-gradient and weight-gradient
    products are the one bf16 rounding of the exact result, whatever the tile
    tails and the number of tiles per round."""
    from flex_shard_amd import hip_ops
    from oracle import eager

    rng = np.random.default_rng(7000 + seed)
    m = int(rng.integers(1, 900))
    n = int(rng.integers(1, 900)) if rng.random() < 0.8 else int(rng.integers(1, 40)) * 128
    k = int(rng.integers(1, 9)) * 128
    gen = torch.Generator().manual_seed(seed)
    kb, nb = k // 128, -(-n // 128)
    pow2 = lambda shape: torch.exp2(torch.randint(-2, 3, shape, generator=gen).float())
    # forward: x [m, k] with scales [k/128, m], weight [n, k] with scales [n/128, k/128]
    xq, wq = _small_int_fp8((m, k), gen, 1), _small_int_fp8((n, k), gen, 1)
    xs, ws = pow2((kb, m)), pow2((nb, kb))
    want = eager.fp8_gemm_1x128_128x128(xq, xs, wq, ws, out_dtype=torch.float32)
    got = hip_ops.fp8_gemm_1x128_128x128(xq.to(device), xs.to(device), wq.to(device), ws.to(device))
    assert torch.equal(got.cpu(), want.bfloat16()), ("forward", m, n, k)
    # input gradient: contraction over the weight's rows (k of them here), its scales read across
    in_dim = -(-n // 16) * 16  # the byte transpose takes widths that are multiples of 16
    gq, gs = _small_int_fp8((m, k), gen, 1), pow2((kb, m))
    w_rows = _small_int_fp8((k, in_dim), gen, 1)  # weight [out = k, in]
    w_scales = pow2((kb, -(-in_dim // 128)))
    wt = hip_ops.fp8_transpose(w_rows.to(device))  # [in, out]
    got = hip_ops.fp8_gemm_1x128_128x128_dgrad(gq.to(device), gs.to(device), wt, w_scales.to(device), in_dim)
    want = eager.fp8_gemm_1x128_128x128(
        gq, gs, w_rows.view(torch.uint8).t().contiguous().view(torch.float8_e4m3fn), w_scales.t().contiguous(),
        out_dtype=torch.float32,
    )
    assert torch.equal(got.cpu(), want.bfloat16()), ("input gradient", m, in_dim, k)
    # weight gradient: both operands with one scale per column and run of 128 along k
    aq, bq = _small_int_fp8((m, k), gen, 4), _small_int_fp8((n, k), gen, 4)
    a_s, b_s = pow2((kb, m)), pow2((kb, n))
    want = eager.fp8_gemm_1x128_128x1(aq, a_s, bq, b_s, out_dtype=torch.float32)
    got = hip_ops.fp8_gemm_1x128_128x1(aq.to(device), a_s.to(device), bq.to(device), b_s.to(device))
    assert torch.equal(got.cpu(), want.bfloat16()), ("weight gradient", m, n, k)


# ------------------------------------------------------------ mixed bucket
@pytest.mark.parametrize("seed", range(30))
def test_random_mixed_bucket_unshard_and_gradients(device, seed):
    """Random mixed buckets (Shard(0) vectors and matrices of random sizes in
    random order around one or two blockwise FP8 matrices, so the FP8 payload
    starts at odd offsets inside the rank rows): on every rank the Shard(0)
    members come back as they were and the FP8 members as the oracle's
    whole-matrix quantization; with every rank contributing the parameters
    themselves as gradients, each rank's reduced gradient is the rank-order
    fold of `world` copies of its own shard times 1 / world."""
    from flex_shard_amd import GradientReduction
    from oracle import eager
    from tests.test_gpu_mixed_bucket import _bucket, _unshard_as

    rng = np.random.default_rng(3000 + seed)
    world = int(rng.choice([2, 3, 4]))
    block = int(rng.choice([4, 8, 16]))
    shapes = []
    for index in range(int(rng.integers(1, 4))):
        rows = world * int(rng.integers(1, 5))  # Shard(0) splits dim 0 evenly here
        shape = (rows,) if rng.random() < 0.5 else (rows, int(rng.integers(1, 9)))
        shapes.append((f"dense{index}", shape, "shard0"))
    for index in range(int(rng.integers(1, 3))):
        rows = int(rng.integers(1, 4)) * block + int(rng.integers(0, block))
        cols = int(rng.integers(1, 4)) * block + int(rng.integers(0, block))
        shapes.append((f"fp8_{index}", (max(rows, 1), max(cols, 1)), "fp8"))
    shapes = [shapes[i] for i in rng.permutation(len(shapes))]
    mixed, raw, member, factory, named, ranks = _bucket(device, world, block, shapes)
    originals = {fqn: p.detach().clone() for fqn, p in named}
    kinds = {fqn: kind for fqn, _, kind in shapes}
    for rank in range(world):
        factory.calls.clear()
        _, result = _unshard_as(mixed, ranks, rank)
        calls = iter(factory.calls)
        for (fqn, _), full in zip(named, result.full_params, strict=True):
            if kinds[fqn] == "shard0":
                assert torch.equal(full, originals[fqn]), (rank, fqn)
            else:
                fp8, scale, orig_dtype, _ = next(calls)
                want_q, want_s = eager.quantize_blockwise(originals[fqn].cpu(), block)
                assert full is fp8 and orig_dtype == torch.bfloat16
                assert torch.equal(fp8.view(torch.uint8).cpu(), want_q.view(torch.uint8)), (rank, fqn)
                assert torch.equal(scale.cpu().view(torch.int32), want_s.view(torch.int32)), (rank, fqn)
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
            # the average of `world` equal contributions, folded in rank order as the reduction folds them
            term = shard.float() * torch.tensor(1.0 / world, dtype=torch.float32)
            want = term.clone()
            for _ in range(world - 1):
                want = want + term
            assert grad.dtype == torch.float32 and torch.equal(grad, want), rank


# ------------------------------------------------------------ runtime slice
@pytest.mark.parametrize("seed", range(12))
def test_random_layer_stacks_under_the_runtime_hooks(device, seed):
    """2-4 FP8 linear layers of random widths, one bucket each, under the
    runtime's hooks with or without prefetch of the next bucket, on one or two
    unshard streams, 1-3 microbatches of which only the last syncs, for two
    steps with an update of the shards in between: outputs, input gradients
    and the reduced shard gradients equal the same kernels called directly on
    one stream, bit for bit (a missing wait or a buffer reused too early would
    show here)."""
    from flex_shard_amd import LocalReduceGroup
    from flex_shard_amd.blockwise_fp8 import (
        BlockwiseFp8Weight,
        Fp8BlockwiseGemms,
        convert_to_flex_shard_float8_blockwise_linear,
        make_blockwise_fp8_weight,
    )
    from flex_shard_amd.custom_placements.fp8_bucketed_block_shard import _quantize_dense_weight_to_blockwise_fp8
    from flex_shard_amd.flex_shard import BucketCommContext, BucketRuntime

    rng = np.random.default_rng(11000 + seed)
    nlayers = int(rng.integers(2, 5))
    widths = [int(rng.integers(1, 4)) * 128 for _ in range(nlayers + 1)]
    tokens = int(rng.integers(1, 4)) * 64
    prefetch = bool(rng.random() < 0.7)
    streams = int(rng.integers(1, 3))
    microbatches = int(rng.integers(1, 4))
    gen = torch.Generator().manual_seed(seed)
    model = nn.Sequential(*[nn.Linear(widths[i], widths[i + 1], bias=False) for i in range(nlayers)])
    with torch.no_grad():
        for p in model.parameters():
            p.copy_(torch.randn(p.shape, generator=gen) * 0.05)
    model = model.to(device=device, dtype=torch.bfloat16)
    full = [p.detach().clone() for p in model.parameters()]
    convert_to_flex_shard_float8_blockwise_linear(model)
    context = BucketCommContext.create(device, unshard_streams=streams)
    runtimes = []
    for index in range(nlayers):
        placement = Fp8BucketedBlockShard(world_size=1, weight_factory=make_blockwise_fp8_weight)
        mesh = FakeMesh(1, 0, LocalReduceGroup(1, 0))
        runtimes.append(BucketRuntime.shard_module_params(model, [f"{index}.weight"], placement, mesh, context))
    for index, (layer, runtime) in enumerate(zip(model, runtimes)):
        runtime.install_hooks(
            layer,
            forward_prefetch=runtimes[index + 1] if prefetch and index + 1 < nlayers else None,
            backward_prefetch=runtimes[index - 1] if prefetch and index > 0 else None,
        )

    def direct(weights, x, grad_out):
        gemms = Fp8BlockwiseGemms(128)
        quantized = []
        for w in weights:
            q, s = _quantize_dense_weight_to_blockwise_fp8(w, 128, torch.float8_e4m3fn)
            quantized.append(BlockwiseFp8Weight(q, s, 128))
        acts = [x]
        for w in quantized:
            acts.append(gemms.forward(acts[-1], w))
        grads, g = [None] * len(weights), grad_out
        for i in reversed(range(len(weights))):
            g, grads[i] = gemms.backward(g, acts[i], quantized[i], True, True)
        return acts[-1], g, grads

    scale = 1.0
    for step in range(2):
        if step:
            scale = 0.5
            with torch.no_grad():
                for runtime in runtimes:
                    for p in runtime.sharded_params:
                        p.mul_(0.5)
                        p.grad = None
        weights = [w * scale for w in full]
        xs = [torch.randn(tokens, widths[0], generator=gen).bfloat16().to(device).requires_grad_() for _ in range(microbatches)]
        gos = [(torch.randn(tokens, widths[-1], generator=gen) * 0.01).bfloat16().to(device) for _ in range(microbatches)]
        wants = [direct(weights, x.detach(), go) for x, go in zip(xs, gos)]
        for k, (x, go) in enumerate(zip(xs, gos)):
            last = k == microbatches - 1
            for runtime in runtimes:
                runtime.set_requires_gradient_sync(last)
            out = model(x)
            out.backward(go)
            assert torch.equal(out.detach(), wants[k][0]), (step, k)
            assert torch.equal(x.grad, wants[k][1]), (step, k)
        context.wait_and_clear_reduce_grad_states()
        for index, runtime in enumerate(runtimes):
            total = None
            for want in wants:  # microbatch gradients add up in fp32 in the order they arrive
                total = want[2][index].float() if total is None else total + want[2][index].float()
            (shard,) = runtime.sharded_params
            assert torch.equal(shard.grad.view(total.shape), total.bfloat16()), (step, index)
            assert not runtime.is_unsharded
    torch.cuda.synchronize()
