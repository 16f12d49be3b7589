"""GPU parity of the fused tile quantize + pack path (through the C ABI) with
the CPU oracle: bit-exact FP8 bytes and scale bits."""

import pytest
import torch
import torch.nn as nn

from flex_shard_amd import Fp8BucketedBlockShard, hip_ops
from flex_shard_amd.custom_placements.fp8_bucketed_block_shard import _quantize_dense_weight_to_blockwise_fp8
from flex_shard_amd.testing import (
    DEEPSEEK_V3_EXPERTS,
    LLAMA3_8B_LAYER,
    FakeMesh,
    add_outliers_and_zero_tiles,
    local_rows,
    make_param_infos,
    prepare_unshard_on_each_rank,
    seeded_bucket,
)
from oracle import cport, eager
from oracle import layout as olayout

pytestmark = pytest.mark.gpu
E4M3 = torch.float8_e4m3fn


def _factory(fp8_data, recip_scale, block_size, *, orig_dtype, requires_grad):
    return fp8_data


def _bits(t):
    return t.contiguous().view(torch.int32)


def _quant_gpu(w, block, eps_mode=hip_ops.EPS_INPUT_DTYPE):
    q, s = _quantize_dense_weight_to_blockwise_fp8(w, block, E4M3, eps_mode=eps_mode)
    return q.view(torch.uint8).cpu(), s.cpu()


def _assert_matches_oracle(w_cpu, block, device, **kw):
    q, s = _quant_gpu(w_cpu.to(device), block)
    oq, osc = cport.quantize_blockwise(w_cpu, block, **kw)
    assert torch.equal(q, oq), f"FP8 bytes differ in {(q != oq).sum().item()} places"
    assert torch.equal(_bits(s), _bits(osc)), "scale bits differ"


def test_config1_plumbing_case(device):
    """bf16 [2048, 2048], N(0, 0.02), 128x128 tiles, world size 1: payload is
    4 194 304 FP8 bytes + [16, 16] scales = 4 195 328 bytes."""
    gen = torch.Generator().manual_seed(0)
    w = (torch.randn(2048, 2048, generator=gen) * 0.02).bfloat16()
    pl = Fp8BucketedBlockShard(world_size=1, weight_factory=_factory)
    param = nn.Parameter(w.to(device), requires_grad=False)
    infos = make_param_infos([("w", param)], pl, FakeMesh(1))
    prepared = pl.prepare_unshard_bucket([param.detach()], infos, FakeMesh(1), None)
    payload = prepared.buffers[0].cpu()
    assert payload.numel() == 4195328 and prepared.buffers[1].numel() == 4195328
    oq, osc = cport.quantize_blockwise(w, 128)
    eq, esc = eager.quantize_blockwise(w, 128)
    assert torch.equal(payload[:4194304], oq.reshape(-1)) and torch.equal(oq, eq.view(torch.uint8))
    assert torch.equal(payload[4194304:].view(torch.float32), osc.reshape(-1))
    assert torch.equal(_bits(osc), _bits(esc)) and osc.shape == (16, 16)


@pytest.mark.parametrize(
    "shape,block",
    [((6, 4), 4), ((12, 6), 4), ((6, 6), 4), ((9, 32), 2), ((256, 384), 128), ((200, 136), 128), ((130, 129), 128),
     ((1, 3), 4), ((128, 8), 128), ((257, 4096), 128), ((64, 64), 16), ((300, 200), 64)],
)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_matches_oracle_on_shapes(device, shape, block, dtype):
    gen = torch.Generator().manual_seed(hash((shape, block)) % 1000)
    w = (torch.randn(shape, generator=gen) * 0.02).to(dtype)
    _assert_matches_oracle(w, block, device)


def test_scale_arithmetic_for_every_bf16_amax(device):
    """One 4x4 tile per non-negative bf16 value (including values below the
    1e-12 floor, the largest finite value and infinity) holding that value as
    its amax: scale bits and bytes must match the oracle for all 32 641."""
    amax = torch.arange(0, 0x7F81, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    n = amax.numel()
    gen = torch.Generator().manual_seed(1)
    frac = torch.rand(n, 4, 4, generator=gen) * 2 - 1
    tiles = (frac * amax.float().clamp(max=3e38).view(n, 1, 1)).bfloat16()
    tiles[:, 1, 2] = amax
    w = tiles.view(n * 4, 4)
    q, s = _quant_gpu(w.to(device), 4)
    oq, osc = cport.quantize_blockwise(w, 4)
    assert torch.equal(_bits(s), _bits(osc))
    finite = ~osc.isinf().view(-1)
    rows = finite.repeat_interleave(4)
    assert torch.equal(q[rows], oq[rows])
    # amax = inf: finite entries become 0, the inf itself NaN (sign aside)
    assert torch.equal(q[~rows] & 0x7F, oq[~rows] & 0x7F)


def test_element_rounding_for_every_bf16_value(device):
    """Tiles whose amax is a power of two (exact scale): every bf16 value with
    |x| <= amax goes through the hardware FP8 conversion and must equal both
    the oracle and torch's own cast of x * scale."""
    all_bf16 = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()
    for k in (0, -7, 6):
        amax = 2.0**k
        values = all_bf16[all_bf16.abs() <= amax]
        values = values[: values.numel() // 16 * 16].view(-1, 4).clone()
        values[0::4, 0] = amax
        w = values.bfloat16()
        q, _ = _quant_gpu(w.to(device), 4)
        oq, _ = cport.quantize_blockwise(w, 4)
        assert torch.equal(q, oq)
        assert torch.equal(q, (w.float() * (448.0 / amax)).to(E4M3).view(torch.uint8))


def test_zero_tile_eps_modes(device, golden):
    g = golden["quant_eps_constants"]
    z = torch.zeros(128, 256, dtype=torch.bfloat16, device=device)
    z[:, 128:] = 0.5
    q, s = _quant_gpu(z, 128)
    assert (q[:, :128] == 0).all() and s.view(torch.int32)[0, 0].item() == int(g["zero_tile_recip_bits_bf16_input"], 16)
    _, s = _quant_gpu(z, 128, hip_ops.EPS_FP32)
    assert s.view(torch.int32)[0, 0].item() == int(g["zero_tile_recip_bits_fp32_input"], 16)
    _, s = _quant_gpu(z.float(), 128)
    assert s.view(torch.int32)[0, 0].item() == int(g["zero_tile_recip_bits_fp32_input"], 16)
    # sub-floor but non-zero amax is clamped too, and tiny values quantize to signed zero
    tiny = torch.full((4, 4), -1e-20, dtype=torch.bfloat16, device=device)
    q, s = _quant_gpu(tiny, 4)
    oq, osc = cport.quantize_blockwise(tiny.cpu(), 4)
    assert torch.equal(q, oq) and torch.equal(_bits(s), _bits(osc)) and (q == 0x80).all()


def test_nan_tile_is_poisoned_like_the_oracle(device):
    w = torch.ones(8, 4).bfloat16()
    w[0, 0] = float("nan")
    q, s = _quant_gpu(w.to(device), 4)
    oq, osc = cport.quantize_blockwise(w, 4)
    assert ((q[:4] & 0x7F) == 0x7F).all() and s[0, 0].isnan()
    assert torch.equal(q[4:], oq[4:]) and torch.equal(_bits(s[1:]), _bits(osc[1:]))


def test_fp32_master_is_quantized_as_bf16(device, golden):
    """Reference known answer: an fp32 shard with param_dtype bf16 quantizes
    its bf16 rounding (and differs from quantizing the fp32 values)."""
    g = golden["fp8_quantizes_param_dtype"]
    block = g["block"]
    full = torch.full((block, block), g["fill"], dtype=torch.float32, device=device)
    full[0, 0] = g["outlier"]
    pl = Fp8BucketedBlockShard(world_size=1, weight_factory=_factory, block_size=block)
    param = nn.Parameter(full.clone())
    (info,) = make_param_infos([("w", param)], pl, FakeMesh(1))
    info.param_dtype = torch.bfloat16
    prepared = pl.prepare_unshard_bucket([full], [info], FakeMesh(1), None)
    md = prepared.placement_state.metadata
    payload = prepared.buffers[0].cpu()
    fp8 = payload[: md.rank_qdata_numels[0]].view(block, block)
    scale = payload[md.rank_scale_byte_offsets[0] : md.rank_packed_nbytes[0]].view(torch.float32)
    ref_q, ref_s = eager.quantize_blockwise(full.cpu().bfloat16(), block)
    _, fp32_s = eager.quantize_blockwise(full.cpu(), block)
    assert torch.equal(fp8, ref_q.view(torch.uint8)) and fp8[0, 0].item() == g["outlier_byte"]
    assert torch.equal(_bits(scale), _bits(ref_s.view(-1))) and scale.item() == torch.tensor(1 / 448.0).item()
    assert not torch.equal(_bits(scale), _bits(fp32_s.view(-1)))
    # larger, vector-path version of the same dtype pair
    gen = torch.Generator().manual_seed(3)
    big = torch.randn(256, 256, generator=gen) * 0.02
    pl = Fp8BucketedBlockShard(world_size=1, weight_factory=_factory)
    param = nn.Parameter(big.to(device))
    (info,) = make_param_infos([("w", param)], pl, FakeMesh(1))
    info.param_dtype = torch.bfloat16
    payload = pl.prepare_unshard_bucket([param.detach()], [info], FakeMesh(1), None).buffers[0].cpu()
    oq, osc = cport.quantize_blockwise(big, 128, cast_to_bf16=True)
    assert torch.equal(payload[: 256 * 256], oq.reshape(-1))
    assert torch.equal(payload[256 * 256 :].view(torch.int32), _bits(osc).view(-1))



@pytest.mark.parametrize("nparams,world", [(3, 1), (9, 2), (26, 1)])
def test_fp32_master_buckets_on_the_vector_kernel(device, nparams, world):
    """fp32 master shards with a bf16 parameter dtype on 128x128 tiles take a
    vector kernel of their own (8- and 24-entry chunk lookup, whole and
    partial tiles), which rounds to bf16 as it loads.  Every element's low 16
    bits are set to one of the tails that decide that rounding (exact, just
    above, just below a tie, ties to even in both directions), and single
    tiles hold fp32 denormals, values that round up to infinity, an infinity,
    and NaNs of both signs; against the C oracle on the values cast by torch.
    A NaN tile's bytes are compared without their sign (a NaN's sign depends on
    the platform), its scale must be NaN."""
    gen = torch.Generator().manual_seed(100 * nparams + world)
    shapes = [((256, 256), (130, 136), (384, 128), (64, 200), (128, 520))[i % 5] for i in range(nparams)]
    tails = torch.tensor([0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF], dtype=torch.int32)
    masters = []
    for shape in shapes:
        bits = (torch.randn(shape, generator=gen) * 0.02).view(torch.int32)
        pick = torch.randint(0, len(tails), shape, generator=gen)
        masters.append(((bits & ~0xFFFF) | tails[pick]).view(torch.float32))
    masters[0][:128, :128] *= 2.0**-120  # fp32 denormals and tiny normals
    masters[0][128, 128] = 3.4e38  # rounds up to the bf16 infinity
    masters[0][128:, :128].view(torch.int32)[5, 7] = 0x7F800000  # an infinity of its own tile
    masters[1][0, 0] = float("nan")
    masters[2][130, 5] = -float("nan")
    nan_tiles = {1: [(0, 0)], 2: [(1, 0)]}
    named = [(f"w{i}", nn.Parameter(m.to(device), requires_grad=False)) for i, m in enumerate(masters)]
    pl = Fp8BucketedBlockShard(world_size=world, weight_factory=_factory)
    lay = olayout.quant_layout(shapes, 128, world)
    qs, ss = zip(*[cport.quantize_blockwise(m, 128, cast_to_bf16=True) for m in masters])
    eq, es = zip(*[cport.quantize_blockwise(m.bfloat16(), 128) for m in masters])
    for a, b, c, d in zip(qs, eq, ss, es):  # the oracle's own rounding equals torch's cast (NaN signs aside)
        assert ((a == b) | (((a & 0x7F) == 0x7F) & ((b & 0x7F) == 0x7F))).all()
        assert ((_bits(c) == _bits(d)) | (c.isnan() & d.isnan())).all()
    for rank in range(world):
        mesh = FakeMesh(world, rank)
        infos = make_param_infos(named, pl, mesh)
        for info in infos:
            info.param_dtype = torch.bfloat16
        shards = [local_rows(p, i) for (_, p), i in zip(named, infos)]
        got = pl.prepare_unshard_bucket(shards, infos, mesh, None).buffers[0].cpu()
        want = olayout.pack_rank_payload(lay, rank, list(qs), list(ss), 128)
        same = got == want
        if not bool(same.all()):
            # only NaN tiles may differ, and only in the sign bit of their bytes
            diff = (~same).nonzero().view(-1)
            assert ((got[diff] & 0x7F) == 0x7F).all() and ((want[diff] & 0x7F) == 0x7F).all(), f"rank {rank}"
    full_q = [q.clone() for q in qs]
    for index, tiles in nan_tiles.items():
        if index < nparams:
            for tr, tc in tiles:
                tile = full_q[index][128 * tr : 128 * tr + 128, 128 * tc : 128 * tc + 128]
                assert ((tile & 0x7F) == 0x7F).all() and ss[index][tr, tc].isnan()


@pytest.mark.parametrize("shape,block", [((6, 4), 4), ((12, 6), 4), ((130, 129), 128), ((256, 384), 128), ((130, 136), 128), ((64, 64), 16), ((1, 3), 4)])
def test_fp16_shards_quantize_like_their_fp32_values(device, shape, block):
    """An fp16 weight (and an fp32 master quantized as fp16) against the eager
    restatement of the reference on fp16 input.  fp16 to fp32 is exact and no
    nonzero fp16 amax lies below the 1e-12 floor, so for every tile with a
    nonzero amax the result also equals the (pinned) C quantization of the
    upcast values.  In fp16 the floor itself rounds to zero: an all-zero tile
    gets scale inf, stored reciprocal 0 and NaN bytes (0 x inf), as the
    reference's arithmetic gives; the sign of that NaN depends on the platform
    and is not compared.  With the fp32 floor the zero tile is finite."""
    gen = torch.Generator().manual_seed(shape[0] * 31 + shape[1])
    w = (torch.randn(shape, generator=gen) * 0.05).half()
    w[0, 0] = 6.1e-5  # subnormal and tiny values keep their exact magnitude
    w[-1, -1] = 65504.0
    oq, osc = eager.quantize_blockwise(w, block)
    q, s = _quant_gpu(w.to(device), block)
    assert torch.equal(q, oq.view(torch.uint8)) and torch.equal(_bits(s), _bits(osc))
    cq, csc = cport.quantize_blockwise(w.float(), block)
    assert torch.equal(q, cq) and torch.equal(_bits(s), _bits(csc))
    # an fp32 master whose parameter dtype is fp16 quantizes its fp16 rounding
    master = w.float() * (1 + 2.0**-13)
    pl = Fp8BucketedBlockShard(world_size=1, weight_factory=_factory, block_size=block)
    param = nn.Parameter(master.to(device))
    (info,) = make_param_infos([("w", param)], pl, FakeMesh(1))
    info.param_dtype = torch.float16
    prepared = pl.prepare_unshard_bucket([param.detach()], [info], FakeMesh(1), None)
    md = prepared.placement_state.metadata
    payload = prepared.buffers[0].cpu()
    rq, rs = eager.quantize_blockwise(master.half(), block)
    assert torch.equal(payload[: md.rank_qdata_numels[0]], rq.view(torch.uint8).reshape(-1))
    assert torch.equal(payload[md.rank_scale_byte_offsets[0] : md.rank_packed_nbytes[0]].view(torch.int32), _bits(rs).view(-1))
    # zero tile
    z = w.clone()
    z[:block, :block] = 0
    q, s = _quant_gpu(z.to(device), block)
    oq, osc = eager.quantize_blockwise(z, block)
    tile = torch.zeros(shape, dtype=torch.bool)
    tile[:block, :block] = True
    assert s[0, 0].item() == 0.0 and osc[0, 0].item() == 0.0
    assert ((q[tile] & 0x7F) == 0x7F).all() and ((oq.view(torch.uint8)[tile] & 0x7F) == 0x7F).all()
    assert torch.equal(q[~tile], oq.view(torch.uint8)[~tile])
    q, s = _quant_gpu(z.to(device), block, eps_mode=hip_ops.EPS_FP32)
    assert (q[tile] == 0).all() and _bits(s)[0, 0].item() == 0x2720D7C5


def test_strided_and_offset_sources(device):
    """Shards that are row-strided views (unit column stride) or start at an
    odd element are read in place; results equal the contiguous copy."""
    gen = torch.Generator().manual_seed(4)
    parent = (torch.randn(300, 400, generator=gen) * 0.02).bfloat16().to(device)
    for view in (parent[:, 8:264], parent[3:259, 1:130], parent[::2, :128]):
        q, s = _quantize_dense_weight_to_blockwise_fp8(view, 128, E4M3)
        oq, osc = cport.quantize_blockwise(view.cpu().contiguous(), 128)
        assert torch.equal(q.view(torch.uint8).cpu(), oq) and torch.equal(_bits(s.cpu()), _bits(osc))


def test_pack_format_and_pad_zeroing(device):
    """The payload of every rank equals the oracle's naive pack of whole-matrix
    quantization, pads included, even when the buffer held garbage."""
    shapes, block, world = [(16, 8), (8, 8), (12, 4), (1, 3)], 4, 8
    gen = torch.Generator().manual_seed(5)
    params = [torch.randn(s, generator=gen).bfloat16() for s in shapes]
    named = [(f"w{i}", nn.Parameter(p.to(device), requires_grad=False)) for i, p in enumerate(params)]
    pl = Fp8BucketedBlockShard(world_size=world, weight_factory=_factory, block_size=block)
    # poison the allocator's free blocks so stale bytes would show up in pads
    junk = torch.full((1 << 20,), 0xAB, dtype=torch.uint8, device=device)
    del junk
    prepared = prepare_unshard_on_each_rank(pl, named, world)
    lay = olayout.quant_layout(shapes, block, world)
    qs, ss = zip(*[cport.quantize_blockwise(p, block) for p in params])
    for rank in range(world):
        want = olayout.pack_rank_payload(lay, rank, list(qs), list(ss), block)
        assert torch.equal(prepared[rank].buffers[0].cpu(), want), f"rank {rank}"
        assert prepared[rank].buffers[1].numel() == world * lay.row_nbytes


def test_many_chunks_split_into_several_launches(device):
    """More chunks than one launch table holds (30 parameters on one rank)."""
    gen = torch.Generator().manual_seed(6)
    params = [(torch.randn(8, 16, generator=gen)).bfloat16() for _ in range(30)]
    named = [(f"w{i}", nn.Parameter(p.to(device), requires_grad=False)) for i, p in enumerate(params)]
    pl = Fp8BucketedBlockShard(world_size=1, weight_factory=_factory, block_size=8)
    (prepared,) = prepare_unshard_on_each_rank(pl, named, 1)
    lay = olayout.quant_layout([(8, 16)] * 30, 8, 1)
    qs, ss = zip(*[cport.quantize_blockwise(p, 8) for p in params])
    assert torch.equal(prepared.buffers[0].cpu(), olayout.pack_rank_payload(lay, 0, list(qs), list(ss), 8))



@pytest.mark.parametrize("nparams,world", [(7, 1), (8, 1), (12, 1), (24, 1), (25, 1), (40, 1), (30, 3)])
def test_vector_kernel_with_many_chunks(device, nparams, world):
    """bf16 shards on 128x128 tiles take the vector kernel, whose chunk lookup
    comes in an 8-entry and a 24-entry form and which is launched once per 24
    chunks: 7, 8, 12, 24, 25 and 40 parameters on one rank, and 30 over three
    ranks, whole and partial tiles, against the oracle's naive pack."""
    gen = torch.Generator().manual_seed(nparams * 10 + world)
    shapes = [((128, 256), (256, 128), (130, 136), (384, 128), (64, 200))[i % 5] for i in range(nparams)]
    params = [(torch.randn(s, generator=gen) * 0.02).bfloat16() for s in shapes]
    named = [(f"w{i}", nn.Parameter(p.to(device), requires_grad=False)) for i, p in enumerate(params)]
    pl = Fp8BucketedBlockShard(world_size=world, weight_factory=_factory)
    prepared = prepare_unshard_on_each_rank(pl, named, world)
    lay = olayout.quant_layout(shapes, 128, world)
    qs, ss = zip(*[cport.quantize_blockwise(p, 128) for p in params])
    for rank in range(world):
        want = olayout.pack_rank_payload(lay, rank, list(qs), list(ss), 128)
        assert torch.equal(prepared[rank].buffers[0].cpu(), want), f"rank {rank}"



@pytest.mark.parametrize("block", [128, 16])
def test_large_pads_of_short_and_empty_ranks_are_zeroed(device, block):
    """One wide single-block-row matrix next to a small one on 3 ranks: the
    ranks that get little or nothing pad their payload up to the longest
    rank's row, hundreds of KB of zeros written by several pad workgroups,
    whatever the buffers held before."""
    shapes = [(block, 300_000), (2 * block, block)]
    gen = torch.Generator().manual_seed(block)
    params = [(torch.randn(s, generator=gen) * 0.02).bfloat16() for s in shapes]
    named = [(f"w{i}", nn.Parameter(p.to(device), requires_grad=False)) for i, p in enumerate(params)]
    pl = Fp8BucketedBlockShard(world_size=3, weight_factory=_factory, block_size=block)
    for _ in range(2):  # the second round takes recycled buffers that held the first round's payloads
        junk = torch.full((64 << 20,), 0xAB, dtype=torch.uint8, device=device)
        del junk
        prepared = prepare_unshard_on_each_rank(pl, named, 3)
        lay = olayout.quant_layout(shapes, block, 3)
        qs, ss = zip(*[cport.quantize_blockwise(p, block) for p in params])
        sizes = []
        for rank in range(3):
            want = olayout.pack_rank_payload(lay, rank, list(qs), list(ss), block)
            got = prepared[rank].buffers[0].cpu()
            assert torch.equal(got, want), f"rank {rank}"
            sizes.append(int((want != 0).sum()))
        assert min(sizes) < max(sizes) // 100  # some rank's row is nearly all padding
        for p in prepared:
            p.buffers[0].fill_(0xCD)  # poison what goes back to the recycled buffers
        del prepared


def test_payload_cache_forward_backward(device):
    """Forward always repacks; a backward graph task may take the cached
    payload back once; compiling bypasses the cache."""
    from unittest.mock import patch

    from flex_shard_amd.custom_placements import blockwise_quant_bucketed_block_shard as mod

    pl = Fp8BucketedBlockShard(world_size=1, weight_factory=_factory, block_size=4)
    param = nn.Parameter(torch.arange(64, dtype=torch.float32, device=device).view(8, 8))
    (info,) = make_param_infos([("w", param)], pl, FakeMesh(1))
    mesh = FakeMesh(1)
    cached = pl.prepare_unshard_bucket([param.detach()], [info], mesh, None)
    with patch.object(torch.compiler, "is_compiling", return_value=True):
        first = pl.prepare_unshard_bucket([param.detach()], [info], mesh, None)
        second = pl.prepare_unshard_bucket([param.detach()], [info], mesh, None)
    with patch.object(mod, "_is_backward_graph_task", return_value=True):
        restored = pl.prepare_unshard_bucket([param.detach()], [info], mesh, None)
        again = pl.prepare_unshard_bucket([param.detach()], [info], mesh, None)
    assert first.buffers[0] is not second.buffers[0] and first.buffers[0] is not cached.buffers[0]
    assert restored.buffers[0] is cached.buffers[0]
    assert again.buffers[0] is not cached.buffers[0]  # the entry is consumed once
    assert torch.equal(again.buffers[0], cached.buffers[0])
    # a source written in place after the forward pack (version counter moved) is packed again
    forward = pl.prepare_unshard_bucket([param.detach()], [info], mesh, None)
    with torch.no_grad():
        param.mul_(-2.0)
    with patch.object(mod, "_is_backward_graph_task", return_value=True):
        repacked = pl.prepare_unshard_bucket([param.detach()], [info], mesh, None)
    assert repacked.buffers[0] is not forward.buffers[0]
    assert not torch.equal(repacked.buffers[0], forward.buffers[0])
    # ... and so is a shard of the same shape at another address
    forward = pl.prepare_unshard_bucket([param.detach()], [info], mesh, None)
    moved = param.detach().clone()
    with patch.object(mod, "_is_backward_graph_task", return_value=True):
        elsewhere = pl.prepare_unshard_bucket([moved], [info], mesh, None)
    assert elsewhere.buffers[0] is not forward.buffers[0] and torch.equal(elsewhere.buffers[0], forward.buffers[0])


def test_two_buckets_in_flight_with_recycled_buffers(device):
    """Three buckets prepared over and over with the current stream alternating
    between two side streams, every payload read on a third stream and handed
    back the way the runtime hands buffers back (the allocation stream waits
    for the reader, then the references go).  Payloads and gather outputs come
    from each stream's recycled buffers, so a buffer reused before its reader
    ran would show up as wrong bytes: every payload must equal the oracle's."""
    from flex_shard_amd.custom_placements import blockwise_quant_bucketed_block_shard as mod
    from flex_shard_amd.flex_shard.bucket_comm import StreamHandoff

    shapes, block, world = [(512, 256), (384, 384), (130, 136)], 128, 2
    pl = Fp8BucketedBlockShard(world_size=world, weight_factory=_factory, block_size=block)
    mesh = FakeMesh(world, 0)
    lay = olayout.quant_layout(shapes, block, world)
    buckets = []
    for b in range(3):
        gen = torch.Generator().manual_seed(40 + b)
        params = [(torch.randn(s, generator=gen) * 0.02).bfloat16() for s in shapes]
        named = [(f"w{i}", nn.Parameter(p.to(device), requires_grad=False)) for i, p in enumerate(params)]
        infos = make_param_infos(named, pl, mesh)
        shards = [local_rows(p, i) for (_, p), i in zip(named, infos)]
        qs, ss = zip(*[cport.quantize_blockwise(p, block) for p in params])
        buckets.append((shards, infos, olayout.pack_rank_payload(lay, 0, list(qs), list(ss), block)))
    sides = [torch.cuda.Stream(device), torch.cuda.Stream(device)]
    reader = torch.cuda.Stream(device)
    main = torch.cuda.current_stream(device)
    rounds = 18
    seen = torch.empty((rounds, lay.row_nbytes), dtype=torch.uint8, device=device)
    addresses = [set(), set()]
    gathered_addresses = [set(), set()]
    try:
        for i in range(rounds):
            shards, infos, _ = buckets[i % 3]
            side = sides[i % 2]
            torch.cuda.set_stream(side)
            prepared = pl.prepare_unshard_bucket(shards, infos, mesh, None)
            packed = torch.cuda.Event()
            packed.record(side)
            addresses[i % 2].add(prepared.buffers[0].data_ptr())
            gathered_addresses[i % 2].add(prepared.buffers[1].data_ptr())
            assert prepared.buffers[1].numel() == world * lay.row_nbytes
            torch.cuda.set_stream(reader)
            reader.wait_event(packed)
            seen[i].copy_(prepared.buffers[0])
            read = torch.cuda.Event()
            read.record(reader)
            StreamHandoff(list(prepared.buffers), (side,)).release_after(read)
            prepared.buffers.clear()
            del prepared
    finally:
        torch.cuda.set_stream(main)
    torch.cuda.synchronize()
    got = seen.cpu()
    for i in range(rounds):
        assert torch.equal(got[i], buckets[i % 3][2]), f"round {i} (bucket {i % 3}, stream {i % 2})"
    # the buffers really were recycled: a handful of addresses served all rounds
    # (the forward payload cache holds one payload per bucket, the rings the rest)
    for side_addresses in addresses:
        assert len(side_addresses) < rounds // 2
    for side_addresses in gathered_addresses:
        assert len(side_addresses) <= mod.GATHER_RING_SLOTS


def test_recycled_payload_is_not_handed_out_while_held(device):
    """A payload (or any view of it) that somebody still holds is never handed
    out again; once dropped, its buffer serves the next call on that stream."""
    pl = Fp8BucketedBlockShard(world_size=1, weight_factory=_factory, block_size=4)
    param = nn.Parameter(torch.arange(64, dtype=torch.float32, device=device).view(8, 8))
    (info,) = make_param_infos([("w", param)], pl, FakeMesh(1))
    mesh = FakeMesh(1)
    shard = param.detach()
    pl.prepare_unshard_bucket([shard], [info], mesh, None)  # first call builds and stores the launch
    held = [pl.prepare_unshard_bucket([shard], [info], mesh, None) for _ in range(6)]
    assert len({p.buffers[0].data_ptr() for p in held}) == 6 and len({p.buffers[1].data_ptr() for p in held}) == 6
    view = held[2].buffers[0][4:12]
    alias = held[3].buffers[0].detach()
    busy = {view.untyped_storage().data_ptr(), alias.untyped_storage().data_ptr()}
    first = held[0].buffers[0].clone()
    del held
    for _ in range(8):
        again = pl.prepare_unshard_bucket([shard], [info], mesh, None)
        assert again.buffers[0].data_ptr() not in busy
        assert torch.equal(again.buffers[0], first)
        del again
    assert torch.equal(view, first[4:12]) and torch.equal(alias, first)


def test_staged_shard_is_read_afresh_on_every_call(device):
    """A shard that cannot be viewed as [rows, in_dim] (a strided slice of a
    stacked parameter) is staged through a temporary copy; the launch of such
    a call is not stored, so the next call reads the shard as it is then and
    never the first call's temporary."""
    pl = Fp8BucketedBlockShard(world_size=1, weight_factory=_factory, block_size=4)
    gen = torch.Generator().manual_seed(9)
    big = torch.randn(2, 8, 32, generator=gen).bfloat16().to(device)
    param = nn.Parameter(torch.empty(2, 8, 16, dtype=torch.bfloat16, device=device), requires_grad=False)
    (info,) = make_param_infos([("experts.w", param)], pl, FakeMesh(1))
    mesh = FakeMesh(1)
    shard = big[:, :, :16]  # [2, 8, 16] with a row stride of 32: reshape to [16, 16] must copy
    assert not shard.is_contiguous()

    def expected():
        oq, osc = cport.quantize_blockwise(shard.cpu().reshape(16, 16), 4)
        return torch.cat([oq.reshape(-1), osc.reshape(-1).view(torch.uint8)])

    first = pl.prepare_unshard_bucket([shard], [info], mesh, None).buffers[0]
    assert torch.equal(first.cpu()[: 256 + 64], expected())
    # whatever now lives where the temporary was must not be read
    junk = [torch.full((16, 16), 7.0, dtype=torch.bfloat16, device=device) for _ in range(8)]
    big.mul_(-3.0)
    second = pl.prepare_unshard_bucket([shard], [info], mesh, None).buffers[0]
    assert torch.equal(second.cpu()[: 256 + 64], expected())
    assert not torch.equal(first.cpu(), second.cpu())
    del junk
    # a lazily negated shard is staged as well (the kernel reads raw bits)
    flat = torch.randn(16, 16, generator=gen).bfloat16().to(device)
    negated = torch._neg_view(flat).view(1, 16, 16)
    param1 = nn.Parameter(torch.empty(1, 16, 16, dtype=torch.bfloat16, device=device), requires_grad=False)
    (info1,) = make_param_infos([("w", param1)], pl, FakeMesh(1))
    got = pl.prepare_unshard_bucket([negated], [info1], mesh, None).buffers[0].cpu()
    oq, osc = cport.quantize_blockwise((-flat).cpu(), 4)
    assert torch.equal(got[:256], oq.reshape(-1))


def test_argument_errors(device):
    pl = Fp8BucketedBlockShard(world_size=1, weight_factory=_factory, block_size=4)
    param = nn.Parameter(torch.zeros(8, 8, device=device))
    infos = make_param_infos([("w", param)], pl, FakeMesh(1))
    with pytest.raises(ValueError, match="one tensor per ParamInfo"):
        pl.prepare_unshard_bucket([], infos, FakeMesh(1), None)
    with pytest.raises((AssertionError, RuntimeError)):
        pl.prepare_unshard_bucket([torch.zeros(4, 8, device=device)], infos, FakeMesh(1), None)
    payload = torch.empty(10, dtype=torch.uint8, device=device)
    spec = hip_ops.QuantChunkSpec(torch.zeros(4, 4, dtype=torch.bfloat16, device=device), 0, 16, hip_ops.SRC_BF16)
    with pytest.raises(RuntimeError, match="outside payload"):
        hip_ops.quantize_pack([spec], payload, ((0, 0), (0, 0)), 4)


# ------------------------------------------------------------ full-size cases
def test_llama_layer_bucket_rank0_and_worst_rank(device, golden):
    """Config 2 at full size: rank 0's share (27 262 976 elements, 4 chunks)
    bit-exact against the C oracle, every rank's payload consistent with
    whole-matrix quantization on the GPU (quantize-then-gather ==
    gather-then-quantize)."""
    g = golden["llama3_8b_layer_plan"]
    named = seeded_bucket(LLAMA3_8B_LAYER, 0.02, 100, device)
    pl = Fp8BucketedBlockShard(world_size=8, weight_factory=_factory)
    prepared = prepare_unshard_on_each_rank(pl, named, 8)
    md = prepared[0].placement_state.metadata
    assert md.packed_send_nbytes_per_rank == g["row_nbytes"] and md.rank_qdata_numels[0] == g["rank0_numel"]
    # rank 0 against the oracle, chunk by chunk
    payload0 = prepared[0].buffers[0].cpu()
    infos0 = make_param_infos(named, pl, FakeMesh(8, 0))
    cursor, scale_cursor = 0, md.rank_scale_byte_offsets[0]
    for (fqn, param), info in zip(named, infos0):
        if info.local_numel == 0:
            continue
        shard = local_rows(param, info).cpu().flatten(0, -2)
        oq, osc = cport.quantize_blockwise(shard, 128)
        assert torch.equal(payload0[cursor : cursor + oq.numel()], oq.reshape(-1)), fqn
        sb = osc.reshape(-1).view(torch.uint8)
        assert torch.equal(payload0[scale_cursor : scale_cursor + sb.numel()], sb), fqn
        cursor += oq.numel()
        scale_cursor += sb.numel()
    assert cursor == g["rank0_numel"] and (payload0[scale_cursor:] == 0).all()
    # every rank against whole-matrix quantization on the GPU
    whole = [_quantize_dense_weight_to_blockwise_fp8(p.detach(), 128, E4M3) for _, p in named]
    data = torch.cat([q.view(torch.uint8).reshape(-1) for q, _ in whole])
    scales = torch.cat([s.reshape(-1) for _, s in whole])
    d_cursor = s_cursor = 0
    for rank in range(8):
        row = prepared[rank].buffers[0]
        n, sn = md.rank_qdata_numels[rank], md.rank_scale_numels[rank]
        assert torch.equal(row[:n], data[d_cursor : d_cursor + n]), f"rank {rank} data"
        s0 = md.rank_scale_byte_offsets[rank]
        assert torch.equal(row[s0 : s0 + 4 * sn].view(torch.float32), scales[s_cursor : s_cursor + sn]), f"rank {rank}"
        d_cursor += n
        s_cursor += sn
    assert d_cursor == g["global_numel"]
    # one whole matrix against the oracle as an anchor for the GPU-vs-GPU check
    oq, osc = cport.quantize_blockwise(named[1][1].detach().cpu(), 128)
    assert torch.equal(whole[1][0].view(torch.uint8).cpu(), oq) and torch.equal(_bits(whole[1][1].cpu()), _bits(osc))


def test_deepseek_expert_bucket_edge_tiles(device):
    """Config 3: stacked [32, 2048, 7168] / [32, 7168, 2048] experts with 50x
    outliers and all-zero tiles; rank 0's share (w1 rows 0..24 575) is checked
    against the oracle on sampled block rows that cover the edge cases."""
    named = seeded_bucket(DEEPSEEK_V3_EXPERTS, 0.006, 300, device)
    for i, (_, p) in enumerate(named):
        add_outliers_and_zero_tiles(p, 400 + i)
    w1 = named[0][1]
    w1.data[0, :128, :] = 0  # one all-zero chunk row band on rank 0
    pl = Fp8BucketedBlockShard(world_size=8, weight_factory=_factory)
    mesh = FakeMesh(8, 0)
    infos = make_param_infos(named, pl, mesh)
    assert infos[0].local_numel == 24576 * 7168 and infos[1].local_numel == 0 and infos[2].local_numel == 0
    shards = [local_rows(p, i) for (_, p), i in zip(named, infos)]
    prepared = pl.prepare_unshard_bucket(shards, infos, mesh, None)
    md = prepared.placement_state.metadata
    assert md.rank_qdata_numels[0] == 176160768 and md.rank_scale_numels[0] == 10752
    payload = prepared.buffers[0]
    flat = w1.detach().flatten(0, -2)
    gen = torch.Generator().manual_seed(7)
    bands = sorted({0, 1, 191, *torch.randint(0, 192, (10,), generator=gen).tolist()})
    s0 = md.rank_scale_byte_offsets[0]
    scales = payload[s0 : s0 + 4 * 10752].view(torch.float32).view(192, 56)
    zero_scale_bits = 0x27212492
    saw_zero_tile = False
    for band in bands:
        rows = flat[band * 128 : (band + 1) * 128].cpu()
        oq, osc = cport.quantize_blockwise(rows, 128)
        got = payload[band * 128 * 7168 : (band + 1) * 128 * 7168].view(128, 7168).cpu()
        assert torch.equal(got, oq), f"band {band}"
        assert torch.equal(_bits(scales[band].cpu()), _bits(osc.view(-1))), f"band {band}"
        saw_zero_tile |= bool((_bits(osc) == zero_scale_bits).any())
    assert saw_zero_tile
    assert (scales[0].view(torch.int32) == zero_scale_bits).all()


def test_deepseek_rank_inside_w2_and_llama_down_against_the_oracle(device):
    """Shares other than rank 0's at full size, on sampled 128-row bands
    against the C oracle: rank 3 of the DeepSeek-V3 expert bucket (its whole
    share lies in w2, in_dim 2048, rows of several experts) and rank 7 of the
    Llama bucket (rows of `down`, in_dim 14336)."""
    gen = torch.Generator().manual_seed(17)
    for spec, std, rank, fqn, seed in (
        (DEEPSEEK_V3_EXPERTS, 0.006, 3, "experts.w2", 310),
        (LLAMA3_8B_LAYER, 0.02, 7, "down", 110),
    ):
        named = seeded_bucket(spec, std, seed, device)
        if spec is DEEPSEEK_V3_EXPERTS:
            for i, (_, p) in enumerate(named):
                add_outliers_and_zero_tiles(p, 410 + i)
        pl = Fp8BucketedBlockShard(world_size=8, weight_factory=_factory)
        mesh = FakeMesh(8, rank)
        infos = make_param_infos(named, pl, mesh)
        live = [i for i in infos if i.local_numel]
        assert [i.fqn for i in live] == [fqn], [i.fqn for i in live]
        shards = [local_rows(p, i) for (_, p), i in zip(named, infos)]
        prepared = pl.prepare_unshard_bucket(shards, infos, mesh, None)
        md = prepared.placement_state.metadata
        payload = prepared.buffers[0]
        index = [i.fqn for i in infos].index(fqn)
        shard = shards[index].flatten(0, -2)
        rows, in_dim = shard.shape
        assert rows * in_dim == md.rank_qdata_numels[rank] and rows % 128 == 0
        tiles_c = in_dim // 128
        s0 = md.rank_scale_byte_offsets[rank]
        scales = payload[s0 : s0 + 4 * md.rank_scale_numels[rank]].view(torch.float32).view(rows // 128, tiles_c)
        bands = sorted({0, rows // 128 - 1, *torch.randint(0, rows // 128, (10,), generator=gen).tolist()})
        for band in bands:
            oq, osc = cport.quantize_blockwise(shard[band * 128 : (band + 1) * 128].cpu(), 128)
            got = payload[band * 128 * in_dim : (band + 1) * 128 * in_dim].view(128, in_dim).cpu()
            assert torch.equal(got, oq), f"{fqn} band {band}"
            assert torch.equal(_bits(scales[band].cpu()), _bits(osc.view(-1))), f"{fqn} band {band}"
        assert (payload[md.rank_qdata_numels[rank] : s0] == 0).all()
        del named, shards, prepared, payload
        torch.cuda.empty_cache()
