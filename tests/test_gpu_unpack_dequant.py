"""GPU parity of the unpack side: rank-row compaction (segment copy), the fused
compaction + dequantization kernel, and the dequantizer, against the oracle."""

import numpy as np
import pytest
import torch
import torch.nn as nn

from flex_shard_amd import Fp8BucketedBlockShard
from flex_shard_amd.blockwise_fp8 import BlockwiseFp8Weight, blockwise_dequant_weight, make_blockwise_fp8_weight
from flex_shard_amd.custom_placements._copy_kernels import SegmentCopyDescriptor, copy_segments, zero_segments
from flex_shard_amd.testing import (
    LLAMA3_8B_LAYER,
    FakeMesh,
    gather_rank_rows,
    make_param_infos,
    prepare_unshard_on_each_rank,
    seeded_bucket,
)
from oracle import cport
from oracle import eager as eager_oracle
from oracle import layout as olayout

pytestmark = pytest.mark.gpu
E4M3 = torch.float8_e4m3fn


class RecordingFactory:
    def __init__(self):
        self.calls = []

    def __call__(self, fp8_data, recip_scale, block_size, *, orig_dtype, requires_grad):
        self.calls.append((fp8_data, recip_scale, block_size, orig_dtype, requires_grad))
        return fp8_data


def _return_fp8(fp8_data, recip_scale, block_size, *, orig_dtype, requires_grad):
    return fp8_data


def _bits(t):
    return t.contiguous().view(torch.int32)


def test_compacts_strided_rank_rows_into_shared_storage(device, golden):
    """Reference case: W=8, block 4, params 16x8, 8x8, 1x3 of arange values,
    gathered rows strided and starting at an odd byte; the compact buffer is
    align16(sum numel) + 4 * sum scales bytes, every factory view shares its
    storage, and bytes/scales equal whole-matrix quantization."""
    g = golden["compact_unshard_case"]
    block, world = g["block"], g["world_size"]
    factory = RecordingFactory()
    pl = Fp8BucketedBlockShard(world_size=world, weight_factory=factory, block_size=block)
    named = []
    for i, shape in enumerate(g["shapes"]):
        n = shape[0] * shape[1]
        named.append((f"w{i + 1}", nn.Parameter(torch.arange(n, dtype=torch.float32, device=device).reshape(shape))))
    prepared_by_rank = prepare_unshard_on_each_rank(pl, named, world)
    prepared = prepared_by_rank[0]
    md = prepared.placement_state.metadata
    row = md.packed_send_nbytes_per_rank
    parent = torch.full((world, row + g["row_extra_bytes"]), 0xFF, dtype=torch.uint8, device=device)
    rank_rows = parent[:, g["row_byte_offset"] : row + g["row_byte_offset"]]
    assert not rank_rows.is_contiguous() and rank_rows.storage_offset() % 4 == 1
    for rank, p in enumerate(prepared_by_rank):
        local = p.buffers[0]
        n, s0, end = md.rank_qdata_numels[rank], md.rank_scale_byte_offsets[rank], md.rank_packed_nbytes[rank]
        rank_rows[rank, :n].copy_(local[:n])
        rank_rows[rank, s0:end].copy_(local[s0:end])
    prepared.persistent = True
    result = pl._finish_unshard_from_rank_rows(prepared, rank_rows)
    (compact,) = result.persistent_buffers
    fp8_nbytes = sum(p.numel() for _, p in named)
    assert fp8_nbytes % 4 != 0 and 0 in md.rank_qdata_numels
    scale_numel = sum(-(-p.shape[0] // block) * -(-p.shape[1] // block) for _, p in named)
    assert compact.dtype == torch.uint8 and compact.numel() == -(-fp8_nbytes // 16) * 16 + 4 * scale_numel
    base = compact.untyped_storage().data_ptr()
    for weight, call, (_, full) in zip(result.full_params, factory.calls, named, strict=True):
        fp8, recip, blk, orig_dtype, requires_grad = call
        oq, osc = cport.quantize_blockwise(full.detach().cpu(), block)
        assert weight is fp8 and blk == block and orig_dtype == full.dtype and requires_grad == full.requires_grad
        assert fp8.is_contiguous() and recip.is_contiguous()
        assert fp8.untyped_storage().data_ptr() == base and recip.untyped_storage().data_ptr() == base
        assert torch.equal(fp8.view(torch.uint8).cpu(), oq) and torch.equal(_bits(recip.cpu()), _bits(osc))
    # a persistent refill writes the same buffer in place and returns it
    prepared.persistent_buffers = [compact]
    compact.fill_(0x55)
    again = pl._finish_unshard_from_rank_rows(prepared, rank_rows)
    assert again.persistent_buffers[0] is compact
    assert torch.equal(factory.calls[-3][0].view(torch.uint8).cpu(), cport.quantize_blockwise(named[0][1].detach().cpu(), block)[0])


def test_stacked_weight_is_quantized_as_flattened_matrix(device):
    factory = RecordingFactory()
    pl = Fp8BucketedBlockShard(world_size=3, weight_factory=factory, block_size=4)
    torch.manual_seed(0)
    param = nn.Parameter(torch.randn(2, 6, 8, device=device))
    prepared = prepare_unshard_on_each_rank(pl, [("w13", param)], 3)
    pl._finish_unshard_from_rank_rows(prepared[0], gather_rank_rows(prepared))
    ((fp8, recip, *_),) = factory.calls
    oq, osc = cport.quantize_blockwise(param.detach().cpu().flatten(0, -2), 4)
    assert fp8.shape == param.shape
    assert torch.equal(fp8.flatten(0, -2).view(torch.uint8).cpu(), oq) and torch.equal(_bits(recip.cpu()), _bits(osc))


def test_fused_copy_out_matches_oracle_for_every_row_layout(device, golden):
    """Aligned and odd region sizes x contiguous / spaced / odd-offset rows:
    the one-launch copy-out equals the oracle's compaction byte for byte, and
    bytes outside the written regions keep their old value."""
    g = golden["fused_copy_out_cases"]
    for case_name, case in g["cases"].items():
        pl = Fp8BucketedBlockShard(world_size=g["world_size"], weight_factory=_return_fp8, block_size=g["block"])
        named = [(f"w{i}", nn.Parameter(torch.empty(tuple(s), device="meta"))) for i, s in enumerate(case["shapes"])]
        infos = make_param_infos(named, pl, FakeMesh(g["world_size"]))
        md = pl._quant_metadata_from_infos(infos)
        lay = olayout.quant_layout(case["shapes"], g["block"], g["world_size"])
        world, row = g["world_size"], md.packed_send_nbytes_per_rank
        assert row == lay.row_nbytes
        for layout_name, (offset, padding) in g["row_layouts"].items():
            gen = torch.Generator().manual_seed(1)
            parent = torch.randint(0, 256, (world, offset + row + padding), dtype=torch.uint8, generator=gen)
            rows_cpu = parent[:, offset : offset + row]
            rows_gpu = parent.to(device)[:, offset : offset + row]
            want = olayout.compact_from_rank_rows(lay, rows_cpu, fill=0xAB)
            fused = torch.full((want.numel(),), 0xAB, dtype=torch.uint8, device=device)
            assert pl._copy_out_rank_rows_fused(md, rows_gpu, fused)
            assert torch.equal(fused.cpu(), want), f"{case_name} / {layout_name}"
            plan = pl._copy_out_plan(md, data_elem_nbytes=1, with_scales=True)
            unit = case["aligned_unit"] if offset == 0 else 1
            assert (rows_gpu.device, rows_gpu.stride(0), unit) in plan.descriptors
            # the torch.cat form used under torch.compile agrees
            cat = torch.full_like(fused, 0xAB)
            data_total = sum(md.rank_qdata_numels)
            pl._copy_out_rank_rows_cat(md, rows_gpu, cat, qdata_nbytes=data_total, scale_byte_offset=-(-data_total // 16) * 16)
            assert torch.equal(cat, fused)


def test_copy_plan_is_built_once_per_row_stride(device):
    pl = Fp8BucketedBlockShard(world_size=8, weight_factory=_return_fp8, block_size=4)
    named = [(f"w{i}", nn.Parameter(torch.empty(s, device="meta"))) for i, s in enumerate([(16, 8), (8, 8), (6, 4)])]
    md = pl._quant_metadata_from_infos(make_param_infos(named, pl, FakeMesh(8)))
    row = md.packed_send_nbytes_per_rank
    compact = torch.empty(row * 8, dtype=torch.uint8, device=device)
    rows = torch.zeros((8, row), dtype=torch.uint8, device=device)
    pl._copy_out_rank_rows_fused(md, rows, compact)
    plan = pl._copy_out_plan(md, data_elem_nbytes=1, with_scales=True)
    (descriptor,) = plan.descriptors.values()
    pl._copy_out_rank_rows_fused(md, rows, compact)
    assert list(plan.descriptors.values()) == [descriptor]
    spaced = torch.zeros((8, row + 16), dtype=torch.uint8, device=device)[:, :row]
    pl._copy_out_rank_rows_fused(md, spaced, compact)
    assert len(plan.descriptors) == 2


def test_copy_out_falls_back_only_while_compiling(device):
    from unittest.mock import patch

    pl = Fp8BucketedBlockShard(world_size=8, weight_factory=_return_fp8, block_size=4)
    named = [("w0", nn.Parameter(torch.empty(16, 8, device="meta")))]
    md = pl._quant_metadata_from_infos(make_param_infos(named, pl, FakeMesh(8)))
    rows = torch.zeros((8, md.packed_send_nbytes_per_rank), dtype=torch.uint8, device=device)
    compact = torch.empty(rows.numel(), dtype=torch.uint8, device=device)
    with patch.object(torch.compiler, "is_compiling", return_value=True):
        assert not pl._copy_out_rank_rows_fused(md, rows, compact)
    with pytest.raises(RuntimeError, match="no CPU compute path"):
        pl._copy_out_rank_rows_fused(md, rows.cpu(), compact)
    with pytest.raises(ValueError, match="shape"):
        prepared = prepare_unshard_on_each_rank(
            pl, [("w0", nn.Parameter(torch.zeros(16, 8, device=device)))], 8
        )[0]
        pl._finish_unshard_from_rank_rows(prepared, rows[:, :-16])
    with pytest.raises(ValueError, match="uint8"):
        pl._finish_unshard_from_rank_rows(prepared, rows.view(torch.int8))


def test_dense_rows_join_with_wider_elements(device):
    """data_elem_nbytes=2 without scales: joins bf16 rank rows (the dense
    all-gather reference layout) in rank order."""
    pl = Fp8BucketedBlockShard(world_size=8, weight_factory=_return_fp8, block_size=4)
    named = [(f"w{i}", nn.Parameter(torch.empty(s, device="meta"))) for i, s in enumerate([(16, 8), (8, 8), (1, 3)])]
    md = pl._quant_metadata_from_infos(make_param_infos(named, pl, FakeMesh(8)))
    for row_numel in (max(md.rank_qdata_numels) + 5, 64):
        rows = torch.randn((8, row_numel), dtype=torch.bfloat16, device=device)
        joined = rows.new_empty(sum(md.rank_qdata_numels))
        assert pl._copy_out_rank_rows_fused(
            md, rows.view(torch.uint8), joined.view(torch.uint8), data_elem_nbytes=2, with_scales=False
        )
        want = torch.cat([rows[r, :n] for r, n in enumerate(md.rank_qdata_numels)])
        assert torch.equal(joined.view(torch.int16), want.view(torch.int16))


def test_segment_copy_splits_long_segments(device, golden):
    g = golden["segment_split_case"]
    gen = torch.Generator().manual_seed(2)
    source = torch.randint(-(2**31), 2**31 - 1, (g["source_numel"],), dtype=torch.int32, generator=gen).to(device)
    segs = g["segments"]
    desc = SegmentCopyDescriptor.create(
        src_offsets=[s for s, _, _ in segs], numels=[n for _, n, _ in segs], dst_offsets=[d for _, _, d in segs],
        device=device, block_size=g["block_size"], max_chunks_per_segment=g["max_chunks_per_segment"],
    )
    assert desc.nsegments > len(segs) and desc.max_segment_numel == g["max_segment_numel"]
    out = torch.zeros(g["output_numel"], dtype=torch.int32, device=device)
    copy_segments(source, out, desc)
    want = torch.zeros_like(out)
    for s, n, d in segs:
        want[d : d + n] = source[s : s + n]
    assert torch.equal(out, want)
    # every unit size, odd relative alignment, and the zero kernel
    for dtype in (torch.uint8, torch.int16, torch.int32, torch.int64):
        src = torch.randint(0, 100, (5000,), generator=gen).to(dtype).to(device)
        dst = torch.full((6000,), 7, dtype=dtype, device=device)
        d2 = SegmentCopyDescriptor.create(src_offsets=[3, 1001], numels=[997, 3333], dst_offsets=[10, 1500], device=device)
        copy_segments(src, dst, d2)
        ref = torch.full((6000,), 7, dtype=dtype, device=device)
        ref[10:1007] = src[3:1000]
        ref[1500:4833] = src[1001:4334]
        assert torch.equal(dst, ref)
        zero_segments(dst, d2)
        ref[10:1007] = 0
        ref[1500:4833] = 0
        assert torch.equal(dst, ref)



@pytest.mark.parametrize("nsegments,longest", [(300, 200_000), (6000, 9_000), (9, 3_000_000)])
def test_segment_copy_shares_slices_of_uneven_segments(device, nsegments, longest):
    """Large launches over segments of very different lengths: a few hundred
    segments, several thousand short ones, and a few long ones, in any address
    order, at every unit size and relative alignment; then the zero kernel
    over the same destinations.  Bytes outside the segments stay."""
    rng = np.random.default_rng(nsegments)
    numels = rng.integers(0, longest, nsegments).tolist()
    numels[nsegments // 2] = longest  # the longest sizes the launch
    numels[0] = 0
    gaps = rng.integers(0, 9, nsegments).tolist()
    src_offs, dst_offs, s_cur, d_cur = [], [], 0, 3
    for n, gap in zip(numels, gaps):
        src_offs.append(s_cur)
        dst_offs.append(d_cur)
        s_cur += n + (gap % 3)
        d_cur += n + gap
    order = rng.permutation(nsegments).tolist()  # segments need not be sorted by address
    pick = lambda values: [values[i] for i in order]
    for dtype in (torch.uint8, torch.int16, torch.int64):
        src_host = torch.from_numpy(rng.integers(0, 120, s_cur + 1).astype(np.int64)).to(dtype)
        dst_host = torch.full((d_cur + 5,), 7, dtype=dtype)
        desc = SegmentCopyDescriptor.create(
            src_offsets=pick(src_offs), numels=pick(numels), dst_offsets=pick(dst_offs), device=device
        )
        dst = dst_host.to(device)
        copy_segments(src_host.to(device), dst, desc)
        want = dst_host.clone()
        for s, n, d in zip(src_offs, numels, dst_offs):
            want[d : d + n] = src_host[s : s + n]
        assert torch.equal(dst.cpu(), want)
        zero_segments(dst, desc)
        for n, d in zip(numels, dst_offs):
            want[d : d + n] = 0
        assert torch.equal(dst.cpu(), want)


# ---------------------------------------------------------------- dequantize
def test_dequant_known_answers(device, golden):
    g = golden["dequant_flat"]
    fp8 = torch.arange(128, dtype=torch.bfloat16).reshape(g["shape"]).to(E4M3).to(device)
    scale = torch.full(g["scale_shape"], g["scale"], dtype=torch.float32, device=device)
    wrapped = BlockwiseFp8Weight(fp8, scale, g["block"], orig_dtype=torch.bfloat16, requires_grad=True)
    assert wrapped.dtype == torch.bfloat16 and wrapped.requires_grad and wrapped.block_size == 4
    assert torch.equal(wrapped.dequantize(torch.float32), fp8.float() * g["scale"])
    assert torch.equal(wrapped.dequantize(), (fp8.float() * g["scale"]).bfloat16())

    g = golden["dequant_stacked"]
    fp8 = torch.arange(96, dtype=torch.bfloat16).reshape(g["shape"]).to(E4M3).to(device)
    scale = torch.tensor(g["scales"], dtype=torch.float32, device=device)
    wrapped = make_blockwise_fp8_weight(fp8, scale, g["block"], orig_dtype=torch.bfloat16, requires_grad=False)
    per_elem = scale.repeat_interleave(4, 0).repeat_interleave(4, 1).view(g["shape"])
    assert wrapped.shape == tuple(g["shape"])
    assert torch.equal(wrapped.dequantize(torch.float32), fp8.float() * per_elem)
    with pytest.raises(ValueError, match="scale shape"):
        BlockwiseFp8Weight(fp8, scale[:2], 4)


@pytest.mark.parametrize("shape,block", [((256, 384), 128), ((200, 136), 128), ((130, 129), 128), ((16, 32), 4), ((300, 208), 64)])
def test_dequant_is_bit_exact_with_oracle(device, shape, block):
    """Every FP8 byte value times random scales, fp32 and bf16 outputs: 0 ULP."""
    gen = torch.Generator().manual_seed(3)
    data = torch.randint(0, 256, shape, dtype=torch.uint8, generator=gen)
    data[(data & 0x7F) == 0x7F] = 0x3C  # NaN encodings are compared separately
    scale = torch.rand(-(-shape[0] // block), -(-shape[1] // block), generator=gen) * 1e-3 + 1e-6
    for dtype in (torch.float32, torch.bfloat16):
        got = blockwise_dequant_weight(data.to(device).view(E4M3), scale.to(device), block, dtype).cpu()
        want = cport.dequant_blockwise(data, scale, block, dtype)
        view = torch.int32 if dtype == torch.float32 else torch.int16
        assert torch.equal(got.view(view), want.view(view))
    # fp16 output: torch's own cast of the fp32 product (these scales put most products among the fp16
    # subnormals, exact ties included, and the larger ones past fp16's range)
    for factor in (1.0, 64.0, 3.0e4):
        got = blockwise_dequant_weight(data.to(device).view(E4M3), (scale * factor).to(device), block, torch.float16).cpu()
        want = eager_oracle.dequant_blockwise(data.view(E4M3), scale * factor, block, torch.float16)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    nan = torch.full((4, 4), 0x7F, dtype=torch.uint8)
    assert blockwise_dequant_weight(nan.to(device).view(E4M3), torch.ones(1, 1, device=device), 4).isnan().all()
    assert blockwise_dequant_weight(nan.to(device).view(E4M3), torch.ones(1, 1, device=device), 4, torch.float16).isnan().all()




@pytest.mark.parametrize("block,shapes", [
    (128, [(256, 128), (130, 136), (384, 256), (128, 128)] * 18),
    (4, [(16, 8), (9, 12), (8, 8), (5, 3), (12, 4)] * 15),
])
def test_fused_unpack_with_more_than_64_chunks(device, block, shapes):
    """The tile-to-chunk lookup resolves up to 64 chunks with one ballot and
    bisects beyond that: 72 and 75 parameters over 8 ranks (a chunk per
    parameter and rank that holds rows of it: more than 64), compact bytes,
    scales and dequantized values against the oracle."""
    world = 8
    factory = RecordingFactory()
    pl = Fp8BucketedBlockShard(world_size=world, weight_factory=factory, block_size=block)
    gen = torch.Generator().manual_seed(len(shapes) + block)
    named = [(f"w{i}", nn.Parameter((torch.randn(s, generator=gen) * 0.02).bfloat16().to(device), requires_grad=False))
             for i, s in enumerate(shapes)]
    prepared = prepare_unshard_on_each_rank(pl, named, world)
    rows = gather_rank_rows(prepared)
    table, starts, total_tiles, _ = pl._unpack_table(pl._unshard_state(prepared[3]), rows.stride(0), rows.device)
    assert table.shape[0] > 64
    _, dequant = pl.finish_prepared_unshard_with_dequant(prepared[3], rows)
    for (_, p), call, deq in zip(named, factory.calls, dequant, strict=True):
        oq, osc = cport.quantize_blockwise(p.detach().cpu(), block)
        assert torch.equal(call[0].view(torch.uint8).cpu(), oq) and torch.equal(_bits(call[1].cpu()), _bits(osc))
        want = cport.dequant_blockwise(oq, osc, block)
        assert torch.equal(deq.cpu().view(torch.int16), want.view(torch.int16))


def test_fp16_bucket_round_trip_and_fp16_dequantization(device):
    """fp16 parameters through pack, gather and unpack on 4 ranks: the factory
    gets the oracle's bytes and scales with orig_dtype fp16, and the fused
    dequantization writes fp16 equal to torch's one rounding of the fp32
    product, from aligned rows and from strided rows at an odd offset."""
    shapes, block, world = [(512, 256), (130, 136), (3, 64, 128)], 128, 4
    factory = RecordingFactory()
    pl = Fp8BucketedBlockShard(world_size=world, weight_factory=factory, block_size=block)
    gen = torch.Generator().manual_seed(8)
    named = [(f"w{i}", nn.Parameter((torch.randn(s, generator=gen) * 0.02).half().to(device), requires_grad=False))
             for i, s in enumerate(shapes)]
    prepared = prepare_unshard_on_each_rank(pl, named, world)
    rows = gather_rank_rows(prepared)
    parent = torch.zeros((world, rows.shape[1] + 5), dtype=torch.uint8, device=device)
    parent[:, 3 : 3 + rows.shape[1]] = rows
    for rank_rows in (rows, parent[:, 3 : 3 + rows.shape[1]]):
        factory.calls.clear()
        _, dequant = pl.finish_prepared_unshard_with_dequant(prepared[1], rank_rows, dequant_dtype=torch.float16)
        for (_, p), call, deq in zip(named, factory.calls, dequant, strict=True):
            flat = p.detach().cpu().flatten(0, -2)
            oq, osc = eager_oracle.quantize_blockwise(flat, block)
            assert call[3] == torch.float16
            assert torch.equal(call[0].flatten(0, -2).view(torch.uint8).cpu(), oq.view(torch.uint8))
            assert torch.equal(_bits(call[1].cpu()), _bits(osc))
            want = eager_oracle.dequant_blockwise(oq, osc, block, torch.float16)
            assert deq.dtype == torch.float16 and deq.shape == p.shape
            assert torch.equal(deq.flatten(0, -2).cpu().view(torch.int16), want.view(torch.int16))
    fp8 = factory.calls[0][0]
    got = blockwise_dequant_weight(fp8.flatten(0, -2), factory.calls[0][1], block, torch.float16)
    assert torch.equal(got.view(torch.int16), dequant[0].flatten(0, -2).view(torch.int16))


def test_fused_unpack_with_dequant_matches_oracle(device):
    """finish_prepared_unshard_with_dequant: FP8 views as in the plain finish,
    plus bf16 weights equal to dequantizing the gathered weight (0 ULP), from
    strided rows at an odd offset as well."""
    for shapes, block, world in (([(16, 8), (8, 8), (1, 3)], 4, 8), ([(512, 256), (256, 384), (130, 136)], 128, 4),
                                 ([(1024, 512), (3, 256, 256)], 128, 8)):
        factory = RecordingFactory()
        pl = Fp8BucketedBlockShard(world_size=world, weight_factory=factory, block_size=block)
        gen = torch.Generator().manual_seed(4)
        named = [
            (f"w{i}", nn.Parameter((torch.randn(s, generator=gen) * 0.02).bfloat16().to(device), requires_grad=False))
            for i, s in enumerate(shapes)
        ]
        prepared = prepare_unshard_on_each_rank(pl, named, world)
        rows = gather_rank_rows(prepared)
        parent = torch.zeros((world, rows.shape[1] + 5), dtype=torch.uint8, device=device)
        parent[:, 3 : 3 + rows.shape[1]] = rows
        for rank_rows in (rows, parent[:, 3 : 3 + rows.shape[1]]):
            factory.calls.clear()
            result, dequant = pl.finish_prepared_unshard_with_dequant(prepared[0], rank_rows)
            plain = pl._finish_unshard_from_rank_rows(prepared[0], rank_rows)
            for (_, p), call, deq, plain_fp8 in zip(named, factory.calls, dequant, plain.full_params):
                oq, osc = cport.quantize_blockwise(p.detach().cpu().flatten(0, -2), block)
                assert torch.equal(call[0].flatten(0, -2).view(torch.uint8).cpu(), oq)
                assert torch.equal(_bits(call[1].cpu()), _bits(osc))
                assert torch.equal(plain_fp8.view(torch.uint8), call[0].view(torch.uint8))
                want = cport.dequant_blockwise(oq, osc, block)
                assert deq.shape == p.shape and deq.dtype == torch.bfloat16
                assert torch.equal(deq.flatten(0, -2).cpu().view(torch.int16), want.view(torch.int16))
        _, only_dequant = pl.finish_prepared_unshard_with_dequant(prepared[0], rows, compact=False)
        assert all(torch.equal(a, b) for a, b in zip(only_dequant, dequant))


def test_llama_gathered_layout_unpack_full_size(device, golden):
    """Config 2 unpack: the 8-rank gathered layout [8, 27 531 840] built from 8
    locally quantized seeded shards; the compact buffer must equal whole-matrix
    quantization, the fused dequant must equal dequantizing it, and
    encode -> gather -> decode must stay within the FP8 error bound."""
    g = golden["llama3_8b_layer_plan"]
    factory = RecordingFactory()
    pl = Fp8BucketedBlockShard(world_size=8, weight_factory=factory)
    named = seeded_bucket(LLAMA3_8B_LAYER, 0.02, 100, device)
    prepared = prepare_unshard_on_each_rank(pl, named, 8)
    rows = gather_rank_rows(prepared)
    assert tuple(rows.shape) == (8, g["row_nbytes"])
    result, dequant = pl.finish_prepared_unshard_with_dequant(prepared[0], rows)
    plain = pl._finish_unshard_from_rank_rows(prepared[0], rows)
    from flex_shard_amd.custom_placements.fp8_bucketed_block_shard import _quantize_dense_weight_to_blockwise_fp8

    for index, ((fqn, p), fp8, deq) in enumerate(zip(named, result.full_params, dequant)):
        wq, ws = _quantize_dense_weight_to_blockwise_fp8(p.detach(), 128, E4M3)
        recip = factory.calls[index][1]
        assert torch.equal(fp8.view(torch.uint8), wq.view(torch.uint8)), fqn
        assert torch.equal(recip.view(torch.int32), ws.view(torch.int32)), fqn
        assert torch.equal(plain.full_params[index].view(torch.uint8), fp8.view(torch.uint8)), fqn
        ref = blockwise_dequant_weight(wq, ws, 128, torch.bfloat16)
        assert torch.equal(deq.view(torch.int16), ref.view(torch.int16)), fqn
        # round trip: |deq - w| <= amax_tile / 16 (+ bf16 rounding of the result)
        tiles_r, tiles_c = p.shape[0] // 128, p.shape[1] // 128
        amax = p.detach().float().view(tiles_r, 128, tiles_c, 128).abs().amax(dim=(1, 3))
        bound = (amax / 16 * 1.01).repeat_interleave(128, 0).repeat_interleave(128, 1)
        assert ((deq.float() - p.detach().float()).abs() <= bound).all(), fqn
    # anchor the widest parameter (`down`, in_dim 14336) against the CPU oracle on sampled 128-row bands
    down = named[6][1].detach()
    gen = torch.Generator().manual_seed(3)
    for band in sorted({0, 31, *torch.randint(0, 32, (4,), generator=gen).tolist()}):
        rows_cpu = down[band * 128 : (band + 1) * 128].cpu()
        oq, osc = cport.quantize_blockwise(rows_cpu, 128)
        got = result.full_params[6].view(torch.uint8)[band * 128 : (band + 1) * 128].cpu()
        assert torch.equal(got, oq), f"down band {band}"
        assert torch.equal(factory.calls[6][1][band].cpu().view(torch.int32), osc.view(-1).view(torch.int32))
        want = cport.dequant_blockwise(oq, osc, 128)
        assert torch.equal(dequant[6][band * 128 : (band + 1) * 128].cpu().view(torch.int16), want.view(torch.int16))
    # anchor one gathered parameter against the CPU oracle
    k = named[1][1].detach().cpu()
    oq, osc = cport.quantize_blockwise(k, 128)
    assert torch.equal(result.full_params[1].view(torch.uint8).cpu(), oq)
    assert torch.equal(dequant[1].cpu().view(torch.int16), cport.dequant_blockwise(oq, osc, 128).view(torch.int16))


@pytest.mark.parametrize("world", [1, 8])
def test_offsets_beyond_two_gib(device, world):
    """A bucket of nine [16384, 16384] matrices (2.4 G elements): byte offsets
    in one rank's payload (world 1), in the gathered rows and in the compact
    buffer pass 2^31, those of the bf16 dequantization pass 2^32.  Bands of 128
    rows from the first, a middle and the last parameter against the C oracle,
    through pack, gather, unpack and dequantization."""
    n, dim = 9, 16384
    spec = tuple((f"w{i}", (dim, dim)) for i in range(n))
    factory = RecordingFactory()
    pl = Fp8BucketedBlockShard(world_size=world, weight_factory=factory)
    named = seeded_bucket(spec, 0.02, 4200, device)
    prepared = prepare_unshard_on_each_rank(pl, named, world)
    rows = gather_rank_rows(prepared)
    assert rows.numel() > 2**31
    del prepared[1:]
    result, dequant = pl.finish_prepared_unshard_with_dequant(prepared[0], rows)
    assert result.full_params[-1].data_ptr() - result.full_params[0].data_ptr() >= 2**31
    assert dequant[-1].data_ptr() - dequant[0].data_ptr() >= 2**32
    for index in (0, 4, n - 1):
        weight = named[index][1].detach()
        for band in (0, 77, dim // 128 - 1):
            lo, hi = band * 128, (band + 1) * 128
            oq, osc = cport.quantize_blockwise(weight[lo:hi].cpu(), 128)
            assert torch.equal(result.full_params[index].view(torch.uint8)[lo:hi].cpu(), oq), (index, band)
            assert torch.equal(factory.calls[index][1][band].cpu().view(torch.int32), osc.view(-1).view(torch.int32))
            want = cport.dequant_blockwise(oq, osc, 128)
            assert torch.equal(dequant[index][lo:hi].cpu().view(torch.int16), want.view(torch.int16)), (index, band)
    # every parameter, on the GPU: the gathered bytes are those of quantizing the whole matrix
    from flex_shard_amd.custom_placements.fp8_bucketed_block_shard import _quantize_dense_weight_to_blockwise_fp8

    for index, (fqn, p) in enumerate(named):
        wq, ws = _quantize_dense_weight_to_blockwise_fp8(p.detach(), 128, E4M3)
        assert torch.equal(result.full_params[index].view(torch.uint8), wq.view(torch.uint8)), fqn
        assert torch.equal(factory.calls[index][1].view(torch.int32), ws.view(torch.int32)), fqn
        del wq, ws


def test_segment_kernels_with_offsets_beyond_two_to_the_32_bytes(device):
    """Copy, zero and casting pack of segments whose source and destination
    offsets lie beyond 2^32 bytes of their buffers (int64 tables end to end)."""
    from flex_shard_amd.custom_placements._copy_kernels import pack_segments_into_flat_buffer

    n = 2**32 + (1 << 22)
    src = torch.empty(n, dtype=torch.uint8, device=device)
    src[-(1 << 22) :].random_(0, 256)
    src[:4096].random_(0, 256)
    dst = torch.full((n,), 9, dtype=torch.uint8, device=device)
    far = 2**32 + 12345
    desc = SegmentCopyDescriptor.create(
        src_offsets=[far, 17], numels=[1_000_001, 3000], dst_offsets=[far + 4097, 2**32 + 5], device=device
    )
    copy_segments(src, dst, desc)
    assert torch.equal(dst[far + 4097 : far + 4097 + 1_000_001], src[far : far + 1_000_001])
    assert torch.equal(dst[2**32 + 5 : 2**32 + 3005], src[17:3017])
    assert (dst[2**32 + 3005 : far + 4097] == 9).all() and (dst[far + 4097 + 1_000_001 :] == 9).all()
    zero_segments(dst, desc)
    assert (dst[far + 4097 : far + 4097 + 1_000_001] == 0).all() and (dst[2**32 + 5 : 2**32 + 3005] == 0).all()
    assert dst[2**32 + 4].item() == 9 and dst[2**32 + 3005].item() == 9
    del src, dst
    # bf16 -> fp32 pack: source element 2^31 + ..., destination element 2^31 + ... (8.6 GB into the output)
    m = 2**31 + (1 << 21)
    grads = torch.empty(m, dtype=torch.bfloat16, device=device)
    grads[-(1 << 21) :].normal_()
    out = torch.ones(m, dtype=torch.float32, device=device)
    start, zeros_at = 2**31 + 1000, 2**31 + 700_000
    keep = pack_segments_into_flat_buffer([grads], [0, -1], [start, 0], [600_000, 5000], [start + 8, zeros_at], out)
    assert keep is not None
    assert torch.equal(out[start + 8 : start + 8 + 600_000], grads[start : start + 600_000].float())
    assert (out[zeros_at : zeros_at + 5000] == 0).all()
    assert (out[start + 8 + 600_000 : zeros_at] == 1).all() and (out[2**31 - 4096 : start + 8] == 1).all()

