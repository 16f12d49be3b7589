"""GPU parity of the gradient path (copy-in, fp32 accumulation, fixed-order
reduce + copy-out) and of the Muon / Newton-Schulz kernels."""

import numpy as np
import pytest
import torch
import torch.nn as nn

from flex_shard_amd import _native  # noqa: E402
from flex_shard_amd import (
    BucketedBlockShard,
    Fp8BucketedBlockShard,
    GradientReduction,
    LocalReduceGroup,
    hip_ops,
)
from flex_shard_amd.custom_placements.utils import gradient_reduce_plan, reduce_grads_on_one_rank
from flex_shard_amd.dist_muon import (
    OwnedMuon,
    _apply_muon_update,
    _compute_muon_direction,
    _estimate_muon_compute_cost,
    _prepare_muon_input,
    _zeropower_via_newtonschulz,
)
from flex_shard_amd.testing import LLAMA3_8B_LAYER, FakeMesh, make_param_infos, seeded_normal
from oracle import cport, eager
from oracle import layout as olayout

pytestmark = pytest.mark.gpu
import torch.distributed as dist  # noqa: E402

COEFFS = (3.4445, -4.7750, 2.0315)


def _factory(fp8_data, recip_scale, block_size, *, orig_dtype, requires_grad):
    return fp8_data


def _bucket(shapes, world, dtype, device_type="meta"):
    pl = Fp8BucketedBlockShard(world_size=world, weight_factory=_factory, block_size=4)
    named = [(f"w{i}", nn.Parameter(torch.empty(tuple(s), device=device_type, dtype=dtype))) for i, s in enumerate(shapes)]
    return pl, make_param_infos(named, pl, FakeMesh(world))


def _expected_rows(pl, grads, infos, dtype):
    layout = infos[0].bucket_layout
    return olayout.reduce_scatter_input(
        [g.cpu() for g in grads],
        [layout.param_layouts[i.fqn].param_offset for i in infos],
        layout.global_numel, layout.rank_offsets, layout.rank_numels, dtype,
    )


def _grads(infos, dtype, device):
    torch.manual_seed(0)
    return [torch.randn(i.global_shape, dtype=dtype, device=device) for i in infos]


# ------------------------------------------------------------------ copy-in
def test_one_pass_copy_in_matches_reference_rows(device, golden):
    cases = golden["reduce_copy_in_cases"]["fp8_layout_cases"]
    for name, case in cases.items():
        for dtype in (torch.bfloat16, torch.float32):
            pl, infos = _bucket(case["shapes"], case["world_size"], dtype)
            grads = _grads(infos, dtype, device)
            prepared = pl.prepare_reduce_grad(grads, infos, FakeMesh(case["world_size"]), None)
            want = _expected_rows(pl, grads, infos, dtype)
            assert torch.equal(prepared.buffers[0].view(want.shape).cpu(), want), f"{name} {dtype}"
            assert len(pl._reduce_copy_in_plans) == 1


def test_copy_in_with_gaps_and_empty_rank(device, golden):
    dense = golden["reduce_copy_in_cases"]["dense_case"]
    pl = BucketedBlockShard(dims=(0,), blocks_per_rank=tuple(dense["blocks_per_rank"]))
    named = [(f"w{i}", nn.Parameter(torch.empty(tuple(s), device="meta", dtype=torch.bfloat16))) for i, s in enumerate(dense["shapes"])]
    infos = make_param_infos(named, pl, FakeMesh(4))
    grads = _grads(infos, torch.bfloat16, device)
    prepared = pl.prepare_reduce_grad(grads, infos, FakeMesh(4), None)
    want = _expected_rows(pl, grads, infos, torch.bfloat16)
    assert torch.equal(prepared.buffers[0].view(want.shape).cpu(), want)
    (plan,) = pl._reduce_copy_in_plans.values()
    assert len(plan.zero_segments) > 4


def test_copy_in_into_wider_rows(device, golden):
    pl, infos = _bucket([(16, 8), (8, 8), (12, 4)], 8, torch.bfloat16)
    grads = _grads(infos, torch.bfloat16, device)
    want = _expected_rows(pl, grads, infos, torch.bfloat16).to(device)
    width = want.size(1)
    for start, extra in golden["reduce_copy_in_cases"]["wider_rows"]:
        rows = torch.full((8, start + width + extra), 7.0, dtype=torch.bfloat16, device=device)
        send = rows[:, start : start + width]
        pl._pack_reduce_scatter_grad(grads, infos, 8, send)
        assert torch.equal(send, want)
        assert (rows[:, :start] == 7.0).all() and (rows[:, start + width :] == 7.0).all()
    assert len(pl._reduce_copy_in_plans) == 3  # one plan per row stride


def test_copy_in_casts_to_the_reduce_dtype_in_the_same_launch(device):
    """bf16 grads with an fp32 reduce dtype: the cast is fused into the copy
    (the reference routes this through a zeroed bucket and a foreach copy)."""
    pl, infos = _bucket([(16, 8), (8, 8), (12, 4)], 8, torch.bfloat16)
    for info in infos:
        info.reduce_dtype = torch.float32
    grads = _grads(infos, torch.bfloat16, device)
    assert pl._packs_reduce_scatter_grad_in_one_pass(grads, torch.float32)
    prepared = pl.prepare_reduce_grad(grads, infos, FakeMesh(8), None)
    want = _expected_rows(pl, grads, infos, torch.float32)
    assert prepared.buffers[0].dtype == torch.float32
    assert torch.equal(prepared.buffers[0].view(want.shape).cpu(), want)
    # fp32 grads into a bf16 reduce dtype round to nearest even like torch
    pl2, infos2 = _bucket([(16, 8), (5, 3)], 4, torch.bfloat16)
    grads32 = _grads(infos2, torch.float32, device)
    prepared = pl2.prepare_reduce_grad(grads32, infos2, FakeMesh(4), None)
    want = _expected_rows(pl2, grads32, infos2, torch.bfloat16)
    assert torch.equal(prepared.buffers[0].view(want.shape).cpu(), want)


@pytest.mark.parametrize("src_dtype,dst_dtype", [(torch.bfloat16, torch.float32), (torch.float32, torch.bfloat16)])
def test_casting_pack_for_any_length_and_alignment(device, src_dtype, dst_dtype):
    """Casting segments move eight elements per thread where both sides are
    16-byte aligned and element by element elsewhere: lengths around the
    group and slice sizes, at source and destination offsets of every
    alignment, plus a zero-fill segment, against torch's cast."""
    gen = torch.Generator().manual_seed(11)
    lengths = [1, 7, 8, 9, 63, 4096, 4101, 8192 + 13, 20000]
    src_offs = [0, 1, 3, 8, 5, 0, 2, 8, 16]
    inputs = [torch.randn(n + o + 3, generator=gen).to(src_dtype).to(device) for n, o in zip(lengths, src_offs)]
    dst_offs, cursor = [], 0
    for k, n in enumerate(lengths):
        cursor += (0, 1, 4, 0, 5, 0, 3, 8, 0)[k]  # gaps that put the destinations at odd alignments
        dst_offs.append(cursor)
        cursor += n
    zero_at, zero_len = cursor + 2, 37
    total = zero_at + zero_len + 5
    out = torch.full((total,), 7.0, dtype=dst_dtype, device=device)
    table = lambda values: torch.tensor(values, dtype=torch.int64, device=device)
    hip_ops.pack_segments(
        table([t.data_ptr() for t in inputs]), table(list(range(len(lengths))) + [-1]), table(src_offs + [0]),
        table(lengths + [zero_len]), table(dst_offs + [zero_at]), max(lengths), src_dtype, out,
    )
    want = torch.full((total,), 7.0, dtype=dst_dtype)
    for t, n, so, do in zip(inputs, lengths, src_offs, dst_offs):
        want[do : do + n] = t[so : so + n].cpu().to(dst_dtype)
    want[zero_at : zero_at + zero_len] = 0
    assert torch.equal(out.cpu(), want)



@pytest.mark.parametrize(
    "src_dtype,dst_dtype",
    [(torch.bfloat16, torch.float32), (torch.float32, torch.bfloat16), (torch.float32, torch.float32),
     (torch.bfloat16, torch.bfloat16)],
)
@pytest.mark.parametrize("nsegments,longest", [(200, 150_000), (5000, 12_000)])
def test_pack_shares_slices_of_uneven_segments(device, src_dtype, dst_dtype, nsegments, longest):
    """A large gather: segments of very different lengths from several inputs,
    zero-fill segments among them, several thousand segments in one launch,
    aligned and unaligned offsets."""
    rng = np.random.default_rng(nsegments + 1)
    ninputs = 5
    numels = rng.integers(0, longest, nsegments)
    numels[nsegments // 3] = longest
    aligned = rng.random(nsegments) < 0.7  # most segments on 8-element boundaries on both sides
    numels = np.where(aligned, numels // 8 * 8, numels).tolist()
    tensor_index = rng.integers(-1, ninputs, nsegments).tolist()
    src_cursor = [0] * ninputs
    src_offs, dst_offs, d_cur = [], [], 0
    for k, (n, t) in enumerate(zip(numels, tensor_index)):
        if not aligned[k]:
            d_cur += int(rng.integers(1, 8))
        if t >= 0:
            if not aligned[k]:
                src_cursor[t] += int(rng.integers(1, 8))
            src_offs.append(src_cursor[t])
            src_cursor[t] += n
            src_cursor[t] = -(-src_cursor[t] // 8) * 8
        else:
            src_offs.append(0)
        dst_offs.append(d_cur)
        d_cur = -(-(d_cur + n) // 8) * 8
    gen = torch.Generator().manual_seed(5)
    inputs_host = [torch.randn(max(c, 8), generator=gen).to(src_dtype) for c in src_cursor]
    inputs = [t.to(device) for t in inputs_host]
    out = torch.full((d_cur + 8,), 7.0, dtype=dst_dtype, device=device)
    table = lambda values: torch.tensor(values, dtype=torch.int64, device=device)
    hip_ops.pack_segments(
        table([t.data_ptr() for t in inputs]), table(tensor_index), table(src_offs), table(numels), table(dst_offs),
        longest, src_dtype, out,
    )
    want = torch.full((d_cur + 8,), 7.0, dtype=dst_dtype)
    for t, s, n, d in zip(tensor_index, src_offs, numels, dst_offs):
        want[d : d + n] = 0 if t < 0 else inputs_host[t][s : s + n].to(dst_dtype)
    view = torch.int32 if dst_dtype == torch.float32 else torch.int16
    assert torch.equal(out.cpu().view(view), want.view(view))


def test_copy_in_through_a_bucket_while_compiling(device):
    from unittest.mock import patch

    pl, infos = _bucket([(16, 8), (8, 8), (12, 4)], 8, torch.bfloat16)
    grads = _grads(infos, torch.bfloat16, device)
    with patch.object(torch.compiler, "is_compiling", return_value=True):
        assert not pl._packs_reduce_scatter_grad_in_one_pass(grads, torch.bfloat16)
        prepared = pl.prepare_reduce_grad(grads, infos, FakeMesh(8), None)
    want = _expected_rows(pl, grads, infos, torch.bfloat16)
    assert torch.equal(prepared.buffers[0].view(want.shape).cpu(), want)
    assert pl._reduce_copy_in_plans == {}


def test_zero_copy_when_grads_view_one_bucket(device):
    pl = BucketedBlockShard(dims=(0,), blocks_per_rank=(1, 1))
    named = [("a", nn.Parameter(torch.empty(4, 4, device="meta"))), ("b", nn.Parameter(torch.empty(4, 4, device="meta")))]
    infos = make_param_infos(named, pl, FakeMesh(2))
    bucket = torch.randn(infos[0].bucket_layout.global_numel, device=device)
    grads = [bucket[0:16].view(4, 4), bucket[16:32].view(4, 4)]
    prepared = pl.prepare_reduce_grad(grads, infos, FakeMesh(2), None)
    assert prepared.buffers[0] is bucket


# -------------------------------------------------- accumulate, reduce, copy-out
def test_fp32_accumulation_known_answer(device, golden):
    g = golden["fp32_accumulation"]
    acc = torch.empty(1000, device=device)
    hip_ops.accumulate_grad(acc, torch.full((1000,), g["first"], device=device).bfloat16(), overwrite=True)
    hip_ops.accumulate_grad(acc, torch.full((1000,), g["second"], device=device).bfloat16())
    assert (acc == g["fp32_sum"]).all()


@pytest.mark.parametrize("n,offset", [(1 << 20, 0), (1000003, 0), (4099, 1), (7, 3)])
def test_accumulate_is_exact_for_any_length_and_alignment(device, n, offset):
    gen = torch.Generator().manual_seed(n)
    grads = [(torch.randn(n + offset, generator=gen) * 1e-3).bfloat16() for _ in range(4)]
    base = torch.zeros(n + offset + 8, device=device)
    acc = base[offset : offset + n]
    for k, g in enumerate(grads):
        hip_ops.accumulate_grad(acc, g.to(device)[offset:], overwrite=(k == 0))
    want = eager.accumulate_microbatches([g[offset:] for g in grads])
    assert torch.equal(acc.cpu(), want)
    check = torch.zeros(n)
    for g in grads:
        cport.accumulate_bf16(check, g[offset:].contiguous())
    assert torch.equal(want, check)
    assert (base[:offset] == 0).all() and (base[offset + n :] == 0).all()
    # fp32 microbatch gradients accumulate too
    g32 = torch.randn(n, generator=gen).to(device)
    before = acc.clone()
    hip_ops.accumulate_grad(acc, g32)
    assert torch.equal(acc, before + g32)


def test_fixed_order_reduce_and_modes(device):
    gen = torch.Generator().manual_seed(5)
    world, seg = 8, 12345
    contrib = torch.randn(world, world * seg, generator=gen).to(device)
    out = torch.empty(seg, device=device)
    for rank in (0, 3, 7):
        rows = [contrib[r, rank * seg : (rank + 1) * seg].cpu().contiguous() for r in range(world)]
        hip_ops.reduce_rows(out, contrib, rank * seg)
        assert torch.equal(out.cpu(), cport.reduce_rows(rows))
        hip_ops.reduce_rows(out, contrib, rank * seg, mode=hip_ops.REDUCE_PREMUL, factor=1 / 3)
        assert torch.equal(out.cpu(), cport.reduce_rows(rows, cport.REDUCE_PREMUL, 1 / 3))
        hip_ops.reduce_rows(out, contrib, rank * seg, mode=hip_ops.REDUCE_POSTDIV, factor=3.0)
        assert torch.equal(out.cpu(), cport.reduce_rows(rows, cport.REDUCE_POSTDIV, 3.0))
        hip_ops.reduce_rows(out, contrib, rank * seg, mode=hip_ops.REDUCE_POSTMUL, factor=0.125)
        assert torch.equal(out.cpu(), cport.reduce_rows(rows, cport.REDUCE_POSTMUL, 0.125))
    # unaligned column offset and odd length take the scalar path
    odd = torch.empty(1001, device=device)
    hip_ops.reduce_rows(odd, contrib, 17)
    assert torch.equal(odd.cpu(), cport.reduce_rows([contrib[r, 17:1018].cpu().contiguous() for r in range(world)]))
    with pytest.raises(ValueError, match="outside rows"):
        hip_ops.reduce_rows(out, contrib, world * seg - 10)


def test_fixed_order_reduce_of_bf16_contributions(device):
    """bf16 contributions: widened to fp32, added in rank order in fp32, rounded
    to bf16 once (checked against that fold written out in torch on the CPU;
    no rounding per hop as a ring in bf16 would have)."""
    gen = torch.Generator().manual_seed(6)
    world, seg = 8, 12344
    contrib = torch.randn(world, world * seg, generator=gen).bfloat16().to(device)
    out = torch.empty(seg, device=device, dtype=torch.bfloat16)

    def fold(rows, pre=None, post=None):
        total = None
        for row in rows:
            term = row.float() if pre is None else row.float() * torch.tensor(pre, dtype=torch.float32)
            total = term if total is None else total + term
        if post is not None:
            total = post(total)
        return total.bfloat16()

    third = float(np.float32(1 / 3))
    for rank in (0, 5):
        rows = [contrib[r, rank * seg : (rank + 1) * seg].cpu() for r in range(world)]
        hip_ops.reduce_rows(out, contrib, rank * seg)
        assert torch.equal(out.cpu(), fold(rows))
        hip_ops.reduce_rows(out, contrib, rank * seg, mode=hip_ops.REDUCE_PREMUL, factor=1 / 3)
        assert torch.equal(out.cpu(), fold(rows, pre=third))
        hip_ops.reduce_rows(out, contrib, rank * seg, mode=hip_ops.REDUCE_POSTMUL, factor=0.125)
        assert torch.equal(out.cpu(), fold(rows, post=lambda t: t * 0.125))
        hip_ops.reduce_rows(out, contrib, rank * seg, mode=hip_ops.REDUCE_POSTDIV, factor=3.0)
        assert torch.equal(out.cpu(), fold(rows, post=lambda t: t / 3.0))
    # groups of eight and a tail of four in one launch
    hip_ops.reduce_rows(out[:12340], contrib, 2 * seg)
    assert torch.equal(out[:12340].cpu(), fold([contrib[r, 2 * seg : 2 * seg + 12340].cpu() for r in range(world)]))
    # unaligned column offset and odd length take the scalar path
    odd = torch.empty(1001, device=device, dtype=torch.bfloat16)
    hip_ops.reduce_rows(odd, contrib, 17)
    assert torch.equal(odd.cpu(), fold([contrib[r, 17:1018].cpu() for r in range(world)]))
    with pytest.raises(NotImplementedError, match="same dtype"):
        hip_ops.reduce_rows(torch.empty(seg, device=device), contrib, 0)
    # through the one-GPU group: averaged bf16 gradients of three ranks
    group = LocalReduceGroup(3, 1)
    sends = [torch.randn(3 * 1000, generator=gen).bfloat16().to(device) for _ in range(3)]
    for r in (0, 2):
        group.deposit(r, sends[r])
    from flex_shard_amd.custom_placements.utils import reduce_scatter_grads

    recv = torch.empty(1000, device=device, dtype=torch.bfloat16)
    reduce_scatter_grads(recv, sends[1], GradientReduction(), group)
    assert torch.equal(recv.cpu(), fold([s[1000:2000].cpu() for s in sends], pre=float(np.float32(1.0) / np.float32(3.0))))


def test_gradient_kernels_index_beyond_two_to_the_31(device):
    """More than 2^31 elements: the accumulation of a bf16 gradient into an
    fp32 bucket and the fixed-order reduction of a rank range whose elements
    lie beyond 2^32 bytes of the contributions, checked on slices at both ends
    against the same arithmetic in torch."""
    n = 2**31 + 4096 + 3
    acc = torch.zeros(n, device=device)
    grad = torch.empty(n, device=device, dtype=torch.bfloat16)
    grad[: 1 << 20].normal_()
    grad[1 << 20 :] = grad[: 1 << 20].repeat((n >> 20) + 1)[: n - (1 << 20)]
    hip_ops.accumulate_grad(acc, grad, overwrite=True)
    hip_ops.accumulate_grad(acc, grad)
    for sl in (slice(0, 5000), slice(2**31 - 2500, 2**31 + 2500), slice(n - 5000, n)):
        assert torch.equal(acc[sl], grad[sl].float() + grad[sl].float())
    del acc, grad
    world, seg = 2, 2**30 + 8
    contrib = torch.empty((world, world * seg), device=device)
    contrib[:, : 1 << 20].normal_()
    contrib[:, 1 << 20 :] = contrib[:, : 1 << 20].repeat(1, (world * seg >> 20) + 1)[:, : world * seg - (1 << 20)]
    contrib[1] *= 3.0
    out = torch.empty(seg, device=device)
    hip_ops.reduce_rows(out, contrib, seg)  # rank 1's range: columns seg .. 2 seg, row 1 starts 2^33 bytes in
    for sl in (slice(0, 5000), slice(seg - 5000, seg)):
        want = contrib[0, seg:][sl] + contrib[1, seg:][sl]
        assert torch.equal(out[sl], want)


def test_reduce_plan_table():
    avg, sm = GradientReduction(), GradientReduction(op=dist.ReduceOp.SUM)
    assert gradient_reduce_plan(sm, 8, torch.float32) == ("sum", None, None)
    assert gradient_reduce_plan(avg, 8, torch.float32) == ("avg", None, None)
    assert gradient_reduce_plan(avg, 1, torch.float32) == ("sum", None, None)
    assert gradient_reduce_plan(GradientReduction(divide_factor=4.0), 1, torch.float32) == ("sum", None, 4.0)
    assert gradient_reduce_plan(GradientReduction(divide_factor=16.0), 8, torch.bfloat16) == ("premul_sum", 16.0, None)
    assert gradient_reduce_plan(GradientReduction(divide_factor=16.0), 8, torch.float16) == ("sum", 4, 4.0)
    with pytest.raises(ValueError, match="requires gradient_reduce_op=AVG"):
        GradientReduction(op=dist.ReduceOp.SUM, divide_factor=2.0)
    with pytest.raises(ValueError, match="positive"):
        GradientReduction(divide_factor=0.0)


def test_reduce_prepared_grad_end_to_end_small(device):
    """8 simulated ranks' copy-in rows, the fixed-order reduction on rank r and
    the copy-out views, for SUM / AVG / a custom divide factor."""
    world = 8
    shapes = [(16, 8), (8, 8), (12, 4)]
    for rank in (0, 5):
        for reduction, post in ((GradientReduction(op=dist.ReduceOp.SUM), 1.0), (GradientReduction(), 8.0),
                                (GradientReduction(divide_factor=16.0), 16.0)):
            group = LocalReduceGroup(world, rank)
            pl = Fp8BucketedBlockShard(world_size=world, weight_factory=_factory, block_size=4)
            named = [(f"w{i}", nn.Parameter(torch.empty(s, device="meta"))) for i, s in enumerate(shapes)]
            infos = make_param_infos(named, pl, FakeMesh(world, rank, group))
            per_rank_grads, prepared_mine = [], None
            for r in range(world):
                torch.manual_seed(100 + r)
                grads = [torch.randn(s, device=device) for s in shapes]
                per_rank_grads.append(grads)
                prepared = pl.prepare_reduce_grad(grads, infos, FakeMesh(world, rank, group), None)
                group.deposit(r, prepared.buffers[0])
                if r == rank:
                    prepared_mine = prepared
            result = pl.reduce_prepared_grad(prepared_mine, reduction)
            layout = infos[0].bucket_layout
            for i, (info, shard) in enumerate(zip(infos, result.sharded_grads)):
                total = None
                for r in range(world):
                    term = per_rank_grads[r][i].cpu() * (1.0 / post) if post != 1.0 else per_rank_grads[r][i].cpu()
                    total = term.clone() if total is None else total + term
                lo = layout.param_layouts[info.fqn].local_global_offset - layout.param_layouts[info.fqn].param_offset
                want = total.reshape(-1)[lo : lo + info.local_numel].view(info.local_shape)
                assert torch.equal(shard.cpu(), want), (rank, i)
                if shard.numel():
                    assert shard.untyped_storage().data_ptr() == result.buffers[0].untyped_storage().data_ptr()
    one = torch.full((4,), 8.0, device=device)
    reduce_grads_on_one_rank(one, GradientReduction(divide_factor=4.0))
    assert (one == 2.0).all()
    with pytest.raises(ValueError, match="missing the contributions"):
        group = LocalReduceGroup(2, 0)
        group.allocate(8, torch.float32, device)
        from flex_shard_amd.custom_placements.utils import reduce_scatter_grads

        reduce_scatter_grads(torch.empty(4, device=device), torch.zeros(8, device=device), GradientReduction(), group)


def test_llama_gradient_bucket_full_size(device, golden):
    """Config 4 at full size, in the real placement layout (218 365 952
    elements including zero gaps, rank range 27 295 744): 4 bf16 microbatches
    accumulate into fp32, then 8 rank contributions are summed in rank order
    into rank 0's range.  Checked against the same left fold in torch fp32 on
    the GPU (bit-exact, and within rtol 1e-6 by construction) and against the C
    oracle on a slice."""
    g = golden["llama3_8b_dense_bucket"]
    world = 8
    pl = BucketedBlockShard(dims=(0,), blocks_per_rank=(1,) * world)
    named = [(n, nn.Parameter(torch.empty(s, device="meta", dtype=torch.bfloat16))) for n, s in LLAMA3_8B_LAYER]
    group = LocalReduceGroup(world, 0)
    infos = make_param_infos(named, pl, FakeMesh(world, 0, group))
    for info in infos:
        info.reduce_dtype = torch.float32
    layout = infos[0].bucket_layout
    total, seg = layout.global_numel, layout.rank_numels[0]
    assert total == g["global_numel"] and seg == g["rank_numel"]

    # fp32 accumulation of 4 microbatches into a gradient bucket in this layout
    acc = torch.zeros(total, device=device)
    micro = [seeded_normal((total,), 1e-3, 500 + k, device) for k in range(4)]
    for k, m in enumerate(micro):
        hip_ops.accumulate_grad(acc, m, overwrite=(k == 0))
    ref = micro[0].float()
    for m in micro[1:]:
        ref = ref + m.float()
    assert torch.equal(acc, ref)
    sl = slice(12345678, 12345678 + 100000)
    check = torch.zeros(100000)
    for m in micro:
        cport.accumulate_bf16(check, m[sl].cpu().contiguous())
    assert torch.equal(acc[sl].cpu(), check)
    del micro, ref

    # grads as views of the accumulated bucket: the copy-in is free
    grads = [acc[layout.param_layouts[i.fqn].param_offset :][: i.global_numel].view(i.global_shape) for i in infos]
    prepared = pl.prepare_reduce_grad(grads, infos, FakeMesh(world, 0, group), None)
    assert prepared.buffers[0] is acc

    # 8 rank contributions (this rank's accumulated bucket plus 7 seeded ones)
    contributions = group.allocate(total, torch.float32, device)
    contributions[0].copy_(acc)
    for r in range(1, world):
        contributions[r].copy_(seeded_normal((total,), 1e-3, 900 + r, device, torch.float32))
    group.mark_deposited(*range(world))
    result = pl.reduce_prepared_grad(prepared, GradientReduction(op=dist.ReduceOp.SUM))
    recv = result.buffers[0]
    want = contributions[0, :seg].clone()
    for r in range(1, world):
        want = want + contributions[r, :seg]
    assert torch.equal(recv, want)
    torch.testing.assert_close(recv, contributions[:, :seg].double().sum(0).float(), rtol=1e-6, atol=1e-8)
    rows = [contributions[r, 777 : 777 + 50000].cpu().contiguous() for r in range(world)]
    assert torch.equal(recv[777 : 777 + 50000].cpu(), cport.reduce_rows(rows))
    # copy-out: q, k, v and the first 504 rows of o land on rank 0 as views of recv
    numels = [i.local_numel for i in infos]
    assert numels[0] == 4096 * 4096 and numels[1] == numels[2] == 1024 * 4096 and sum(numels) < seg
    for info, shard in zip(infos, result.sharded_grads):
        assert shard.shape == info.local_shape
        if shard.numel():
            start = info.byte_offset // 2
            assert shard.data_ptr() == recv.data_ptr() + 4 * start


# ------------------------------------------------------------ Newton-Schulz
@pytest.mark.parametrize("shape", [(128, 256), (256, 128), (256, 256), (64, 96), (200, 136), (3, 512, 256), (2, 128, 384)])
def test_newton_schulz_matches_torch_muon_routine(device, shape, golden):
    from torch.optim._muon import _zeropower_via_newtonschulz as torch_ns

    tol = golden["muon_tolerance"]["atol"]
    gen = torch.Generator().manual_seed(3)
    g = torch.randn(shape, generator=gen).bfloat16()
    mine = _zeropower_via_newtonschulz(g.to(device)).cpu()
    mats = g.view(-1, *shape[-2:])
    ref = torch.stack([torch_ns(m, COEFFS, 5, 1e-7) for m in mats]).view(shape)
    assert mine.shape == g.shape and mine.dtype == torch.bfloat16
    assert (mine.float() - ref.float()).abs().max().item() <= tol
    small = cport.newton_schulz(mats[0]) if mats[0].numel() <= 128 * 256 else None
    if small is not None:
        assert (mine.view(-1, *shape[-2:])[0].float() - small.float()).abs().max().item() <= tol


@pytest.mark.parametrize("shape,steps", [((20, 1024, 1280), 5), ((20, 1280, 1024), 5), ((24, 1024, 1024), 4), ((20, 1280, 1024), 1)])
def test_newton_schulz_with_one_orientation_carried(device, shape, steps, golden):
    """Batches with whole 256 x 256 x 64 tiles and at least 192 of them carry
    only X^T between steps (G from its k-major rows; a wide input's last step
    written as X' = P X): wide, tall and square inputs, odd, even and single
    step counts, first and last matrix against torch's routine."""
    from torch.optim._muon import _zeropower_via_newtonschulz as torch_ns

    tol = golden["muon_tolerance"]["atol"]
    gen = torch.Generator().manual_seed(8)
    g = torch.randn(shape, generator=gen).bfloat16()
    keep = g.clone()
    on_gpu = g.to(device)
    mine = _zeropower_via_newtonschulz(on_gpu, ns_steps=steps).cpu()
    assert torch.equal(on_gpu.cpu(), keep)
    for index in (0, shape[0] - 1):
        ref = torch_ns(g[index], COEFFS, steps, 1e-7)
        assert (mine[index].float() - ref.float()).abs().max().item() <= tol
    # every matrix of the batch went through the same launches: same result for equal inputs
    twice = torch.stack([g[0], g[0]] * (shape[0] // 2)).contiguous().to(device)
    out = _zeropower_via_newtonschulz(twice, ns_steps=steps)
    assert torch.equal(out[0], out[1]) and torch.equal(out[0], out[-1]) and torch.equal(out[0].cpu(), mine[0])


@pytest.mark.parametrize("batch,m,n,k,symmetric", [(3, 2048, 2048, 320, False), (6, 2048, 2048, 448, True), (1, 4096, 3584, 64, False)])
def test_gemm_k_major_equals_the_k_contiguous_form(device, batch, m, n, k, symmetric):
    """Operands given as [k, m] and [k, n]: the fragments come out of LDS
    through the transposing read, the products and their order are those of
    the k-contiguous form on the transposed operands -- bit-identical."""
    gen = torch.Generator().manual_seed(9)
    a_km = torch.randn(batch, k, m, generator=gen).bfloat16().to(device)
    b_km = a_km if symmetric else torch.randn(batch, k, n, generator=gen).bfloat16().to(device)
    a_nt, b_nt = a_km.transpose(1, 2).contiguous(), b_km.transpose(1, 2).contiguous()
    want = hip_ops.gemm_nt(a_nt, b_nt, symmetric=symmetric)
    got = hip_ops.gemm_nt(a_km, b_km, symmetric=symmetric, k_major=True)
    assert torch.equal(got, want)
    ref = torch.bmm(a_nt.float(), b_nt.float().transpose(1, 2))
    assert ((got.float() - ref).abs().max() / ref.abs().max()).item() < 5e-3
    if symmetric:
        assert torch.equal(got, got.transpose(1, 2))


def test_gemm_k_major_needs_the_large_tile_kernel(device):
    a = torch.randn(1, 64, 256, device=device).bfloat16()
    with pytest.raises(RuntimeError, match="k-major operands need whole 256 x 256 x 64 tiles"):
        hip_ops.gemm_nt(a, a, k_major=True)  # one tile
    b = torch.randn(3, 64, 2048 + 8, device=device).bfloat16()
    with pytest.raises(RuntimeError, match="k-major operands need whole 256 x 256 x 64 tiles"):
        hip_ops.gemm_nt(b, b, k_major=True)  # ragged tiles


def test_newton_schulz_leaves_its_input_untouched_and_handles_zero(device):
    g = torch.randn(128, 128, device=device).bfloat16()
    keep = g.clone()
    _zeropower_via_newtonschulz(g)
    assert torch.equal(g, keep)
    z = _zeropower_via_newtonschulz(torch.zeros(64, 128, device=device, dtype=torch.bfloat16))
    assert (z == 0).all()
    # the C entry itself works on 16-byte rows (the Python wrapper pads other shapes)
    odd = torch.randn(1, 12, 20, device=device).bfloat16()
    work = torch.empty(hip_ops.newton_schulz_workspace_bytes(1, 12, 20), dtype=torch.uint8, device=device)
    status = _native.lib().fsh_newton_schulz(
        odd.data_ptr(), 1, 12, 20, *COEFFS, 5, 1e-7, work.data_ptr(), work.numel(), hip_ops.stream_ptr(device)
    )
    assert status != 0 and b"multiples of 8" in _native.lib().fsh_last_error()


def test_gemm_building_block(device):
    gen = torch.Generator().manual_seed(4)
    a = torch.randn(2, 200, 64, generator=gen).bfloat16().to(device)
    b = torch.randn(2, 136, 64, generator=gen).bfloat16().to(device)
    d = torch.randn(2, 200, 136, generator=gen).bfloat16().to(device)
    ct = torch.empty(2, 136, 200, device=device, dtype=torch.bfloat16)
    c = hip_ops.gemm_nt(a, b, d=d, alpha=0.5, beta=2.0, out_t=ct)
    ref = 0.5 * (a.double() @ b.double().transpose(1, 2)) + 2.0 * d.double()
    assert torch.allclose(c.double(), ref, rtol=2.0**-8, atol=1e-2)  # one bf16 rounding of the fp32 result
    assert torch.equal(ct, c.transpose(1, 2).contiguous())
    big = hip_ops.gemm_nt(a[0].repeat(3, 8)[:512], a[0].repeat(3, 8)[:384])
    want = (a[0].repeat(3, 8)[:512].double() @ a[0].repeat(3, 8)[:384].double().t())
    assert torch.allclose(big.double(), want, rtol=2.0**-7, atol=0.5)


def _gemm_reference(a, b, d=None, alpha=1.0, beta=0.0):
    ref = alpha * (a.cpu().double() @ b.cpu().double().transpose(-1, -2))
    return ref + beta * d.cpu().double() if d is not None else ref


@pytest.mark.parametrize(
    "batch,m,n,k",
    [
        (6, 1536, 1536, 192),  # 256x256x64 whole-tile kernel, 3 k-tiles
        (7, 1536, 1280, 64),  # same kernel, single k-tile, padding workgroups in the grid
        (1, 512, 384, 96),  # 128x128x32 whole-tile kernel
        (9, 1544, 1288, 72),  # 256x256 predicated kernel
    ],
)
def test_gemm_tile_paths(device, batch, m, n, k):
    gen = torch.Generator().manual_seed(batch * 1000 + k)
    a = torch.randn(batch, m, k, generator=gen).bfloat16().to(device)
    b = torch.randn(batch, n, k, generator=gen).bfloat16().to(device)
    d = torch.randn(batch, m, n, generator=gen).bfloat16().to(device)
    # guard bands around both outputs: a tile path must not write outside them
    pad = 2048
    c_buf = torch.full((batch * m * n + 2 * pad,), 7.0, dtype=torch.bfloat16, device=device)
    t_buf = torch.full((batch * m * n + 2 * pad,), 7.0, dtype=torch.bfloat16, device=device)
    c = c_buf[pad:-pad].view(batch, m, n)
    ct = t_buf[pad:-pad].view(batch, n, m)
    hip_ops.gemm_nt(a, b, d=d, alpha=0.5, beta=2.0, out=c, out_t=ct)
    ref = _gemm_reference(a, b, d, 0.5, 2.0)
    assert torch.allclose(c.cpu().double(), ref, rtol=2.0**-8, atol=2e-2)  # one bf16 rounding of the fp32 result
    assert torch.equal(ct, c.transpose(1, 2).contiguous())
    for buf in (c_buf, t_buf):
        assert (buf[:pad] == 7).all() and (buf[-pad:] == 7).all()


@pytest.mark.parametrize("batch,n,k", [(6, 1536, 192), (1, 512, 96), (9, 1544, 72), (40, 520, 64)])
def test_gemm_symmetric_mode_mirrors_the_upper_triangle(device, batch, n, k):
    gen = torch.Generator().manual_seed(n + k)
    a = torch.randn(batch, n, k, generator=gen).bfloat16().to(device)
    full = hip_ops.gemm_nt(a, a)
    sym = hip_ops.gemm_nt(a, a, symmetric=True)
    assert torch.equal(sym, sym.transpose(1, 2))
    assert torch.equal(torch.triu(sym), torch.triu(full))  # the computed tiles are the same work
    assert torch.allclose(sym.float(), full.float(), rtol=2.0**-7, atol=1e-2)
    # with a symmetric addend, as in P = b G + c G G
    p_full = hip_ops.gemm_nt(sym, sym, d=sym, alpha=-0.05, beta=0.3)
    p_sym = hip_ops.gemm_nt(sym, sym, d=sym, alpha=-0.05, beta=0.3, symmetric=True)
    assert torch.equal(p_sym, p_sym.transpose(1, 2))
    assert torch.equal(torch.triu(p_sym), torch.triu(p_full))
    ref = _gemm_reference(sym, sym, sym, -0.05, 0.3)
    assert torch.allclose(p_sym.cpu().double(), ref, rtol=2.0**-7, atol=2e-2 * ref.abs().max().item() / 8)
    with pytest.raises(RuntimeError, match="symmetric"):
        hip_ops.gemm_nt(a, a[:, : n - 8].contiguous(), symmetric=True)


@pytest.mark.parametrize(
    "batch,n,k,symmetric",
    [(10, 1536, 128, True), (7, 1536, 192, False), (1, 512, 96, True), (3, 264, 72, False)],
)
def test_gemm_diagonal_addend(device, batch, n, k, symmetric):
    """C = alpha A B^T + beta D + diag_add I on every kernel: the addend enters
    in fp32 before the one rounding, on the diagonal only (this is how the
    iteration carries `a X` inside `P X`)."""
    gen = torch.Generator().manual_seed(n + k)
    a = torch.randn(batch, n, k, generator=gen).bfloat16().to(device)
    b = a if symmetric else torch.randn(batch, n, k, generator=gen).bfloat16().to(device)
    d = torch.randn(batch, n, n, generator=gen).bfloat16().to(device)
    if symmetric:
        d = torch.triu(d) + torch.triu(d, 1).transpose(1, 2)
    plain = hip_ops.gemm_nt(a, b, d=d, alpha=0.25, beta=-0.5, symmetric=symmetric)
    shifted = hip_ops.gemm_nt(a, b, d=d, alpha=0.25, beta=-0.5, symmetric=symmetric, diag_add=3.4445)
    eye = torch.eye(n, dtype=torch.bool, device=device).expand(batch, n, n)
    assert torch.equal(shifted[~eye], plain[~eye])
    ref = _gemm_reference(a, b, d, 0.25, -0.5) + 3.4445 * torch.eye(n, dtype=torch.float64)
    assert torch.allclose(shifted.cpu().double(), ref, rtol=2.0**-8, atol=2e-2)
    # one rounding: the diagonal is within about half a bf16 ulp of the exact value
    want = ref[eye.cpu()]
    ulp = torch.exp2(torch.floor(torch.log2(want.abs())) - 7)
    assert ((shifted[eye].cpu().double() - want).abs() <= 0.51 * ulp + 1e-3).all()


def test_gemm_group_equals_separate_calls(device):
    """Problems of different shapes and kernels in one call: the ones on the
    large-tile kernel share a launch (longest k first), every result is bit
    for bit what a call of its own gives, and nothing outside the outputs is
    written."""
    gen = torch.Generator().manual_seed(21)
    specs = [
        # (batch, m, n, k, symmetric, with d, with out_t)
        (10, 1536, 1536, 128, True, False, False),  # large tile, short k
        (7, 1536, 1280, 320, False, True, True),  # large tile, long k, all outputs
        (1, 512, 384, 96, False, True, False),  # 128x128 whole-tile kernel
        (10, 1536, 1536, 192, True, True, False),  # large tile, symmetric with addend
        (2, 264, 136, 72, False, False, True),  # predicated kernel
        (8, 1280, 1280, 64, False, False, False),  # large tile, one k-tile
    ]
    pad = 1024
    problems, buffers = [], []
    for batch, m, n, k, symmetric, with_d, with_t in specs:
        a = torch.randn(batch, m, k, generator=gen).bfloat16().to(device)
        b = a if symmetric else torch.randn(batch, n, k, generator=gen).bfloat16().to(device)
        d = None
        if with_d:
            d = torch.randn(batch, m, n, generator=gen).bfloat16().to(device)
            if symmetric:
                d = torch.triu(d) + torch.triu(d, 1).transpose(1, 2)
        c_buf = torch.full((batch * m * n + 2 * pad,), 7.0, dtype=torch.bfloat16, device=device)
        t_buf = torch.full((batch * m * n + 2 * pad,), 7.0, dtype=torch.bfloat16, device=device) if with_t else None
        buffers += [c_buf] + ([t_buf] if with_t else [])
        problems.append(dict(
            a=a, b=b, d=d, alpha=0.75, beta=-1.5, symmetric=symmetric, out=c_buf[pad:-pad].view(batch, m, n),
            out_t=t_buf[pad:-pad].view(batch, n, m) if with_t else None,
        ))
    outs = hip_ops.gemm_nt_group(problems)
    for q, out in zip(problems, outs):
        alone = hip_ops.gemm_nt(q["a"], q["b"], d=q["d"], alpha=q["alpha"], beta=q["beta"], symmetric=q["symmetric"])
        assert torch.equal(out, alone)
        if q["out_t"] is not None:
            assert torch.equal(q["out_t"], out.transpose(1, 2).contiguous())
        ref = _gemm_reference(q["a"], q["b"], q["d"], q["alpha"], q["beta"])
        assert torch.allclose(out.cpu().double(), ref, rtol=2.0**-7, atol=0.25)
    for buf in buffers:
        assert (buf[:pad] == 7).all() and (buf[-pad:] == 7).all()
    assert hip_ops.gemm_nt_group([]) == []


def test_gemm_static_schedule_when_tiles_are_equally_long(device):
    """More large tiles than compute units, all with the same k: one resident
    workgroup per compute unit walks the tiles of both problems (next tile's
    operands requested during the epilogue).  Against fp64 and against the
    symmetric / transposed identities, with guard bands."""
    gen = torch.Generator().manual_seed(33)
    batch, m, n, k = 11, 1536, 1792, 192  # 6 x 7 x 11 = 462 tiles
    a = torch.randn(batch, m, k, generator=gen).bfloat16().to(device)
    b = torch.randn(batch, n, k, generator=gen).bfloat16().to(device)
    d = torch.randn(batch, m, n, generator=gen).bfloat16().to(device)
    s = torch.randn(9, 1280, k, generator=gen).bfloat16().to(device)  # 15 x 9 = 135 symmetric tiles
    pad = 4096
    c_buf = torch.full((batch * m * n + 2 * pad,), 7.0, dtype=torch.bfloat16, device=device)
    t_buf = torch.full((batch * m * n + 2 * pad,), 7.0, dtype=torch.bfloat16, device=device)
    s_buf = torch.full((9 * 1280 * 1280 + 2 * pad,), 7.0, dtype=torch.bfloat16, device=device)
    c, ct, sc = c_buf[pad:-pad].view(batch, m, n), t_buf[pad:-pad].view(batch, n, m), s_buf[pad:-pad].view(9, 1280, 1280)
    hip_ops.gemm_nt_group([
        dict(a=a, b=b, d=d, alpha=0.5, beta=2.0, out=c, out_t=ct),
        dict(a=s, b=s, alpha=1.0, symmetric=True, out=sc),
    ])
    ref = _gemm_reference(a, b, d, 0.5, 2.0)
    assert torch.allclose(c.cpu().double(), ref, rtol=2.0**-8, atol=2e-2)
    assert torch.equal(ct, c.transpose(1, 2).contiguous())
    assert torch.equal(sc, sc.transpose(1, 2))
    assert torch.allclose(sc.cpu().double(), _gemm_reference(s, s), rtol=2.0**-8, atol=2e-2)
    for buf in (c_buf, t_buf, s_buf):
        assert (buf[:pad] == 7).all() and (buf[-pad:] == 7).all()
    # in place, as the iteration uses it: X' = a X + P X with C = D
    x = d.clone()
    hip_ops.gemm_nt(a, b, d=x, alpha=0.5, beta=2.0, out=x)
    assert torch.equal(x, c)


def test_newton_schulz_multi_equals_one_call_per_shape(device):
    """Shape groups iterated together (each product issued for all groups at
    once) against one call per group: identical bits, tall, wide and square,
    large-tile and small-tile kernels mixed."""
    shapes = [(40, 1024, 768), (48, 768, 768), (5, 256, 1024), (1, 64, 96)]  # the first two fill the large tile
    inputs = [seeded_normal(shape, 1.0, 30 + i, device) for i, shape in enumerate(shapes)]
    together = [x.clone() for x in inputs]
    hip_ops.newton_schulz_multi([(x, None) for x in together], COEFFS, 5, 1e-7)
    for x, y in zip(inputs, together):
        alone = hip_ops.newton_schulz(x.clone(), COEFFS, 5, 1e-7)
        assert torch.equal(alone, y)
    from torch.optim._muon import _zeropower_via_newtonschulz as torch_ns

    want = torch_ns(inputs[0][0].cpu(), COEFFS, 5, 1e-7)
    assert (together[0][0].cpu().float() - want.float()).abs().max().item() <= 2e-2
    hip_ops.newton_schulz_multi([], COEFFS, 5, 1e-7)
    with pytest.raises(RuntimeError, match="multiples of 8"):
        hip_ops.newton_schulz_multi([(together[0], None), (torch.zeros(2, 12, 20, device=device, dtype=torch.bfloat16), None)], COEFFS, 5, 1e-7)


def test_newton_schulz_full_size_invariants(device):
    """Config 5 shapes: [7168, 2048] (tall, iterated as its transpose) and
    [2048, 2048].  Singular values of the result lie in the quintic's band and
    the result correlates with the exact polar factor."""
    for shape in ((7168, 2048), (2048, 2048)):
        g = seeded_normal(shape, 1.0, 11, device)
        x = _zeropower_via_newtonschulz(g).float()
        sv = torch.linalg.svdvals(x)
        assert sv.max().item() < 1.3
        if shape[0] != shape[1]:
            # a square Gaussian matrix has singular values near zero that five
            # steps cannot lift; a 3.5:1 one does not
            assert sv.min().item() > 0.3
        u, _, vh = torch.linalg.svd(g.float(), full_matrices=False)
        polar = u @ vh
        cos = (x * polar).sum() / (x.norm() * polar.norm())
        assert cos.item() > (0.97 if shape[0] != shape[1] else 0.9)
    # one full-size matrix against torch's routine on the GPU (its hipBLAS path)
    from torch.optim._muon import _zeropower_via_newtonschulz as torch_ns

    g = seeded_normal((2048, 2048), 1.0, 12, device)
    assert (_zeropower_via_newtonschulz(g).float() - torch_ns(g, COEFFS, 5, 1e-7).float()).abs().max().item() <= 2e-2


# --------------------------------------------------------------- Muon steps
def test_muon_elementwise_kernels(device):
    """Momentum / Nesterov interpolation and the decayed update against the
    same torch tensor ops the reference issues, run by torch on the GPU (the
    reference's own execution target) and on the CPU.  bf16 results may differ
    by one ulp where torch fuses a multiply-add; they must agree almost
    everywhere.  (torch's CPU kernel rounds the decay factor 0.9999 to bf16,
    i.e. to 1.0, so only the GPU comparison is tight for the update.)"""
    gen = torch.Generator().manual_seed(6)
    n = 100003
    grad = torch.randn(n, generator=gen).bfloat16()
    mom = (torch.randn(n, generator=gen) * 0.1).bfloat16()
    for nesterov in (True, False):
        m_gpu, out = mom.to(device), torch.empty(n, dtype=torch.bfloat16, device=device)
        _prepare_muon_input(grad.to(device), m_gpu, momentum=0.95, nesterov=nesterov, out=out)
        for where in (device, torch.device("cpu")):
            m_ref, g_ref = mom.to(where).clone(), grad.to(where)
            m_ref.lerp_(g_ref, 1 - 0.95)
            o_ref = torch.lerp(g_ref, m_ref, 0.95) if nesterov else m_ref.clone()
            assert torch.allclose(m_gpu.cpu().float(), m_ref.cpu().float(), rtol=2.0**-7, atol=1e-6)
            assert torch.allclose(out.cpu().float(), o_ref.cpu().float(), rtol=2.0**-7, atol=1e-5)
            assert (m_gpu.cpu() != m_ref.cpu()).float().mean() < 0.01
            assert (out.cpu() != o_ref.cpu()).float().mean() < 0.02
    p = (torch.randn(n, generator=gen) * 0.02).bfloat16()
    d = torch.randn(n, generator=gen).bfloat16()
    p_gpu = p.to(device)
    _apply_muon_update(p_gpu.view(1, n), d.to(device).view(1, n), lr=1e-3, weight_decay=0.1, adjust_lr_fn=None,
                       compute_matrix_shape=(7168, 2048))
    alpha = -eager.adjusted_lr(1e-3, None, (7168, 2048))
    p_ref = p.to(device).clone()
    p_ref.mul_(1 - 1e-3 * 0.1)
    p_ref.add_(d.to(device), alpha=alpha)
    assert torch.allclose(p_gpu.float(), p_ref.float(), rtol=2.0**-7, atol=2e-5)
    assert (p_gpu != p_ref).float().mean() < 0.01
    p_cpu = p.clone()
    p_cpu.mul_(1 - 1e-3 * 0.1)
    p_cpu.add_(d, alpha=alpha)
    assert torch.allclose(p_gpu.cpu().float(), p_cpu.float(), rtol=2.0**-7, atol=2e-5)


def test_owned_muon_step_matches_torch_optim_muon(device, golden):
    """Three steps on whole matrices of two shapes against torch.optim.Muon's
    single-tensor path (same defaults), the reference's own oracle and bar."""
    tol = golden["muon_tolerance"]["atol"]
    gen = torch.Generator().manual_seed(7)
    shapes = [(256, 128), (128, 128), (256, 128), (128, 128)]
    start = [(torch.randn(s, generator=gen) * 0.02).bfloat16() for s in shapes]
    mine = [p.clone().to(device) for p in start]
    theirs = [nn.Parameter(p.clone()) for p in start]
    opt_mine = OwnedMuon(mine)
    opt_theirs = torch.optim.Muon(theirs, lr=1e-3, weight_decay=0.1, momentum=0.95, nesterov=True)
    for _ in range(3):
        grads = [torch.randn(s, generator=gen).bfloat16() for s in shapes]
        opt_mine.step([g.to(device) for g in grads])
        for p, g in zip(theirs, grads):
            p.grad = g.clone()
        opt_theirs.step()
    for a, b in zip(mine, theirs):
        assert (a.cpu().float() - b.detach().float()).abs().max().item() <= tol
        assert torch.allclose(a.cpu().float(), b.detach().float(), atol=1e-3)  # a few bf16 ulps of the weights
    assert opt_mine.flops_per_step() == 2 * (
        _estimate_muon_compute_cost((2, 256, 128), 5) + _estimate_muon_compute_cost((2, 128, 128), 5)
    )
    with pytest.raises(RuntimeError, match="no gradient"):
        before = [p.clone() for p in mine]
        opt_mine.step([None] + [torch.zeros_like(p) for p in mine[1:]])
    assert all(torch.equal(a, b) for a, b in zip(mine, before))



def test_muon_elementwise_kernels_on_fp32_masters(device):
    """fp32 gradient, momentum buffer and parameter (the dtype of the
    reference's own optimizer tests): the momentum and the parameter are
    updated in fp32, bit for bit the interpolation and the decayed update
    written as separate fp32 multiplies and adds, and within an fp32 ulp of the
    operands of torch.lerp / mul_ / add_ (which may fuse a multiply-add); the
    orthogonalization's bf16 input is the one rounding of the fp32 blend."""
    gen = torch.Generator().manual_seed(16)
    n = 100003
    grad = torch.randn(n, generator=gen)
    mom = torch.randn(n, generator=gen) * 0.1

    def lerp(start, end, w):  # torch.lerp's two branches, every operation rounded on its own
        diff = end - start
        w32 = torch.tensor(w, dtype=torch.float32)  # the weight and 1 - weight are fp32 values
        return start + w32 * diff if w < 0.5 else end - diff * (1 - w32)

    for nesterov in (True, False):
        m_gpu, out = mom.to(device), torch.empty(n, dtype=torch.bfloat16, device=device)
        _prepare_muon_input(grad.to(device), m_gpu, momentum=0.95, nesterov=nesterov, out=out)
        w_small = torch.tensor(1 - 0.95, dtype=torch.float32)
        m_ref = mom + w_small * (grad - mom)
        u_ref = lerp(grad, m_ref, 0.95) if nesterov else m_ref
        assert torch.equal(m_gpu.cpu(), m_ref)
        assert torch.equal(out.cpu(), u_ref.bfloat16())
        m_torch = mom.clone().lerp_(grad, 1 - 0.95)
        assert torch.allclose(m_gpu.cpu(), m_torch, rtol=1e-6, atol=1e-6)  # a fused multiply-add moves an fp32 ulp of the operands
        o_torch = (torch.lerp(grad, m_torch, 0.95) if nesterov else m_torch).bfloat16()
        assert (out.cpu() != o_torch).float().mean() < 1e-3
    p = torch.randn(n, generator=gen) * 0.02
    d = torch.randn(n, generator=gen).bfloat16()
    alpha = -eager.adjusted_lr(1e-3, None, (7168, 2048))
    for scale in (1.0, 0.5303300858899106):
        p_gpu = p.to(device)
        hip_ops.muon_apply(p_gpu, d.to(device), decay_factor=1 - 1e-3 * 0.1, neg_adjusted_lr=alpha, direction_scale=scale)
        f32 = lambda v: torch.tensor(v, dtype=torch.float32)
        dd = d.float() if scale == 1.0 else d.float() * f32(scale)
        want = p * f32(1 - 1e-3 * 0.1) + f32(alpha) * dd
        assert torch.equal(p_gpu.cpu(), want)
        p_torch = p.clone().mul_(1 - 1e-3 * 0.1).add_(dd, alpha=alpha)
        assert torch.allclose(p_gpu.cpu(), p_torch, rtol=1e-6, atol=1e-6)
    with pytest.raises(ValueError, match="differ in dtype"):
        _prepare_muon_input(grad.to(device), mom.bfloat16().to(device), momentum=0.95, nesterov=True,
                            out=torch.empty(n, dtype=torch.bfloat16, device=device))


def test_owned_muon_on_fp32_masters_matches_torch_optim_muon(device, golden):
    """Three steps on fp32 whole matrices (two shapes for the batched step,
    one whose sides are not multiples of 8 for the per-matrix path, and a bf16
    parameter beside them) against torch.optim.Muon on the host; the batched
    step gives the bits of the per-matrix kernels."""
    tol = golden["muon_tolerance"]["atol"]
    gen = torch.Generator().manual_seed(17)
    shapes = [(256, 128), (128, 128), (256, 128), (100, 36), (128, 128)]
    dtypes = [torch.float32, torch.float32, torch.float32, torch.float32, torch.bfloat16]
    start = [(torch.randn(s, generator=gen) * 0.02).to(dt) for s, dt in zip(shapes, dtypes)]
    mine = [p.clone().to(device) for p in start]
    by_hand = [p.clone().to(device) for p in start]
    hand_momentum = [torch.zeros_like(p) for p in by_hand]
    theirs = [nn.Parameter(p.clone()) for p in start]
    opt_mine = OwnedMuon(mine)
    assert all(m.dtype == p.dtype for m, p in zip(opt_mine.momentum_buffers, mine))
    opt_theirs = torch.optim.Muon(theirs, lr=1e-3, weight_decay=0.1, momentum=0.95, nesterov=True)
    for _ in range(3):
        grads = [torch.randn(s, generator=gen).to(dt) for s, dt in zip(shapes, dtypes)]
        opt_mine.step([g.to(device) for g in grads])
        for p, m, g in zip(by_hand, hand_momentum, grads):
            direction = _prepare_muon_input(g.to(device), m, momentum=0.95, nesterov=True,
                                            out=torch.empty(p.shape, dtype=torch.bfloat16, device=device))
            _compute_muon_direction(direction)
            _apply_muon_update(p, direction, lr=1e-3, weight_decay=0.1, adjust_lr_fn=None, compute_matrix_shape=p.shape)
        for p, g in zip(theirs, grads):
            p.grad = g.clone()
        opt_theirs.step()
    for a, h, b in zip(mine, by_hand, theirs):
        assert torch.equal(a, h)
        assert (a.cpu().float() - b.detach().float()).abs().max().item() <= tol
        assert torch.allclose(a.cpu().float(), b.detach().float(), atol=1e-3)
    for m, h in zip(opt_mine.momentum_buffers, hand_momentum):
        assert torch.equal(m, h)
    with pytest.raises(ValueError, match="does not match parameter"):
        opt_mine.step([torch.zeros_like(p).bfloat16() if p.dtype == torch.float32 else torch.zeros_like(p) for p in mine])
    with pytest.raises(NotImplementedError, match="bf16 or fp32"):
        OwnedMuon([torch.zeros(8, 8, dtype=torch.float16, device=device)])



def test_owned_muon_takes_stacked_parameters_as_batches_of_matrices(device, golden):
    """A parameter with leading dimensions ([experts, rows, cols]) is updated
    as its matrices would be on their own (dist_muon/optimizer.py:2082-2091
    views it as a batch): same bits as an optimizer over the unbound
    matrices, for the batched step and for the per-matrix path of shapes that
    are not multiples of 8, and within the reference's bar of its step in
    eager torch on the host."""
    tol = golden["muon_tolerance"]["atol"]
    gen = torch.Generator().manual_seed(19)
    shapes = [(3, 64, 128), (2, 100, 36), (128, 64), (2, 2, 64, 128)]
    dtypes = [torch.float32, torch.bfloat16, torch.bfloat16, torch.bfloat16]
    start = [(torch.randn(s, generator=gen) * 0.02).to(dt) for s, dt in zip(shapes, dtypes)]
    stacked = [p.clone().to(device) for p in start]
    separate = [m.clone() for p in start for m in p.to(device).reshape(-1, *p.shape[-2:]).unbind(0)]
    host = [m.clone() for p in start for m in p.reshape(-1, *p.shape[-2:]).unbind(0)]
    host_momentum = [torch.zeros_like(m) for m in host]
    opt_stacked, opt_separate = OwnedMuon(stacked, adjust_lr_fn="match_rms_adamw"), OwnedMuon(separate, adjust_lr_fn="match_rms_adamw")
    assert opt_stacked.flops_per_step() == opt_separate.flops_per_step()
    for _ in range(2):
        grads = [torch.randn(s, generator=gen).to(dt) for s, dt in zip(shapes, dtypes)]
        opt_stacked.step([g.to(device) for g in grads])
        flat = [m.contiguous() for g in grads for m in g.reshape(-1, *g.shape[-2:]).unbind(0)]
        opt_separate.step([g.to(device) for g in flat])
        for p, g, m in zip(host, flat, host_momentum):
            eager.muon_step(p, g, m, adjust_lr_fn="match_rms_adamw")
    ours = [m for p in stacked for m in p.reshape(-1, *p.shape[-2:]).unbind(0)]
    for a, b, c in zip(ours, separate, host, strict=True):
        assert torch.equal(a, b)
        assert (a.cpu().float() - c.float()).abs().max().item() <= tol
    # a stacked parameter whose storage is replaced between steps is followed
    moved = stacked[0].clone()
    stacked[0].data = moved
    grads = [torch.randn(s, generator=gen).to(dt) for s, dt in zip(shapes, dtypes)]
    opt_stacked.step([g.to(device) for g in grads])
    opt_separate.step([m.contiguous().to(device) for g in grads for m in g.reshape(-1, *g.shape[-2:]).unbind(0)])
    assert stacked[0].data_ptr() == moved.data_ptr()
    for a, b in zip(stacked[0].unbind(0), separate[:3], strict=True):
        assert torch.equal(a, b)
    with pytest.raises(ValueError, match="Muon updates matrices"):
        OwnedMuon([torch.zeros(64, device=device, dtype=torch.bfloat16)])


def test_newton_schulz_batch_beyond_two_to_the_32_bytes(device):
    """160 matrices of [7168, 2048]: the batch (4.7 GB) and every workspace
    buffer pass 2^32 bytes.  The first and the last 24 matrices must come out
    with the bits of a 24-matrix call on their own (same kernels and k order;
    only the addresses differ)."""
    batch, rows, cols = 160, 7168, 2048
    x = torch.empty((batch, rows, cols), device=device, dtype=torch.bfloat16)
    x[:24].normal_()
    x[-24:].normal_()
    x[24:-24] = x[:8].repeat((batch - 48) // 8, 1, 1)
    assert x.numel() * 2 > 2**32
    first, last = x[:24].clone(), x[-24:].clone()
    hip_ops.newton_schulz(x, (3.4445, -4.7750, 2.0315), 5, 1e-7)
    hip_ops.newton_schulz(first, (3.4445, -4.7750, 2.0315), 5, 1e-7)
    hip_ops.newton_schulz(last, (3.4445, -4.7750, 2.0315), 5, 1e-7)
    assert torch.equal(x[:24], first)
    assert torch.equal(x[-24:], last)
    assert torch.equal(x[24:32], x[:8]) and torch.equal(x[-32:-24], x[:8])


# ------------------------------------------- config 5 at the benchmarked size
CONFIG5_SHAPES = [(7168, 2048)] * 24 + [(2048, 2048)] * 24


def _direction_error(mine: torch.Tensor, ref: torch.Tensor) -> tuple[float, float]:
    diff = mine.float() - ref.float()
    return diff.abs().max().item(), (diff.norm() / ref.float().norm()).item()


def test_newton_schulz_multi_config5_batches_match_torch_routine(device, golden):
    """The two batches the benchmark times, 24 x [7168, 2048] and
    24 x [2048, 2048], in one newton_schulz_multi call (the launches shared by
    both shape groups, one orientation carried, k-major operands, resident
    workgroups): first and last matrix of each shape, element by element,
    against torch's own Newton-Schulz (the reference's 2-D branch,
    dist_muon/optimizer.py:2120-2151) at the reference's bar
    (tests/test_dist_muon_optimizer.py:206-212), plus a relative Frobenius
    bound so that the comparison has teeth on entries of size 0.02."""
    from torch.optim._muon import _zeropower_via_newtonschulz as torch_ns

    tol = golden["muon_tolerance"]["atol"]
    batches = [seeded_normal((24, 7168, 2048), 1.0, 41, device), seeded_normal((24, 2048, 2048), 1.0, 42, device)]
    inputs = {(b.shape[1], index): b[index].cpu() for b in batches for index in (0, 23)}
    hip_ops.newton_schulz_multi([(b, None) for b in batches], COEFFS, 5, 1e-7)
    for b in batches:
        for index in (0, 23):
            ref = torch_ns(inputs[(b.shape[1], index)], COEFFS, 5, 1e-7)
            worst, rel = _direction_error(b[index].cpu(), ref)
            print(f"config 5 NS {tuple(b.shape[1:])}[{index}]: max abs {worst:.3e}, rel Frobenius {rel:.3e}", flush=True)
            assert worst <= tol
            assert rel <= 2e-2
        # equal inputs in different batch slots give equal bits
    again = torch.stack([inputs[(7168, 0)]] * 24).to(device)
    hip_ops.newton_schulz_multi([(again, None), (batches[1].normal_(), None)], COEFFS, 5, 1e-7)
    assert torch.equal(again[0], again[23]) and torch.equal(again[0], batches[0][0])


def test_owned_muon_step_config5_matches_reference_step(device, golden):
    """One OwnedMuon.step over the 48 matrices of config 5 (gradients N(0, 1),
    momentum 0.95, Nesterov, 5 steps): orthogonalized direction and updated
    parameter of the first and last matrix of each shape against the
    reference step in eager torch on the host (dist_muon/optimizer.py
    :2049-2151)."""
    tol = golden["muon_tolerance"]["atol"]
    params = [seeded_normal(s, 0.02, 2000 + i, device) for i, s in enumerate(CONFIG5_SHAPES)]
    grads = [seeded_normal(s, 1.0, 3000 + i, device) for i, s in enumerate(CONFIG5_SHAPES)]
    checked = (0, 23, 24, 47)
    before = {i: params[i].cpu() for i in checked}
    opt = OwnedMuon(params)
    opt.step(grads)
    # The step applies the update from the last product's epilogue and never
    # stores the direction; the same kernels give it here for the comparison.
    batches = {
        key[:2]: torch.stack([
            _prepare_muon_input(grads[i], torch.zeros_like(grads[i]), momentum=0.95, nesterov=True,
                                out=torch.empty_like(grads[i]))
            for i in members
        ])
        for key, members in opt._groups.items()
    }
    hip_ops.newton_schulz_multi([(b, None) for b in batches.values()], COEFFS, 5, 1e-7)
    for i in checked:
        shape = CONFIG5_SHAPES[i]
        slot = opt._groups[(*shape, torch.bfloat16)].index(i)
        direction = batches[shape][slot].cpu()
        momentum = torch.zeros(shape, dtype=torch.bfloat16)
        g = grads[i].cpu()
        momentum.lerp_(g, 1 - 0.95)
        update = torch.lerp(g, momentum, 0.95)
        ref_direction = eager.newton_schulz(update, COEFFS, 5, 1e-7)
        worst, rel = _direction_error(direction, ref_direction)
        print(f"config 5 Muon {shape}[{i}]: direction max abs {worst:.3e}, rel Frobenius {rel:.3e}", flush=True)
        assert worst <= tol
        assert rel <= 2e-2
        assert torch.equal(opt.momentum_buffers[i].cpu(), momentum)
        p_ref = before[i].clone()
        p_ref.mul_(1 - 1e-3 * 0.1)
        p_ref.add_(ref_direction, alpha=-eager.adjusted_lr(1e-3, None, shape))
        assert (params[i].cpu().float() - p_ref.float()).abs().max().item() <= tol
        assert torch.allclose(params[i].cpu().float(), p_ref.float(), rtol=2.0**-7, atol=2e-5)  # one bf16 ulp
    assert opt.flops_per_step() == 2 * (
        _estimate_muon_compute_cost((24, 7168, 2048), 5) + _estimate_muon_compute_cost((24, 2048, 2048), 5)
    )


@pytest.mark.parametrize("nesterov", [True, False])
def test_fused_muon_step_equals_the_per_matrix_kernels(device, nesterov):
    """OwnedMuon.step is one fsh_muon_step call (batched momentum kernel that
    also leaves the norm partials, Newton-Schulz over all groups, the update
    applied by the last product's epilogue for the large-tile groups and by a
    batched kernel for the others).  It must give the bits of the per-matrix sequence
    _prepare_muon_input -> newton_schulz_multi -> _apply_muon_update: wide,
    tall and small matrices, a batch large enough for the large-tile
    one-orientation flow, two steps (the second with momentum in place and
    gradients at new addresses)."""
    shapes = [(1024, 1280)] * 20 + [(768, 256)] * 3 + [(64, 96)] + [(256, 256)] * 2
    start = [seeded_normal(s, 0.02, 700 + i, device) for i, s in enumerate(shapes)]
    mine = [p.clone() for p in start]
    theirs = [p.clone() for p in start]
    opt = OwnedMuon(mine, nesterov=nesterov, lr=2e-3, weight_decay=0.05)
    momenta = [torch.zeros_like(p) for p in theirs]
    groups: dict[tuple[int, int], list[int]] = {}
    for i, s in enumerate(shapes):
        groups.setdefault(s, []).append(i)
    for step in range(2):
        grads = [seeded_normal(s, 1.0, 800 + 100 * step + i, device) for i, s in enumerate(shapes)]
        opt.step(grads)
        batches = {s: torch.empty((len(m), *s), dtype=torch.bfloat16, device=device) for s, m in groups.items()}
        for s, members in groups.items():
            for slot, i in enumerate(members):
                _prepare_muon_input(grads[i], momenta[i], momentum=0.95, nesterov=nesterov, out=batches[s][slot])
        hip_ops.newton_schulz_multi([(batches[s], None) for s in groups], COEFFS, 5, 1e-7)
        for s, members in groups.items():
            for slot, i in enumerate(members):
                _apply_muon_update(theirs[i], batches[s][slot], lr=2e-3, weight_decay=0.05, adjust_lr_fn=None,
                                   compute_matrix_shape=s)
        for i in range(len(shapes)):
            assert torch.equal(opt.momentum_buffers[i], momenta[i]), f"momentum {i} differs at step {step}"
            assert torch.equal(mine[i], theirs[i]), f"parameter {i} differs at step {step}"
    assert not torch.equal(mine[0], start[0])


# ------------------------------------- shapes that are not multiples of 8, schedules, scaled directions
@pytest.mark.parametrize("shape", [(100, 36), (33, 77), (130, 64), (2, 21, 50), (7, 7)])
def test_newton_schulz_takes_any_shape(device, shape, golden):
    """Rows or columns that are not multiples of 8 are zero-padded inside the
    wrapper (zero rows and columns stay zero through the iteration and leave
    the norm unchanged); against torch's own routine, the reference's bar."""
    from torch.optim._muon import _zeropower_via_newtonschulz as torch_ns

    tol = golden["muon_tolerance"]["atol"]
    gen = torch.Generator().manual_seed(12)
    g = torch.randn(shape, generator=gen).bfloat16()
    on_gpu = g.to(device)
    mine = _zeropower_via_newtonschulz(on_gpu).cpu()
    assert mine.shape == g.shape and torch.equal(on_gpu.cpu(), g)  # the input is left as it was
    ref = torch.stack([torch_ns(m, COEFFS, 5, 1e-7) for m in g.clone().view(-1, *shape[-2:])]).view(shape)
    assert (mine.float() - ref.float()).abs().max().item() <= tol


def test_owned_muon_with_odd_shapes_and_a_learning_rate_schedule(device, golden):
    """Matrices the batched step cannot take (rows or columns not multiples of
    8) go through the per-matrix kernels beside the batched groups, and a
    learning rate changed between steps moves the step size and the weight
    decay together: three steps against torch.optim.Muon under the same
    schedule."""
    tol = golden["muon_tolerance"]["atol"]
    gen = torch.Generator().manual_seed(21)
    shapes = [(256, 128), (100, 36), (128, 128), (33, 77), (256, 128)]
    start = [(torch.randn(s, generator=gen) * 0.02).bfloat16() for s in shapes]
    mine = [p.clone().to(device) for p in start]
    theirs = [nn.Parameter(p.clone()) for p in start]
    opt_mine = OwnedMuon(mine, lr=1e-3)
    opt_theirs = torch.optim.Muon(theirs, lr=1e-3, weight_decay=0.1, momentum=0.95, nesterov=True)
    for lr in (1e-3, 5e-2, 2e-4):
        opt_mine.lr = lr
        for group in opt_theirs.param_groups:
            group["lr"] = lr
        grads = [torch.randn(s, generator=gen).bfloat16() for s in shapes]
        opt_mine.step([g.to(device) for g in grads])
        for p, g in zip(theirs, grads):
            p.grad = g.clone()
        opt_theirs.step()
    for a, b, p0 in zip(mine, theirs, start):
        assert (a.cpu().float() - b.detach().float()).abs().max().item() <= tol
        assert torch.allclose(a.cpu().float(), b.detach().float(), atol=4e-3)
        # the 5e-2 step moved every entry by about lr x sqrt(rows/cols) x |direction|: a frozen step size would not
        assert (a.cpu().float() - p0.float()).abs().mean().item() > 1e-3


def test_muon_step_plan_with_scaled_directions_equals_the_per_matrix_kernels(device):
    """A direction scale other than 1 (a matrix whose learning-rate factor
    differs from its reference shape's): the update in the last product's
    epilogue (large-tile group) and the batched update kernel (small group)
    must give the bits of prepare -> Newton-Schulz -> apply(direction_scale)."""
    groups = [((1024, 1280), 20, -3e-3, 0.75), ((64, 96), 2, -1.5e-3, 1.5)]
    plan = hip_ops.MuonStepPlan(groups, device)
    params, momenta, grads, ref_params, ref_momenta = [], [], [], [], []
    for gi, (shape, n, _, _) in enumerate(groups):
        params.append([seeded_normal(shape, 0.02, 900 + 50 * gi + i, device) for i in range(n)])
        momenta.append([seeded_normal(shape, 0.5, 1900 + 50 * gi + i, device) for i in range(n)])
        grads.append([seeded_normal(shape, 1.0, 2900 + 50 * gi + i, device) for i in range(n)])
        ref_params.append([p.clone() for p in params[-1]])
        ref_momenta.append([m.clone() for m in momenta[-1]])
    decay = 1 - 2e-3 * 0.05
    plan.step(params, momenta, grads, lerp_weight=0.05, nesterov_weight=0.95, nesterov=True, decay_factor=decay,
              coefficients=COEFFS, steps=5, eps=1e-7)
    batches = [torch.empty((n, *shape), dtype=torch.bfloat16, device=device) for shape, n, _, _ in groups]
    for gi, (shape, n, _, _) in enumerate(groups):
        for i in range(n):
            _prepare_muon_input(grads[gi][i], ref_momenta[gi][i], momentum=0.95, nesterov=True, out=batches[gi][i])
    hip_ops.newton_schulz_multi([(b, None) for b in batches], COEFFS, 5, 1e-7)
    for gi, (shape, n, neg_lr, scale) in enumerate(groups):
        for i in range(n):
            hip_ops.muon_apply(ref_params[gi][i], batches[gi][i], decay_factor=decay, neg_adjusted_lr=neg_lr,
                               direction_scale=scale)
            assert torch.equal(momenta[gi][i], ref_momenta[gi][i]), f"momentum {gi}/{i}"
            assert torch.equal(params[gi][i], ref_params[gi][i]), f"parameter {gi}/{i}"
    # the per-step override replaces what the plan was built with
    plan.step(params, momenta, grads, lerp_weight=0.05, nesterov_weight=0.95, nesterov=True, decay_factor=decay,
              coefficients=COEFFS, steps=5, eps=1e-7, neg_adjusted_lrs=[0.0, 0.0], direction_scales=[1.0, 1.0])
    for gi in range(len(groups)):
        for i in range(groups[gi][1]):
            want = (ref_params[gi][i].float() * decay).bfloat16()
            assert torch.equal(params[gi][i], want), f"zero step size {gi}/{i}"
