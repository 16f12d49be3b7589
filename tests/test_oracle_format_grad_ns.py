"""Pins of the oracle's payload format, gradient arithmetic and Newton-Schulz
(CPU only)."""

import math

import pytest
import torch

from oracle import cport, eager
from oracle import layout as olayout


def _quantized_bucket(shapes, block, seed=0):
    gen = torch.Generator().manual_seed(seed)
    params = [(torch.randn(s, generator=gen) * 0.02).bfloat16() for s in shapes]
    qs, ss = zip(*[cport.quantize_blockwise(p.flatten(0, -2), block) for p in params])
    return params, list(qs), list(ss)


@pytest.mark.parametrize(
    "shapes,block,world",
    [([(16, 8), (8, 8), (1, 3)], 4, 8), ([(2, 6, 8)], 4, 3), ([(9, 32)], 2, 2), ([(16, 8), (8, 8), (2, 4)], 4, 8), ([(4, 4)], 4, 4)],
)
def test_pack_gather_compact_equals_whole_matrix_quantization(shapes, block, world):
    """Packing each rank's units, stacking the payload rows and compacting them
    rebuilds exactly [all FP8 bytes | pad | all scales] of whole-matrix
    quantization, also through strided rows at an odd byte offset."""
    _, qs, ss = _quantized_bucket(shapes, block)
    lay = olayout.quant_layout(shapes, block, world)
    rows = torch.stack([olayout.pack_rank_payload(lay, r, qs, ss, block) for r in range(world)])
    want = olayout.compact_from_full(qs, ss)
    got = olayout.compact_from_rank_rows(lay, rows)
    assert torch.equal(got, want)
    parent = torch.full((world, lay.row_nbytes + 3), 0xFF, dtype=torch.uint8)
    parent[:, 1 : lay.row_nbytes + 1] = rows
    assert torch.equal(olayout.compact_from_rank_rows(lay, parent[:, 1 : lay.row_nbytes + 1]), want)
    # payload invariants: pads are zero, sizes follow the 16-byte rule
    for r in range(world):
        n, s0, end = lay.rank_numels[r], lay.rank_scale_byte_offsets[r], lay.rank_packed_nbytes[r]
        assert s0 == -(-n // 16) * 16 and end == s0 + 4 * lay.rank_scale_numels[r]
        assert (rows[r, n:s0] == 0).all() and (rows[r, end:] == 0).all()
    assert lay.row_nbytes % 16 == 0 and lay.row_nbytes >= max(lay.rank_packed_nbytes)


def test_per_rank_quantization_equals_slices_of_whole_quantization():
    """What a rank quantizes locally (its row range) is byte-identical to the
    slice of the whole-matrix result that pack_rank_payload copies."""
    shapes, block, world = [(16, 8), (8, 8), (12, 4)], 4, 8
    params, qs, ss = _quantized_bucket(shapes, block, seed=3)
    lay = olayout.quant_layout(shapes, block, world)
    for rank in range(world):
        payload = olayout.pack_rank_payload(lay, rank, qs, ss, block)
        cursor, scale_cursor = 0, lay.rank_scale_byte_offsets[rank]
        for p, (lo, hi) in enumerate(olayout.local_row_ranges(lay, rank, len(shapes))):
            if hi == lo:
                continue
            q, s = cport.quantize_blockwise(params[p][lo:hi], block)
            assert torch.equal(payload[cursor : cursor + q.numel()], q.reshape(-1))
            sb = s.reshape(-1).view(torch.uint8)
            assert torch.equal(payload[scale_cursor : scale_cursor + sb.numel()], sb)
            cursor += q.numel()
            scale_cursor += sb.numel()


def test_segment_copy_and_zero(golden):
    g = golden["segment_split_case"]
    gen = torch.Generator().manual_seed(1)
    source = torch.randint(-(2**31), 2**31 - 1, (g["source_numel"],), dtype=torch.int32, generator=gen)
    out = torch.zeros(g["output_numel"], dtype=torch.int32)
    segs = g["segments"]
    cport.copy_segments(
        source.view(torch.uint8), out.view(torch.uint8),
        [4 * s for s, _, _ in segs], [4 * n for _, n, _ in segs], [4 * d for _, _, d in segs],
    )
    want = torch.zeros_like(out)
    for s, n, d in segs:
        want[d : d + n] = source[s : s + n]
    assert torch.equal(out, want)
    cport.zero_segments(out.view(torch.uint8), [4 * 10], [4 * 241])
    want[241:251] = 0
    assert torch.equal(out, want)


def test_reduce_scatter_input_rows(golden):
    """Rows are each rank's range of the zeroed param-major bucket, zero padded
    to the longest range (checked against a direct element-by-element build)."""
    dense = golden["reduce_copy_in_cases"]["dense_case"]
    lay = olayout.dense_bucket_layout(dense["shapes"], dense["blocks_per_rank"])
    gen = torch.Generator().manual_seed(0)
    grads = [torch.randn(s, generator=gen).bfloat16() for s in dense["shapes"]]
    rows = olayout.reduce_scatter_input(
        grads, lay.param_offsets, lay.global_numel, lay.rank_offsets, lay.rank_numels, torch.bfloat16
    )
    assert rows.shape == (4, max(lay.rank_numels))
    for rank in range(4):
        for col in range(rows.shape[1]):
            g_index = lay.rank_offsets[rank] + col
            want = 0.0
            if col < lay.rank_numels[rank]:
                for grad, offset in zip(grads, lay.param_offsets):
                    if offset <= g_index < offset + grad.numel():
                        want = grad.reshape(-1)[g_index - offset].item()
            assert rows[rank, col].item() == want
    assert (rows[2] == 0).all()  # rank 2 owns no blocks


def test_fp32_accumulation_known_answer(golden):
    g = golden["fp32_accumulation"]
    grads = [torch.full((8,), g["first"]).bfloat16(), torch.full((8,), g["second"]).bfloat16()]
    acc = torch.zeros(8)
    for grad in grads:
        cport.accumulate_bf16(acc, grad)
    assert (acc == g["fp32_sum"]).all()
    assert (eager.accumulate_microbatches(grads) == g["fp32_sum"]).all()
    assert ((grads[0] + grads[1]) == g["bf16_sum"]).all()  # bf16 accumulation would lose the 1


def test_accumulate_and_fold_orders():
    gen = torch.Generator().manual_seed(6)
    grads = [(torch.randn(4099, generator=gen) * 1e-3).bfloat16() for _ in range(4)]
    acc = torch.zeros(4099)
    for grad in grads:
        cport.accumulate_bf16(acc, grad)
    assert torch.equal(acc, eager.accumulate_microbatches(grads))
    # exactness: every partial sum of four bf16 values of this size is exact in fp64
    exact = sum(g.double() for g in grads)
    assert torch.allclose(acc.double(), exact, rtol=1e-6, atol=0)

    rows = [torch.randn(1000, generator=gen) for _ in range(8)]
    folded = cport.reduce_rows(rows)
    want = rows[0].clone()
    for r in rows[1:]:
        want = want + r
    assert torch.equal(folded, want)
    assert torch.equal(folded, eager.reduce_rank_contributions([r for r in rows], 0, 1000))
    # the association matters: a pairwise tree gives different bits somewhere
    tree = ((rows[0] + rows[1]) + (rows[2] + rows[3])) + ((rows[4] + rows[5]) + (rows[6] + rows[7]))
    assert not torch.equal(tree, folded)
    # divide-factor variants
    avg = cport.reduce_rows(rows, cport.REDUCE_PREMUL, 1.0 / 8)
    assert torch.equal(avg, want / 8)  # power-of-two factor commutes with rounding
    post = cport.reduce_rows(rows, cport.REDUCE_POSTDIV, 3.0)
    assert torch.equal(post, want / 3.0)
    pre = cport.reduce_rows(rows, cport.REDUCE_PREMUL, 1.0 / 3)
    assert torch.equal(pre, eager.reduce_rank_contributions(rows, 0, 1000, premultiply=1.0 / 3))


# ------------------------------------------------------------ Newton-Schulz
COEFFS = (3.4445, -4.7750, 2.0315)


def test_eager_newton_schulz_equals_torch_muon_routine():
    from torch.optim._muon import _zeropower_via_newtonschulz as torch_ns

    gen = torch.Generator().manual_seed(8)
    for shape in ((64, 96), (96, 64), (80, 80)):
        g = torch.randn(shape, generator=gen).bfloat16()
        assert torch.equal(eager.newton_schulz(g), torch_ns(g, COEFFS, 5, 1e-7))
    batch = torch.randn(3, 48, 64, generator=gen).bfloat16()
    per_matrix = torch.stack([torch_ns(m, COEFFS, 5, 1e-7) for m in batch])
    assert (eager.newton_schulz(batch).float() - per_matrix.float()).abs().max() <= 2e-2


def test_c_newton_schulz_within_reference_tolerance(golden):
    from torch.optim._muon import _zeropower_via_newtonschulz as torch_ns

    tol = golden["muon_tolerance"]["atol"]
    gen = torch.Generator().manual_seed(9)
    for shape in ((24, 40), (40, 24), (32, 32)):
        g = torch.randn(shape, generator=gen).bfloat16()
        got = cport.newton_schulz(g)
        assert got.shape == g.shape
        assert (got.float() - torch_ns(g, COEFFS, 5, 1e-7).float()).abs().max() <= tol


def test_newton_schulz_invariants():
    """Independent of any implementation: singular values land near 1, the
    singular vectors are those of the input (polar factor), NS(G^T) = NS(G)^T,
    and NS(alpha G) = NS(G) up to bf16 noise."""
    gen = torch.Generator().manual_seed(10)
    g = torch.randn(48, 80, generator=gen)
    for ns in (eager.newton_schulz, cport.newton_schulz):
        x = ns(g.bfloat16()).double()
        sv = torch.linalg.svdvals(x)
        assert sv.min() > 0.3 and sv.max() < 1.6
        u, _, vh = torch.linalg.svd(g.double(), full_matrices=False)
        polar = u @ vh
        # the quintic leaves singular values in a band around 1, so compare directions
        cos = (x * polar).sum() / (x.norm() * polar.norm())
        assert cos > 0.97
        xt = ns(g.t().contiguous().bfloat16()).double()
        assert (xt - x.t()).abs().max() <= 2e-2
        scaled = ns((g * 37.0).bfloat16()).double()
        assert (scaled - x).abs().max() <= 3e-2


def test_adjusted_lr_and_muon_step_match_torch_optim_muon():
    gen = torch.Generator().manual_seed(12)
    for shape in ((32, 64), (64, 32)):
        p0 = (torch.randn(shape, generator=gen) * 0.02).bfloat16()
        mine, theirs = p0.clone(), torch.nn.Parameter(p0.clone())
        buf = torch.zeros_like(p0)
        opt = torch.optim.Muon([theirs], lr=1e-3, weight_decay=0.1, momentum=0.95, nesterov=True)
        for _ in range(3):
            grad = torch.randn(shape, generator=gen).bfloat16()
            eager.muon_step(mine, grad, buf)
            theirs.grad = grad.clone()
            opt.step()
        assert (mine.float() - theirs.detach().float()).abs().max() <= 2e-2
        assert torch.allclose(mine.float(), theirs.detach().float(), atol=1e-4)
    assert eager.adjusted_lr(1.0, None, (7168, 2048)) == math.sqrt(3.5)
    assert eager.adjusted_lr(1.0, "match_rms_adamw", (2048, 7168)) == 0.2 * math.sqrt(7168)
    with pytest.raises(ValueError):
        eager.adjusted_lr(1.0, "nope", (2, 2))
