"""Pins of the oracle's activation quantizer (1x128 runs) and scaled FP8 GEMM.

Both restate kernels of torchao (absent here), so they are pinned through what
is already pinned and through closed forms: a run is a one-row tile of the
tile quantizer; constant and zero runs have known bytes and scales; with unit
scales and small integers the GEMM is an exact integer product; a single
non-unit scale moves exactly the contributions of its k-block and row (or
column block).
"""

import torch

from oracle import cport, eager

E4M3 = torch.float8_e4m3fn


def bits32(t: torch.Tensor) -> torch.Tensor:
    return t.contiguous().view(torch.int32)


def test_a_run_is_a_one_row_tile_of_the_tile_quantizer():
    gen = torch.Generator().manual_seed(5)
    x = (torch.randn(37, 300, generator=gen) * 0.02).bfloat16()
    x[3, 128:256] = 0  # an all-zero run
    x[5, 17] = 3.0  # an outlier
    q, s = eager.act_quant_1x128(x)
    assert q.shape == (37, 384) and s.shape == (3, 37)
    assert (q[:, 300:].view(torch.uint8) == 0).all()
    padded = torch.zeros(37, 384)
    padded[:, :300] = x.float()
    for row in (0, 3, 5, 36):
        for run in range(3):
            # the run alone in a 128x128 tile (rows 1..127 zero), through the C tile quantizer in fp32
            tile = torch.zeros(128, 128)
            tile[0] = padded[row, run * 128 : (run + 1) * 128]
            tq, ts = cport.quantize_blockwise(tile, 128)
            assert torch.equal(tq[0].view(torch.uint8), q[row, run * 128 : (run + 1) * 128].view(torch.uint8))
            assert bits32(ts)[0, 0] == bits32(s)[run, row]


def test_constant_and_zero_runs_closed_form():
    x = torch.full((2, 256), 0.375).bfloat16()
    x[1, :128] = -0.375
    x[1, 128:] = 0
    q, s = eager.act_quant_1x128(x)
    assert (q[0].view(torch.uint8) == 0x7E).all() and (q[1, :128].view(torch.uint8) == 0xFE).all()
    want = 1.0 / torch.tensor(448.0 / 0.375, dtype=torch.float64).to(torch.float32)
    assert bits32(s[:, 0])[0] == bits32(want.reshape(1))[0] and bits32(s[0, 1:2])[0] == bits32(want.reshape(1))[0]
    assert (q[1, 128:].view(torch.uint8) == 0).all()
    assert bits32(s[1, 1:2])[0].item() == 0x2720D7C5  # 1 / fp32(448 / fp32(1e-12))


def _small_int_fp8(shape, gen, high=4):
    return torch.randint(-high, high + 1, shape, generator=gen).to(torch.float32).to(E4M3)


def test_gemm_with_unit_scales_is_the_integer_product():
    gen = torch.Generator().manual_seed(9)
    xq, wq = _small_int_fp8((70, 384), gen), _small_int_fp8((200, 384), gen)
    xs, ws = torch.ones(3, 70), torch.ones(2, 3)
    out = eager.fp8_gemm_1x128_128x128(xq, xs, wq, ws, out_dtype=torch.float32)
    assert torch.equal(out, (xq.float().long() @ wq.float().long().t()).float())


def test_one_scale_moves_exactly_its_block():
    gen = torch.Generator().manual_seed(10)
    xq, wq = _small_int_fp8((20, 256), gen), _small_int_fp8((260, 256), gen)
    per_block = [xq[:, kb * 128 : (kb + 1) * 128].float() @ wq[:, kb * 128 : (kb + 1) * 128].float().t() for kb in (0, 1)]
    xs, ws = torch.ones(2, 20), torch.ones(3, 2)
    xs[1, 7] = 2.0  # activation row 7, k-block 1
    ws[2, 0] = 0.5  # weight rows 256.., k-block 0
    out = eager.fp8_gemm_1x128_128x128(xq, xs, wq, ws, out_dtype=torch.float32)
    want = per_block[0] + per_block[1]
    want[7] += per_block[1][7]
    want[:, 256:] -= 0.5 * per_block[0][:, 256:]
    assert torch.equal(out, want)


def test_gemm_equals_the_product_of_the_dequantized_operands():
    gen = torch.Generator().manual_seed(11)
    x = (torch.randn(48, 512, generator=gen)).bfloat16()
    w = (torch.randn(300, 512, generator=gen) * 0.02).bfloat16()
    xq, xs = eager.act_quant_1x128(x)
    wq, ws = eager.quantize_blockwise(w, 128)
    out = eager.fp8_gemm_1x128_128x128(xq, xs, wq, ws, out_dtype=torch.float32)
    x_deq = xq.double() * xs.t().double().repeat_interleave(128, dim=1)
    w_deq = eager.dequant_blockwise(wq, ws, 128, torch.float64)
    exact = x_deq @ w_deq.t()
    assert torch.allclose(out.double(), exact, rtol=1e-5, atol=1e-6)
    # and the quantized product is close to the bf16 one (FP8 has 3 mantissa bits)
    dense = x.double() @ w.double().t()
    assert (out.double() - dense).abs().max() <= 0.08 * dense.abs().max()


# ---------------------------------------------------------------- backward
def test_token_run_quantizer_is_the_row_run_quantizer_of_the_transpose():
    gen = torch.Generator().manual_seed(21)
    x = (torch.randn(300, 40, generator=gen) * 0.3).bfloat16()
    x[128:256, 3] = 0  # an all-zero run
    x[17, 5] = 40.0
    q, s = eager.act_quant_128x1_transposed(x)
    q2, s2 = eager.act_quant_1x128(x.t().contiguous())
    assert q.shape == (40, 384) and s.shape == (3, 40)
    assert torch.equal(q.view(torch.uint8), q2.view(torch.uint8))
    assert torch.equal(bits32(s), bits32(s2))
    assert (q[:, 300:].view(torch.uint8) == 0).all()


def test_a_token_run_is_a_one_column_tile_of_the_tile_quantizer():
    gen = torch.Generator().manual_seed(22)
    x = (torch.randn(200, 9, generator=gen) * 0.02).bfloat16()
    q, s = eager.act_quant_128x1_transposed(x)
    for col in (0, 4, 8):
        tq, ts = cport.quantize_blockwise(x[:, col : col + 1].float().contiguous(), 128)  # tiles of 128 x 1
        assert torch.equal(tq[:, 0].view(torch.uint8), q[col, :200].view(torch.uint8))
        assert torch.equal(bits32(ts)[:, 0], bits32(s)[:, col])


def test_column_scaled_gemm_closed_forms():
    gen = torch.Generator().manual_seed(23)
    aq, bq = _small_int_fp8((50, 256), gen), _small_int_fp8((70, 256), gen)
    per_block = [aq[:, kb * 128 : (kb + 1) * 128].float() @ bq[:, kb * 128 : (kb + 1) * 128].float().t() for kb in (0, 1)]
    a_s, b_s = torch.ones(2, 50), torch.ones(2, 70)
    assert torch.equal(eager.fp8_gemm_1x128_128x1(aq, a_s, bq, b_s, out_dtype=torch.float32), per_block[0] + per_block[1])
    a_s[0, 9] = 4.0  # row 9, k-block 0
    b_s[1, 33] = 0.25  # column 33, k-block 1
    want = per_block[0] + per_block[1]
    want[9] += 3.0 * per_block[0][9]
    want[:, 33] -= 0.75 * per_block[1][:, 33]
    assert torch.equal(eager.fp8_gemm_1x128_128x1(aq, a_s, bq, b_s, out_dtype=torch.float32), want)
    # column scales that are constant over a 128-column block are the tile-scaled product
    aq, bq = _small_int_fp8((20, 256), gen), _small_int_fp8((260, 256), gen)
    a_s = torch.rand(2, 20, generator=gen) + 0.5
    ws = torch.rand(3, 2, generator=gen) + 0.5
    b_s = ws.t()[:, torch.arange(260) // 128].contiguous()
    assert torch.equal(
        eager.fp8_gemm_1x128_128x1(aq, a_s, bq, b_s, out_dtype=torch.float32),
        eager.fp8_gemm_1x128_128x128(aq, a_s, bq, ws, out_dtype=torch.float32),
    )


def test_backward_equals_the_products_of_the_dequantized_operands():
    """Every scale meets the bytes it was computed from, in both products: the
    results equal fp64 products of the dequantized operands, and are close to
    the unquantized gradients (a transposed or mis-indexed operand fails both)."""
    gen = torch.Generator().manual_seed(24)
    tokens, out_dim, in_dim = 150, 200, 136
    weight = (torch.randn(out_dim, in_dim, generator=gen) * 0.05).bfloat16()
    x = torch.randn(tokens, in_dim, generator=gen).bfloat16()
    grad_out = (torch.randn(tokens, out_dim, generator=gen) * 0.01).bfloat16()
    wq, ws = eager.quantize_blockwise(weight, 128)
    grad_x, grad_w = eager.fp8_linear_backward(grad_out, x, wq, ws, out_dtype=torch.float32)
    assert grad_x.shape == (tokens, in_dim) and grad_w.shape == (out_dim, in_dim)

    w_deq = eager.dequant_blockwise(wq, ws, 128, out_dtype=torch.float64)
    gq, gs = eager.act_quant_1x128(grad_out)
    g_deq = (gq.double().view(tokens, 2, 128) * gs.t().double()[:, :, None]).view(tokens, 256)[:, :out_dim]
    want_x = g_deq @ w_deq
    assert torch.allclose(grad_x.double(), want_x, rtol=1e-5, atol=1e-6 * want_x.abs().max().item())

    gtq, gts = eager.act_quant_128x1_transposed(grad_out)  # [out, 256], [2, out]
    xtq, xts = eager.act_quant_128x1_transposed(x)
    gt_deq = gtq.double().view(out_dim, 2, 128) * gts.t().double()[:, :, None]
    xt_deq = xtq.double().view(in_dim, 2, 128) * xts.t().double()[:, :, None]
    want_w = gt_deq.view(out_dim, 256) @ xt_deq.view(in_dim, 256).t()
    assert torch.allclose(grad_w.double(), want_w, rtol=1e-5, atol=1e-6 * want_w.abs().max().item())

    exact_x = grad_out.double() @ weight.double()
    exact_w = grad_out.double().t() @ x.double()
    assert (grad_x.double() - exact_x).norm() <= 0.06 * exact_x.norm()
    assert (grad_w.double() - exact_w).norm() <= 0.06 * exact_w.norm()
