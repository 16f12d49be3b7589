"""GPU parity of the prequantized-weight linear forward: the 1x128 activation
quantizer (bit-exact against the oracle) and the scaled FP8 GEMM (fp32
accumulation of FP8 products, one bf16 rounding: relative 2^-7 against the
oracle's fp32 result, exact where the arithmetic is exact)."""

import pytest
import torch

from flex_shard_amd import hip_ops
from flex_shard_amd.blockwise_fp8 import BlockwiseFp8Weight, Fp8BlockwiseGemms
from oracle import eager

pytestmark = pytest.mark.gpu
E4M3 = torch.float8_e4m3fn


def _bits(t):
    return t.contiguous().view(torch.int32)


@pytest.mark.parametrize("rows,cols", [(64, 512), (1, 128), (37, 300 - 4), (200, 1024 + 136), (1000, 4096), (65, 8)])
def test_act_quant_is_bit_exact(device, rows, cols):
    gen = torch.Generator().manual_seed(rows * 7 + cols)
    x = (torch.randn(rows, cols, generator=gen) * 0.5).bfloat16()
    x[torch.rand(rows, cols, generator=gen) < 0.002] *= 60  # outliers
    if cols >= 256:
        x[rows // 2, 128:256] = 0  # an all-zero run
    x[0, 0] = 0.0
    q, s = hip_ops.act_quant_1x128(x.to(device))
    oq, os_ = eager.act_quant_1x128(x)
    assert q.shape == oq.shape and s.shape == os_.shape
    assert torch.equal(q.cpu().view(torch.uint8), oq.view(torch.uint8))
    assert torch.equal(_bits(s.cpu()), _bits(os_))


def test_act_quant_strided_rows_and_eps_switch(device):
    gen = torch.Generator().manual_seed(3)
    wide = (torch.randn(70, 640, generator=gen)).bfloat16().to(device)
    view = wide[:, 128:512]  # row stride 640, offset 128 elements
    q, s = hip_ops.act_quant_1x128(view)
    oq, os_ = eager.act_quant_1x128(view.cpu())
    assert torch.equal(q.cpu().view(torch.uint8), oq.view(torch.uint8)) and torch.equal(_bits(s.cpu()), _bits(os_))
    zeros = torch.zeros(4, 128, dtype=torch.bfloat16, device=device)
    _, s32 = hip_ops.act_quant_1x128(zeros)
    _, s16 = hip_ops.act_quant_1x128(zeros, eps_fp32=False)
    assert (_bits(s32.cpu()) == 0x2720D7C5).all() and (_bits(s16.cpu()) == 0x27212492).all()
    with pytest.raises(ValueError, match="bf16"):
        hip_ops.act_quant_1x128(zeros.float())
    with pytest.raises(RuntimeError, match="multiples of 8"):
        hip_ops.act_quant_1x128(torch.zeros(4, 100, dtype=torch.bfloat16, device=device))


def _small_int_fp8(shape, gen, high=4):
    return torch.randint(-high, high + 1, shape, generator=gen).to(torch.float32).to(E4M3)


@pytest.mark.parametrize(
    "m,n,k",
    [
        (128, 256, 128), (70, 200, 384), (300, 520, 256), (1, 8, 128), (129, 257, 1024),
        (3072, 3000, 256),  # 144 tiles on 256 CUs: more than half a round, every tile computed whole
        (4352, 4096, 128),  # 272 tiles: one round of whole tiles, the 16 left over as 32 half tiles
        (2200, 4096, 128),  # 144 tiles whose last tile row ends in its first half
    ],
)
def test_gemm_integer_products_are_exact(device, m, n, k):
    """Small integers and power-of-two scales: every product, scaled partial
    sum and running sum is exact in fp32 whatever the order, so the output is
    the one bf16 rounding of the exact result, tails and scale indexing
    included."""
    gen = torch.Generator().manual_seed(m + n + k)
    xq, wq = _small_int_fp8((m, k), gen, 1), _small_int_fp8((n, k), gen, 1)
    xs = torch.exp2(torch.randint(-2, 3, (k // 128, m), generator=gen).float())
    ws = torch.exp2(torch.randint(-2, 3, (-(-n // 128), k // 128), generator=gen).float())
    want = eager.fp8_gemm_1x128_128x128(xq, xs, wq, ws, out_dtype=torch.float32)
    pad = 512
    buf = torch.full((m * n + 2 * pad,), 7.0, dtype=torch.bfloat16, device=device)
    out = buf[pad:-pad].view(m, n)
    hip_ops.fp8_gemm_1x128_128x128(xq.to(device), xs.to(device), wq.to(device), ws.to(device), out=out)
    assert torch.equal(out.cpu(), want.bfloat16())
    assert (buf[:pad] == 7).all() and (buf[-pad:] == 7).all()


@pytest.mark.parametrize("m,n,k", [(256, 512, 512), (200, 384, 256), (1024, 1024, 4096), (77, 130, 128)])
def test_gemm_matches_the_oracle(device, m, n, k):
    gen = torch.Generator().manual_seed(m * 3 + n + k)
    x = torch.randn(m, k, generator=gen).bfloat16()
    w = (torch.randn(n, k, generator=gen) * 0.02).bfloat16()
    xq, xs = eager.act_quant_1x128(x)
    wq, ws = eager.quantize_blockwise(w, 128)
    want = eager.fp8_gemm_1x128_128x128(xq, xs, wq, ws, out_dtype=torch.float32)
    out = hip_ops.fp8_gemm_1x128_128x128(xq.to(device), xs.to(device), wq.to(device), ws.to(device))
    # one bf16 rounding (2^-8 relative) plus fp32 summation-order noise
    assert torch.allclose(out.cpu().float(), want, rtol=2.0**-7, atol=1e-3 * want.abs().max().item())


def test_forward_of_the_prequantized_linear(device):
    """Fp8BlockwiseGemms.forward: against the oracle's two steps, against the
    bf16 product, and the reference's own property: a stacked [2, F, D] weight
    gives exactly the flattened [2F, D] result (F % 128 != 0)."""
    gen = torch.Generator().manual_seed(0)
    num_linears, out_dim, in_dim = 2, 192, 256
    w = torch.randn(num_linears * out_dim, in_dim, generator=gen).bfloat16()
    wq, ws = eager.quantize_blockwise(w, 128)
    x = torch.randn(128, in_dim, generator=gen).bfloat16()
    gemms = Fp8BlockwiseGemms(block_size=128, out_dtype=torch.bfloat16)
    flat = BlockwiseFp8Weight(wq.to(device), ws.to(device), 128, orig_dtype=torch.bfloat16)
    stacked = BlockwiseFp8Weight(wq.to(device).view(num_linears, out_dim, in_dim), ws.to(device), 128, orig_dtype=torch.bfloat16)
    out_flat = gemms.forward(x.to(device), flat)
    out_stacked = gemms.forward(x.to(device), stacked)
    assert out_flat.shape == (128, num_linears * out_dim) and out_flat.dtype == torch.bfloat16
    assert torch.equal(out_flat, out_stacked)
    xq, xs = eager.act_quant_1x128(x)
    want = eager.fp8_gemm_1x128_128x128(xq, xs, wq, ws, out_dtype=torch.float32)
    assert torch.allclose(out_flat.cpu().float(), want, rtol=2.0**-7, atol=1e-3 * want.abs().max().item())
    dense = x.float() @ w.float().t()
    assert (out_flat.cpu().float() - dense).abs().max() <= 0.08 * dense.abs().max()
    # an input width that is not a whole number of runs: activation and weight are padded with zeros
    w2 = torch.randn(256, 200, generator=gen).bfloat16()
    w2q, w2s = eager.quantize_blockwise(w2, 128)
    x2 = torch.randn(40, 200, generator=gen).bfloat16()
    out2 = gemms.forward(x2.to(device), BlockwiseFp8Weight(w2q.to(device), w2s.to(device), 128))
    x2q, x2s = eager.act_quant_1x128(x2)
    w2q_padded = torch.zeros(256, 256, dtype=torch.uint8)
    w2q_padded[:, :200] = w2q.view(torch.uint8)
    want2 = eager.fp8_gemm_1x128_128x128(x2q, x2s, w2q_padded.view(E4M3), w2s, out_dtype=torch.float32)
    assert torch.allclose(out2.cpu().float(), want2, rtol=2.0**-7, atol=1e-3 * want2.abs().max().item())
    with pytest.raises(ValueError, match="block_size"):
        Fp8BlockwiseGemms(block_size=64).forward(x.to(device), flat)
    with pytest.raises(ValueError, match="input dim"):
        gemms.forward(x.to(device)[:, :128].contiguous(), flat)
    with pytest.raises(ValueError, match="block_size"):
        Fp8BlockwiseGemms(block_size=64).backward(x.to(device), x.to(device), flat, True, True)


def test_gemm_rejects_what_the_kernel_cannot_take(device):
    """k that is not a multiple of 128 fails with a message instead of launching."""
    xq = torch.zeros((8, 192), dtype=torch.uint8, device=device)
    xs = torch.ones((1, 8), dtype=torch.float32, device=device)
    wq = torch.zeros((8, 192), dtype=torch.uint8, device=device)
    ws = torch.ones((1, 1), dtype=torch.float32, device=device)
    with pytest.raises(RuntimeError, match="multiple of 128"):
        hip_ops.fp8_gemm_1x128_128x128(xq, xs, wq, ws)


def test_contraction_longer_than_one_window_of_weight_scales(device):
    """The block-scale variant keeps 256 k-tiles of weight scales in LDS and
    refills the window when the loop crosses it: k = 2 windows + 3 k-tiles,
    every weight scale different, against the oracle's product; forward and
    input-gradient (scale table read across) forms."""
    gen = torch.Generator().manual_seed(5)
    m, n, k = 96, 384, 2 * 32768 + 384
    x = torch.randn(m, k, generator=gen).bfloat16()
    w = (torch.randn(n, k, generator=gen) * 0.02).bfloat16()
    xq, xs = eager.act_quant_1x128(x)
    wq, ws = eager.quantize_blockwise(w, 128)
    ws = ws * (1.0 + torch.arange(ws.numel(), dtype=torch.float32).view(ws.shape) / ws.numel())  # no two alike
    want = eager.fp8_gemm_1x128_128x128(xq, xs, wq, ws, out_dtype=torch.float32)
    got = hip_ops.fp8_gemm_1x128_128x128(xq.to(device), xs.to(device), wq.to(device), ws.to(device))
    assert torch.allclose(got.cpu().float(), want, rtol=2.0**-7, atol=1e-3 * want.abs().max().item())
    # the same product as an input gradient: operand w as [k, n]^T with the table [k / 128, n / 128] read across
    got_t = hip_ops.fp8_gemm_1x128_128x128_dgrad(
        xq.to(device), xs.to(device), wq.to(device), ws.t().contiguous().to(device), in_dim=n
    )
    assert torch.equal(got_t, got)


def test_projections_that_share_an_activation_quantize_it_once(device):
    """q, k and v read the same activation: the second and third forward (and
    weight-gradient) products take the first one's quantization.  Same bits as
    with the sharing switched off; a changed activation (in place, or another
    tensor at another address) is quantized again."""
    from unittest.mock import patch

    from flex_shard_amd.blockwise_fp8.fp8_blockwise_linear import shared_activation_quantizer as shared

    gen = torch.Generator().manual_seed(8)
    x = torch.randn(256, 384, generator=gen).bfloat16().to(device)
    grad = (torch.randn(256, 256, generator=gen) * 0.01).bfloat16().to(device)
    weights = []
    for _ in range(3):
        wq, ws = eager.quantize_blockwise((torch.randn(256, 384, generator=gen) * 0.02).bfloat16(), 128)
        weights.append(BlockwiseFp8Weight(wq.to(device), ws.to(device), 128, orig_dtype=torch.bfloat16))
    gemms = Fp8BlockwiseGemms(block_size=128)

    def run():
        outs = [gemms.forward(x, w) for w in weights]
        grads = [gemms.backward(grad, x, w, True, True) for w in weights]
        return outs, grads

    shared.clear()
    calls = {"rows": 0, "tokens": 0}
    real_rows, real_tokens = hip_ops.act_quant_1x128, hip_ops.act_quant_128x1_transposed

    def count_rows(t, **kw):
        calls["rows"] += 1
        return real_rows(t, **kw)

    def count_tokens(t, **kw):
        calls["tokens"] += 1
        return real_tokens(t, **kw)

    with patch.object(hip_ops, "act_quant_1x128", count_rows), patch.object(hip_ops, "act_quant_128x1_transposed", count_tokens):
        outs, grads = run()
        assert calls == {"rows": 1, "tokens": 1}  # x once per form (the output gradient goes through act_quant_both)
        x.mul_(2.0)  # in place: the version counter moves
        outs2, _ = run()
        assert calls == {"rows": 2, "tokens": 2}
        moved = x.clone()
        gemms.forward(moved, weights[0])
        assert calls["rows"] == 3
    shared.enabled = False
    try:
        plain_outs, plain_grads = run()
    finally:
        shared.enabled = True
        shared.clear()
    for a, b in zip(outs2, plain_outs):
        assert torch.equal(a, b)
    assert not torch.equal(outs[0], outs2[0])
    x.div_(2.0)
    again_outs, again_grads = run()
    for (gx, gw), (px, pw) in zip(again_grads, grads):
        assert torch.equal(gx, px) and torch.equal(gw, pw)


def test_products_whose_output_passes_two_to_the_32_bytes(device):
    """65 536 tokens x 32 768 outputs (4.3 GB of bf16), a short contraction:
    the corners of the forward product and of the weight-gradient product
    with small-integer operands and power-of-two scales, where every order of
    summation gives the same bits, against the eager restatement on the host."""
    gen = torch.Generator().manual_seed(41)
    m, n, k = 65536, 32768, 128
    ints = lambda shape, high: torch.randint(-high, high + 1, shape, generator=gen).float().to(torch.float8_e4m3fn)
    pow2 = lambda shape: torch.exp2(torch.randint(-2, 3, shape, generator=gen).float())
    xq, wq, xs, ws = ints((m, k), 1), ints((n, k), 1), pow2((1, m)), pow2((n // 128, 1))
    got = hip_ops.fp8_gemm_1x128_128x128(xq.to(device), xs.to(device), wq.to(device), ws.to(device))
    assert got.numel() * got.element_size() >= 2**32
    for rows, cols in ((slice(0, 300), slice(0, 384)), (slice(m - 300, m), slice(n - 384, n)), (slice(0, 130), slice(n - 128, n))):
        blocks = slice(cols.start // 128, cols.stop // 128)  # the selected output columns are whole scale blocks
        want = eager.fp8_gemm_1x128_128x128(xq[rows], xs[:, rows], wq[cols], ws[blocks], out_dtype=torch.float32)
        assert torch.equal(got[rows, cols].cpu(), want.bfloat16())
    del got
    # weight gradient [n, m2] over 128 tokens: outputs beyond 2^32 bytes as well
    m2 = 65536
    aq, bq, a_s, b_s = ints((n, k), 2), ints((m2, k), 2), pow2((1, n)), pow2((1, m2))
    got = hip_ops.fp8_gemm_1x128_128x1(aq.to(device), a_s.to(device), bq.to(device), b_s.to(device))
    assert tuple(got.shape) == (n, m2)
    for rows, cols in ((slice(0, 300), slice(0, 300)), (slice(n - 300, n), slice(m2 - 300, m2))):
        want = eager.fp8_gemm_1x128_128x1(aq[rows], a_s[:, rows], bq[cols], b_s[:, cols], out_dtype=torch.float32)
        assert torch.equal(got[rows, cols].cpu(), want.bfloat16())

