"""GPU parity of the backward products of the prequantized-weight linear: the
byte transpose and the token-run quantizer are bit-exact against the oracle,
the two scaled FP8 GEMMs are within one bf16 rounding plus summation-order
noise of the oracle's fp32 result (relative 2^-7) and exact where the
arithmetic is exact."""

import pytest
import torch

from flex_shard_amd import hip_ops
from flex_shard_amd.blockwise_fp8 import (
    BlockwiseFp8Weight,
    FlexShardFloat8BlockwiseLinear,
    Fp8BlockwiseGemms,
    prequantized_linear,
)
from oracle import eager

pytestmark = pytest.mark.gpu
E4M3 = torch.float8_e4m3fn
RTOL = 2.0**-7


def _bits(t):
    return t.contiguous().view(torch.int32)


def _close(got, want):
    return torch.allclose(got.cpu().float(), want, rtol=RTOL, atol=1e-3 * want.abs().max().item())


def _small_int_fp8(shape, gen, high=1):
    return torch.randint(-high, high + 1, shape, generator=gen).to(torch.float32).to(E4M3)


@pytest.mark.parametrize("rows,cols", [(128, 128), (384, 256), (130, 144), (1, 16), (500, 1040), (4096, 1024)])
def test_transpose_is_exact(device, rows, cols):
    gen = torch.Generator().manual_seed(rows + cols)
    src = torch.randint(0, 256, (rows, cols), generator=gen, dtype=torch.uint8)
    got = hip_ops.fp8_transpose(src.to(device)).cpu()
    padded = -(-rows // 128) * 128
    assert got.shape == (cols, padded)
    assert torch.equal(got[:, :rows], src.t())
    assert (got[:, rows:] == 0).all()


def test_transpose_of_a_strided_view_and_errors(device):
    gen = torch.Generator().manual_seed(1)
    wide = torch.randint(0, 256, (200, 512), generator=gen, dtype=torch.uint8).to(device)
    view = wide[:, 64:320].view(E4M3)
    got = hip_ops.fp8_transpose(view)
    assert got.dtype == E4M3 and torch.equal(got.view(torch.uint8)[:, :200].cpu(), wide[:, 64:320].t().cpu())
    with pytest.raises(RuntimeError, match="multiples of 16"):
        hip_ops.fp8_transpose(wide[:, :40])
    with pytest.raises(ValueError, match="contiguous rows"):
        hip_ops.fp8_transpose(wide.t())
    assert hip_ops.fp8_transpose(wide[:0]).shape == (512, 0)


@pytest.mark.parametrize("rows,cols", [(128, 128), (256, 384), (130, 136), (77, 8), (1000, 520), (4096, 256), (1, 128)])
def test_token_run_quantizer_is_bit_exact(device, rows, cols):
    gen = torch.Generator().manual_seed(rows * 5 + cols)
    x = (torch.randn(rows, cols, generator=gen) * 0.5).bfloat16()
    x[torch.rand(rows, cols, generator=gen) < 0.002] *= 60  # outliers
    if rows >= 256:
        x[128:256, cols // 2] = 0  # an all-zero run
    x[0, 0] = 0.0
    x[rows - 1, cols - 1] = 3.0e38  # the largest magnitudes saturate nothing: amax scales them to 448
    x[rows // 2, 1] = 1e-40  # a subnormal input
    q, s = hip_ops.act_quant_128x1_transposed(x.to(device))
    oq, os_ = eager.act_quant_128x1_transposed(x)
    assert q.shape == oq.shape and s.shape == os_.shape
    assert torch.equal(q.cpu().view(torch.uint8), oq.view(torch.uint8))
    assert torch.equal(_bits(s.cpu()), _bits(os_))


@pytest.mark.parametrize("rows,cols", [(128, 128), (256, 384), (130, 136), (77, 8), (1000, 520), (4096, 256), (1, 128)])
def test_both_forms_in_one_pass_equal_the_two_quantizers(device, rows, cols):
    """One read of the matrix, both outputs: bit for bit what the row-run and
    the token-run quantizer write on their own (pads included), and the
    oracle's bytes."""
    gen = torch.Generator().manual_seed(rows * 7 + cols)
    x = (torch.randn(rows, cols, generator=gen) * 0.5).bfloat16()
    x[torch.rand(rows, cols, generator=gen) < 0.002] *= 60
    if rows >= 256:
        x[128:256, cols // 2] = 0
        x[3, :] = 0  # an all-zero row run
    x[rows - 1, cols - 1] = 3.0e38
    xd = x.to(device)
    q_rows, s_rows, q_cols, s_cols = hip_ops.act_quant_both(xd)
    want_q_rows, want_s_rows = hip_ops.act_quant_1x128(xd)
    want_q_cols, want_s_cols = hip_ops.act_quant_128x1_transposed(xd)
    for got, want in ((q_rows, want_q_rows), (q_cols, want_q_cols)):
        assert got.shape == want.shape and torch.equal(got.view(torch.uint8), want.view(torch.uint8))
    for got, want in ((s_rows, want_s_rows), (s_cols, want_s_cols)):
        assert got.shape == want.shape and torch.equal(_bits(got.cpu()), _bits(want.cpu()))
    oq, os_ = eager.act_quant_1x128(x)
    assert torch.equal(q_rows.cpu().view(torch.uint8), oq.view(torch.uint8)) and torch.equal(_bits(s_rows.cpu()), _bits(os_))
    # strided rows and the bf16-rounded floor
    wide = torch.randn(300, 640, generator=gen).bfloat16().to(device)
    view = wide[:, 128:512]
    a = hip_ops.act_quant_both(view, eps_fp32=False)
    b = hip_ops.act_quant_1x128(view, eps_fp32=False) + hip_ops.act_quant_128x1_transposed(view, eps_fp32=False)
    assert all(torch.equal(u.view(torch.uint8) if u.dtype != torch.float32 else u, v.view(torch.uint8) if v.dtype != torch.float32 else v)
               for u, v in zip(a, b))


def test_token_run_quantizer_strided_rows_and_eps_switch(device):
    gen = torch.Generator().manual_seed(4)
    wide = torch.randn(300, 640, generator=gen).bfloat16().to(device)
    view = wide[:, 128:512]
    q, s = hip_ops.act_quant_128x1_transposed(view)
    oq, os_ = eager.act_quant_128x1_transposed(view.cpu())
    assert torch.equal(q.cpu().view(torch.uint8), oq.view(torch.uint8)) and torch.equal(_bits(s.cpu()), _bits(os_))
    zeros = torch.zeros(128, 8, dtype=torch.bfloat16, device=device)
    _, s32 = hip_ops.act_quant_128x1_transposed(zeros)
    _, s16 = hip_ops.act_quant_128x1_transposed(zeros, eps_fp32=False)
    assert (_bits(s32.cpu()) == 0x2720D7C5).all() and (_bits(s16.cpu()) == 0x27212492).all()
    with pytest.raises(RuntimeError, match="multiples of 8"):
        hip_ops.act_quant_128x1_transposed(torch.zeros(128, 12, dtype=torch.bfloat16, device=device))


@pytest.mark.parametrize(
    "m,n,k",
    [
        (128, 256, 128), (70, 200, 384), (300, 520, 256), (1, 8, 128), (129, 257, 1024),
        (128, 256, 32768 + 128),  # more tokens than the block-scale variant's k limit: this variant takes any length
    ],
)
def test_column_scaled_gemm_integer_products_are_exact(device, m, n, k):
    gen = torch.Generator().manual_seed(m + n + k + 1)
    aq, bq = _small_int_fp8((m, k), gen), _small_int_fp8((n, k), gen)
    a_s = torch.exp2(torch.randint(-2, 3, (k // 128, m), generator=gen).float())
    b_s = torch.exp2(torch.randint(-2, 3, (k // 128, n), generator=gen).float())
    want = eager.fp8_gemm_1x128_128x1(aq, a_s, bq, b_s, out_dtype=torch.float32)
    got = hip_ops.fp8_gemm_1x128_128x1(aq.to(device), a_s.to(device), bq.to(device), b_s.to(device))
    assert torch.equal(got.cpu(), want.bfloat16())


@pytest.mark.parametrize(
    "m,n,k",
    [
        (256, 512, 512), (200, 384, 256), (1024, 1032, 2048), (77, 130, 128),
        (3072, 3000, 256),  # 144 tiles on 256 CUs: more than half a round, every tile computed whole
        (4352, 4096, 128),  # 272 tiles: one round of whole tiles, the 16 left over as 32 half tiles
        (2200, 4096, 128),  # 144 tiles whose last tile row ends in its first half
    ],
)
def test_column_scaled_gemm_matches_the_oracle(device, m, n, k):
    gen = torch.Generator().manual_seed(m * 3 + n + k + 1)
    a = torch.randn(k, m, generator=gen).bfloat16()
    b = (torch.randn(k, n, generator=gen) * 0.02).bfloat16()
    aq, a_s = eager.act_quant_128x1_transposed(a)
    bq, b_s = eager.act_quant_128x1_transposed(b)
    want = eager.fp8_gemm_1x128_128x1(aq, a_s, bq, b_s, out_dtype=torch.float32)
    got = hip_ops.fp8_gemm_1x128_128x1(aq.to(device), a_s.to(device), bq.to(device), b_s.to(device))
    assert _close(got, want)


@pytest.mark.parametrize("tokens,out_dim,in_dim", [(128, 256, 256), (70, 384, 200), (300, 128, 520), (1000, 1024, 1024)])
def test_input_gradient_product(device, tokens, out_dim, in_dim):
    """Against the oracle, and bit for bit against the forward kernel fed with
    explicitly transposed copies of the weight bytes AND scales (the kernel
    reads the scale table across instead)."""
    gen = torch.Generator().manual_seed(tokens + out_dim + in_dim)
    w = (torch.randn(out_dim, in_dim, generator=gen) * 0.05).bfloat16()
    g = (torch.randn(tokens, out_dim, generator=gen) * 0.01).bfloat16()
    wq, ws = eager.quantize_blockwise(w, 128)
    gq, gs = eager.act_quant_1x128(g)
    in_pad = -(-in_dim // 16) * 16
    wq_dev = torch.zeros(out_dim, in_pad, dtype=torch.uint8, device=device)
    wq_dev[:, :in_dim] = wq.view(torch.uint8).to(device)
    wt = hip_ops.fp8_transpose(wq_dev.view(E4M3))
    got = hip_ops.fp8_gemm_1x128_128x128_dgrad(gq.to(device), gs.to(device), wt, ws.to(device), in_dim=in_dim)
    assert got.shape == (tokens, in_dim)
    want = eager.fp8_gemm_1x128_128x128(gq, gs, wq.t().contiguous(), ws.t().contiguous(), out_dtype=torch.float32)
    assert _close(got, want)
    same = hip_ops.fp8_gemm_1x128_128x128(gq.to(device), gs.to(device), wt[:in_dim], ws.t().contiguous().to(device))
    assert torch.equal(got, same)


def _case(gen, tokens, out_shape, in_dim, device):
    out_dim = 1
    for extent in out_shape:
        out_dim *= extent
    w = (torch.randn(out_dim, in_dim, generator=gen) * 0.05).bfloat16()
    x = torch.randn(tokens, in_dim, generator=gen).bfloat16()
    g = (torch.randn(tokens, out_dim, generator=gen) * 0.01).bfloat16()
    wq, ws = eager.quantize_blockwise(w, 128)
    weight = BlockwiseFp8Weight(wq.to(device).view(*out_shape, in_dim), ws.to(device), 128, orig_dtype=torch.bfloat16)
    return w, x, g, wq, ws, weight


@pytest.mark.parametrize(
    "tokens,out_shape,in_dim", [(256, (256,), 384), (77, (200,), 136), (150, (2, 192), 256), (130, (72,), 100)]
)
def test_backward_of_the_prequantized_linear(device, tokens, out_shape, in_dim):
    """Fp8BlockwiseGemms.backward against the oracle's restatement of the
    reference's steps and, loosely, against the unquantized gradients; odd
    token counts and widths exercise every padding branch, the stacked weight
    returns a gradient of the parameter's shape."""
    gen = torch.Generator().manual_seed(tokens * 3 + in_dim)
    w, x, g, wq, ws, weight = _case(gen, tokens, out_shape, in_dim, device)
    gemms = Fp8BlockwiseGemms(block_size=128)
    grad_x, grad_w = gemms.backward(g.to(device), x.to(device), weight, True, True)
    want_x, want_w = eager.fp8_linear_backward(g, x, wq, ws, out_dtype=torch.float32)
    assert grad_x.shape == x.shape and grad_x.dtype == torch.bfloat16
    assert grad_w.shape == weight.shape and grad_w.dtype == torch.bfloat16 and grad_w.is_contiguous()
    assert _close(grad_x, want_x)
    assert _close(grad_w.view(w.shape), want_w)
    exact_x, exact_w = g.double() @ w.double(), g.double().t() @ x.double()
    assert (grad_x.cpu().double() - exact_x).norm() <= 0.06 * exact_x.norm()
    assert (grad_w.view(w.shape).cpu().double() - exact_w).norm() <= 0.06 * exact_w.norm()
    only_x = gemms.backward(g.to(device), x.to(device), weight, True, False)
    only_w = gemms.backward(g.to(device), x.to(device), weight, False, True)
    assert only_x[1] is None and only_w[0] is None
    assert torch.equal(only_x[0], grad_x) and torch.equal(only_w[1], grad_w)
    with pytest.raises(ValueError, match="grad_output"):
        gemms.backward(g.to(device)[:, :8], x.to(device), weight, True, True)
    with pytest.raises(ValueError, match="activation"):
        gemms.backward(g.to(device), x.to(device)[:-1], weight, True, True)


def test_autograd_through_the_prequantized_linear(device):
    gen = torch.Generator().manual_seed(11)
    w, x, g, wq, ws, _ = _case(gen, 96, (256,), 128, device)
    weight = BlockwiseFp8Weight(wq.to(device), ws.to(device), 128, orig_dtype=torch.bfloat16, requires_grad=True)
    bias = torch.randn(256, generator=gen).bfloat16().to(device).requires_grad_()
    x_dev = x.to(device).view(4, 24, 128).requires_grad_()
    out = prequantized_linear(x_dev, weight, bias)
    assert out.shape == (4, 24, 256)
    out.backward(g.to(device).view(4, 24, 256))
    gemms = Fp8BlockwiseGemms(block_size=128)
    want_x, want_w = gemms.backward(g.to(device), x.to(device), weight.detach(), True, True)
    assert torch.equal(x_dev.grad.view(96, 128), want_x)
    assert torch.equal(weight.grad, want_w)
    assert torch.equal(bias.grad, g.to(device).sum(dim=0))
    plain = gemms.forward(x.to(device), weight.detach())
    assert torch.equal(out.detach().view(96, 256), plain + bias.detach())

    linear = torch.nn.Linear(128, 256, bias=False, device=device, dtype=torch.bfloat16)
    module = FlexShardFloat8BlockwiseLinear.from_float(linear)
    with pytest.raises(TypeError, match="BlockwiseFp8Weight"):
        module(x.to(device))
    module._parameters["weight"] = weight  # what an FP8 unshard installs for the span of a forward/backward
    assert torch.equal(module(x.to(device)).detach(), plain)



@pytest.mark.parametrize("tokens,in_dim", [(96, 128), (77, 100), (300, 392)])
def test_weight_gradient_from_the_forward_pass_token_runs(device, tokens, in_dim):
    """With a weight gradient to come the forward quantizes the activation in
    both forms at once and keeps the token-run form instead of the activation:
    the gradients are bit for bit those of a backward that is handed the
    activation, for ragged token counts and widths too; without a weight
    gradient, and with a GEMM object that has only the reference's two methods,
    the activation is kept as before."""
    gen = torch.Generator().manual_seed(tokens + in_dim)
    w, x, g, wq, ws, _ = _case(gen, tokens, (256,), in_dim, device)
    gemms = Fp8BlockwiseGemms(block_size=128)

    def run(requires_grad, gemms_object):
        weight = BlockwiseFp8Weight(wq.to(device), ws.to(device), 128, orig_dtype=torch.bfloat16, requires_grad=requires_grad)
        x_dev = x.to(device).clone().requires_grad_()
        out = prequantized_linear(x_dev, weight, None, gemms_object)
        saved = [t for t in out.grad_fn.saved_tensors if t is not None]
        out.backward(g.to(device))
        return out.detach(), x_dev.grad, weight.grad, saved

    want_x, want_w = gemms.backward(g.to(device), x.to(device), BlockwiseFp8Weight(wq.to(device), ws.to(device), 128, orig_dtype=torch.bfloat16), True, True)
    out, grad_x, grad_w, saved = run(True, gemms)
    assert torch.equal(grad_x, want_x) and torch.equal(grad_w, want_w)
    assert not any(t.dtype == torch.bfloat16 and t.shape == x.shape for t in saved)  # x itself is not kept
    padded_in, padded_tokens = -(-in_dim // 8) * 8, -(-tokens // 128) * 128
    assert any(t.dtype == E4M3 and tuple(t.shape) == (padded_in, padded_tokens) for t in saved)
    out2, grad_x2, grad_w2, saved2 = run(False, gemms)
    assert torch.equal(out2, out) and torch.equal(grad_x2, want_x) and grad_w2 is None
    assert any(t.shape == x.shape and t.dtype == torch.bfloat16 for t in saved2)

    class ReferenceInterfaceOnly:
        block_size = 128
        forward = staticmethod(gemms.forward)
        backward = staticmethod(gemms.backward)

    out3, grad_x3, grad_w3, saved3 = run(True, ReferenceInterfaceOnly())
    assert torch.equal(out3, out) and torch.equal(grad_x3, want_x) and torch.equal(grad_w3, want_w)
    assert any(t.shape == x.shape and t.dtype == torch.bfloat16 for t in saved3)
    with pytest.raises(ValueError, match="x_token_runs"):
        gemms.backward(g.to(device), None, BlockwiseFp8Weight(wq.to(device), ws.to(device), 128, orig_dtype=torch.bfloat16),
                       True, True, x_token_runs=(torch.empty(8, 128, dtype=E4M3, device=device), torch.empty(1, 8, device=device)))
    with pytest.raises(ValueError, match="token-run form"):
        gemms.backward(g.to(device), None, BlockwiseFp8Weight(wq.to(device), ws.to(device), 128, orig_dtype=torch.bfloat16), True, True)



def test_strided_output_gradient_is_read_in_place(device):
    """The gradient of an output that was concatenated with another tensor is
    a column slice of a wider matrix (row stride 2 x its width): the backward
    reads it as it lies and gives the bits of the contiguous copy."""
    gen = torch.Generator().manual_seed(21)
    w, x, g, wq, ws, _ = _case(gen, 200, (256,), 384, device)
    weight = BlockwiseFp8Weight(wq.to(device), ws.to(device), 128, orig_dtype=torch.bfloat16, requires_grad=True)
    x_dev = x.to(device).requires_grad_()
    out = prequantized_linear(x_dev, weight)
    other = torch.zeros_like(out).requires_grad_()
    wide_grad = torch.randn(200, 512, generator=gen).bfloat16().to(device) * 0.01
    seen = []
    out.register_hook(lambda grad: seen.append((grad.stride(), grad.is_contiguous())))
    torch.cat([other, out], dim=-1).backward(wide_grad)
    assert seen == [((512, 1), False)]
    want_x, want_w = Fp8BlockwiseGemms(block_size=128).backward(
        wide_grad[:, 256:].contiguous(), x.to(device), weight.detach(), True, True
    )
    assert torch.equal(x_dev.grad, want_x) and torch.equal(weight.grad, want_w)


def test_llama_sized_gradients_on_sampled_entries(device):
    """At the size the measurements quote (8192 tokens, a [4096, 14336]
    weight gradient and its input gradient) a sample of output entries is
    checked against fp64 dot products of the dequantized operands."""
    gen = torch.Generator(device=device).manual_seed(5)
    tokens, out_dim, in_dim = 8192, 4096, 14336
    x = torch.randn(tokens, in_dim, generator=gen, device=device, dtype=torch.float32).bfloat16()
    g = (torch.randn(tokens, out_dim, generator=gen, device=device, dtype=torch.float32) * 0.01).bfloat16()
    wq = torch.randint(0, 256, (out_dim, in_dim), generator=gen, device=device, dtype=torch.uint8)
    wq[(wq & 0x7F) == 0x7F] = 0x3C  # no NaN encodings
    ws = torch.rand(out_dim // 128, in_dim // 128, generator=gen, device=device) * 1e-3 + 1e-4
    weight = BlockwiseFp8Weight(wq.view(E4M3), ws, 128, orig_dtype=torch.bfloat16)
    grad_x, grad_w = Fp8BlockwiseGemms(block_size=128).backward(g, x, weight, True, True)

    gq, gs = hip_ops.act_quant_1x128(g)
    gtq, gts = hip_ops.act_quant_128x1_transposed(g)
    xtq, xts = hip_ops.act_quant_128x1_transposed(x)
    cpu_gen = torch.Generator().manual_seed(6)
    rows = torch.randint(0, tokens, (64,), generator=cpu_gen).tolist()
    cols = torch.randint(0, in_dim, (64,), generator=cpu_gen).tolist()
    outs = torch.randint(0, out_dim, (64,), generator=cpu_gen).tolist()
    for t, i, o in zip(rows, cols, outs):
        # grad_x[t, i] = sum_o deq(g)[t, o] * deq(w)[o, i]
        g_row = (gq[t].double().view(-1, 128) * gs[:, t].double()[:, None]).view(-1)
        w_col = wq.view(E4M3)[:, i].double() * ws[:, i // 128].double().repeat_interleave(128)
        want = float(g_row @ w_col)
        scale = float(g_row.abs() @ w_col.abs())
        assert abs(float(grad_x[t, i]) - want) <= RTOL * abs(want) + 1e-5 * scale
        # grad_w[o, i] = sum_t deq(g^T)[o, t] * deq(x^T)[i, t]
        g_col = (gtq[o].double().view(-1, 128) * gts[:, o].double()[:, None]).view(-1)
        x_col = (xtq[i].double().view(-1, 128) * xts[:, i].double()[:, None]).view(-1)
        want = float(g_col @ x_col)
        scale = float(g_col.abs() @ x_col.abs())
        assert abs(float(grad_w[o, i]) - want) <= RTOL * abs(want) + 1e-5 * scale


def test_quantizers_and_transpose_on_a_matrix_beyond_two_to_the_32_bytes(device):
    """[65536, 32768] bf16 (4.3 GB): both quantizers, the one-pass form of both
    and the byte transpose, whose input and output offsets pass 2^31 elements;
    corners against the eager restatement on the host."""
    rows, cols = 65536, 32768
    x = torch.empty((rows, cols), device=device, dtype=torch.bfloat16)
    x[:512].normal_()
    x[512:] = x[:512].repeat(rows // 512 - 1, 1)
    x[-384:].normal_()
    q, s = hip_ops.act_quant_1x128(x)
    qt, st = hip_ops.act_quant_128x1_transposed(x)
    both = hip_ops.act_quant_both(x)
    for a, b in zip(both, (q, s, qt, st)):
        assert torch.equal(a.view(torch.uint8) if a.dtype != torch.float32 else a.view(torch.int32),
                           b.view(torch.uint8) if b.dtype != torch.float32 else b.view(torch.int32))
    del both
    for r, c in ((slice(0, 256), slice(0, 256)), (slice(rows - 256, rows), slice(cols - 256, cols))):
        corner = x[r, c].cpu()
        wq, ws = eager.act_quant_1x128(corner)
        assert torch.equal(q[r, c].cpu().view(torch.uint8), wq.view(torch.uint8))
        assert torch.equal(s[c.start // 128 : c.stop // 128, r].cpu().view(torch.int32), ws.view(torch.int32))
        wqt, wst = eager.act_quant_128x1_transposed(corner)
        assert torch.equal(qt[c, r].cpu().view(torch.uint8), wqt.view(torch.uint8))
        assert torch.equal(st[r.start // 128 : r.stop // 128, c].cpu().view(torch.int32), wst.view(torch.int32))
    t = hip_ops.fp8_transpose(q)
    assert tuple(t.shape) == (cols, rows)
    for r, c in ((slice(0, 300), slice(0, 300)), (slice(rows - 300, rows), slice(cols - 300, cols))):
        assert torch.equal(t[c, r].view(torch.uint8), q[r, c].view(torch.uint8).t())

