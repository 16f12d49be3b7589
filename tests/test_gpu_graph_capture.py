"""The library's entry points queue kernels and nothing else (no allocation,
no memset or copy nodes, no host synchronization), so a caller may record them
into a HIP graph.  Each test records a few calls with ``torch.cuda.graph``,
replays the graph several times with other eager work and synchronizations
between the replays, and requires every replay to reproduce the eager result
bit for bit on the inputs of that replay."""

import pytest
import torch

from flex_shard_amd import hip_ops
from flex_shard_amd.testing import seeded_normal
from oracle import cport

pytestmark = pytest.mark.gpu

COEFFS = (3.4445, -4.7750, 2.0315)


def _eager_noise(device):
    """Unrelated eager work between two replays."""
    junk = torch.randn(1 << 20, device=device)
    (junk * 2).sum().item()
    torch.cuda.synchronize()


def test_allocation_free_newton_schulz_in_a_graph(device):
    inputs = [seeded_normal((6, 256, 384), 1.0, 900 + i, device) for i in range(3)]
    want = [hip_ops.newton_schulz(x.clone(), COEFFS, 5, 1e-7) for x in inputs]
    static = inputs[0].clone()
    hip_ops.newton_schulz_noalloc(static, COEFFS, 5, 1e-7)  # resolves the scratch address and sizes the kernels' LDS
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    static.copy_(inputs[0])
    with torch.cuda.graph(graph):
        hip_ops.newton_schulz_noalloc(static, COEFFS, 5, 1e-7)
    for replay in range(4):
        static.copy_(inputs[replay % 3])
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static, want[replay % 3]), replay
        _eager_noise(device)


def test_quantize_pack_and_gradient_kernels_in_a_graph(device):
    gen = torch.Generator().manual_seed(77)
    shapes = [(256, 384), (130, 136)]
    weights = [(torch.randn(s, generator=gen) * 0.02).bfloat16().to(device) for s in shapes]
    numel = sum(w.numel() for w in weights)
    scales = sum(-(-w.shape[0] // 128) * -(-w.shape[1] // 128) for w in weights)
    scale_at = -(-numel // 16) * 16
    nbytes = -(-(scale_at + 4 * scales) // 16) * 16 + 48
    chunks, q_off, s_off = [], 0, scale_at
    for w in weights:
        chunks.append(hip_ops.QuantChunkSpec(w, q_off, s_off, hip_ops.SRC_BF16))
        q_off += w.numel()
        s_off += 4 * (-(-w.shape[0] // 128) * -(-w.shape[1] // 128))
    plan = hip_ops.QuantPackPlan(chunks, nbytes, ((numel, scale_at), (s_off, nbytes)), 128, keep_alive=True)
    payload = torch.full((nbytes,), 0xAB, dtype=torch.uint8, device=device)
    acc = torch.zeros(numel, device=device)
    grad = torch.empty(numel, device=device, dtype=torch.bfloat16)
    contrib = torch.empty((4, 4 * 1000), device=device)
    reduced = torch.empty(1000, device=device)
    # one eager round first (code objects loaded, nothing left to set up under capture)
    plan.launch(payload)
    hip_ops.accumulate_grad(acc, grad, overwrite=True)
    hip_ops.reduce_rows(reduced, contrib, 2000)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        plan.launch(payload)
        hip_ops.accumulate_grad(acc, grad, overwrite=True)
        hip_ops.accumulate_grad(acc, grad)
        hip_ops.reduce_rows(reduced, contrib, 2000)
    for replay in range(4):
        for w in weights:
            w.copy_((torch.randn(w.shape, generator=gen) * 0.02 * (replay + 1)).bfloat16())
        grad.copy_(torch.randn(numel, generator=gen).bfloat16())
        contrib.copy_(torch.randn(contrib.shape, generator=gen))
        payload.fill_(0xCD)
        graph.replay()
        torch.cuda.synchronize()
        got = payload.cpu()
        q_off, s_off = 0, scale_at
        for w in weights:
            oq, osc = cport.quantize_blockwise(w.cpu(), 128)
            assert torch.equal(got[q_off : q_off + w.numel()], oq.reshape(-1)), replay
            assert torch.equal(got[s_off : s_off + 4 * osc.numel()].view(torch.int32), osc.reshape(-1).view(torch.int32))
            q_off += w.numel()
            s_off += 4 * osc.numel()
        assert (got[numel:scale_at] == 0).all() and (got[s_off:] == 0).all()
        assert torch.equal(acc, grad.float() + grad.float())
        rows = [contrib[r, 2000:3000].cpu().contiguous() for r in range(4)]
        assert torch.equal(reduced.cpu(), cport.reduce_rows(rows))
        _eager_noise(device)


def test_fp8_linear_forward_and_backward_kernels_in_a_graph(device):
    """Activation quantizers, byte transpose and the three scaled products
    (their outputs come from the graph's own memory pool)."""
    gen = torch.Generator().manual_seed(78)
    tokens, out_dim, in_dim = 300, 384, 256
    x = torch.empty((tokens, in_dim), device=device, dtype=torch.bfloat16)
    g = torch.empty((tokens, out_dim), device=device, dtype=torch.bfloat16)
    w = (torch.randn(out_dim, in_dim, generator=gen) * 0.02).bfloat16().to(device)
    wq, ws = hip_ops.act_quant_1x128(w)
    ws = ws.t().contiguous()[: out_dim // 128].contiguous()  # a [out / 128, in / 128] table of valid scales

    def run():
        xq, xs = hip_ops.act_quant_1x128(x)
        y = hip_ops.fp8_gemm_1x128_128x128(xq, xs, wq, ws)
        gq, gs, gtq, gts = hip_ops.act_quant_both(g)
        dx = hip_ops.fp8_gemm_1x128_128x128_dgrad(gq, gs, hip_ops.fp8_transpose(wq), ws, in_dim)
        xtq, xts = hip_ops.act_quant_128x1_transposed(x)
        dw = hip_ops.fp8_gemm_1x128_128x1(gtq, gts, xtq, xts)
        return y, dx, dw

    x.normal_()
    g.normal_()
    run()  # eager round first
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outputs = run()
    for replay in range(3):
        x.copy_(torch.randn(x.shape, generator=gen).bfloat16())
        g.copy_((torch.randn(g.shape, generator=gen) * 0.01).bfloat16())
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outputs]
        want = run()
        torch.cuda.synchronize()
        for a, b in zip(got, want, strict=True):
            assert torch.equal(a, b), replay
        _eager_noise(device)

