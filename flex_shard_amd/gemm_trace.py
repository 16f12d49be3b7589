"""Per-workgroup timing of the two MFMA tile kernels from a trace build.

The kernels carry time stamps behind ``#ifdef FSH_TRACE`` (``s_memrealtime``,
a 100 MHz counter, and ``s_memtime``, the shader clock).  A trace build is a
second library next to the product one::

    make -C flex_shard_amd/csrc EXTRA=-DFSH_TRACE BUILD=build_trace TARGET=../libflexshard_hip_trace.so
    python -m flex_shard_amd.gemm_trace fp8      # scaled FP8 GEMM: forward and weight gradient, 8192 x [14336, 4096]
    python -m flex_shard_amd.gemm_trace bf16     # Newton-Schulz products of 24 x [7168, 2048]

The stamps go to a device buffer whose address the library reads from the
environment variable ``FSH_GEMM_TRACE`` at launch.  ``fp8`` prints, per launch:
time from a workgroup's entry to its first k-tile being ready, the k loop (and
per k-tile), from the loop's end to the last wave's last store being
acknowledged, the gap between one workgroup's end and the next one's entry on
the same CU, and the k loop split into compute, wait for operands and barrier.
``bf16`` prints per launch the workgroup duration, the shader clock (core
ticks over real time) and the shares of the k loop, operand waits, barriers
and epilogues in a workgroup's core ticks.
"""

from __future__ import annotations

import argparse
import collections
import os

TRACE_LIB = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libflexshard_hip_trace.so")


def _load(lib_path: str):
    from . import _native

    if not os.path.exists(lib_path):
        raise SystemExit(f"{lib_path} is missing; build it with the make command in this module's docstring")
    _native.LIB_PATH = lib_path
    from . import hip_ops

    return hip_ops


def _traced(fn, trace, warmup: int = 3):
    """Run fn() untraced a few times, then once with stamps; returns the stamps as a numpy array."""
    import torch

    os.environ.pop("FSH_GEMM_TRACE", None)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    trace.zero_()
    torch.cuda.synchronize()
    os.environ["FSH_GEMM_TRACE"] = str(trace.data_ptr())
    try:
        fn()
        torch.cuda.synchronize()
    finally:
        os.environ.pop("FSH_GEMM_TRACE", None)
    return trace.cpu().numpy()


def trace_fp8(hip_ops, tokens: int = 8192, out_dim: int = 14336, in_dim: int = 4096) -> None:
    import numpy as np
    import torch

    dev = torch.device("cuda:0")
    trace = torch.zeros(8192 * 8 * 8, dtype=torch.int64, device=dev)
    x = torch.randn(tokens, in_dim, device=dev).bfloat16()
    g = torch.randn(tokens, out_dim, device=dev).bfloat16()
    w = torch.randn(out_dim, in_dim, device=dev).bfloat16()
    gq, gs = hip_ops.act_quant_128x1_transposed(g)
    xq, xs = hip_ops.act_quant_128x1_transposed(x)
    aq, a_s = hip_ops.act_quant_1x128(x)
    wq, _ = hip_ops.act_quant_1x128(w)
    ws = torch.rand(out_dim // 128, in_dim // 128, device=dev) + 0.5

    def report(name, fn, ktiles):
        t = _traced(fn, trace).reshape(-1, 8, 8)
        t = t[t[:, 0, 0] != 0]  # per workgroup: 8 waves x 8 slots (10 ns ticks)
        w0 = t[:, 0, :]
        entry, begin, loop_end, exit_ = w0[:, 5] * 10.0, w0[:, 0] * 10.0, w0[:, 4] * 10.0, t[:, :, 6].max(1) * 10.0
        cu = (w0[:, 7] >> 32) * 256 + ((w0[:, 7] >> 8) & 0xFF)
        per_cu = collections.defaultdict(list)
        for i in range(len(t)):
            per_cu[int(cu[i])].append((entry[i], exit_[i]))
        gaps = []
        for spans in per_cu.values():
            spans.sort()
            gaps += [b[0] - a[1] for a, b in zip(spans, spans[1:])]
        compute, wait, barrier = (t[:, :, k].mean() * 10.0 / ktiles for k in (1, 2, 3))
        print(f"{name}: {len(t)} workgroups on {len(per_cu)} CUs, launch {(exit_.max() - entry.min()) / 1e3:.1f} us")
        print(f"   entry -> first k-tile ready {np.mean(begin - entry) / 1e3:.2f} us; k loop {np.mean(loop_end - begin) / 1e3:.2f} us "
              f"({np.mean(loop_end - begin) / ktiles:.0f} ns per k-tile: compute {compute:.0f}, wait for operands {wait:.0f}, "
              f"barrier {barrier:.0f}); loop end -> last store acknowledged {np.mean(exit_ - loop_end) / 1e3:.2f} us")
        if gaps:
            print(f"   end of a workgroup -> entry of the next on the same CU: mean {np.mean(gaps) / 1e3:.2f} us "
                  f"(min {np.min(gaps) / 1e3:.2f}, max {np.max(gaps) / 1e3:.2f})", flush=True)

    report(f"weight gradient [{out_dim}, {in_dim}], k = {tokens}", lambda: hip_ops.fp8_gemm_1x128_128x1(gq, gs, xq, xs), tokens // 128)
    report(f"forward [{tokens}, {out_dim}], k = {in_dim}", lambda: hip_ops.fp8_gemm_1x128_128x128(aq, a_s, wq, ws), in_dim // 128)


def trace_bf16(hip_ops, batch: int = 24, short: int = 2048, long: int = 7168) -> None:
    import torch

    dev = torch.device("cuda:0")
    trace = torch.zeros(16384 * 16, dtype=torch.int64, device=dev)
    for name, (m, n, k) in (("X'^T = X^T P", (long, short, short)), ("G = X X^T (plain NT form)", (short, short, long))):
        a = torch.randn(batch, m, k, device=dev).bfloat16()
        b = torch.randn(batch, n, k, device=dev).bfloat16()
        out = torch.empty(batch, m, n, device=dev, dtype=torch.bfloat16)
        t = _traced(lambda: hip_ops.gemm_nt(a, b, out=out), trace).reshape(-1, 16).astype("float64")
        t = t[t[:, 12] != 0]  # resident workgroups: sums over all their tiles, stamps of the last one
        core = t[:, 12]
        real_ns = (t[:, 4] - t[:, 1]) * 10.0  # last tile's end against the first tile's start
        clock_mhz = (core / real_ns).mean() * 1e3
        tiles = t[:, 10].mean()
        share = lambda col: 100.0 * (t[:, col] / core).mean()
        print(f"{name} [{batch} x {m} x {n} x {k}]: {len(t)} workgroups, {tiles:.1f} tiles each, {real_ns.mean() / 1e3:.1f} us per "
              f"workgroup, shader clock {clock_mhz:.0f} MHz")
        print(f"   share of a workgroup's core ticks: k loops {share(11):.1f} % (of which waiting for operands {share(13):.1f} %, "
              f"k-tile barriers {share(14):.1f} %), epilogues {share(7):.1f} %, tile hand-over wait + barrier "
              f"{share(8) + share(9):.1f} %", flush=True)


def main(argv=None) -> None:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("kernel", choices=("fp8", "bf16"))
    ap.add_argument("--lib", default=TRACE_LIB, help="the trace build of the library")
    args = ap.parse_args(argv)
    hip_ops = _load(args.lib)
    (trace_fp8 if args.kernel == "fp8" else trace_bf16)(hip_ops)


if __name__ == "__main__":
    main()
