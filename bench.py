#!/usr/bin/env python3
"""Benchmark of the single-GPU hot path on one MI355X.

Headline: fused FP8 tile quantize + pack of one rank's share (rank 0 of 8) of a
Llama-3-8B layer bucket: q, k, v and the first 512 rows of o = 27 262 976 bf16
elements in 4 chunks, packed into a 27 531 840-byte payload.  A step is one
pass over `--layers` distinct layer buckets, one such launch per layer (what a
training step does with the layers of a model), so the inputs of every launch
come from HBM, not from the 256 MB last-level cache.  Before anything is
timed, every layer bucket is packed twice (launch tables cached, allocator
blocks in place), whatever `--warmup` says.  `value` is algorithmic bytes moved
per second over the whole timed region, inputs resident in HBM.

One JSON line is printed.  Besides the contract fields it carries
  roofline      the dominant kernel against the 8 TB/s HBM peak, timed with
                events on the launch stream over the same timed region
  contract_entry / two_buckets_in_flight
                the same launches through `prepare_unshard_bucket` itself
                (host time of the contract included) and alternating over two
                streams (the per-launch ramp of one overlaps the other's tail)
  cpu_baseline  the oracle's eager-torch restatement of the reference path on
                the host cores, on the same rank-0 share (the gradient path
                and Newton-Schulz have their own CPU legs under `secondary`)
  secondary     unpack+dequant of the 8-rank gathered layout, the fp32
                gradient path, the 48-matrix Muon / Newton-Schulz step, and the
                forward and backward products of the prequantized-weight
                linear (activation quantizers + scaled FP8 GEMMs) on
                Llama-3-8B shapes
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, vendor figure
BF16_MFMA_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, vendor figure
FP8_MFMA_PEAK_TFLOPS = 5000.0  # MI355X dense fp8, vendor figure
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "quantize_pack_bf16_kernel_llama3_8b_layer_rank0.md")


def profiled_traffic(elems: int, payload_nbytes: int):
    """HBM bytes per launch of the dominant kernel as the counter runs
    (FETCH_SIZE, then WRITE_SIZE, each scaled by the same counter's reading for
    a plain copy of known size) found them.  Counters cannot be read inside a
    timed run, so the figure is read from the committed summary of those runs,
    which names the workload and the commit of the kernel it was measured on:
    a line `traffic_bytes_per_launch: <bytes> elems=<n> payload_nbytes=<n> commit=<sha>`.
    Returns (bytes, commit) or (None, None) when the summary has no line for
    this workload."""
    import re

    try:
        with open(TRAFFIC_PROFILE) as fh:
            text = fh.read()
    except OSError:
        return None, None
    for m in re.finditer(r"traffic_bytes_per_launch:\s*(\d+)\s+elems=(\d+)\s+payload_nbytes=(\d+)\s+commit=(\w+)", text):
        if int(m.group(2)) == elems and int(m.group(3)) == payload_nbytes:
            return int(m.group(1)), m.group(4)
    return None, None


def _factory(fp8_data, recip_scale, block_size, *, orig_dtype, requires_grad):
    return fp8_data


def _event_ms(fn, steps: int, warmup: int) -> tuple[float, float]:
    """(wall ms, event ms) for `steps` calls of fn(i) after `warmup` calls."""
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for i in range(steps):
        fn(i)
    stop.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3
    return wall, start.elapsed_time(stop)


def _steady_us(fn, reps: int, settle_ms: float = 25.0) -> float:
    """us per call of fn(i) over `reps` calls, after untimed calls that last
    about `settle_ms`: after lighter work a compute-bound kernel runs slower
    for its first 15-20 ms (the same GEMM measured 139 us right after a 5 ms
    settle and 118 us from then on)."""
    _, est_ms = _event_ms(fn, 3, 2)
    settle = max(2, int(settle_ms / max(est_ms / 3, 1e-3)))
    _, ms = _event_ms(fn, reps, settle)
    return ms / reps * 1e3


def build_quant_workload(device, layers: int, rank: int = 0, spec=None, std: float = 0.02,
                         master_dtype: torch.dtype = torch.bfloat16):
    """Per layer: one rank's local shards as views of one flat storage (the
    sharded bucket storage layout; bf16, or fp32 masters that are quantized as
    bf16), their ParamInfos, and a reusable payload."""
    import torch.nn as nn

    from flex_shard_amd import Fp8BucketedBlockShard
    from flex_shard_amd.testing import LLAMA3_8B_LAYER, FakeMesh, make_param_infos, seeded_normal

    placement = Fp8BucketedBlockShard(world_size=8, weight_factory=_factory)
    mesh = FakeMesh(8, rank)
    meta = [(n, nn.Parameter(torch.empty(s, device="meta", dtype=master_dtype)))
            for n, s in (spec or LLAMA3_8B_LAYER)]
    infos = make_param_infos(meta, placement, mesh)
    for info in infos:
        info.param_dtype = torch.bfloat16
    local_numel = infos[0].bucket_layout.local_numel
    size = master_dtype.itemsize
    work = []
    for layer in range(layers):
        storage = seeded_normal((local_numel,), std, 1000 + layer, device, master_dtype)
        shards = [
            storage[i.byte_offset // size : i.byte_offset // size + i.local_numel].view(i.local_shape) for i in infos
        ]
        work.append((storage, shards))
    return placement, mesh, infos, work


def bench_quant_pack(device, steps, warmup, layers, rank: int = 0, spec=None, std: float = 0.02, extras: bool = False,
                     master_dtype: torch.dtype = torch.bfloat16):
    """One step = one pass over the `layers` layer buckets: one fused
    quantize+pack launch per bucket through the placement's contract entry,
    `prepare_unshard_bucket` (payload-cache bookkeeping, the launch, the
    W x row gather output).  The two most recent prepared unshards are held,
    as a runtime with one bucket prefetched holds them."""
    import collections

    placement, mesh, infos, work = build_quant_workload(device, layers, rank, spec, std, master_dtype)
    metadata = placement._quant_metadata_from_infos(infos)
    plan = metadata.rank_pack_plans[rank]
    elems = plan.qdata_numel
    scales = sum(sum(c.scale_numels) for c in plan.chunks)
    # 2 B (4 B of an fp32 master) read + 1 B written per element, 4 B per tile scale
    algo_bytes = (master_dtype.itemsize + 1) * elems + 4 * scales
    held = collections.deque(maxlen=2)

    def launch(layer):
        held.append(placement.prepare_unshard_bucket(work[layer][1], infos, mesh, None))

    def step(i):
        for layer in range(len(work)):
            launch(layer)

    # Steady state first, independent of --warmup: every bucket's launch is
    # stored and the recycled buffers exist before the clock starts.
    for _ in range(2):
        step(0)
    torch.cuda.synchronize()
    wall_ms, event_ms = _event_ms(step, steps, warmup)
    out = {
        "elems": elems,
        "algo_bytes": algo_bytes,
        "launches_per_step": len(work),
        "wall_ms": wall_ms,
        "event_ms": event_ms,
        "payload_nbytes": metadata.packed_send_nbytes_per_rank,
        "chunks": len(plan.chunks),
        "work": (placement, infos, work, metadata, mesh),
    }
    if not extras:
        return out
    n = steps * len(work)
    # Hot-cache variant (one layer over and over) for the record.
    _, hot_ms = _event_ms(lambda i: launch(0), n, 5)
    out["hot_us"] = hot_ms / n * 1e3

    # Host time of the contract entry: the time the calls take to issue
    # (nothing waits for the GPU inside them), the queue drained first.
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(n):
        launch(i % len(work))
    out["contract_host_us"] = (time.perf_counter() - t0) / n * 1e6
    torch.cuda.synchronize()

    # Two buckets in flight: the same contract calls with torch's current
    # stream alternating between two side streams of the same (default)
    # priority, the way a runtime that prefetches the next bucket issues them;
    # the ramp and drain of one launch overlap the other's.  Payloads and
    # gather outputs come from each stream's own recycled buffers.
    streams = [torch.cuda.Stream(device), torch.cuda.Stream(device)]
    main = torch.cuda.current_stream(device)
    held2 = [collections.deque(maxlen=2), collections.deque(maxlen=2)]

    def issue(i):
        torch.cuda.set_stream(streams[i % 2])
        held2[i % 2].append(placement.prepare_unshard_bucket(work[i % len(work)][1], infos, mesh, None))

    try:
        for rep in range(2):  # the first repetition creates both streams' buffers
            torch.cuda.synchronize()
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record(streams[0])
            fence = torch.cuda.Event()
            fence.record(streams[0])
            streams[1].wait_event(fence)
            t0 = time.perf_counter()
            for i in range(n):
                issue(i)
            host = time.perf_counter() - t0
            joined = torch.cuda.Event()
            joined.record(streams[1])
            streams[0].wait_event(joined)
            stop.record(streams[0])
            torch.cuda.synchronize()
    finally:
        torch.cuda.set_stream(main)
    out["two_stream_us"] = start.elapsed_time(stop) / n * 1e3
    out["two_stream_host_us"] = host / n * 1e6
    out["two_stream_last"] = (held2, streams)
    return out


def bench_other_shares(device):
    """The same launch on other shares: the largest rank share of the Llama
    bucket (rank 6: rows of `down`, in_dim 14336), rank 0 of the DeepSeek-V3
    expert bucket (stacked w1 rows), and the headline share kept as fp32
    masters that are quantized as bf16 (4 B read + 1 B written per element)."""
    from flex_shard_amd.testing import DEEPSEEK_V3_EXPERTS

    out = {}
    for name, kwargs, steps in (
        ("llama3_8b_rank6", dict(layers=8, rank=6), 25),
        ("deepseek_v3_experts_rank0", dict(layers=2, rank=0, spec=DEEPSEEK_V3_EXPERTS, std=0.006), 20),
        ("llama3_8b_rank0_fp32_masters", dict(layers=8, rank=0, master_dtype=torch.float32), 25),
    ):
        q = bench_quant_pack(device, steps, 2, **kwargs)
        q.pop("work")
        us = q["event_ms"] / (steps * q["launches_per_step"]) * 1e3
        out[name] = {"elems": q["elems"], "chunks": q["chunks"], "algorithmic_bytes": q["algo_bytes"],
                     "us_per_launch": us, "GBps": q["algo_bytes"] / us / 1e3,
                     "frac_of_hbm_peak": q["algo_bytes"] / us / 1e3 / HBM_PEAK_GBPS}
        torch.cuda.empty_cache()
    return out


def check_against_oracle(placement, infos, work, metadata, mesh, prepared=None):
    """Bit-exactness gate before any timing is reported: one chunk of a
    payload produced through the contract entry against the C oracle.
    `prepared`: a prepared unshard of layer bucket 0 to check instead of a
    fresh one."""
    from oracle import cport

    storage, shards = work[0]
    if prepared is None:
        prepared = placement.prepare_unshard_bucket(shards, infos, mesh, None)
    payload = prepared.buffers[0].cpu()
    k = shards[1].detach().cpu().flatten(0, -2)
    oq, osc = cport.quantize_blockwise(k, 128)
    start = shards[0].numel()
    ok = torch.equal(payload[start : start + oq.numel()], oq.reshape(-1))
    s0 = metadata.rank_scale_byte_offsets[0] + 4 * (32 * 32)
    ok &= torch.equal(payload[s0 : s0 + 4 * osc.numel()].view(torch.float32), osc.reshape(-1))
    if not ok:
        raise SystemExit("bench: GPU payload differs from the oracle; refusing to report a timing")


def cpu_baseline_quant(work, infos, metadata, budget_s: float = 10.0):
    """The reference path in eager torch on the host: per chunk quantize
    (pad, amax, clamp, fp64 divide, multiply, clamp, cast), then copy data and
    scale bytes into the payload.  Same rank-0 share as the GPU step."""
    from oracle import eager

    torch.set_num_threads(os.cpu_count() or 1)
    _, shards = work[0]
    cpu_shards = [s.detach().cpu() for s in shards]
    plan = metadata.rank_pack_plans[0]
    payload = torch.zeros(metadata.packed_send_nbytes_per_rank, dtype=torch.uint8)

    def run():
        cursor, scale_cursor = 0, plan.scale_byte_offset
        for chunk in plan.chunks:
            q, s = eager.quantize_blockwise(cpu_shards[chunk.param_index].reshape(chunk.local_shape), 128)
            payload[cursor : cursor + q.numel()] = q.view(torch.uint8).reshape(-1)
            sb = s.reshape(-1).view(torch.uint8)
            payload[scale_cursor : scale_cursor + sb.numel()] = sb
            cursor += q.numel()
            scale_cursor += sb.numel()

    run()  # warm-up
    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < 5 or (time.perf_counter() < t_end and len(times) < 1000):  # about 10 s of host work
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    times.sort()
    return times[len(times) // 2], len(times), torch.get_num_threads()


def cpu_baseline_gradients(reps: int = 15):
    """Config 4 on the host cores, on a bounded sample: one rank range
    (27 295 744 elements, an eighth of the layer bucket) through the oracle's
    eager restatement of the fp32 microbatch accumulation (4 bf16 microbatches)
    and of the fixed-order 8-way fold."""
    from oracle import eager

    torch.set_num_threads(os.cpu_count() or 1)
    seg, world = 27295744, 8
    gen = torch.Generator().manual_seed(7)
    micro = [(torch.randn(seg, generator=gen) * 1e-3).bfloat16() for _ in range(4)]
    eager.accumulate_microbatches(micro)
    acc_t = []
    for _ in range(reps):
        t0 = time.perf_counter()
        eager.accumulate_microbatches(micro)
        acc_t.append(time.perf_counter() - t0)
    del micro
    contrib = [torch.randn(seg, generator=gen) * 1e-3 for _ in range(world)]
    eager.reduce_rank_contributions(contrib, 0, seg)
    red_t = []
    for _ in range(reps):
        t0 = time.perf_counter()
        eager.reduce_rank_contributions(contrib, 0, seg)
        red_t.append(time.perf_counter() - t0)
    acc_s, red_s = sorted(acc_t)[reps // 2], sorted(red_t)[reps // 2]
    return {
        "kind": "port",
        "cores": torch.get_num_threads(),
        "sample": f"one rank range of {seg} elements (1/8 of the bucket): 4 bf16 microbatches accumulated in fp32, "
        f"then the 8-way fixed-order fold of that range; eager torch, median of {reps}",
        "accumulate_ms_per_microbatch_on_sample": round(acc_s / 4 * 1e3, 3),
        "accumulate_GBps": round(10 * seg * 4 / acc_s / 1e9, 3),
        "reduce_ms": round(red_s * 1e3, 3),
        "reduce_GBps": round(36 * seg / red_s / 1e9, 3),
    }


def cpu_baseline_newton_schulz(flops_full: int, per_shape: int = 2, reps: int = 3):
    """Config 5 on the host cores, on a bounded sample: `per_shape` matrices
    of each of the two shapes through torch's own Newton-Schulz
    (torch.optim._muon._zeropower_via_newtonschulz, the routine the oracle is
    pinned to), scaled linearly to the 24 + 24 matrices."""
    from torch.optim._muon import _zeropower_via_newtonschulz as torch_ns

    torch.set_num_threads(os.cpu_count() or 1)
    gen = torch.Generator().manual_seed(11)
    coeffs, steps, eps = (3.4445, -4.7750, 2.0315), 5, 1e-7
    total_s = 0.0
    for shape in ((7168, 2048), (2048, 2048)):
        mats = [torch.randn(shape, generator=gen).bfloat16() for _ in range(per_shape)]
        torch_ns(mats[0], coeffs, steps, eps)
        times = []
        for _ in range(reps):
            t0 = time.perf_counter()
            for m in mats:
                torch_ns(m, coeffs, steps, eps)
            times.append(time.perf_counter() - t0)
        total_s += sorted(times)[reps // 2] * (24 / per_shape)
    return {
        "kind": "port",
        "cores": torch.get_num_threads(),
        "sample": f"{per_shape} matrices of [7168, 2048] and {per_shape} of [2048, 2048] through "
        f"torch.optim._muon._zeropower_via_newtonschulz in bf16 on the host, median of {reps}, scaled by "
        f"{24 // per_shape} to the 24 + 24 matrices",
        "newton_schulz_ms_scaled_to_full_config": round(total_s * 1e3, 1),
        "TFLOPs": round(flops_full / total_s / 1e12, 4),
    }


def bench_unpack(device, placement, infos, reps=10):
    """Unpack of the 8-rank gathered layout + bf16 dequant: 218 103 808 FP8
    elements, 1 B read + 1 B compact write + 2 B dequant write per element."""
    import torch.nn as nn

    from flex_shard_amd.testing import LLAMA3_8B_LAYER, FakeMesh, make_param_infos

    md = placement._quant_metadata_from_infos(infos)
    # Three gathered buffers (0.66 GB): rotating over them, every launch reads
    # its rows from HBM; repeating one, from the last-level cache, where a
    # gather that has just written them would leave them.
    gathered = []
    for _ in range(3):
        rows = torch.randint(0, 120, (8, md.packed_send_nbytes_per_rank), dtype=torch.uint8, device=device)
        for r in range(8):
            s0 = md.rank_scale_byte_offsets[r]
            rows[r, s0 : s0 + 4 * md.rank_scale_numels[r]].view(torch.float32).fill_(1e-4)
        gathered.append(rows)
    from flex_shard_amd.placement_contract import PlacementPreparedUnshard

    state = placement._QuantUnshardState(infos=infos, pg=None, debug_fqn=None, metadata=md)
    rows = gathered[0]
    prep = PlacementPreparedUnshard(placement=placement, buffers=[rows[0], rows.view(-1)], placement_state=state)
    total = sum(i.global_numel for i in infos)
    out = torch.empty(total, dtype=torch.bfloat16, device=device)
    prep.persistent = True
    result, _ = placement.finish_prepared_unshard_with_dequant(prep, rows, dequant_out=out)
    prep.persistent_buffers = result.persistent_buffers
    reps = 3 * ((reps + 2) // 3)
    _, fused_ms = _event_ms(
        lambda i: placement.finish_prepared_unshard_with_dequant(prep, gathered[i % 3], dequant_out=out), reps, 3)
    _, fused_hot_ms = _event_ms(lambda i: placement.finish_prepared_unshard_with_dequant(prep, rows, dequant_out=out), reps, 3)
    _, compact_ms = _event_ms(lambda i: placement._finish_unshard_from_rank_rows(prep, gathered[i % 3]), reps, 3)
    scales = sum(md.rank_scale_numels)
    return {
        "elems": total,
        "fused_unpack_dequant_ms": fused_ms / reps,
        "fused_GBps": (4 * total + 8 * scales) / (fused_ms / reps) / 1e6,
        "fused_unpack_dequant_ms_rows_in_cache": fused_hot_ms / reps,
        "fused_GBps_rows_in_cache": (4 * total + 8 * scales) / (fused_hot_ms / reps) / 1e6,
        "compact_only_ms": compact_ms / reps,
        "compact_GBps": (2 * total + 8 * scales) / (compact_ms / reps) / 1e6,
    }


def bench_gradient_copy_in(device, reps=5):
    """One-pass copy-in of a Llama-3-8B layer's separate full-parameter
    gradients into the [8, rank range] reduce-scatter input (one
    `pack_segments_kernel` launch, zero gaps included): fp32 gradients as
    they accumulate under an fp32 reduce dtype, and bf16 gradients cast to
    fp32 on the way."""
    import torch.nn as nn

    from flex_shard_amd import BucketedBlockShard, LocalReduceGroup
    from flex_shard_amd.testing import LLAMA3_8B_LAYER, FakeMesh, make_param_infos

    world = 8
    placement = BucketedBlockShard(dims=(0,), blocks_per_rank=(1,) * world)
    named = [(n, nn.Parameter(torch.empty(s, device="meta", dtype=torch.bfloat16))) for n, s in LLAMA3_8B_LAYER]
    mesh = FakeMesh(world, 0, LocalReduceGroup(world, 0))
    infos = make_param_infos(named, placement, mesh)
    for info in infos:
        info.reduce_dtype = torch.float32
    total = sum(i.global_numel for i in infos)
    out = {}
    for key, dtype in (("copy_in_fp32", torch.float32), ("copy_in_bf16_to_fp32", torch.bfloat16)):
        grads = [torch.randn(i.global_shape, device=device, dtype=dtype) for i in infos]
        _, ms = _event_ms(lambda i: placement.prepare_reduce_grad(grads, infos, mesh, None), reps, 2)
        out[key + "_ms"] = ms / reps
        out[key + "_GBps"] = total * (dtype.itemsize + 4) / (ms / reps) / 1e6
        del grads
    return out


def bench_gradients(device, reps=5):
    """Config 4: 4 bf16 microbatches accumulated in fp32 over the 218 365 952
    element bucket (placement layout), then the 8-way fixed-order reduction of
    rank 0's 27 295 744-element range."""
    from flex_shard_amd import hip_ops
    from flex_shard_amd.testing import seeded_normal

    total, seg, world = 218365952, 27295744, 8
    acc = torch.zeros(total, device=device)
    micro = [seeded_normal((total,), 1e-3, 500 + k, device) for k in range(4)]
    _, acc_ms = _event_ms(lambda i: hip_ops.accumulate_grad(acc, micro[i % 4], overwrite=(i % 4 == 0)), 4 * reps, 4)
    del micro
    contrib = torch.empty((world, total), device=device)
    contrib.normal_(0, 1e-3)
    out = torch.empty(seg, device=device)
    _, red_ms = _event_ms(lambda i: hip_ops.reduce_rows(out, contrib, 0), reps * 4, 2)
    acc_per = acc_ms / (4 * reps)
    red_per = red_ms / (reps * 4)
    del acc, contrib, out
    copy_in = bench_gradient_copy_in(device, reps)
    return {
        **copy_in,
        "accumulate_ms_per_microbatch": acc_per,
        "accumulate_GBps": 10 * total / acc_per / 1e6,  # 2 B grad + 4 B read + 4 B write (6 B on the first)
        "reduce_ms": red_per,
        "reduce_GBps": 36 * seg / red_per / 1e6,  # 8 x 4 B read + 4 B write per output element
    }


def bench_muon(device, reps=4):
    """Config 5: 24 x [7168, 2048] + 24 x [2048, 2048] bf16 whole matrices, one
    Muon step (momentum, Nesterov, 5 Newton-Schulz steps, update)."""
    from flex_shard_amd.dist_muon import OwnedMuon
    from flex_shard_amd.testing import seeded_normal

    shapes = [(7168, 2048)] * 24 + [(2048, 2048)] * 24
    params = [seeded_normal(s, 0.02, 2000 + i, device) for i, s in enumerate(shapes)]
    grads = [seeded_normal(s, 1.0, 3000 + i, device) for i, s in enumerate(shapes)]
    opt = OwnedMuon(params)
    _, ms = _event_ms(lambda i: opt.step(grads), reps, 2)  # two untimed steps: the clock settles over the first
    per = ms / reps
    flops = opt.flops_per_step()
    # The orthogonalization alone (normalization + 5 iterations on all 48
    # matrices, one fsh_newton_schulz_multi call), without the momentum and
    # update kernels around it: inputs restored outside the timed region.
    from flex_shard_amd import hip_ops

    problems = [(opt._batch[shape], opt._workspace[shape]) for shape in opt._groups]
    saved = [torch.stack([grads[i] for i in opt._groups[shape]]) for shape in opt._groups]
    ns_ms = 0.0
    for rep in range(reps + 2):
        for (batch, _), keep in zip(problems, saved):
            batch.copy_(keep)
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        hip_ops.newton_schulz_multi(problems, opt.ns_coefficients, opt.ns_steps, opt.eps)
        stop.record()
        torch.cuda.synchronize()
        if rep >= 2:  # two warm-up calls: the second still runs 2 % slower than the ones behind it
            ns_ms += start.elapsed_time(stop)
    ns_per = ns_ms / reps
    return {"step_ms": per, "ns_flop": flops, "ns_TFLOPs": flops / per / 1e9,
            "frac_of_bf16_mfma_peak": flops / per / 1e9 / BF16_MFMA_PEAK_TFLOPS,
            "newton_schulz_only_ms": ns_per, "newton_schulz_only_TFLOPs": flops / ns_per / 1e9,
            "newton_schulz_only_frac_of_bf16_mfma_peak": flops / ns_per / 1e9 / BF16_MFMA_PEAK_TFLOPS}


def bench_side_stream_copies(device, gemms: int = 12, copies: int = 6, nbytes: int = 220 << 20):
    """What a copy on a side stream costs the MFMA kernels on the main stream:
    twelve FP8 forward GEMMs (8192 tokens, gate/up [14336, 4096]) alone, beside
    six 220 MB segment copies, and beside six torch ``copy_`` kernels of the
    same bytes.  Each figure is the best of three runs (the first launch of a
    kernel in a process loads its code object, milliseconds that are not the
    kernels' own)."""
    from flex_shard_amd import hip_ops
    from flex_shard_amd.custom_placements._copy_kernels import SegmentCopyDescriptor, copy_segments
    from flex_shard_amd.testing import seeded_normal

    tokens, n, k = 8192, 14336, 4096
    x = seeded_normal((tokens, k), 1.0, 4000, device)
    w = seeded_normal((n, k), 0.02, 4100, device)
    wq, ws = hip_ops.act_quant_1x128(w)
    ws = ws.t().contiguous()[: n // 128].contiguous()
    xq, xs = hip_ops.act_quant_1x128(x)
    y = torch.empty((tokens, n), dtype=torch.bfloat16, device=device)
    src = torch.randint(0, 255, (nbytes // 4,), dtype=torch.int32, device=device)
    dst = torch.empty_like(src)
    desc = SegmentCopyDescriptor.create(src_offsets=[0], numels=[src.numel()], dst_offsets=[0], device=device)
    side = torch.cuda.Stream(device)
    side_work = {
        "segment_copies": lambda: copy_segments(src, dst, desc),
        "torch_copies": lambda: dst.copy_(src),
    }

    def run(kind):
        for _ in range(3):
            hip_ops.fp8_gemm_1x128_128x128(xq, xs, wq, ws, out=y)
        torch.cuda.synchronize()
        start, end, side_end = (torch.cuda.Event(enable_timing=True) for _ in range(3))
        start.record()
        if kind:
            side.wait_event(start)
            with torch.cuda.stream(side):
                for _ in range(copies):
                    side_work[kind]()
                side_end.record()
        for _ in range(gemms):
            hip_ops.fp8_gemm_1x128_128x128(xq, xs, wq, ws, out=y)
        end.record()
        torch.cuda.synchronize()
        return start.elapsed_time(end), (start.elapsed_time(side_end) if kind else 0.0)

    def alone(kind):
        side_work[kind]()
        torch.cuda.synchronize()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(copies):
            side_work[kind]()
        end.record()
        torch.cuda.synchronize()
        return start.elapsed_time(end)

    out = {"gemms": gemms, "copies": copies, "copy_MB": nbytes / 1e6,
           "gemms_alone_ms": min(run(None)[0] for _ in range(3))}
    for kind in side_work:
        main_ms, side_ms = min(run(kind) for _ in range(3))
        out[kind] = {
            "copies_alone_ms": alone(kind),
            "gemms_beside_copies_ms": main_ms,
            "copies_done_at_ms": side_ms,
        }
    return out


def bench_fp8_linear(device, tokens: int = 8192, reps: int = 10):
    """Forward of the blockwise FP8 linear on the layer's projections: 8192
    tokens against q/o [4096, 4096], gate/up [14336, 4096] and down
    [4096, 14336], weights quantized by the tile quantizer."""
    from flex_shard_amd import hip_ops
    from flex_shard_amd.testing import seeded_normal

    out = {}
    for name, (n, k) in (("q_o_4096x4096", (4096, 4096)), ("gate_up_14336x4096", (14336, 4096)),
                         ("down_4096x14336", (4096, 14336))):
        x = seeded_normal((tokens, k), 1.0, 4000 + n, device)
        w = seeded_normal((n, k), 0.02, 4100 + k, device)
        wq, ws = hip_ops.act_quant_1x128(w)  # any valid FP8 operand: bytes and fp32 scales of the right shapes
        ws = ws.t().contiguous()[: n // 128].contiguous()  # [n / 128, k / 128] table for the timing
        _, q_ms = _event_ms(lambda i: hip_ops.act_quant_1x128(x), reps, 2)
        xq, xs = hip_ops.act_quant_1x128(x)
        y = torch.empty((tokens, n), dtype=torch.bfloat16, device=device)
        g_us = _steady_us(lambda i: hip_ops.fp8_gemm_1x128_128x128(xq, xs, wq, ws, out=y), 2 * reps)
        q_us = q_ms / reps * 1e3
        flop = 2 * tokens * n * k
        out[name] = {
            "act_quant_us": q_us,
            "act_quant_GBps": tokens * k * (3 + 4 / 128) / q_us / 1e3,  # 2 B read + 1 B + 4/128 B written per element
            "gemm_us": g_us,
            "gemm_TFLOPs": flop / g_us / 1e6,
            "frac_of_fp8_mfma_peak": flop / g_us / 1e6 / FP8_MFMA_PEAK_TFLOPS,
        }
        del x, w, wq, ws, xq, xs, y
    return out


def bench_fp8_linear_backward(device, tokens: int = 8192, reps: int = 10):
    """Backward of the same linear, per kernel: the input gradient
    (1x128 quantizer on grad_out, byte transpose of the weight, GEMM) and the
    weight gradient (token-run quantizer on grad_out and on x, GEMM)."""
    from flex_shard_amd import hip_ops
    from flex_shard_amd.testing import seeded_normal

    out = {}
    for name, (n, k) in (("q_o_4096x4096", (4096, 4096)), ("gate_up_14336x4096", (14336, 4096)),
                         ("down_4096x14336", (4096, 14336))):
        x = seeded_normal((tokens, k), 1.0, 4200 + n, device)
        g = seeded_normal((tokens, n), 0.01, 4300 + k, device)
        w = seeded_normal((n, k), 0.02, 4400 + k, device)
        wq, ws = hip_ops.act_quant_1x128(w)  # any valid FP8 operand of the right shape
        ws = ws.t().contiguous()[: n // 128].contiguous()
        del w
        us = {}
        _, ms = _event_ms(lambda i: hip_ops.fp8_transpose(wq), reps, 2)
        us["transpose"] = ms / reps * 1e3
        _, ms = _event_ms(lambda i: hip_ops.act_quant_128x1_transposed(g), reps, 2)
        us["quant_grad_t"] = ms / reps * 1e3
        _, ms = _event_ms(lambda i: hip_ops.act_quant_128x1_transposed(x), reps, 2)
        us["quant_x_t"] = ms / reps * 1e3
        _, ms = _event_ms(lambda i: hip_ops.act_quant_1x128(g), reps, 2)
        us["quant_grad"] = ms / reps * 1e3
        _, ms = _event_ms(lambda i: hip_ops.act_quant_both(g), reps, 2)
        us["quant_grad_both"] = ms / reps * 1e3
        wt = hip_ops.fp8_transpose(wq)
        gq, gs = hip_ops.act_quant_1x128(g)
        us["dgrad_gemm"] = _steady_us(lambda i: hip_ops.fp8_gemm_1x128_128x128_dgrad(gq, gs, wt, ws), 2 * reps)
        del wt, gq, gs
        gtq, gts = hip_ops.act_quant_128x1_transposed(g)
        xtq, xts = hip_ops.act_quant_128x1_transposed(x)
        us["wgrad_gemm"] = _steady_us(lambda i: hip_ops.fp8_gemm_1x128_128x1(gtq, gts, xtq, xts), 2 * reps)
        flop = 2 * tokens * n * k
        out[name] = {
            "transpose_us": us["transpose"],
            "transpose_GBps": 2 * n * k / us["transpose"] / 1e3,  # 1 B read + 1 B written per element
            "quant_grad_transposed_us": us["quant_grad_t"],
            "quant_grad_transposed_GBps": tokens * n * (3 + 4 / 128) / us["quant_grad_t"] / 1e3,
            # the output gradient in both forms: one pass (what the backward runs) against the two separate quantizers
            "quant_grad_both_forms_us": us["quant_grad_both"],
            "quant_grad_both_forms_GBps": tokens * n * (4 + 8 / 128) / us["quant_grad_both"] / 1e3,  # 2 B read + 2 x (1 B + 4/128 B) written
            "quant_grad_rows_plus_transposed_us": us["quant_grad"] + us["quant_grad_t"],
            "quant_x_transposed_us": us["quant_x_t"],
            "quant_x_transposed_GBps": tokens * k * (3 + 4 / 128) / us["quant_x_t"] / 1e3,
            "dgrad_gemm_us": us["dgrad_gemm"],
            "dgrad_gemm_TFLOPs": flop / us["dgrad_gemm"] / 1e6,
            "wgrad_gemm_us": us["wgrad_gemm"],
            "wgrad_gemm_TFLOPs": flop / us["wgrad_gemm"] / 1e6,
            "wgrad_frac_of_fp8_mfma_peak": flop / us["wgrad_gemm"] / 1e6 / FP8_MFMA_PEAK_TFLOPS,
        }
        del x, g, wq, ws, gtq, gts, xtq, xts
    return out


def bench_runtime_layer_step(device, tokens: int = 8192, layers: int = 2, steps: int = 5, warmup: int = 2):
    """The pieces composed: forward + backward of `layers` blocks of the seven
    Llama-3-8B projections at 8192 tokens, each block one FP8 bucket of rank 0
    of an 8-rank mesh under `BucketRuntime.install_hooks` (pack -> local
    all-gather of the 8 payload rows -> unpack -> FP8 linears forward; again in
    the backward, then gradient copy-in and the fixed-order 8-way reduction of
    rank 0's range, the other ranks' rows and contributions deposited once in
    the one-GPU group).  Each block's unshard is prefetched on a side stream
    under the previous block's compute.  Reports the span per step, the host
    time spent inside the runtime's hooks, and the share of the span in which
    the host was issuing work (the rest it waits for the GPU at the end)."""
    import torch.nn as nn

    from flex_shard_amd import Fp8BucketedBlockShard, GradientReduction, LocalReduceGroup
    from flex_shard_amd.blockwise_fp8 import convert_to_flex_shard_float8_blockwise_linear, make_blockwise_fp8_weight
    from flex_shard_amd.flex_shard import BucketCommContext, BucketRuntime
    from flex_shard_amd.testing import LLAMA3_8B_LAYER, FakeMesh, local_rows, make_param_infos, seeded_normal

    world = 8

    class Projections(nn.Module):
        """q/k/v/o and gate/up/down of one block, joined by elementwise ops
        (attention itself and the norms are not part of the measured path)."""

        def __init__(self) -> None:
            super().__init__()
            for name, (out_dim, in_dim) in LLAMA3_8B_LAYER:
                setattr(self, name, nn.Linear(in_dim, out_dim, bias=False, device="meta", dtype=torch.bfloat16))

        def forward(self, x):
            kv = torch.cat([self.k(x), self.v(x)], dim=-1)
            h = self.o(self.q(x) + kv.repeat(1, 2))
            return self.down(self.gate(h) * self.up(h))

    context = BucketCommContext.create(device)
    blocks, runtimes, groups = [], [], []
    for index in range(layers):
        block = Projections()
        for j, (name, (out_dim, in_dim)) in enumerate(LLAMA3_8B_LAYER):
            weight = seeded_normal((out_dim, in_dim), 0.02, 7000 + 10 * index + j, device)
            getattr(block, name).weight = nn.Parameter(weight)
        convert_to_flex_shard_float8_blockwise_linear(block)
        fqns = [f"{name}.weight" for name, _ in LLAMA3_8B_LAYER]
        named = [(fqn, block.get_parameter(fqn)) for fqn in fqns]
        placement = Fp8BucketedBlockShard(world_size=world, weight_factory=make_blockwise_fp8_weight)
        group = LocalReduceGroup(world, 0)
        for other in range(1, world):  # what the other ranks would send: their quantized, packed shards
            mesh_o = FakeMesh(world, other)
            infos_o = make_param_infos(named, placement, mesh_o)
            shards_o = [local_rows(p, i) for (_, p), i in zip(named, infos_o)]
            group.gather_rows[other] = placement.prepare_unshard_bucket(shards_o, infos_o, mesh_o, None).buffers[0]
        runtime = BucketRuntime.shard_module_params(
            block, fqns, placement, FakeMesh(world, 0, group), context, GradientReduction()
        )
        del named
        blocks.append(block)
        runtimes.append(runtime)
        groups.append(group)
    model = nn.Sequential(*blocks)
    for index, (block, runtime) in enumerate(zip(blocks, runtimes)):
        runtime.install_hooks(
            block,
            forward_prefetch=runtimes[index + 1] if index + 1 < layers else None,
            backward_prefetch=runtimes[index - 1] if index > 0 else None,
        )
    torch.cuda.empty_cache()

    # host time inside the runtime's entry points, by name
    host_us: dict[str, float] = {}
    calls: dict[str, int] = {}

    def timed(obj, name):
        inner = getattr(obj, name)

        def wrapper(*args, **kwargs):
            t0 = time.perf_counter()
            try:
                return inner(*args, **kwargs)
            finally:
                host_us[name] = host_us.get(name, 0.0) + (time.perf_counter() - t0) * 1e6
                calls[name] = calls.get(name, 0) + 1

        setattr(obj, name, wrapper)

    for runtime in runtimes:
        for name in ("unshard", "prefetch", "reshard", "reduce_grads"):
            timed(runtime, name)

    x = seeded_normal((tokens, 4096), 1.0, 7900, device).requires_grad_()
    grad_out = seeded_normal((tokens, 4096), 0.01, 7901, device)

    # The other ranks' reduce-scatter inputs: one [world, world x widest rank range] fp32 tensor
    # shared by the blocks' groups; row 0 is written by every reduction's copy-in.
    widest = max(runtimes[0].infos[0].bucket_layout.rank_numels)
    contributions = torch.empty((world, world * widest), dtype=torch.float32, device=device)
    contributions[1:].normal_(0.0, 1e-3)
    for group in groups:
        group.contributions = contributions

    def step():
        for group in groups:
            group.mark_deposited(*range(1, world))
        x.grad = None
        for runtime in runtimes:
            for p in runtime.sharded_params:
                p.grad = None
        model(x).backward(grad_out)
        context.wait_and_clear_reduce_grad_states()

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    host_us.clear()
    calls.clear()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        step()
    t_issued = time.perf_counter()
    stop.record()
    torch.cuda.synchronize()
    t_done = time.perf_counter()
    span_ms = start.elapsed_time(stop) / steps
    flop = 3 * 2 * tokens * sum(o * i for _, (o, i) in LLAMA3_8B_LAYER) * layers
    return {
        "workload": f"{layers} blocks of the seven Llama-3-8B projections, {tokens} tokens, forward + backward, rank 0 of "
        f"{world} (LocalReduceGroup), Fp8BucketedBlockShard under BucketRuntime.install_hooks with prefetch, "
        "fp32 gradient reduction",
        "span_ms_per_step": round(span_ms, 3),
        "host_issue_ms_per_step": round((t_issued - t0) * 1e3 / steps, 3),
        "host_issue_share_of_span": round((t_issued - t0) / max(t_done - t0, 1e-9), 3),
        "gemm_flop_per_step": flop,
        "gemm_TFLOPs_over_span": round(flop / span_ms / 1e9, 1),
        "host_us_per_call_in_runtime_entry": {k: round(v / calls[k], 1) for k, v in sorted(host_us.items())},
        "runtime_entry_calls_per_step": {k: v // steps for k, v in sorted(calls.items())},
    }


def calibrate_copy(device, nbytes: int = 256 << 20, reps: int = 4) -> None:
    """A plain copy of known size through copy_segments_kernel: reads `nbytes`
    and writes `nbytes` per launch."""
    from flex_shard_amd.custom_placements._copy_kernels import SegmentCopyDescriptor, copy_segments

    src = torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device=device)
    dst = torch.empty_like(src)
    desc = SegmentCopyDescriptor.create(src_offsets=[0], numels=[nbytes // 4], dst_offsets=[0], device=device)
    for _ in range(reps):
        copy_segments(src.view(torch.int32), dst.view(torch.int32), desc)
    torch.cuda.synchronize()
    if not torch.equal(src, dst):
        raise SystemExit("bench: calibration copy produced wrong bytes")


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50, help="timed passes over the layer buckets")
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--layers", type=int, default=8, help="distinct layer buckets the steps rotate over")
    ap.add_argument("--skip-cpu", action="store_true")
    ap.add_argument("--skip-secondary", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB -> 256 MiB segment copy, the known-size kernel that the "
                    "FETCH_SIZE / WRITE_SIZE counter readings are scaled by")
    ap.add_argument("--only", choices=("muon", "fp8_linear", "runtime_layer_step", "unpack", "gradients",
                                       "side_stream_copies", "other_shares"),
                    help="profiling aid: run only this secondary section (for counter runs, which slow "
                    "every kernel down) and print its figures instead of the benchmark line")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit(
            "bench.py measures one rank's share of the path on one GPU; this build has no collectives, "
            "so --gpus must be 1."
        )
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs an MI355X; no GPU is visible.")
    from flex_shard_amd import _native

    _native.lib()  # fail loudly if the HIP library is missing
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)

    if args.calibrate_copy:
        calibrate_copy(device)
    if args.only in ("unpack", "gradients"):
        if args.only == "unpack":
            placement, mesh, infos, work = build_quant_workload(device, 1)
            del work
            out = {"unpack_gathered_layout": bench_unpack(device, placement, infos)}
        else:
            out = {"gradient_path": bench_gradients(device)}
        print(json.dumps(out))
        return
    if args.only == "muon":
        print(json.dumps({"muon_newton_schulz": bench_muon(device)}))
        return
    if args.only == "other_shares":
        print(json.dumps({"quantize_pack_other_shares": bench_other_shares(device)}))
        return
    if args.only == "runtime_layer_step":
        print(json.dumps({"runtime_layer_step": bench_runtime_layer_step(device)}))
        return
    if args.only == "side_stream_copies":
        print(json.dumps({"side_stream_copies": bench_side_stream_copies(device)}))
        return
    if args.only == "fp8_linear":
        print(json.dumps({"fp8_linear_forward_8192_tokens": bench_fp8_linear(device),
                          "fp8_linear_backward_8192_tokens": bench_fp8_linear_backward(device)}))
        return
    q = bench_quant_pack(device, args.steps, args.warmup, args.layers, extras=True)
    placement, infos, work, metadata, mesh = q.pop("work")
    check_against_oracle(placement, infos, work, metadata, mesh)
    q.pop("two_stream_last")
    launches = args.steps * q["launches_per_step"]
    step_bytes = q["algo_bytes"] * q["launches_per_step"]
    ms_per_step = q["wall_ms"] / args.steps
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    kernel_ms = q["event_ms"] / launches
    achieved = q["algo_bytes"] / (kernel_ms * 1e-3) / 1e9
    traffic, traffic_commit = profiled_traffic(q["elems"], q["payload_nbytes"])

    result = {
        "metric": "FP8 quantize+pack GB/s (% HBM peak), Llama-3-8B layer bucket; Muon NS TFLOP/s",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16->fp8_e4m3fn (fp32 scales)",
        "data": "synthetic: seeded N(0, 0.02) bf16 shards, random-init",
        "config": {
            "workload": "Llama-3-8B layer bucket (q,k,v,o,gate,up,down), rank 0 of 8: q, k, v, o[0:512] = "
            f"{q['elems']} bf16 elements in {q['chunks']} chunks -> {q['payload_nbytes']}-byte FP8 payload, "
            f"128x128 tiles; one step = one pass over {args.layers} layer buckets, one launch each (cold HBM); "
            "every bucket packed twice untimed before the warm-up (launch tables and allocator blocks in place)",
            "launches_per_step": q["launches_per_step"],
            "device": torch.cuda.get_device_name(0),
            "percent_of_hbm_peak": round(100 * value / HBM_PEAK_GBPS, 1),
        },
        "roofline": {
            "bound": "hbm",
            "kernel": "quantize_pack_bf16_kernel",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "traffic": traffic,
            "traffic_measured_at_commit": traffic_commit,
            "algorithmic_bytes_per_launch": q["algo_bytes"],
            "avg_launch_us": round(kernel_ms * 1e3, 2),
            "avg_launch_us_hot_cache": round(q["hot_us"], 2),
        },
        # The same launch through the contract method (payload-cache
        # bookkeeping, pack, allocation of the W x row gather output), the host
        # time either call takes to issue, and the rate with two buckets in
        # flight on two default-priority streams.
        "contract_entry": {
            "entry": "Fp8BucketedBlockShard.prepare_unshard_bucket (what `value` and `roofline` are timed through)",
            "prepare_unshard_bucket_host_us_per_call": round(q["contract_host_us"], 2),
            "two_buckets_in_flight": {
                "how": "the same calls with torch's current stream alternating between two default-priority "
                "side streams (torch.cuda.set_stream), payloads from each stream's recycled buffers",
                "streams": 2,
                "us_per_launch": round(q["two_stream_us"], 2),
                "host_us_per_call": round(q["two_stream_host_us"], 2),
                "GBps": round(q["algo_bytes"] / q["two_stream_us"] / 1e3, 1),
                "frac_of_hbm_peak": round(q["algo_bytes"] / q["two_stream_us"] / 1e3 / HBM_PEAK_GBPS, 4),
            },
        },
    }
    if not args.skip_cpu:
        median_s, reps, threads = cpu_baseline_quant(work, infos, metadata)
        result["cpu_baseline"] = {
            "value": round(q["algo_bytes"] / median_s / 1e9, 3),
            "unit": "GB/s",
            "cores": threads,
            "kind": "port",
            "sample": f"eager-torch restatement of the reference path on the same rank-0 share "
            f"({q['elems']} elements), median of {reps} runs, {threads} threads of {os.cpu_count()} logical CPUs",
        }
    del work
    torch.cuda.empty_cache()
    if not args.skip_secondary:
        secondary = {}
        secondary["quantize_pack_other_shares"] = {
            name: {k: (round(v, 4) if isinstance(v, float) else v) for k, v in d.items()}
            for name, d in bench_other_shares(device).items()
        }
        torch.cuda.empty_cache()
        secondary["unpack_gathered_layout"] = {k: round(v, 3) if isinstance(v, float) else v
                                               for k, v in bench_unpack(device, placement, infos).items()}
        torch.cuda.empty_cache()
        secondary["gradient_path"] = {k: round(v, 3) for k, v in bench_gradients(device).items()}
        torch.cuda.empty_cache()
        muon = bench_muon(device)
        secondary["muon_newton_schulz"] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in muon.items()}
        if not args.skip_cpu:
            secondary["gradient_path"]["cpu_baseline"] = cpu_baseline_gradients()
            secondary["muon_newton_schulz"]["cpu_baseline"] = cpu_baseline_newton_schulz(muon["ns_flop"])
        torch.cuda.empty_cache()
        secondary["fp8_linear_forward_8192_tokens"] = {
            name: {k: round(v, 4) for k, v in d.items()} for name, d in bench_fp8_linear(device).items()
        }
        torch.cuda.empty_cache()
        secondary["fp8_linear_backward_8192_tokens"] = {
            name: {k: round(v, 4) for k, v in d.items()} for name, d in bench_fp8_linear_backward(device).items()
        }
        torch.cuda.empty_cache()
        secondary["runtime_layer_step"] = bench_runtime_layer_step(device)
        torch.cuda.empty_cache()
        secondary["side_stream_copies"] = {
            k: ({kk: round(vv, 3) for kk, vv in v.items()} if isinstance(v, dict) else round(v, 3) if isinstance(v, float) else v)
            for k, v in bench_side_stream_copies(device).items()
        }
        result["secondary"] = secondary
    print(json.dumps(result))


if __name__ == "__main__":
    main()
