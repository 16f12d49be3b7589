"""The torch.distributed branch of the two exchange wrappers on a 2-rank gloo
group on the CPU (the branch a multi-GPU run takes with RCCL): equal payload
rows are gathered in rank order, and a SUM reduce-scatter of packed gradients
gives every rank its range of the element-wise sum.  The one-GPU stand-in
(LocalReduceGroup) is covered by the GPU tests."""

import os
import socket

import pytest
import torch
import torch.distributed as dist
import torch.multiprocessing as mp

from flex_shard_amd import GradientReduction
from flex_shard_amd.custom_placements.utils import all_gather_rows, group_size, reduce_scatter_grads

WORLD = 2


def _free_port() -> int:
    with socket.socket() as s:
        s.bind(("127.0.0.1", 0))
        return s.getsockname()[1]


def _worker(rank: int, port: int, failures) -> None:
    os.environ["MASTER_ADDR"], os.environ["MASTER_PORT"] = "127.0.0.1", str(port)
    dist.init_process_group("gloo", rank=rank, world_size=WORLD)
    try:
        group = dist.group.WORLD
        assert group_size(group) == WORLD
        row = 37
        payload = torch.arange(row, dtype=torch.uint8) + 100 * rank
        gathered = torch.zeros(WORLD * row, dtype=torch.uint8)
        work = all_gather_rows(gathered, payload, group)
        assert work is None
        want = torch.cat([torch.arange(row, dtype=torch.uint8) + 100 * r for r in range(WORLD)])
        assert torch.equal(gathered, want), "rows are not in rank order"
        handle = all_gather_rows(gathered.zero_(), payload, group, async_op=True)
        handle.wait()
        assert torch.equal(gathered, want)
        # reduce-scatter of [WORLD, segment] packed gradients, SUM
        segment = 11
        send = (torch.arange(WORLD * segment, dtype=torch.float32) + 1000.0 * rank).contiguous()
        out = torch.empty(segment, dtype=torch.float32)
        try:
            reduce_scatter_grads(out, send, GradientReduction(op="sum"), group)
        except RuntimeError as exc:  # a gloo build without reduce_scatter_tensor
            if "not support" not in str(exc).lower() and "unsupported" not in str(exc).lower():
                raise
        else:
            total = sum(torch.arange(WORLD * segment, dtype=torch.float32) + 1000.0 * r for r in range(WORLD))
            assert torch.equal(out, total[rank * segment : (rank + 1) * segment])
    except Exception as exc:  # noqa: BLE001 - reported to the parent
        failures.put(f"rank {rank}: {type(exc).__name__}: {exc}")
    finally:
        dist.destroy_process_group()


def test_exchange_wrappers_on_a_two_rank_gloo_group():
    ctx = mp.get_context("spawn")
    failures = ctx.Queue()
    port = _free_port()
    procs = [ctx.Process(target=_worker, args=(rank, port, failures)) for rank in range(WORLD)]
    for p in procs:
        p.start()
    for p in procs:
        p.join(120)
        if p.is_alive():
            p.terminate()
            pytest.fail("a rank did not finish")
    problems = []
    while not failures.empty():
        problems.append(failures.get())
    assert not problems, "; ".join(problems)
    assert all(p.exitcode == 0 for p in procs)


def test_wrappers_refuse_a_missing_group():
    with pytest.raises(ValueError, match="needs a process group"):
        all_gather_rows(torch.zeros(4, dtype=torch.uint8), torch.zeros(2, dtype=torch.uint8), None)
    with pytest.raises(ValueError, match="needs a process group"):
        reduce_scatter_grads(torch.zeros(2), torch.zeros(4), GradientReduction(), None)
