"""CPU checks of the boundary: the shared library loads and exports exactly the
symbols include/flexshard_hip.h declares (no compute calls), the package
refuses to compute off the GPU, and the owner placement's host math."""

import ctypes
import os
import re

import pytest
import torch
import torch.nn as nn

from flex_shard_amd import BucketedOwned, BucketedOwnedSegmentSpec, _native, hip_ops
from flex_shard_amd.custom_placements import (
    BlockShard,
    make_bucketed_owned_expert_block_segments,
    make_bucketed_owned_full_param_segments,
)
from flex_shard_amd.custom_placements.owner_balance import assign_to_hosts_then_ranks, lpt_owners, mesh_rank_hosts
from flex_shard_amd.testing import FakeMesh, make_param_infos
from oracle import layout as olayout

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "flexshard_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fsh_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    declared = _declared_symbols()
    assert len(declared) >= 14
    handle = ctypes.CDLL(_native.LIB_PATH)
    for name in declared:
        assert hasattr(handle, name), f"{name} is declared in the header but not exported"
    assert sorted(_native.SIGNATURES) == declared
    lib = _native.lib()
    assert lib.fsh_version() >= 1
    assert isinstance(lib.fsh_last_error(), bytes)  # empty until a call of this thread has failed


def test_struct_sizes_match_the_header():
    assert ctypes.sizeof(_native.QuantChunk) == 56
    assert ctypes.sizeof(_native.UnpackChunk) == 56
    assert ctypes.sizeof(_native.GemmDesc) == 5 * 8 + 14 * 8 + 2 * 4 + 2 * 4 + 2 * 4
    assert ctypes.sizeof(_native.MuonGroup) == 9 * 8 + 2 * 4 + 2 * 4
    assert ctypes.sizeof(_native.NsProblem) == 6 * 8


def test_host_side_argument_checks_need_no_gpu():
    lib = _native.lib()
    assert lib.fsh_quantize_pack(None, 99, None, 0, 0, 0, 0, 0, 128, 0, None) == -22
    assert b"nchunks" in lib.fsh_last_error()
    assert lib.fsh_quantize_pack(None, 0, None, 0, 0, 0, 0, 0, 0, 0, None) == -22
    assert lib.fsh_copy_segments(None, None, None, None, None, 1, 1, 3, None) == -22
    assert b"unit_nbytes" in lib.fsh_last_error()
    assert lib.fsh_newton_schulz(None, 1, 7, 8, 1.0, 1.0, 1.0, 5, 1e-7, None, 0, None) == -22
    assert lib.fsh_newton_schulz_workspace_bytes(24, 7168, 2048) > 2 * 24 * 7168 * 2048 * 2
    assert lib.fsh_accumulate_grad(None, None, 0, 0, 0, None) == 0  # empty is a no-op
    # whole Muon step: list and group checks come before any launch
    assert lib.fsh_muon_step(None, 1, 0.05, 0.95, 1, 1.0, 1.0, 1.0, 1.0, 5, 1e-7, None) == -22
    assert b"null list" in lib.fsh_last_error()
    assert lib.fsh_muon_step(None, 0, 0.05, 0.95, 1, 1.0, 1.0, 1.0, 1.0, 5, 1e-7, None) == 0  # no group: nothing to do
    group = _native.MuonGroup()
    group.batch, group.rows, group.cols = 1, 12, 8  # rows not a multiple of 8
    assert lib.fsh_muon_step(ctypes.byref(group), 1, 0.05, 0.95, 1, 1.0, 1.0, 1.0, 1.0, 5, 1e-7, None) == -22
    assert b"multiples of 8" in lib.fsh_last_error()
    group.rows = 16
    assert lib.fsh_muon_step(ctypes.byref(group), 1, 0.05, 0.95, 1, 1.0, 1.0, 1.0, 1.0, 5, 1e-7, None) == -22
    assert b"null pointer" in lib.fsh_last_error()
    # FP8 GEMM limits
    assert lib.fsh_fp8_gemm_1x128_128x1(None, None, None, None, None, 8, 8, 100, 128, 128, 8, None) == -22


def test_more_argument_checks_that_need_no_gpu():
    """Sizes, null pointers and modes are refused before anything is queued,
    so these calls are safe where there is no GPU; an empty request is a no-op."""
    lib = _native.lib()
    fake = 4096  # an aligned address that is never dereferenced: every call below fails (or returns) before a launch
    EINVAL, ENOTSUP = -22, -95
    assert lib.fsh_reduce_rows_f32(None, None, 0, 0, 0, 4, 0, 1.0, None) == EINVAL  # world 0
    assert lib.fsh_reduce_rows_f32(None, None, 8, 2, 0, 4, 0, 1.0, None) == EINVAL  # null pointers
    assert lib.fsh_reduce_rows_f32(fake, fake, 8, 2, 0, 4, 9, 1.0, None) == EINVAL
    assert b"mode" in lib.fsh_last_error()
    assert lib.fsh_reduce_rows_f32(None, None, 8, 2, 0, 0, 0, 1.0, None) == 0
    assert lib.fsh_reduce_rows_bf16(None, None, 0, 0, 0, 4, 0, 1.0, None) == EINVAL
    assert lib.fsh_reduce_rows_bf16(fake, fake, 8, 2, 0, 8, 9, 1.0, None) == EINVAL
    assert b"fsh_reduce_rows_bf16" in lib.fsh_last_error()
    assert lib.fsh_reduce_rows_bf16(None, None, 8, 2, 0, 0, 0, 1.0, None) == 0
    assert lib.fsh_zero_segments(None, None, None, 1, 1, 4, None) == EINVAL
    assert lib.fsh_zero_segments(None, None, None, 0, 1, 4, None) == 0
    assert lib.fsh_pack_segments(None, None, None, None, None, 1, 1, 0, 1, None, None) == EINVAL
    assert lib.fsh_pack_segments(fake, fake, fake, fake, fake, 1, 1, 7, 1, fake, None) == EINVAL  # unknown dtype pair
    assert lib.fsh_pack_segments(None, None, None, None, None, 0, 0, 0, 1, None, None) == 0
    assert lib.fsh_quant_pack_plan_create(None, 1, 0, 0, 0, 0, 0, 128, 0, None) == EINVAL  # no place for the handle
    handle = ctypes.c_void_p()
    assert lib.fsh_quant_pack_plan_create(None, 1, 0, 0, 0, 0, 0, 128, 0, ctypes.byref(handle)) == EINVAL
    assert handle.value is None
    assert lib.fsh_quant_pack_plan_launch(None, None, None) == EINVAL
    lib.fsh_quant_pack_plan_destroy(None)  # destroying nothing is allowed
    # the allocation-free Newton-Schulz refuses what its fixed scratch cannot hold
    assert lib.fsh_newton_schulz_noalloc(fake, 0, 8, 8, 1.0, 1.0, 1.0, 5, 1e-7, None) == EINVAL
    assert lib.fsh_newton_schulz_noalloc(fake, 24, 7168, 2048, 1.0, 1.0, 1.0, 5, 1e-7, None) == ENOTSUP
    assert b"static scratch" in lib.fsh_last_error()
    assert lib.fsh_newton_schulz_noalloc(fake, 1 << 20, 8, 8, 1.0, 1.0, 1.0, 5, 1e-7, None) == ENOTSUP


def test_no_cpu_compute_path():
    with pytest.raises(RuntimeError, match="GPU"):
        hip_ops.accumulate_grad(torch.zeros(4), torch.zeros(4, dtype=torch.bfloat16))
    from flex_shard_amd import Fp8BucketedBlockShard

    pl = Fp8BucketedBlockShard(world_size=1, weight_factory=lambda *a, **k: a[0], block_size=4)
    param = nn.Parameter(torch.zeros(4, 4))
    infos = make_param_infos([("w", param)], pl, FakeMesh(1))
    with pytest.raises(RuntimeError, match="no CPU compute path"):
        pl.prepare_unshard_bucket([param.detach()], infos, FakeMesh(1), None)
    from flex_shard_amd.dist_muon import _zeropower_via_newtonschulz

    with pytest.raises(RuntimeError, match="GPU"):
        _zeropower_via_newtonschulz(torch.zeros(8, 8))


# ------------------------------------------------------------- BucketedOwned
def _named(shapes, dtype=torch.bfloat16):
    return [(f"p{i}", nn.Parameter(torch.empty(s, device="meta", dtype=dtype))) for i, s in enumerate(shapes)]


def test_lpt_owner_assignment():
    numels = [9, 7, 7, 5, 3, 3, 1]
    owners = lpt_owners(numels, 3)
    assert owners == olayout.lpt_owners(numels, 3)
    loads = [sum(n for n, o in zip(numels, owners) if o == r) for r in range(3)]
    assert max(loads) <= 13  # LPT bound for this instance: optimum is 12
    assert lpt_owners([4, 4, 4], 3) == [0, 1, 2]  # ties go to the lower rank, equal sizes keep order
    assert lpt_owners([5, 5], 2, carried_loads=[10, 0]) == [1, 1]


def test_host_then_rank_assignment():
    assert mesh_rank_hosts([0, 1, 2, 3, 8, 9], ranks_per_host=4) == (0, 0, 0, 0, 1, 1)
    hosts = mesh_rank_hosts(list(range(8)), ranks_per_host=2)  # 4 hosts of 2
    owners = assign_to_hosts_then_ranks([8, 7, 6, 5], hosts)
    # largest loads go to hosts 0, 2, 1, 3 (even-first tie order), first rank of each
    assert owners == [0, 4, 2, 6]
    with pytest.raises(ValueError, match="numbered"):
        assign_to_hosts_then_ranks([1], [0, 2])
    with pytest.raises(ValueError, match="don't fit"):
        assign_to_hosts_then_ranks([1, 1, 1], [0, 0], one_per_rank=True)
    assert sorted(assign_to_hosts_then_ranks([3, 2], [0, 0], one_per_rank=True)) == [0, 1]


def test_full_param_segments_and_lowering():
    named = _named([(7168, 2048), (2048, 2048), (7168, 2048), (2048, 2048)])
    segments = make_bucketed_owned_full_param_segments(named, 2)
    assert {f: s[0].owner_rank for f, s in segments.items()} == {"p0": 0, "p2": 1, "p1": 0, "p3": 1}
    placement = BucketedOwned(segments)
    assert placement == BucketedOwned(segments) and hash(placement) == hash(BucketedOwned(segments))
    assert repr(placement) == "BucketedOwned(num_params=4, view_kind='full_param')"
    lowered = placement._lower_to_block_shards({f: tuple(p.shape) for f, p in named}, 2)
    assert lowered["p0"] == BlockShard((1, 0)) and lowered["p2"] == BlockShard((0, 1))
    assert placement.owned_fqns(0) == ["p0", "p1"]
    with pytest.raises(ValueError, match="view_kind"):
        BucketedOwned(segments, view_kind="bogus")
    with pytest.raises(ValueError, match="at least one segment"):
        BucketedOwned({"p0": []})
    bad = BucketedOwnedSegmentSpec("x", "other", 0, 4, 0)
    with pytest.raises(ValueError, match="names FQN"):
        BucketedOwned({"p0": [bad]})
    with pytest.raises(NotImplementedError, match="mixed-bucket"):
        placement.prepare_unshard_bucket([], [], FakeMesh(2), None)


def test_owned_storage_layout_is_the_owner_row():
    """Each owner stores its whole parameters back to back, grouped by owner in
    first-appearance order; non-owners store nothing."""
    shapes = [(8, 4), (4, 4), (8, 4), (4, 4), (2, 4)]
    named = _named(shapes, torch.float32)
    placement = BucketedOwned(make_bucketed_owned_full_param_segments(named, 2))
    owners = {f: s[0].owner_rank for f, s in placement.segments_by_fqn.items()}
    for rank in range(2):
        infos = make_param_infos(named, placement, FakeMesh(2, rank))
        cursor = 0
        for (fqn, param), info in zip(named, infos):
            if owners[fqn] == rank:
                assert tuple(info.local_shape) == tuple(param.shape) and info.byte_offset == cursor * 4
                cursor += param.numel()
                layout = placement.global_layout(info, rank, 2)
                assert layout.global_offsets == ((0, 0),) and layout.local_sizes == (tuple(param.shape),)
            else:
                assert info.local_numel == 0 and info.storage_nbytes == 0
    with pytest.raises(ValueError, match="match the bucket FQNs"):
        placement.bucket_storage_layout(named[:2], {f: (placement,) for f, _ in named[:2]}, FakeMesh(2))


def test_expert_block_segments():
    named = [
        ("moe.w1", nn.Parameter(torch.empty(4, 2, 6, device="meta"))),
        ("moe.w2", nn.Parameter(torch.empty(4, 6, 2, device="meta"))),
        ("moe.w3", nn.Parameter(torch.empty(4, 2, 6, device="meta"))),
    ]
    segments = make_bucketed_owned_expert_block_segments(named, 2)
    assert [s.owner_rank for s in segments["moe.w1"]] == [0, 0, 1, 1]
    assert [s.param_offset for s in segments["moe.w2"]] == [0, 12, 24, 36]
    placement = BucketedOwned(segments, view_kind="expert_block")
    lowered = placement._lower_to_block_shards({f: tuple(p.shape) for f, p in named}, 2)
    assert lowered["moe.w3"] == BlockShard((2, 2))
    with pytest.raises(ValueError, match="at least 3 dims"):
        make_bucketed_owned_expert_block_segments([("x.w1", nn.Parameter(torch.empty(4, 2, device="meta")))], 2)


def test_block_shard_layout_math():
    shard = BlockShard(blocks_per_rank=(2, 1))
    assert shard.compute_local_shape(torch.Size((6, 4)), 0, 2) == torch.Size((4, 4))
    assert shard.compute_local_shape(torch.Size((6, 4)), 1, 2) == torch.Size((2, 4))
    full = torch.arange(24.0).view(6, 4)
    assert torch.equal(shard.extract_local_shard(full, 1, 2), full[4:])
    with pytest.raises(ValueError, match="divisible"):
        shard.compute_local_shape(torch.Size((7, 4)), 0, 2)
    with pytest.raises(ValueError, match="world size"):
        shard.compute_local_shape(torch.Size((6, 4)), 0, 3)
    assert repr(BlockShard((1, 0), dim=1)) == "BlockShard(blocks_per_rank=(1, 0), dim=1)"


def test_bench_refuses_more_than_one_gpu():
    """One rank's share on one GPU is all the benchmark measures: asking for
    more exits with a message before anything touches a device."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    run = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert run.returncode != 0
    assert "--gpus must be 1" in (run.stdout + run.stderr)
