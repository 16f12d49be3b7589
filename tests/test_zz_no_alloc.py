"""The allocation-free Newton-Schulz entry point (static device scratch)
against the workspace-taking entry point it is a variant of: same kernels, so
the results must be equal bit for bit.  Two calls in a row share the scratch,
the second with a smaller input that finds the first call's contents there."""

import pytest
import torch

from flex_shard_amd import _native, hip_ops
from flex_shard_amd.testing import seeded_normal

pytestmark = pytest.mark.gpu

COEFFS = (3.4445, -4.7750, 2.0315)


def _with_workspace(x):
    return hip_ops.newton_schulz(x.clone(), COEFFS, 5, 1e-7)


def test_noalloc_newton_schulz_equals_the_workspace_entry_point(device):
    torch.cuda.synchronize()
    # large-tile, one-orientation flow: 192 matrices of 256 x 256 (96.2 MB of scratch) ...
    first = seeded_normal((192, 256, 256), 1.0, 51, device)
    # ... then a smaller, tall batch on the small-tile kernels, over what the first call left behind
    second = seeded_normal((3, 200, 136), 1.0, 52, device)
    third = seeded_normal((2, 512, 768), 1.0, 53, device)
    want = [_with_workspace(x) for x in (first, second, third)]
    assert hip_ops.newton_schulz_workspace_bytes(192, 256, 256) <= _native.NS_STATIC_SCRATCH_BYTES
    got_first = hip_ops.newton_schulz_noalloc(first.clone(), COEFFS, 5, 1e-7)
    got_second = hip_ops.newton_schulz_noalloc(second.clone(), COEFFS, 5, 1e-7)
    got_third = hip_ops.newton_schulz_noalloc(third.clone(), COEFFS, 5, 1e-7)
    again_first = hip_ops.newton_schulz_noalloc(first.clone(), COEFFS, 5, 1e-7)
    torch.cuda.synchronize()
    assert torch.equal(got_first, want[0])
    assert torch.equal(got_second, want[1])
    assert torch.equal(got_third, want[2])
    assert torch.equal(again_first, want[0])
    # and against torch's own routine, at the reference's bar
    from torch.optim._muon import _zeropower_via_newtonschulz as torch_ns

    ref = torch_ns(second[0].cpu(), COEFFS, 5, 1e-7)
    assert (got_second[0].cpu().float() - ref.float()).abs().max().item() <= 2e-2


def test_noalloc_newton_schulz_allocates_nothing_and_rejects_oversize(device):
    x = seeded_normal((4, 256, 384), 1.0, 54, device)
    hip_ops.newton_schulz_noalloc(x.clone(), COEFFS, 5, 1e-7)  # first call on the device resolves the scratch address
    y = x.clone()
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats(device)["allocation.all.allocated"]
    free_before, _ = torch.cuda.mem_get_info(device)
    hip_ops.newton_schulz_noalloc(y, COEFFS, 5, 1e-7)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info(device)
    assert torch.cuda.memory_stats(device)["allocation.all.allocated"] == before
    assert free_after == free_before
    # 24 x [2048, 2048] needs 805 MB of workspace: beyond the static scratch
    big = torch.empty((24, 2048, 2048), dtype=torch.bfloat16, device=device)
    assert hip_ops.newton_schulz_workspace_bytes(24, 2048, 2048) > _native.NS_STATIC_SCRATCH_BYTES
    with pytest.raises(_native.NativeError, match="static scratch"):
        hip_ops.newton_schulz_noalloc(big, COEFFS, 5, 1e-7)
    with pytest.raises(_native.NativeError, match="static scratch"):
        _native.check(
            _native.lib().fsh_newton_schulz_noalloc(big.data_ptr(), 65535, 1 << 20, 1 << 20, *COEFFS, 5, 1e-7, 0),
            "fsh_newton_schulz_noalloc",
        )
