"""Single-process harness pieces: a mesh that needs no process group, ParamInfo
construction for any rank, and the synthetic workloads of the benchmarks.

``FakeMesh`` and ``make_param_infos`` have the behaviour of the reference's test
helpers (tests/common.py:260-305); the rank-loop helpers build a gathered
buffer on one GPU from locally quantized seeded shards, the way the reference's
``_prepare_unshard_on_each_rank`` (tests/test_flex_shard_fp8_allgather.py
:191-207) does.
"""

from __future__ import annotations

import math
from collections.abc import Sequence

import torch
import torch.nn as nn

from .bucket_storage import ParamInfo, create_param_infos
from .placement_contract import Placement


class FakeMesh:
    """The three mesh methods the placements call, without a process group."""

    def __init__(self, size: int, rank: int = 0, group=None) -> None:
        self._size, self._rank, self._group = size, rank, group

    def size(self) -> int:
        return self._size

    def get_local_rank(self) -> int:
        return self._rank

    def get_group(self):
        return self._group


def make_param_infos(named_params: list[tuple[str, nn.Parameter]], placement: Placement, mesh) -> list[ParamInfo]:
    """ParamInfos of parameters sharing one placement's bucket storage layout."""
    return create_param_infos(named_params, {fqn: (placement,) for fqn, _ in named_params}, mesh)[0]


def make_mixed_param_infos(
    named_params: list[tuple[str, nn.Parameter]], param_placements: dict[str, tuple[Placement, ...]], mesh
) -> list[ParamInfo]:
    """ParamInfos of a bucket whose parameters carry different member
    placements of one bucket-scoped placement (a mixed bucket): the first
    parameter's placement lays out the bucket."""
    return create_param_infos(named_params, param_placements, mesh)[0]


def local_rows(param: torch.Tensor, info: ParamInfo) -> torch.Tensor:
    """The rank's shard of ``param``: a row range of its flattened matrix."""
    if info.local_numel == 0:
        return param.new_empty(info.local_shape)
    layout = info.bucket_layout.param_layouts[info.fqn]
    in_dim = param.shape[-1]
    start = (layout.local_global_offset - layout.param_offset) // in_dim
    rows = info.local_numel // in_dim
    return param.detach().flatten(0, -2)[start : start + rows].reshape(info.local_shape)


def prepare_unshard_on_each_rank(placement, named_params, world_size: int) -> list:
    """Run ``prepare_unshard_bucket`` as every rank of a ``world_size`` mesh."""
    prepared = []
    for rank in range(world_size):
        mesh = FakeMesh(world_size, rank)
        infos = make_param_infos(named_params, placement, mesh)
        shards = [local_rows(p, i) for (_, p), i in zip(named_params, infos, strict=True)]
        prepared.append(placement.prepare_unshard_bucket(shards, infos, mesh, None))
    return prepared


def gather_rank_rows(prepared_by_rank: Sequence) -> torch.Tensor:
    """The gathered [W, row] buffer built on one GPU from every rank's payload."""
    return torch.stack([p.buffers[0] for p in prepared_by_rank])


# ------------------------------------------------------------------ workloads
LLAMA3_8B_LAYER = (
    ("q", (4096, 4096)),
    ("k", (1024, 4096)),
    ("v", (1024, 4096)),
    ("o", (4096, 4096)),
    ("gate", (14336, 4096)),
    ("up", (14336, 4096)),
    ("down", (4096, 14336)),
)

DEEPSEEK_V3_EXPERTS = (
    ("experts.w1", (32, 2048, 7168)),
    ("experts.w2", (32, 7168, 2048)),
    ("experts.w3", (32, 2048, 7168)),
)


def seeded_normal(shape, std: float, seed: int, device, dtype=torch.bfloat16) -> torch.Tensor:
    """N(0, std) values from a seeded generator on ``device``."""
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    out = torch.empty(shape, dtype=torch.float32, device=device)
    out.normal_(0.0, std, generator=gen)
    return out.to(dtype)


def seeded_bucket(spec, std: float, seed: int, device, dtype=torch.bfloat16) -> list[tuple[str, nn.Parameter]]:
    return [
        (name, nn.Parameter(seeded_normal(shape, std, seed + 1000 * i, device, dtype), requires_grad=False))
        for i, (name, shape) in enumerate(spec)
    ]


def add_outliers_and_zero_tiles(weight: torch.Tensor, seed: int, block: int = 128) -> None:
    """In place: multiply 0.1% of the entries by 50 and zero a seeded set of
    whole tiles of the flattened matrix (scale edge cases)."""
    gen = torch.Generator(device=weight.device)
    gen.manual_seed(seed)
    flat = weight.data.view(-1, weight.shape[-1])
    mask = torch.rand(flat.shape, generator=gen, device=weight.device) < 1e-3
    flat[mask] = (flat[mask].float() * 50).to(flat.dtype)
    rows, cols = flat.shape
    tiles_r, tiles_c = math.ceil(rows / block), math.ceil(cols / block)
    picks = torch.randint(0, tiles_r * tiles_c, (8,), generator=gen, device=weight.device).tolist()
    for pick in picks:
        tr, tc = divmod(pick, tiles_c)
        flat[tr * block : (tr + 1) * block, tc * block : (tc + 1) * block] = 0
