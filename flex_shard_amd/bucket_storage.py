"""Bucket metadata types the placements read and write.

Only the part of the reference's ``flex_shard/bucket_storage.py`` that crosses
the placement boundary is mirrored: ``BucketParamLayout`` / ``BucketLayout``
(:261-277) and the ``ParamInfo`` fields and dtype properties the hot path uses
(:280-343), and ``create_param_infos`` (``ShardedBucketStorage.create_param_infos``,
:478-650: the bucket's layout from the first placement, or one parameter after
the other when it declares none).  The storage engine itself
(``ShardedBucketStorage``) is the caller's side of the boundary and is not
part of this package.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import TYPE_CHECKING, Any

import torch

if TYPE_CHECKING:
    from .placement_contract import GlobalLayout, Placement


@dataclass(frozen=True)
class BucketParamLayout:
    """Element offsets of one parameter in the bucket-global flat layout:
    where the parameter starts and where this rank's part of it starts."""

    param_offset: int
    local_global_offset: int


@dataclass(frozen=True)
class BucketLayout:
    """The flat layout shared by every parameter of a bucket."""

    global_numel: int
    local_numel: int
    rank_offsets: tuple[int, ...]
    rank_numels: tuple[int, ...]
    param_layouts: dict[str, BucketParamLayout]


@dataclass
class ParamInfo:
    """Per-parameter metadata handed to every placement hook."""

    fqn: str
    global_shape: torch.Size
    global_stride: tuple[int, ...]
    dtype: torch.dtype
    requires_grad: bool
    placements: tuple["Placement", ...]
    param_dtype: torch.dtype | None = None
    reduce_dtype: torch.dtype | None = None
    local_shape: torch.Size = field(default_factory=lambda: torch.Size([]))
    local_numel: int = 0
    byte_offset: int = 0
    storage_nbytes: int = 0
    global_numel: int = 0
    bucket_layout: BucketLayout | None = None
    outer_layout: "GlobalLayout | None" = None
    partial_grad_group: Any | None = None
    param_attrs: dict[str, Any] = field(default_factory=dict)
    has_explicit_grad_dtype: bool = False
    grad_dtype_override: torch.dtype | None = None
    shared_fqns: tuple[str, ...] = ()
    bucket_reduce_dtype: torch.dtype | None = None

    @property
    def placement(self) -> "Placement":
        if len(self.placements) != 1:
            raise ValueError(f"Expected exactly one placement for {self.fqn!r}, got {len(self.placements)}.")
        return self.placements[0]

    @property
    def unsharded_dtype(self) -> torch.dtype:
        """Dtype of the full parameter the forward sees."""
        return self.param_dtype or self.dtype

    @property
    def unsharded_grad_dtype(self) -> torch.dtype | None:
        """Dtype full-parameter gradients accumulate in (None: any)."""
        if self.reduce_dtype is not None:
            return self.reduce_dtype
        if self.has_explicit_grad_dtype:
            return self.grad_dtype_override
        return self.dtype

    @property
    def grad_reduce_dtype(self) -> torch.dtype:
        """Dtype the gradient is reduced in."""
        return self.bucket_reduce_dtype or self.unsharded_grad_dtype or self.unsharded_dtype


def create_param_infos(
    named_params: list[tuple[str, "torch.nn.Parameter"]],
    param_placements: dict[str, tuple["Placement", ...]],
    mesh: Any,
) -> tuple[list[ParamInfo], int]:
    """ParamInfos of one bucket on this rank, in ``named_params`` order, and
    the bucket's local byte size.  The first parameter's placement lays the
    bucket out (``bucket_storage_layout``); a placement that declares no bucket
    layout gets its parameters one after the other, each as its
    ``local_storage_layout`` says.  A layout the parameter already declares (it
    is a shard of an outer sharding) is kept as ``outer_layout``."""
    from .placement_contract import get_global_layout, get_partial_grad_group

    if not named_params:
        return [], 0
    rank, world_size = mesh.get_local_rank(), mesh.size()
    first = param_placements[named_params[0][0]][0]
    bucket = first.bucket_storage_layout(named_params, param_placements, mesh)
    if bucket is not None:
        expected, actual = {fqn for fqn, _ in named_params}, set(bucket.param_layouts)
        if expected != actual:
            raise ValueError(
                "Placement bucket_storage_layout() must return layouts for exactly the provided parameters; "
                f"missing {sorted(expected - actual)}, unexpected {sorted(actual - expected)}."
            )
    infos, cursor = [], 0
    for fqn, param in named_params:
        placements = param_placements[fqn]
        if bucket is not None:
            layout = bucket.param_layouts[fqn]
            local_shape, local_numel = layout.local_shape, layout.local_numel
            byte_offset, storage_nbytes, bucket_layout = layout.byte_offset, layout.storage_nbytes, layout.bucket_layout
            if min(local_numel, byte_offset, storage_nbytes) < 0:
                raise ValueError(f"Placement bucket_storage_layout() returned a negative size or offset for {fqn!r}.")
            if storage_nbytes > 0 and byte_offset + storage_nbytes > bucket.total_bytes:
                raise ValueError(
                    f"Placement bucket_storage_layout() returned storage for parameter {fqn!r} outside the bucket byte range."
                )
        else:
            if len(placements) != 1:
                raise ValueError(f"Expected exactly one placement for {fqn!r}, got {len(placements)}.")
            local = placements[0].local_storage_layout(param.shape, param.dtype, rank, world_size)
            if local.local_numel < 0 or local.storage_nbytes < 0:
                raise ValueError(f"Placement {placements[0]!r} returned a negative size for parameter {fqn!r}.")
            local_shape, local_numel, storage_nbytes, bucket_layout = (
                local.local_shape, local.local_numel, local.storage_nbytes, None,
            )
            byte_offset = cursor if storage_nbytes else 0
            cursor += storage_nbytes
        infos.append(
            ParamInfo(
                fqn=fqn,
                global_shape=param.shape,
                global_stride=tuple(param.stride()),
                dtype=param.dtype,
                requires_grad=param.requires_grad,
                placements=placements,
                local_shape=local_shape,
                local_numel=local_numel,
                byte_offset=byte_offset,
                storage_nbytes=storage_nbytes,
                global_numel=param.numel(),
                bucket_layout=bucket_layout,
                outer_layout=get_global_layout(param),
                partial_grad_group=get_partial_grad_group(param),
            )
        )
    return infos, (bucket.total_bytes if bucket is not None else cursor)


__all__ = ["BucketLayout", "BucketParamLayout", "ParamInfo", "create_param_infos"]
