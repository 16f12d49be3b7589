"""Bucket metadata types the placements read and write.

Only the part of the reference's ``flex_shard/bucket_storage.py`` that crosses
the placement boundary is mirrored: ``BucketParamLayout`` / ``BucketLayout``
(:261-277) and the ``ParamInfo`` fields and dtype properties the hot path uses
(:280-343).  The storage engine itself (``ShardedBucketStorage``) is the
caller's side of the boundary and is not part of this package.
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


__all__ = ["BucketLayout", "BucketParamLayout", "ParamInfo"]
