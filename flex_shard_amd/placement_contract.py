"""The placement contract: the drop-in boundary of this package.

Same names, fields and call signatures as the reference's
``flex_shard/placement_contract.py`` (dataclasses :25-63, :152-177, :381-454;
``Placement`` :180-378), so a bucket runtime written against the reference can
drive the placements in :mod:`flex_shard_amd.custom_placements` unchanged.
Only the five collective-lifecycle hooks, the storage-layout hooks and the
checkpoint layout hook exist here; the collectives themselves are out of scope
(single GPU), so ``run_prepared_unshard`` on these placements needs a process
group supplied by the caller.
"""

from __future__ import annotations

import math
from abc import ABC, abstractmethod
from dataclasses import dataclass, field
from typing import TYPE_CHECKING, Any, ClassVar

import torch
import torch.distributed as dist

if TYPE_CHECKING:
    import torch.nn as nn

    from .bucket_storage import ParamInfo


@dataclass(frozen=True)
class LocalStorageLayout:
    """Local storage of one parameter under a per-parameter placement."""

    local_shape: torch.Size
    local_numel: int
    storage_nbytes: int


@dataclass(frozen=True)
class BucketParamStorageLayout:
    """Where one parameter's local shard sits in its bucket's byte storage."""

    local_shape: torch.Size
    local_numel: int
    byte_offset: int
    storage_nbytes: int
    bucket_layout: Any | None = None


@dataclass(frozen=True)
class BucketStorageLayout:
    """Per-parameter storage layouts of a bucket and the bucket's local size."""

    param_layouts: dict[str, BucketParamStorageLayout]
    total_bytes: int


@dataclass(frozen=True)
class GlobalLayout:
    """Boxes of the full parameter held by one rank's local tensor (the field
    names of DCP's checkpointable-tensor protocol)."""

    global_shape: tuple[int, ...]
    global_offsets: tuple[tuple[int, ...], ...]
    local_offsets: tuple[tuple[int, ...], ...]
    local_sizes: tuple[tuple[int, ...], ...]


_LAYOUT_FIELDS = ("global_shape", "global_offsets", "local_offsets", "local_sizes")


def get_global_layout(tensor: torch.Tensor) -> GlobalLayout | None:
    """The layout ``tensor`` declares through its attributes, if any."""
    if not all(hasattr(tensor, name) for name in _LAYOUT_FIELDS):
        return None
    return GlobalLayout(
        global_shape=tuple(tensor.global_shape),
        global_offsets=tuple(tuple(o) for o in tensor.global_offsets),
        local_offsets=tuple(tuple(o) for o in tensor.local_offsets),
        local_sizes=tuple(tuple(s) for s in tensor.local_sizes),
    )


def set_global_layout(tensor: torch.Tensor, layout: GlobalLayout) -> None:
    """Declare where ``tensor`` sits in the full parameter."""
    for name in _LAYOUT_FIELDS:
        setattr(tensor, name, getattr(layout, name))


_PARTIAL_GRAD_GROUP_ATTR = "_flex_shard_partial_grad_group"


def set_partial_grad_group(tensor: torch.Tensor, group: Any) -> None:
    """Mark ``tensor``'s gradient as partial over ``group`` (summed before the
    bucket reduction)."""
    setattr(tensor, _PARTIAL_GRAD_GROUP_ATTR, group)


def get_partial_grad_group(tensor: torch.Tensor) -> Any | None:
    return getattr(tensor, _PARTIAL_GRAD_GROUP_ATTR, None)


def compose_global_layouts(outer: GlobalLayout, inner: GlobalLayout) -> GlobalLayout:
    """Express ``inner`` (local -> intermediate) in ``outer``'s (intermediate
    -> global) coordinates: one box per overlapping pair of boxes."""
    g_offsets, l_offsets, sizes = [], [], []
    for o_glob, o_loc, o_size in zip(outer.global_offsets, outer.local_offsets, outer.local_sizes, strict=True):
        for i_glob, i_loc, i_size in zip(inner.global_offsets, inner.local_offsets, inner.local_sizes, strict=True):
            lo = [max(a, b) for a, b in zip(i_glob, o_loc)]
            hi = [min(ig + isz, ol + osz) for ig, isz, ol, osz in zip(i_glob, i_size, o_loc, o_size)]
            if any(h <= l for l, h in zip(lo, hi)):
                continue
            g_offsets.append(tuple(og + l - ol for og, l, ol in zip(o_glob, lo, o_loc)))
            l_offsets.append(tuple(il + l - ig for il, l, ig in zip(i_loc, lo, i_glob)))
            sizes.append(tuple(h - l for l, h in zip(lo, hi)))
    return GlobalLayout(outer.global_shape, tuple(g_offsets), tuple(l_offsets), tuple(sizes))


GradientReduceOp = Any  # dist.ReduceOp.AVG or dist.ReduceOp.SUM


@dataclass(frozen=True)
class GradientReduction:
    """What a bucket's gradient reduction must produce: the sum over the mesh,
    divided by ``divide_factor`` (default: the mesh size) when ``op`` is AVG."""

    op: GradientReduceOp = dist.ReduceOp.AVG
    divide_factor: float | None = None

    def __post_init__(self) -> None:
        if self.divide_factor is None:
            return
        if not math.isfinite(self.divide_factor) or self.divide_factor <= 0:
            raise ValueError(f"gradient_divide_factor must be a positive number, got {self.divide_factor!r}.")
        if self.op == dist.ReduceOp.SUM:
            raise ValueError("gradient_divide_factor requires gradient_reduce_op=AVG; SUM does not divide gradients.")


class Placement(ABC):
    """Base class of placement strategies.

    Subclasses must be value types: ``__eq__`` and ``__hash__`` are abstract,
    and a subclass that overrides ``__eq__`` without ``__hash__`` is rejected
    at class creation.
    """

    #: True when only ``finish_prepared_unshard`` writes a refill's persistent
    #: buffers (a copy-out on the current stream); the runtime then
    #: re-allocates their storage right before finish.
    refills_persistent_buffers_in_finish: ClassVar[bool] = False

    def __init_subclass__(cls) -> None:
        super().__init_subclass__()
        if "__eq__" in cls.__dict__ and cls.__dict__.get("__hash__") is None:
            raise TypeError(f"{cls.__name__} must define __hash__ when overriding __eq__.")

    @abstractmethod
    def __eq__(self, other: object) -> bool:
        raise NotImplementedError

    @abstractmethod
    def __hash__(self) -> int:
        raise NotImplementedError

    def bucket_compatibility_key(self) -> object:
        """Placements with equal keys can share one bucket collective."""
        return self

    def compute_local_shape(self, global_shape: torch.Size, rank: int, world_size: int) -> torch.Size:
        raise NotImplementedError

    def compute_local_numel(self, global_shape: torch.Size, rank: int, world_size: int) -> int:
        return math.prod(self.compute_local_shape(global_shape, rank, world_size))

    def extract_local_shard(self, param: torch.Tensor, rank: int, world_size: int) -> torch.Tensor:
        """This rank's part of the full parameter (may be a non-contiguous view)."""
        raise NotImplementedError

    def local_storage_layout(
        self, global_shape: torch.Size, dtype: torch.dtype, rank: int, world_size: int
    ) -> LocalStorageLayout:
        shape = self.compute_local_shape(global_shape, rank, world_size)
        numel = self.compute_local_numel(global_shape, rank, world_size)
        return LocalStorageLayout(local_shape=shape, local_numel=numel, storage_nbytes=numel * dtype.itemsize)

    def bucket_storage_layout(
        self,
        named_params: list[tuple[str, "nn.Parameter"]],
        param_placements: dict[str, tuple["Placement", ...]],
        mesh: Any,
    ) -> BucketStorageLayout | None:
        """A bucket-global layout, or None for the default sequential one."""
        return None

    def copy_param_to_storage(
        self, byte_storage: torch.Tensor, info: "ParamInfo", param: torch.Tensor, rank: int, world_size: int
    ) -> None:
        """Write this rank's part of ``param`` into the bucket byte storage."""
        data = param.detach()
        if data.device.type == "meta":
            return
        shard = self.extract_local_shard(data, rank, world_size)
        if shard.numel() == 0:
            return
        shard = shard.contiguous()
        nbytes = shard.numel() * shard.element_size()
        if nbytes > info.storage_nbytes:
            raise ValueError(
                f"Placement {self!r} produced {nbytes} bytes for {info.fqn!r}, "
                f"but its storage layout only reserved {info.storage_nbytes} bytes."
            )
        byte_storage[info.byte_offset : info.byte_offset + nbytes].copy_(shard.view(-1).view(torch.uint8))

    def make_local_storage_view(self, byte_storage: torch.Tensor, info: "ParamInfo") -> torch.Tensor:
        """The local parameter as a typed view of the bucket byte storage."""
        nbytes = info.local_numel * info.dtype.itemsize
        window = byte_storage[info.byte_offset : info.byte_offset + nbytes]
        return window.view(info.dtype).view(info.local_shape)

    def global_layout(self, info: "ParamInfo", rank: int, world_size: int) -> GlobalLayout:
        raise NotImplementedError(f"{self!r} does not support distributed checkpointing.")

    # -- collective lifecycle ------------------------------------------------
    def prepare_unshard_bucket(
        self, tensors: list[torch.Tensor], infos: list["ParamInfo"], mesh: Any, debug_fqn: str | None
    ) -> "PlacementPreparedUnshard":
        raise NotImplementedError

    def run_prepared_unshard(self, prepared: "PlacementPreparedUnshard", *, async_op: bool = False) -> Any | None:
        raise NotImplementedError

    def finish_prepared_unshard(self, prepared: "PlacementPreparedUnshard") -> "PlacementUnshardResult":
        raise NotImplementedError

    def prepare_reduce_grad(
        self, tensors: list[torch.Tensor], infos: list["ParamInfo"], mesh: Any, debug_fqn: str | None
    ) -> "PlacementPreparedReduceGrad":
        raise NotImplementedError

    def reduce_prepared_grad(
        self, prepared: "PlacementPreparedReduceGrad", reduction: GradientReduction
    ) -> "PlacementReduceGradResult":
        raise NotImplementedError

    def reduces_grads_in_param_layout(self, infos: list["ParamInfo"], world_size: int) -> bool:
        """Whether the reduction reads grads laid out as views of one zeroed
        buffer at the unsharded params' offsets, without a copy-in."""
        return False


@dataclass
class PlacementPreparedUnshard:
    """A prepared bucket unshard.  ``buffers`` live until finish has queued its
    last use; ``placement_state`` is private to the placement.  ``persistent``
    asks finish to back the full params with buffers the caller keeps; on
    refills the caller passes them back in ``persistent_buffers`` and the
    placement writes them in place."""

    placement: Placement
    buffers: list[torch.Tensor]
    placement_state: Any
    persistent: bool = False
    persistent_buffers: list[torch.Tensor] | None = None


@dataclass
class PlacementUnshardResult:
    """Full parameters, temporaries created by finish, and (persistent
    unshards) the buffers backing the full parameters."""

    full_params: list[torch.Tensor]
    buffers: list[torch.Tensor] = field(default_factory=list)
    persistent_buffers: list[torch.Tensor] = field(default_factory=list)


@dataclass
class PlacementPreparedReduceGrad:
    """A prepared bucket gradient reduction."""

    placement: Placement
    buffers: list[torch.Tensor]
    placement_state: Any


@dataclass
class PlacementReduceGradResult:
    """Reduced local gradient shards and the buffers they view."""

    sharded_grads: list[torch.Tensor]
    buffers: list[torch.Tensor] = field(default_factory=list)


__all__ = [
    "BucketParamStorageLayout",
    "BucketStorageLayout",
    "GlobalLayout",
    "GradientReduceOp",
    "GradientReduction",
    "LocalStorageLayout",
    "Placement",
    "PlacementPreparedReduceGrad",
    "PlacementPreparedUnshard",
    "PlacementReduceGradResult",
    "PlacementUnshardResult",
    "compose_global_layouts",
    "get_global_layout",
    "get_partial_grad_group",
    "set_global_layout",
    "set_partial_grad_group",
]
