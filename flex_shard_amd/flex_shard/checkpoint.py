"""Checkpoint layouts of sharded buckets: where each parameter's local shard
sits in the full parameter, declared on state-dict and optimizer-state tensors
through the attribute protocol a distributed checkpoint writer reads.

Mirrors ``src/flex_shard/flex_shard/checkpoint.py`` of the reference
(``get_flex_shard_global_layouts`` :25-54, ``set_state_dict_global_layouts``
:57-70, ``register_optimizer_checkpoint_hook`` :73-118 and the state hook
:134-160) over this package's :class:`BucketRuntime` objects instead of the
reference's module tree.  ``copy_shard_into_full`` / ``copy_full_into_shard``
apply a layout box by box; they are what a checkpoint writer does with the
declared fields, and the tests use them to re-shard between mesh sizes.
"""

from __future__ import annotations

from functools import partial
from typing import Any, Iterable

import torch

from ..placement_contract import GlobalLayout, compose_global_layouts, set_global_layout

# Their states other than ``step`` are elementwise, with the parameter's shape.
_CHECKPOINTABLE_OPTIMIZERS = (torch.optim.Adam, torch.optim.AdamW)
_OPTIMIZER_CHECKPOINT_HOOK_ATTR = "_flex_shard_optimizer_checkpoint_hook"


def get_flex_shard_global_layouts(runtimes: Iterable[Any]) -> dict[str, GlobalLayout]:
    """Layout of every sharded parameter of ``runtimes`` (objects with
    ``infos`` and ``mesh``), keyed by ``ParamInfo.fqn`` and every name the
    parameter is shared under.  A layout the parameter declared before it was
    sharded (it was already a shard of an outer sharding) is composed in.
    Computed from the current state on every call; raises
    ``NotImplementedError`` for a placement without ``global_layout``."""
    layouts: dict[str, GlobalLayout] = {}
    for runtime in runtimes:
        rank, world_size = runtime.mesh.get_local_rank(), runtime.mesh.size()
        for info in runtime.infos:
            layout = info.placement.global_layout(info, rank, world_size)
            if info.outer_layout is not None:
                layout = compose_global_layouts(info.outer_layout, layout)
            for fqn in (info.fqn, *info.shared_fqns):
                layouts[fqn] = layout
    return layouts


def set_state_dict_global_layouts(runtimes: Iterable[Any], state_dict: dict[str, Any]) -> None:
    """Declare each sharded parameter's layout on its ``state_dict`` tensor
    (for the dict passed to both the save and the load).  Parameters missing
    from ``state_dict`` are skipped."""
    for fqn, layout in get_flex_shard_global_layouts(runtimes).items():
        if fqn in state_dict:
            set_global_layout(state_dict[fqn], layout)


def register_optimizer_checkpoint_hook(optimizer: torch.optim.Optimizer, runtimes: Iterable[Any]) -> None:
    """Register a ``state_dict`` post-hook on ``optimizer`` that declares each
    sharded parameter's layout on its state tensors; ``step`` is left without
    one (replicated).  Calling it again replaces the hook.

    Raises ``NotImplementedError`` for optimizers other than Adam and AdamW;
    the hook raises it for a state that does not have its parameter's shape."""
    if not isinstance(optimizer, _CHECKPOINTABLE_OPTIMIZERS):
        raise NotImplementedError(
            f"FlexShard optimizer checkpointing supports Adam and AdamW, got {type(optimizer).__name__}."
        )
    runtimes = list(runtimes)
    layouts = get_flex_shard_global_layouts(runtimes)
    param_layouts: dict[torch.Tensor, tuple[str, GlobalLayout]] = {}
    for runtime in runtimes:
        for bucket_param in runtime.bucket_params:
            param_layouts[bucket_param.sharded_param] = (bucket_param.info.fqn, layouts[bucket_param.info.fqn])
    handle = getattr(optimizer, _OPTIMIZER_CHECKPOINT_HOOK_ATTR, None)
    if handle is not None:
        handle.remove()
    handle = optimizer.register_state_dict_post_hook(partial(_set_optimizer_state_layouts, param_layouts=param_layouts))
    setattr(optimizer, _OPTIMIZER_CHECKPOINT_HOOK_ATTR, handle)


def _set_optimizer_state_layouts(
    optimizer: torch.optim.Optimizer,
    state_dict: dict[str, Any],
    *,
    param_layouts: dict[torch.Tensor, tuple[str, GlobalLayout]],
) -> None:
    # the state dict lists each group's parameters as indices, in the order of the live groups
    for group, saved_group in zip(optimizer.param_groups, state_dict["param_groups"], strict=True):
        for param, param_id in zip(group["params"], saved_group["params"], strict=True):
            entry = param_layouts.get(param)
            if entry is None:
                continue
            fqn, layout = entry
            for state_name, value in state_dict["state"].get(param_id, {}).items():
                if state_name == "step" or not isinstance(value, torch.Tensor):
                    continue
                if value.shape != param.shape:
                    raise NotImplementedError(
                        f"Optimizer state {state_name!r} of FlexShard parameter {fqn!r} has shape "
                        f"{tuple(value.shape)}, but the local shard has shape {tuple(param.shape)}."
                    )
                set_global_layout(value, layout)


def _boxes(layout: GlobalLayout):
    for g_off, l_off, size in zip(layout.global_offsets, layout.local_offsets, layout.local_sizes, strict=True):
        g_box = tuple(slice(o, o + s) for o, s in zip(g_off, size, strict=True))
        l_box = tuple(slice(o, o + s) for o, s in zip(l_off, size, strict=True))
        yield g_box, l_box


def copy_shard_into_full(full: torch.Tensor, local: torch.Tensor, layout: GlobalLayout) -> None:
    """Write the boxes of ``local`` that ``layout`` names into ``full``."""
    if tuple(full.shape) != tuple(layout.global_shape):
        raise ValueError(f"Expected a full tensor of shape {tuple(layout.global_shape)}, got {tuple(full.shape)}.")
    for g_box, l_box in _boxes(layout):
        full[g_box].copy_(local[l_box])


def copy_full_into_shard(local: torch.Tensor, full: torch.Tensor, layout: GlobalLayout) -> None:
    """Fill the boxes of ``local`` that ``layout`` names from ``full``."""
    if tuple(full.shape) != tuple(layout.global_shape):
        raise ValueError(f"Expected a full tensor of shape {tuple(layout.global_shape)}, got {tuple(full.shape)}.")
    for g_box, l_box in _boxes(layout):
        local[l_box].copy_(full[g_box])


__all__ = [
    "copy_full_into_shard",
    "copy_shard_into_full",
    "get_flex_shard_global_layouts",
    "register_optimizer_checkpoint_hook",
    "set_state_dict_global_layouts",
]
