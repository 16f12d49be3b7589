"""Profiler ranges around the hot path, named as the reference names them
(flex_shard/utils.py:35-78: ``FlexShard::copy_in``, ``::copy_out``,
``::all_gather``, ``::post_backward_reduce``, ``::reduce_scatter_copy_in/out``),
suppressed while compiling."""

from __future__ import annotations

import contextlib

import torch


_NO_RANGE = contextlib.nullcontext()


def record_range(name: str, debug_fqn: str | None = None):
    # A range costs several microseconds of host time per call even when
    # nobody listens; torch keeps this flag current while a profiler runs.
    if not torch.autograd.profiler._is_profiler_enabled or torch.compiler.is_compiling():
        return _NO_RANGE
    label = name if debug_fqn is None else f"{name} ({debug_fqn})"
    return torch.profiler.record_function(label)


def record_copy_in(debug_fqn: str | None = None):
    return record_range("FlexShard::copy_in", debug_fqn)


def record_copy_out(debug_fqn: str | None = None):
    return record_range("FlexShard::copy_out", debug_fqn)


def record_comm(name: str, debug_fqn: str | None = None):
    return record_range(name, debug_fqn)
