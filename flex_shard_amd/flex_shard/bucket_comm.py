"""Stream hand-off between a bucket's consumer stream and the side streams its
unshard and gradient reduction run on.

Mirror of the reference's ``flex_shard/bucket_comm.py``: ``begin_bucket_unshard``
(:94-146), ``begin_reduce_grad`` (:149-181), ``begin_explicit_bucket_unshard``
(:184-220), the handles they return (:239-413) and ``StreamHandoff``
(:421-452).  The graph-capture (``torch.compile``) branches are left out: the
kernels behind the placements are opaque HIP launches.

Ordering rules, all expressed with HIP events (no host synchronisation):

* the side stream waits for an event recorded on the consumer stream before
  the placement reads the local shards (copy-in / quantize + pack);
* the consumer stream waits for the event recorded after the placement's side
  stream work before it unpacks (``finish``);
* temporaries allocated on one stream and last read on another are released
  through :class:`StreamHandoff`: every allocation stream waits for an event
  recorded after the last reader, then the references are dropped, so the
  caching allocator of either stream cannot hand the memory out early.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import TYPE_CHECKING, Any

import torch

from ..placement_contract import PlacementPreparedUnshard, PlacementUnshardResult

if TYPE_CHECKING:
    from ..bucket_storage import ParamInfo
    from ..placement_contract import GradientReduction, Placement


class UnshardHandle:
    """Handle of a bucket unshard in flight."""

    def finish(self) -> PlacementUnshardResult:
        """Wait for the unshard and return its full params (once)."""
        raise NotImplementedError

    def wait(self) -> None:
        """Make the current stream wait until the unshard's result is usable."""
        raise NotImplementedError

    def release_buffers(self) -> None:
        """Release the buffers of an unshard that will not be finished."""
        raise NotImplementedError


class ReduceGradHandle:
    """Handle of a bucket gradient reduction in flight."""

    def finish(self) -> list[torch.Tensor]:
        raise NotImplementedError

    def wait(self) -> None:
        raise NotImplementedError

    def synchronize(self) -> None:
        raise NotImplementedError

    def release_buffers(self, release_sharded_grads: bool) -> None:
        raise NotImplementedError

    def record_sharded_grads(self, sharded_grads: list[torch.Tensor], stream: torch.cuda.Stream) -> None:
        raise NotImplementedError


def _first_tensor_device(*tensor_groups: list[torch.Tensor]) -> torch.device | None:
    for tensors in tensor_groups:
        if tensors:
            return tensors[0].device
    return None


def _get_bucket_placement(infos: list["ParamInfo"], operation: str) -> "Placement":
    placement = infos[0].placement
    key = placement.bucket_compatibility_key()
    for info in infos[1:]:
        if info.placement.bucket_compatibility_key() != key:
            raise ValueError(
                f"FlexShard bucket {operation} requires all parameters in a bucket to use compatible placements, "
                f"but {infos[0].fqn!r} uses {placement!r} and {info.fqn!r} uses {info.placement!r}."
            )
    return placement


def _run_refilling(prepared: PlacementPreparedUnshard, persistent_buffers: list[torch.Tensor] | None, **kwargs: Any):
    """``run_prepared_unshard``; a refill may write the persistent buffers the
    unsharded params view, which autograd may have saved before a reshard, so
    their version counters are preserved."""
    if persistent_buffers is None:
        return prepared.placement.run_prepared_unshard(prepared, **kwargs)
    with (
        torch.inference_mode(False),
        torch.no_grad(),
        torch.autograd._unsafe_preserve_version_counter(tuple(persistent_buffers)),
    ):
        return prepared.placement.run_prepared_unshard(prepared, **kwargs)


def begin_bucket_unshard(
    tensors: list[torch.Tensor],
    infos: list["ParamInfo"],
    mesh: Any,
    unshard_stream: torch.cuda.Stream,
    debug_fqn: str | None = None,
    persistent_buffers: list[torch.Tensor] | None = None,
) -> UnshardHandle:
    """Begin a bucket unshard on ``unshard_stream`` and return its handle.

    The unshard is persistent (see ``PlacementPreparedUnshard``).  Given the
    ``persistent_buffers`` of an earlier unshard it refills them, in run or in
    finish as the placement chooses; their storage has been re-allocated on the
    current stream already, or is re-allocated before finish."""
    placement = _get_bucket_placement(infos, "unshard")
    device = tensors[0].device
    copy_in_done = torch.cuda.Event()
    copy_in_done.record(torch.cuda.current_stream(device))
    with torch.cuda.stream(unshard_stream):
        unshard_stream.wait_event(copy_in_done)
        prepared = placement.prepare_unshard_bucket(tensors, infos, mesh, debug_fqn)
        prepared.persistent = True
        prepared.persistent_buffers = persistent_buffers
        _run_refilling(prepared, persistent_buffers)
        event = torch.cuda.Event()
        event.record(unshard_stream)
    return AsyncUnshardResult(prepared=prepared, event=event, unshard_stream=unshard_stream)


def begin_reduce_grad(
    tensors: list[torch.Tensor],
    infos: list["ParamInfo"],
    mesh: Any,
    reduction: "GradientReduction",
    reduce_grad_stream: torch.cuda.Stream,
    debug_fqn: str | None = None,
) -> ReduceGradHandle:
    """Copy the full-parameter gradients in on the current stream, reduce them
    on ``reduce_grad_stream`` and return the handle of the local shards."""
    placement = _get_bucket_placement(infos, "reduce-grad")
    prepared = placement.prepare_reduce_grad(tensors, infos, mesh, debug_fqn)
    device = prepared.buffers[0].device
    copy_in_stream = torch.cuda.current_stream(device)
    copy_in_done = torch.cuda.Event()
    copy_in_done.record(copy_in_stream)
    with torch.cuda.stream(reduce_grad_stream):
        reduce_grad_stream.wait_event(copy_in_done)
        result = prepared.placement.reduce_prepared_grad(prepared, reduction)
        event = torch.cuda.Event()
        event.record(reduce_grad_stream)
    return AsyncReduceGradResult(
        sharded_grads=result.sharded_grads,
        event=event,
        buffers=[*prepared.buffers, *result.buffers],
        allocation_streams=(copy_in_stream, reduce_grad_stream),
    )


def begin_explicit_bucket_unshard(
    tensors: list[torch.Tensor],
    infos: list["ParamInfo"],
    mesh: Any,
    *,
    async_op: bool,
    debug_fqn: str | None = None,
    persistent_buffers: list[torch.Tensor] | None = None,
) -> UnshardHandle:
    """Begin a bucket unshard on the current stream: copy-in, exchange buffers
    and copy-out all belong to it, so its memory pool gets the buffers back
    after the copy-out.  With ``async_op`` the exchange may be asynchronous."""
    placement = _get_bucket_placement(infos, "unshard")
    prepared = placement.prepare_unshard_bucket(tensors, infos, mesh, debug_fqn)
    prepared.persistent = True
    prepared.persistent_buffers = persistent_buffers
    work = _run_refilling(prepared, persistent_buffers, async_op=async_op)
    return ExplicitUnshardResult(prepared=prepared, work=work)


@dataclass
class AsyncUnshardResult(UnshardHandle):
    """State needed to finish an unshard launched on a side stream."""

    prepared: PlacementPreparedUnshard
    event: torch.cuda.Event
    unshard_stream: torch.cuda.Stream
    _device: torch.device | None = field(default=None, init=False)
    _finished: bool = field(default=False, init=False)

    def __post_init__(self) -> None:
        self._device = _first_tensor_device(self.prepared.buffers)

    def finish(self) -> PlacementUnshardResult:
        if self._finished:
            raise RuntimeError("An unshard may only be finished once.")
        self._finished = True
        self.wait()
        result = self.prepared.placement.finish_prepared_unshard(self.prepared)
        # Only work queued so far on the current stream (the copy-out) reads
        # the prepare and finish buffers.
        self._release([*self.prepared.buffers, *result.buffers])
        self.prepared.buffers.clear()
        result.buffers.clear()
        return result

    def wait(self) -> None:
        if self._device is not None:
            torch.cuda.current_stream(self._device).wait_event(self.event)

    def release_buffers(self) -> None:
        self._release(list(self.prepared.buffers))
        self.prepared.buffers.clear()

    def _release(self, tensors: list[torch.Tensor]) -> None:
        if not tensors:
            return
        current = torch.cuda.current_stream(tensors[0].device)
        StreamHandoff(tensors, (self.unshard_stream, current)).release_after_current_stream()


@dataclass
class ExplicitUnshardResult(UnshardHandle):
    """An unshard begun on the current stream; ``work`` is the asynchronous
    exchange's handle or ``None``."""

    prepared: PlacementPreparedUnshard
    work: Any | None
    _finished: bool = field(default=False, init=False)

    def finish(self) -> PlacementUnshardResult:
        if self._finished:
            raise RuntimeError("An unshard may only be finished once.")
        self._finished = True
        self.wait()
        result = self.prepared.placement.finish_prepared_unshard(self.prepared)
        # The current stream queued the exchange and the copy-out, so its pool
        # can reuse the buffers once these references drop.
        self.prepared.buffers.clear()
        result.buffers.clear()
        return result

    def wait(self) -> None:
        if self.work is not None:
            self.work.wait()
            self.work = None

    def release_buffers(self) -> None:
        self.wait()
        self.prepared.buffers.clear()


@dataclass
class AsyncReduceGradResult(ReduceGradHandle):
    """State needed to finish a gradient reduction launched on a side stream."""

    sharded_grads: list[torch.Tensor]
    event: torch.cuda.Event | None
    buffers: list[torch.Tensor]
    allocation_streams: tuple[torch.cuda.Stream, ...]
    _device: torch.device | None = field(default=None, init=False)

    def __post_init__(self) -> None:
        self._device = _first_tensor_device(self.sharded_grads, self.buffers)

    def finish(self) -> list[torch.Tensor]:
        self.wait()
        return self.sharded_grads

    def wait(self) -> None:
        if self._device is not None and self.event is not None:
            torch.cuda.current_stream(self._device).wait_event(self.event)

    def synchronize(self) -> None:
        if self.event is not None:
            self.event.synchronize()

    def release_buffers(self, release_sharded_grads: bool) -> None:
        tensors = list(self.buffers)
        self.buffers.clear()
        if release_sharded_grads:
            tensors.extend(self.sharded_grads)
            self.sharded_grads.clear()
        if tensors:
            StreamHandoff(tensors, self.allocation_streams).release_after_current_stream()

    def record_sharded_grads(self, sharded_grads: list[torch.Tensor], stream: torch.cuda.Stream) -> None:
        self.sharded_grads = sharded_grads
        self._device = _first_tensor_device(self.sharded_grads, self.buffers) or self._device
        self.event = torch.cuda.Event()
        self.event.record(stream)


class StreamHandoff:
    """Keeps tensors alive until their allocation streams own the final wait."""

    __slots__ = ("_tensors", "_allocation_streams", "_released")

    def __init__(self, tensors: list[torch.Tensor], allocation_streams: tuple[torch.cuda.Stream, ...]) -> None:
        self._tensors = tensors
        self._allocation_streams = allocation_streams
        self._released = False

    def release_after(self, event: torch.cuda.Event) -> None:
        """Order every allocation stream after ``event``, then drop the references."""
        if self._released:
            return
        seen: set[int] = set()
        for stream in self._allocation_streams:
            if stream.cuda_stream in seen:
                continue
            seen.add(stream.cuda_stream)
            stream.wait_event(event)
        self._released = True
        self._tensors.clear()

    def release_after_current_stream(self) -> None:
        """Record the final consumer point on the current stream and release after it."""
        if self._released:
            return
        if not self._tensors:
            self._released = True
            return
        event = torch.cuda.Event()
        event.record(torch.cuda.current_stream(self._tensors[0].device))
        self.release_after(event)


__all__ = [
    "AsyncReduceGradResult", "AsyncUnshardResult", "ExplicitUnshardResult", "ReduceGradHandle", "StreamHandoff",
    "UnshardHandle", "begin_bucket_unshard", "begin_explicit_bucket_unshard", "begin_reduce_grad",
]
