"""Hand-off of a bucket's unshard and gradient reduction between HIP streams.

Serves the callers of the reference's ``flex_shard/bucket_comm.py``
(``begin_bucket_unshard`` :94-146, ``begin_reduce_grad`` :149-181,
``begin_explicit_bucket_unshard`` :184-220, ``StreamHandoff`` :421-452) with
the same entry names and argument meaning.  The placements' kernels are plain
HIP launches, so there is one eager code path and one handle type per
operation, both built from two small pieces:

``_Fence``
    an event recorded after some work, and the streams that must not run
    ahead of it;
``_on_side_stream``
    "after what the current stream has queued, run this block on that stream,
    and give me the fence of its end".

Ordering uses events only; nothing here blocks the host:

* a side stream starts after the consumer stream's queued work (the local
  shards or the gradients are ready) and the consumer stream waits for the
  side stream's fence before it touches the result;
* a temporary allocated on one stream and last read on another is released by
  making every stream that allocated it wait for a fence recorded after its
  last reader, then dropping the reference (``StreamHandoff``), so neither
  stream's caching-allocator pool can hand the memory out early.
"""

from __future__ import annotations

import contextlib
from typing import TYPE_CHECKING, Any

import torch

from ..placement_contract import PlacementPreparedUnshard, PlacementUnshardResult

if TYPE_CHECKING:
    from ..bucket_storage import ParamInfo
    from ..placement_contract import GradientReduction, Placement


_STREAM_OBJECTS: dict[tuple[int, int, int], torch.cuda.Stream] = {}


def _current_stream(device: torch.device | None) -> torch.cuda.Stream:
    """``torch.cuda.current_stream(device)`` without building a new Stream
    object per call: the objects are kept by (stream id, device index, device
    type), which is what identifies a stream to torch."""
    index = torch.cuda.current_device() if device is None or device.index is None else device.index
    key = torch._C._cuda_getCurrentStream(index)
    stream = _STREAM_OBJECTS.get(key)
    if stream is None:
        if len(_STREAM_OBJECTS) >= 64:
            _STREAM_OBJECTS.clear()
        stream = _STREAM_OBJECTS[key] = torch.cuda.Stream(stream_id=key[0], device_index=key[1], device_type=key[2])
    return stream


class _Fence:
    """A point in one stream's queue that other streams can be ordered after."""

    __slots__ = ("event",)

    def __init__(self, stream: torch.cuda.Stream | None, event: torch.cuda.Event | None = None) -> None:
        """The end of what ``stream`` has queued so far, or a given ``event``."""
        if event is None:
            event = torch.cuda.Event()
            event.record(stream)
        self.event = event

    def hold_back(self, *streams: torch.cuda.Stream) -> None:
        """Order each distinct stream of ``streams`` after this point."""
        if len(streams) == 1:
            streams[0].wait_event(self.event)
            return
        done: set[int] = set()
        for stream in streams:
            if stream.cuda_stream not in done:
                done.add(stream.cuda_stream)
                stream.wait_event(self.event)


class _on_side_stream:
    """Run the block on ``side`` after everything the current stream has
    queued so far.  ``with _on_side_stream(side, device) as done``: ``done`` is
    a list that holds the fence of the block's end once the block has run.
    The current stream is switched with ``torch.cuda.set_stream`` (a fraction
    of what the ``torch.cuda.stream`` context costs) and always restored."""

    __slots__ = ("_side", "_previous", "_done")

    def __init__(self, side: torch.cuda.Stream, device: torch.device) -> None:
        self._side = side
        self._previous = _current_stream(device)
        self._done: list[_Fence] = []

    def __enter__(self) -> list[_Fence]:
        _Fence(self._previous).hold_back(self._side)
        torch.cuda.set_stream(self._side)
        return self._done

    def __exit__(self, exc_type, exc, tb) -> None:
        try:
            if exc_type is None:
                self._done.append(_Fence(self._side))
        finally:
            torch.cuda.set_stream(self._previous)


class StreamHandoff:
    """References to tensors that were allocated on ``allocation_streams`` and
    are last read by work queued on some other stream.  Releasing orders every
    allocation stream after that last reader and then drops the references;
    releasing twice is harmless."""

    __slots__ = ("_tensors", "_allocation_streams")

    def __init__(self, tensors: list[torch.Tensor], allocation_streams: tuple[torch.cuda.Stream, ...]) -> None:
        self._tensors: list[torch.Tensor] | None = tensors
        self._allocation_streams = allocation_streams

    def release_after(self, event: torch.cuda.Event) -> None:
        """The last reader finished at ``event``."""
        if self._tensors is None:
            return
        _Fence(None, event).hold_back(*self._allocation_streams)
        self._tensors.clear()
        self._tensors = None

    def release_after_current_stream(self) -> None:
        """The last reader is whatever the current stream has queued so far."""
        if self._tensors is None:
            return
        if self._tensors:
            _Fence(_current_stream(self._tensors[0].device)).hold_back(*self._allocation_streams)
            self._tensors.clear()
        self._tensors = None


def _get_bucket_placement(infos: list["ParamInfo"], operation: str) -> "Placement":
    """The placement that runs a bucket's collective lifecycle: the first
    parameter's, provided every other parameter's is compatible with it."""
    lead = infos[0]
    wanted = lead.placement.bucket_compatibility_key()
    for info in infos[1:]:
        if info.placement.bucket_compatibility_key() != wanted:
            raise ValueError(
                f"FlexShard bucket {operation} requires all parameters in a bucket to use compatible placements, "
                f"but {lead.fqn!r} uses {lead.placement!r} and {info.fqn!r} uses {info.placement!r}."
            )
    return lead.placement


def _prepare_and_run(
    placement: "Placement",
    tensors: list[torch.Tensor],
    infos: list["ParamInfo"],
    mesh: Any,
    debug_fqn: str | None,
    persistent_buffers: list[torch.Tensor] | None,
    async_op: bool,
) -> tuple[PlacementPreparedUnshard, Any | None]:
    """Copy-in and exchange of a persistent unshard on the current stream.
    A refill writes buffers that autograd may have saved before a reshard, so
    their version counters are left as they are."""
    prepared = placement.prepare_unshard_bucket(tensors, infos, mesh, debug_fqn)
    prepared.persistent = True
    prepared.persistent_buffers = persistent_buffers
    if persistent_buffers is None:
        return prepared, placement.run_prepared_unshard(prepared, async_op=async_op)
    with contextlib.ExitStack() as guards:
        guards.enter_context(torch.inference_mode(False))
        guards.enter_context(torch.no_grad())
        guards.enter_context(torch.autograd._unsafe_preserve_version_counter(tuple(persistent_buffers)))
        work = placement.run_prepared_unshard(prepared, async_op=async_op)
    return prepared, work


class UnshardHandle:
    """A bucket unshard between its exchange and its copy-out.

    ``side_stream`` is the stream copy-in and exchange were queued on when that
    is not the consumer's; ``fence`` marks their end there.  ``work`` is the
    handle of an exchange that was started asynchronously on the consumer's own
    stream (a ``torch.distributed`` work object), or ``None``.
    """

    def __init__(
        self,
        prepared: PlacementPreparedUnshard,
        *,
        side_stream: torch.cuda.Stream | None = None,
        fence: _Fence | None = None,
        work: Any | None = None,
    ) -> None:
        self.prepared = prepared
        self._side_stream = side_stream
        self._fence = fence
        self._work = work
        self._finished = False
        self._device = prepared.buffers[0].device if prepared.buffers else None

    def wait(self) -> None:
        """Order the current stream after the exchange."""
        if self._work is not None:
            self._work.wait()
            self._work = None
        if self._fence is not None and self._device is not None:
            _current_stream(self._device).wait_event(self._fence.event)

    def finish(self) -> PlacementUnshardResult:
        """Copy out on the current stream and hand the temporaries back to the
        pools they came from.  An unshard is finished once."""
        if self._finished:
            raise RuntimeError("An unshard may only be finished once.")
        self._finished = True
        self.wait()
        result = self.prepared.placement.finish_prepared_unshard(self.prepared)
        self._drop([*self.prepared.buffers, *result.buffers])
        self.prepared.buffers.clear()
        result.buffers.clear()
        return result

    def release_buffers(self) -> None:
        """Give up an unshard that will not be finished."""
        if self._work is not None:
            self.wait()
        self._drop(list(self.prepared.buffers))
        self.prepared.buffers.clear()

    def _drop(self, tensors: list[torch.Tensor]) -> None:
        # On the consumer's own stream the pool may reuse the buffers as soon
        # as the references go: all their readers are queued on that stream.
        # Buffers of a side stream were last read by the copy-out just queued
        # on the current stream.
        if tensors and self._side_stream is not None:
            current = _current_stream(tensors[0].device)
            StreamHandoff(tensors, (self._side_stream, current)).release_after_current_stream()


def begin_bucket_unshard(
    tensors: list[torch.Tensor],
    infos: list["ParamInfo"],
    mesh: Any,
    unshard_stream: torch.cuda.Stream | None,
    debug_fqn: str | None = None,
    persistent_buffers: list[torch.Tensor] | None = None,
    *,
    async_op: bool = False,
) -> UnshardHandle:
    """Copy-in (for the FP8 placement: quantize + pack) and exchange of a
    bucket on ``unshard_stream``, behind the work the current stream has
    queued; the copy-out happens in ``finish`` on the stream current then.

    The unshard is persistent (see ``PlacementPreparedUnshard``).  Given the
    ``persistent_buffers`` of an earlier unshard it refills them, in run or in
    finish as the placement chooses; their storage has been re-allocated on
    the current stream already, or is re-allocated before finish.  With
    ``unshard_stream=None`` everything is queued on the current stream, whose
    pool then gets the buffers back after the copy-out; only there may the
    exchange be asynchronous (``async_op``)."""
    placement = _get_bucket_placement(infos, "unshard")
    if unshard_stream is None:
        prepared, work = _prepare_and_run(placement, tensors, infos, mesh, debug_fqn, persistent_buffers, async_op)
        return UnshardHandle(prepared, work=work)
    if async_op:
        raise ValueError("an unshard on a side stream is ordered by events; async_op applies to the current stream only")
    with _on_side_stream(unshard_stream, tensors[0].device) as done:
        prepared, _ = _prepare_and_run(placement, tensors, infos, mesh, debug_fqn, persistent_buffers, False)
    return UnshardHandle(prepared, side_stream=unshard_stream, fence=done[0])


def begin_explicit_bucket_unshard(
    tensors: list[torch.Tensor],
    infos: list["ParamInfo"],
    mesh: Any,
    *,
    async_op: bool,
    debug_fqn: str | None = None,
    persistent_buffers: list[torch.Tensor] | None = None,
) -> UnshardHandle:
    """``begin_bucket_unshard`` on the current stream (the reference's entry
    for unshards the user asks for explicitly)."""
    return begin_bucket_unshard(tensors, infos, mesh, None, debug_fqn, persistent_buffers, async_op=async_op)


class ReduceGradHandle:
    """A bucket gradient reduction in flight: this rank's reduced shards, the
    fence after which they hold data, and the buffers the reduction reads and
    writes together with the streams that allocated them."""

    def __init__(
        self,
        sharded_grads: list[torch.Tensor],
        fence: _Fence | None,
        buffers: list[torch.Tensor],
        allocation_streams: tuple[torch.cuda.Stream, ...],
    ) -> None:
        self.sharded_grads = sharded_grads
        self.buffers = buffers
        self._fence = fence
        self._allocation_streams = allocation_streams

    def _device(self) -> torch.device | None:
        for group in (self.sharded_grads, self.buffers):
            if group:
                return group[0].device
        return None

    def wait(self) -> None:
        """Order the current stream after the reduction."""
        device = self._device()
        if device is not None and self._fence is not None:
            _current_stream(device).wait_event(self._fence.event)

    def finish(self) -> list[torch.Tensor]:
        self.wait()
        return self.sharded_grads

    def synchronize(self) -> None:
        """Block the host until the reduction has run (checkpointing, tests)."""
        if self._fence is not None:
            self._fence.event.synchronize()

    def record_sharded_grads(self, sharded_grads: list[torch.Tensor], stream: torch.cuda.Stream) -> None:
        """The shards were post-processed on ``stream`` (accumulated into
        ``.grad``): that work is now what a consumer has to wait for."""
        self.sharded_grads = sharded_grads
        self._fence = _Fence(stream)

    def release_buffers(self, release_sharded_grads: bool) -> None:
        """Hand the reduction's buffers (and, if asked, the shards) back once
        the current stream's queued work has run."""
        going = list(self.buffers)
        self.buffers.clear()
        if release_sharded_grads:
            going += self.sharded_grads
            self.sharded_grads.clear()
        if going:
            StreamHandoff(going, self._allocation_streams).release_after_current_stream()


def begin_reduce_grad(
    tensors: list[torch.Tensor],
    infos: list["ParamInfo"],
    mesh: Any,
    reduction: "GradientReduction",
    reduce_grad_stream: torch.cuda.Stream,
    debug_fqn: str | None = None,
) -> ReduceGradHandle:
    """Copy the full-parameter gradients into the reduce-scatter input on the
    current stream (they were produced there), reduce on
    ``reduce_grad_stream`` behind it, and return the handle of the shards."""
    placement = _get_bucket_placement(infos, "reduce-grad")
    prepared = placement.prepare_reduce_grad(tensors, infos, mesh, debug_fqn)
    device = prepared.buffers[0].device
    copy_in_stream = _current_stream(device)
    with _on_side_stream(reduce_grad_stream, device) as done:
        result = placement.reduce_prepared_grad(prepared, reduction)
    return ReduceGradHandle(
        result.sharded_grads, done[0], [*prepared.buffers, *result.buffers], (copy_in_stream, reduce_grad_stream)
    )


__all__ = [
    "ReduceGradHandle", "StreamHandoff", "UnshardHandle", "begin_bucket_unshard", "begin_explicit_bucket_unshard",
    "begin_reduce_grad",
]
