"""The slice of the bucket runtime that drives a placement under a real
forward and backward on one GPU: persistent unsharded parameters, their refill,
reshard, and the gradient reduction, with the stream hand-off of
``bucket_comm``.

Mirror of the reference's ``flex_shard/bucket_runtime.py``: ``begin_unshard``
(:749-792), ``reduce_grads`` (:794-837), ``unshard`` / ``finish_unshard`` /
``_create_unsharded_params`` (:843-940), ``_swap_in_params`` / ``reshard`` /
persistent storage (:951-980), ``_accumulate_sharded_grads`` (:1686-1724) and
the reduce-grad bookkeeping of ``BucketCommContext`` (:524-576).  What is not
here: prefetch ordering, module-tree hook discovery, activation-checkpoint
recompute, ``torch.compile`` capture and the storage
engine -- a bucket is built from an explicit list of parameters of one module,
and one pair of hooks (``install_hooks``) covers one forward and one backward
per step.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any

import torch
import torch.nn as nn
from torch.utils._python_dispatch import is_traceable_wrapper_subclass

from ..bucket_storage import ParamInfo, create_param_infos
from ..placement_contract import GradientReduction, Placement
from .bucket_comm import (
    ReduceGradHandle,
    UnshardHandle,
    begin_bucket_unshard,
    begin_reduce_grad,
)


def _alloc_storage(tensor: torch.Tensor, nbytes: int) -> None:
    storage = tensor.untyped_storage()
    if storage.size() != nbytes:
        storage.resize_(nbytes)


def _free_storage(tensor: torch.Tensor) -> None:
    storage = tensor.untyped_storage()
    if storage.size() != 0:
        storage.resize_(0)


def _inner_tensors(tensor: torch.Tensor) -> list[torch.Tensor]:
    """The plain tensors holding a (possibly wrapper-subclass) tensor's data."""
    if is_traceable_wrapper_subclass(tensor):
        attrs, _ = tensor.__tensor_flatten__()
        return [inner for attr in attrs for inner in _inner_tensors(getattr(tensor, attr))]
    return [tensor]


def _match_param_grad_layout(grad: torch.Tensor, param: nn.Parameter) -> torch.Tensor:
    dtype = getattr(param, "grad_dtype", None) or grad.dtype
    if grad.dtype != dtype or grad.device != param.device:
        grad = grad.to(device=param.device, dtype=dtype)
    if grad.stride() != param.stride():
        aligned = torch.empty_strided(tuple(param.shape), tuple(param.stride()), dtype=dtype, device=param.device)
        aligned.copy_(grad)
        grad = aligned
    return grad


def _accumulate_sharded_grads(sharded_params: list[nn.Parameter], sharded_grads: list[torch.Tensor]) -> list[torch.Tensor]:
    """Cast the reduced shards to the parameters' gradient dtype and layout and
    accumulate them into ``.grad``."""
    stored = []
    for param, grad in zip(sharded_params, sharded_grads, strict=True):
        grad = _match_param_grad_layout(grad, param)
        stored.append(grad)
        if param.grad is None:
            param.grad = grad
        else:
            param.grad += grad
    return stored


@dataclass
class PendingReduceGrad:
    result: ReduceGradHandle


@dataclass
class BucketCommContext:
    """Streams and in-flight reductions shared by the buckets of one model.

    ``unshard_streams``: the side streams unshards are begun on, taken in turn
    (``next_unshard_stream``).  With two of them, a prefetched bucket's
    quantize + pack launch overlaps the ramp and drain of the previous
    bucket's (an 82 MB launch alone spends a fifth of its time there); all
    streams have the default priority."""

    device: torch.device
    unshard_streams: list[torch.cuda.Stream]
    reduce_grad_stream: torch.cuda.Stream
    reduce_grad_release_stream: torch.cuda.Stream
    max_pending_reduce_grads: int = 2
    reduce_grad_states: list[PendingReduceGrad] = field(default_factory=list)
    retired_reduce_grad_states: list[PendingReduceGrad] = field(default_factory=list)
    _unshard_turn: int = 0

    @classmethod
    def create(
        cls, device: torch.device, max_pending_reduce_grads: int = 2, unshard_streams: int = 2
    ) -> "BucketCommContext":
        if unshard_streams < 1:
            raise ValueError(f"a context needs at least one unshard stream, got {unshard_streams}")
        # default priorities only
        return cls(
            device=device,
            unshard_streams=[torch.cuda.Stream(device) for _ in range(unshard_streams)],
            reduce_grad_stream=torch.cuda.Stream(device),
            reduce_grad_release_stream=torch.cuda.Stream(device),
            max_pending_reduce_grads=max_pending_reduce_grads,
        )

    @property
    def unshard_stream(self) -> torch.cuda.Stream:
        """The first unshard stream (the only one of a one-stream context)."""
        return self.unshard_streams[0]

    def next_unshard_stream(self) -> torch.cuda.Stream:
        """The side stream for the next unshard: the streams take turns."""
        stream = self.unshard_streams[self._unshard_turn % len(self.unshard_streams)]
        self._unshard_turn += 1
        return stream

    def wait_and_release_reduce_grad_state(self, pending: PendingReduceGrad, *, wait_current_stream: bool) -> None:
        if wait_current_stream:
            pending.result.wait()
        with torch.cuda.stream(self.reduce_grad_release_stream):
            pending.result.wait()
            pending.result.release_buffers(release_sharded_grads=True)

    def drain_reduce_grad_states_if_needed(self) -> None:
        """Bound the memory held by reductions in flight."""
        if self.max_pending_reduce_grads <= 0:
            return
        while len(self.reduce_grad_states) >= self.max_pending_reduce_grads:
            pending = self.reduce_grad_states.pop(0)
            self.wait_and_release_reduce_grad_state(pending, wait_current_stream=False)
            self.retired_reduce_grad_states.append(pending)

    def wait_and_clear_reduce_grad_states(self) -> None:
        """Order the reduced gradients before their use on the current stream
        (the optimizer step) and release the reductions' buffers."""
        for pending in self.retired_reduce_grad_states:
            pending.result.wait()
        self.retired_reduce_grad_states.clear()
        for pending in self.reduce_grad_states:
            self.wait_and_release_reduce_grad_state(pending, wait_current_stream=True)
        self.reduce_grad_states.clear()


@dataclass
class BucketParam:
    module: nn.Module
    param_name: str
    info: ParamInfo
    sharded_param: nn.Parameter


class BucketRuntime:
    """Runtime state of one bucket: this rank's sharded parameters (views of one
    flat storage at their ``ParamInfo.byte_offset``), the unsharded parameters
    of a persistent unshard and the buffers behind them."""

    def __init__(
        self,
        bucket_params: list[BucketParam],
        mesh: Any,
        context: BucketCommContext,
        gradient_reduction: GradientReduction,
        storage: torch.Tensor,
        debug_fqn: str | None = None,
    ) -> None:
        self.bucket_params = bucket_params
        self._infos = [bp.info for bp in bucket_params]
        self._sharded_params = [bp.sharded_param for bp in bucket_params]
        self.mesh = mesh
        self.context = context
        self.gradient_reduction = gradient_reduction
        self.storage = storage
        self.debug_fqn = debug_fqn
        self.unsharded_params: list[nn.Parameter] | None = None
        self.persistent_buffers: list[torch.Tensor] = []
        self.persistent_buffer_nbytes: list[int] = []
        self.is_unsharded = False
        self._hook_handles: list[Any] = []
        self._grads_seen = 0
        self._reduce_when_grads_arrive = False
        self._pending_unshard: UnshardHandle | None = None
        #: False: backwards keep their full-parameter gradients (microbatch
        #: accumulation); the next backward with this set reduces them.
        self.requires_gradient_sync = True
        self.needs_sync = False

    # ------------------------------------------------------------ construction
    @classmethod
    def shard_module_params(
        cls,
        root: nn.Module,
        fqns: list[str],
        placement: "Placement | dict[str, Placement]",
        mesh: Any,
        context: BucketCommContext,
        gradient_reduction: GradientReduction | None = None,
        reduce_dtype: torch.dtype | None = torch.float32,
    ) -> "BucketRuntime":
        """Cut this rank's rows out of the full parameters ``fqns`` of ``root``,
        lay them out in one flat storage as the placement's bucket layout says,
        and install them as the modules' parameters.  ``reduce_dtype`` is the
        mixed-precision policy's gradient dtype: full-parameter gradients
        accumulate and are reduced in it."""
        named = [(fqn, root.get_parameter(fqn)) for fqn in fqns]
        if isinstance(placement, dict):  # member placements of one bucket-scoped placement, by fqn
            param_placements = {fqn: (placement[fqn],) for fqn in fqns}
        else:
            param_placements = {fqn: (placement,) for fqn in fqns}
        infos, total_bytes = create_param_infos(named, param_placements, mesh)
        for info in infos:
            info.reduce_dtype = reduce_dtype
        rank, world_size = mesh.get_local_rank(), mesh.size()
        storage = torch.zeros(max(total_bytes, 1), dtype=torch.uint8, device=named[0][1].device)
        bucket_params = []
        for (fqn, param), info in zip(named, infos, strict=True):
            # the placement writes this rank's part of the parameter into the storage and views it
            info.placement.copy_param_to_storage(storage, info, param, rank, world_size)
            local = info.placement.make_local_storage_view(storage, info)
            sharded = nn.Parameter(local, requires_grad=param.requires_grad)
            module_path, _, name = fqn.rpartition(".")
            module = root.get_submodule(module_path) if module_path else root
            module._parameters[name] = sharded
            bucket_params.append(BucketParam(module=module, param_name=name, info=info, sharded_param=sharded))
        return cls(bucket_params, mesh, context, gradient_reduction or GradientReduction(), storage,
                   debug_fqn=fqns[0] if fqns else None)

    @property
    def infos(self) -> list[ParamInfo]:
        return self._infos

    @property
    def sharded_params(self) -> list[nn.Parameter]:
        return self._sharded_params

    def _local_shards(self) -> list[torch.Tensor]:
        return [p.detach() for p in self._sharded_params]

    # ---------------------------------------------------------------- unshard
    def begin_unshard(self, *, on_current_stream: bool = False, async_op: bool = False) -> UnshardHandle:
        """Begin this bucket's unshard on the shared unshard stream or, with
        ``on_current_stream``, on the current stream.  A refill re-allocates
        the persistent storage on the current stream (the one that frees it on
        reshard) before the unshard stream waits on it, unless the placement
        writes it only in finish."""
        persistent_buffers = None
        if self.unsharded_params is not None:
            if not self.infos[0].placement.refills_persistent_buffers_in_finish:
                self._alloc_persistent_storage()
            persistent_buffers = self.persistent_buffers
        return begin_bucket_unshard(
            self._local_shards(), self.infos, self.mesh,
            None if on_current_stream else self.context.next_unshard_stream(),
            debug_fqn=self.debug_fqn, persistent_buffers=persistent_buffers, async_op=async_op and on_current_stream,
        )

    def finish_unshard(self, result: UnshardHandle) -> None:
        """Finish ``result`` into the persistent buffers.  The first unshard
        creates the unsharded params from the placement's full params; later
        ones write the same buffers without bumping their version counters
        (autograd may have saved the params in forward before a reshard)."""
        with torch.inference_mode(False), torch.no_grad():
            if self.unsharded_params is None:
                unshard = result.finish()
                self._create_unsharded_params(unshard.full_params, unshard.persistent_buffers)
            else:
                if self.infos[0].placement.refills_persistent_buffers_in_finish:
                    self._alloc_persistent_storage()
                with torch.autograd._unsafe_preserve_version_counter(tuple(self.persistent_buffers)):
                    refill = result.finish()
                if len(refill.persistent_buffers) != len(self.persistent_buffers) or any(
                    a is not b for a, b in zip(refill.persistent_buffers, self.persistent_buffers)
                ):
                    raise AssertionError(
                        f"Placement {self.infos[0].placement!r} did not refill the persistent buffers it was given."
                    )
            for bp, unsharded in zip(self.bucket_params, self.unsharded_params, strict=True):
                if unsharded.requires_grad != bp.sharded_param.requires_grad:
                    unsharded.requires_grad_(bp.sharded_param.requires_grad)
        self.is_unsharded = True

    def prefetch(self) -> None:
        """Begin this bucket's unshard on the unshard stream ahead of its use
        (the quantize + pack and the exchange then run under the consumer
        stream's work); the next ``unshard`` finishes it instead of beginning
        one (reference: ``BucketCommContext.prefetch`` / ``take_pending_unshard``,
        bucket_runtime.py:300-396)."""
        if not self.is_unsharded and self._pending_unshard is None:
            self._pending_unshard = self.begin_unshard()

    def release_prefetch(self) -> None:
        """Drop a prefetched unshard that will not be used."""
        if self._pending_unshard is not None:
            self._pending_unshard.release_buffers()
            self._pending_unshard = None
            if self.unsharded_params is not None:
                self.free_persistent_storage()

    def unshard(self, *, on_current_stream: bool = False) -> None:
        """Make the unsharded params hold data and swap them into the modules."""
        if not self.is_unsharded:
            result, self._pending_unshard = self._pending_unshard, None
            if result is None:
                result = self.begin_unshard(on_current_stream=on_current_stream)
            self.finish_unshard(result)
        self._swap_in_params(self.unsharded_params)

    def _create_unsharded_params(self, full_params: list[torch.Tensor], persistent_buffers: list[torch.Tensor]) -> None:
        if not persistent_buffers:
            raise AssertionError(
                f"Placement {self.infos[0].placement!r} returned no persistent buffers for a persistent unshard."
            )
        buffer_storages = {b.untyped_storage().data_ptr() for b in persistent_buffers}
        unsharded_params = []
        for bp, full in zip(self.bucket_params, full_params, strict=True):
            # Refills write into the persistent buffers, so the params (or a
            # wrapper subclass's inner tensors) must view them.
            if any(
                inner.numel() and inner.untyped_storage().data_ptr() not in buffer_storages
                for inner in _inner_tensors(full)
            ):
                raise AssertionError(
                    f"Placement {bp.info.placement!r} returned full param {bp.info.fqn!r}, which does not view its "
                    "persistent buffers, so refills would not reach it."
                )
            unsharded = nn.Parameter(full, requires_grad=bp.sharded_param.requires_grad)
            for name, value in bp.info.param_attrs.items():
                setattr(unsharded, name, value)
            # autograd casts each incoming gradient before accumulating it
            unsharded.grad_dtype = bp.info.unsharded_grad_dtype
            unsharded_params.append(unsharded)
        self.unsharded_params = unsharded_params
        self.persistent_buffers = list(persistent_buffers)
        self.persistent_buffer_nbytes = [b.untyped_storage().size() for b in persistent_buffers]
        if self._reduce_when_grads_arrive:
            self._register_grad_hooks()

    def _swap_in_params(self, params: list[torch.Tensor]) -> None:
        for bp, param in zip(self.bucket_params, params, strict=True):
            bp.module._parameters[bp.param_name] = param

    def reshard(self) -> None:
        """Swap the local shards back in and free the persistent storage."""
        self._swap_in_params(self.sharded_params)
        self.free_persistent_storage()
        self.is_unsharded = False

    def _alloc_persistent_storage(self) -> None:
        with torch.inference_mode(False):
            for buffer, nbytes in zip(self.persistent_buffers, self.persistent_buffer_nbytes, strict=True):
                _alloc_storage(buffer, nbytes)

    def free_persistent_storage(self) -> None:
        """Consumers of the storage were queued on the current stream, which
        also allocated it (a refill's unshard stream writes it only after
        waiting on this stream), so the caching allocator orders the reuse."""
        for buffer in self.persistent_buffers:
            _free_storage(buffer)

    # --------------------------------------------------------------- gradients
    def reduce_grads(self, grads: list[torch.Tensor] | None = None) -> None:
        """Reduce the full-parameter gradients and accumulate this rank's
        shards into the sharded parameters' ``.grad``.  Without ``grads`` the
        unsharded parameters' ``.grad`` are taken (and cleared)."""
        if grads is None:
            assert self.unsharded_params is not None
            pairs = [(bp, up) for bp, up in zip(self.bucket_params, self.unsharded_params) if up.grad is not None]
            grads = [up.grad for _, up in pairs]
            for _, up in pairs:
                up.grad = None
            chosen = [bp for bp, _ in pairs]
        else:
            chosen = list(self.bucket_params)
        if not grads:
            return
        if len(chosen) != len(self.bucket_params):
            missing = sorted({bp.info.fqn for bp in self.bucket_params} - {bp.info.fqn for bp in chosen})
            raise RuntimeError(f"bucket parameters {missing} have no gradient; this slice reduces whole buckets")
        infos = [bp.info for bp in chosen]
        sharded_params = [bp.sharded_param for bp in chosen]
        with torch.no_grad():
            self.context.drain_reduce_grad_states_if_needed()
            # A 1-rank mesh has nothing to exchange: reduce on the current stream.
            stream = (
                torch.cuda.current_stream(grads[0].device) if self.mesh.size() == 1 else self.context.reduce_grad_stream
            )
            result = begin_reduce_grad(grads, infos, self.mesh, self.gradient_reduction, stream, debug_fqn=self.debug_fqn)
            with torch.cuda.stream(stream):
                sharded_grads = result.finish()
                result.record_sharded_grads(_accumulate_sharded_grads(sharded_params, sharded_grads), stream)
            self.context.reduce_grad_states.append(PendingReduceGrad(result))

    def set_requires_gradient_sync(self, requires_gradient_sync: bool) -> None:
        """Whether a backward reduces this bucket's gradients (the last
        microbatch) or only accumulates them on the unsharded parameters."""
        self.requires_gradient_sync = requires_gradient_sync

    def _set_unsharded_grad_dtypes(self, *, defer_upcast: bool) -> None:
        """Defer or restore the upcast of gradients that accumulate in a wider
        dtype than the parameter computes in (reference:
        ``_set_unsharded_grad_dtypes``, bucket_runtime.py:1062-1108).

        Deferred (``grad_dtype = None``), in a backward that reduces or that
        adds to a kept gradient, autograd leaves the gradients in the compute
        dtype: the reduce-scatter copy-in widens them as it copies (one cast
        launch per parameter less, and half the bytes read by the copy-in) and
        AccumulateGrad adds them in place to a wider kept gradient.  A backward
        without sync that starts a gradient keeps the upcast, so that the sum
        over microbatches is taken in the wider dtype.  Restoring upcasts a new
        gradient that was not reduced, once."""
        for bp, param in zip(self.bucket_params, self.unsharded_params or [], strict=False):
            dtype, compute_dtype = bp.info.unsharded_grad_dtype, bp.info.unsharded_dtype
            if (
                dtype is None
                or not param.requires_grad
                or not dtype.is_floating_point
                or not compute_dtype.is_floating_point
                or dtype.itemsize <= compute_dtype.itemsize
            ):
                continue
            if defer_upcast:
                if param.grad is not None or self.requires_gradient_sync:
                    param.grad_dtype = None
                continue
            grad = param.grad
            if grad is not None and grad.dtype != dtype:
                param.grad = grad.to(dtype)
            param.grad_dtype = dtype

    # ------------------------------------------------------------------- hooks
    def install_hooks(
        self,
        module: nn.Module,
        *,
        forward_prefetch: "BucketRuntime | None" = None,
        backward_prefetch: "BucketRuntime | None" = None,
    ) -> None:
        """Unshard before ``module``'s forward, reshard after it, unshard again
        when its backward starts, and reduce + reshard once every parameter of
        the bucket has its gradient (one use of each parameter per forward).
        ``forward_prefetch`` / ``backward_prefetch``: the bucket used next in
        the forward / in the backward; its unshard is begun on a side stream as
        soon as this bucket's own is finished, so that its quantize + pack and
        exchange run under this module's compute (the explicit form of the
        reference's prefetch order, bucket_runtime.py:300-396)."""

        def pre_forward(mod: nn.Module, args: Any) -> None:
            self.unshard()
            self._grads_seen = 0
            if forward_prefetch is not None:
                forward_prefetch.prefetch()

        def pre_backward(_grads: Any) -> None:
            self.unshard()
            self._set_unsharded_grad_dtypes(defer_upcast=True)
            if backward_prefetch is not None:
                backward_prefetch.prefetch()

        def post_forward(mod: nn.Module, args: Any, output: Any) -> Any:
            self.reshard()
            tensors = [t for t in (output if isinstance(output, (tuple, list)) else (output,))
                       if isinstance(t, torch.Tensor) and t.requires_grad]
            if tensors:
                torch.autograd.graph.register_multi_grad_hook(tensors, pre_backward, mode="any")
            return output

        self._hook_handles.append(module.register_forward_pre_hook(pre_forward))
        self._hook_handles.append(module.register_forward_hook(post_forward))
        self._reduce_when_grads_arrive = True
        if self.unsharded_params is not None:
            self._register_grad_hooks()

    def _on_param_grad(self, _param: torch.Tensor) -> None:
        self._grads_seen += 1
        expected = sum(1 for p in self.unsharded_params if p.requires_grad)
        if self._grads_seen == expected:
            if self.requires_gradient_sync:
                self.needs_sync = False
                self.reduce_grads()  # takes the gradients; the copy-in casts them to the reduce dtype
                self._set_unsharded_grad_dtypes(defer_upcast=False)
                self.reshard()
            else:
                self.needs_sync = True
                self.reshard()
                # after the reshard, so that a deferred gradient's upcast never coexists with the full parameters
                self._set_unsharded_grad_dtypes(defer_upcast=False)

    def _register_grad_hooks(self) -> None:
        for param in self.unsharded_params:
            if param.requires_grad:
                self._hook_handles.append(param.register_post_accumulate_grad_hook(self._on_param_grad))


__all__ = ["BucketCommContext", "BucketParam", "BucketRuntime", "PendingReduceGrad"]
