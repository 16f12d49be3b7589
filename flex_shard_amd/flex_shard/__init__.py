"""Stream hand-off and the per-bucket runtime slice that drive the placements
under a forward and a backward on one GPU."""

from .bucket_comm import (
    ReduceGradHandle,
    StreamHandoff,
    UnshardHandle,
    begin_bucket_unshard,
    begin_explicit_bucket_unshard,
    begin_reduce_grad,
)
from .checkpoint import (
    copy_full_into_shard,
    copy_shard_into_full,
    get_flex_shard_global_layouts,
    register_optimizer_checkpoint_hook,
    set_state_dict_global_layouts,
)
from .bucket_runtime import BucketCommContext, BucketParam, BucketRuntime, PendingReduceGrad

__all__ = [
    "BucketCommContext", "BucketParam", "BucketRuntime", "PendingReduceGrad", "ReduceGradHandle", "StreamHandoff", "UnshardHandle",
    "begin_bucket_unshard", "begin_explicit_bucket_unshard", "begin_reduce_grad", "copy_full_into_shard",
    "copy_shard_into_full", "get_flex_shard_global_layouts", "register_optimizer_checkpoint_hook",
    "set_state_dict_global_layouts",
]
