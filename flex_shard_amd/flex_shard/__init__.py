"""Stream hand-off and the per-bucket runtime slice that drive the placements
under a forward and a backward on one GPU."""

from .bucket_comm import (
    AsyncReduceGradResult,
    AsyncUnshardResult,
    ExplicitUnshardResult,
    ReduceGradHandle,
    StreamHandoff,
    UnshardHandle,
    begin_bucket_unshard,
    begin_explicit_bucket_unshard,
    begin_reduce_grad,
)
from .bucket_runtime import BucketCommContext, BucketParam, BucketRuntime, PendingReduceGrad

__all__ = [
    "AsyncReduceGradResult", "AsyncUnshardResult", "BucketCommContext", "BucketParam", "BucketRuntime",
    "ExplicitUnshardResult", "PendingReduceGrad", "ReduceGradHandle", "StreamHandoff", "UnshardHandle",
    "begin_bucket_unshard", "begin_explicit_bucket_unshard", "begin_reduce_grad",
]
