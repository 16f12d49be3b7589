"""Placements on the single-GPU hot path: FP8 bucketed block shard, dense
bucketed block shard, and the owner placement (layout side)."""

from .block_shard import BlockShard, BucketedBlockShard, make_bucketed_block_placement_fn
from .blockwise_quant_bucketed_block_shard import BlockwiseQuantBucketedBlockShard
from .fp8_bucketed_block_shard import (
    BlockwiseFp8WeightFactory,
    Fp8BucketedBlockShard,
    make_fp8_bucketed_block_placement_fn,
)
from .mixed_bucket import MixedBucketPlacement
from .owned import (
    BucketedOwned,
    BucketedOwnedSegmentSpec,
    make_bucketed_owned_expert_block_placement_fn,
    make_bucketed_owned_expert_block_segments,
    make_bucketed_owned_full_param_placement_fn,
    make_bucketed_owned_full_param_segments,
)
from .shard import Shard, make_shard_placement_fn
from .utils import LocalReduceGroup

__all__ = [
    "BlockShard",
    "BlockwiseFp8WeightFactory",
    "BlockwiseQuantBucketedBlockShard",
    "BucketedBlockShard",
    "BucketedOwned",
    "BucketedOwnedSegmentSpec",
    "Fp8BucketedBlockShard",
    "LocalReduceGroup",
    "MixedBucketPlacement",
    "Shard",
    "make_bucketed_block_placement_fn",
    "make_bucketed_owned_expert_block_placement_fn",
    "make_bucketed_owned_expert_block_segments",
    "make_bucketed_owned_full_param_placement_fn",
    "make_bucketed_owned_full_param_segments",
    "make_fp8_bucketed_block_placement_fn",
    "make_shard_placement_fn",
]
