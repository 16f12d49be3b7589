"""MI355X-native hot path of FlexShard's bucketed placements.

Python host code keeps the reference's placement contract and the
``Fp8BucketedBlockShard`` / ``BucketedBlockShard`` / ``BucketedOwned`` placements
as the drop-in surface; all device work is hand-written HIP for gfx950 behind
the C ABI of ``libflexshard_hip.so`` (``include/flexshard_hip.h``).
"""

from .bucket_storage import BucketLayout, BucketParamLayout, ParamInfo, create_param_infos
from .custom_placements import (
    BlockShard,
    BucketedBlockShard,
    BucketedOwned,
    BucketedOwnedSegmentSpec,
    Fp8BucketedBlockShard,
    LocalReduceGroup,
    MixedBucketPlacement,
    Shard,
    make_bucketed_block_placement_fn,
    make_bucketed_owned_full_param_placement_fn,
    make_fp8_bucketed_block_placement_fn,
)
from .placement_contract import (
    BucketParamStorageLayout,
    BucketStorageLayout,
    GlobalLayout,
    GradientReduction,
    LocalStorageLayout,
    Placement,
    PlacementPreparedReduceGrad,
    PlacementPreparedUnshard,
    PlacementReduceGradResult,
    PlacementUnshardResult,
    compose_global_layouts,
    get_global_layout,
    set_global_layout,
)

__all__ = [
    "BlockShard",
    "BucketLayout",
    "BucketParamLayout",
    "BucketParamStorageLayout",
    "BucketStorageLayout",
    "BucketedBlockShard",
    "BucketedOwned",
    "BucketedOwnedSegmentSpec",
    "Fp8BucketedBlockShard",
    "GlobalLayout",
    "GradientReduction",
    "LocalReduceGroup",
    "LocalStorageLayout",
    "MixedBucketPlacement",
    "ParamInfo",
    "Placement",
    "PlacementPreparedReduceGrad",
    "PlacementPreparedUnshard",
    "PlacementReduceGradResult",
    "PlacementUnshardResult",
    "Shard",
    "compose_global_layouts",
    "create_param_infos",
    "get_global_layout",
    "make_bucketed_block_placement_fn",
    "make_bucketed_owned_full_param_placement_fn",
    "make_fp8_bucketed_block_placement_fn",
    "set_global_layout",
]
