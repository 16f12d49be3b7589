from .blockwise_fp8_weight import BlockwiseFp8Weight, blockwise_dequant_weight, make_blockwise_fp8_weight
from .fp8_blockwise_linear import (
    FlexShardFloat8BlockwiseLinear,
    Fp8BlockwiseGemms,
    convert_to_flex_shard_float8_blockwise_linear,
    prequantized_linear,
)

__all__ = [
    "BlockwiseFp8Weight", "FlexShardFloat8BlockwiseLinear", "Fp8BlockwiseGemms", "blockwise_dequant_weight",
    "convert_to_flex_shard_float8_blockwise_linear", "make_blockwise_fp8_weight", "prequantized_linear",
]
