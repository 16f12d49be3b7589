from .blockwise_fp8_weight import BlockwiseFp8Weight, blockwise_dequant_weight, make_blockwise_fp8_weight
from .fp8_blockwise_linear import Fp8BlockwiseGemms

__all__ = ["BlockwiseFp8Weight", "Fp8BlockwiseGemms", "blockwise_dequant_weight", "make_blockwise_fp8_weight"]
