from .blockwise_fp8_weight import BlockwiseFp8Weight, blockwise_dequant_weight, make_blockwise_fp8_weight

__all__ = ["BlockwiseFp8Weight", "blockwise_dequant_weight", "make_blockwise_fp8_weight"]
