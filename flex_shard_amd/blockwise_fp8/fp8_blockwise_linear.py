"""Blockwise FP8 linear consumer for weights prequantized by the FP8 unshard.

Mirror of the reference's ``blockwise_fp8/fp8_blockwise_linear.py:42-91``
(``Fp8BlockwiseGemms.forward``): the activation is quantized in runs of 1x128
and multiplied with the gathered 128x128-scaled FP8 weight on the FP8 matrix
cores, both scale sets applied per k-block in fp32.  The reference takes both
kernels from torchao (``triton_fp8_blockwise_act_quant_lhs``,
``triton_fp8_gemm_1x128_128x128``); here they are ``fsh_act_quant_1x128`` and
``fsh_fp8_gemm_1x128_128x128`` of the HIP library.  The backward products
(:93-162 of the reference file) are not built yet and raise.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .. import hip_ops
from .blockwise_fp8_weight import BlockwiseFp8Weight


def _pad_last_dim_to(tensor: torch.Tensor, target_dim: int) -> torch.Tensor:
    """Zero-pad the last dimension (reference: blockwise_quant/linear.py:49-62)."""
    if tensor.shape[-1] == target_dim:
        return tensor
    if tensor.shape[-1] > target_dim:
        raise ValueError(f"Cannot pad last dim from {tensor.shape[-1]} down to {target_dim}.")
    padded = torch.zeros((*tensor.shape[:-1], target_dim), dtype=tensor.dtype, device=tensor.device)
    padded[..., : tensor.shape[-1]].copy_(tensor)
    return padded


@dataclass(frozen=True)
class Fp8BlockwiseGemms:
    """1x128 activation / 128x128 weight blockwise FP8 GEMMs."""

    block_size: int
    out_dtype: torch.dtype = torch.bfloat16

    def forward(self, x_2d: torch.Tensor, weight: BlockwiseFp8Weight) -> torch.Tensor:
        """``x_2d @ weight_matrix.T`` with shape ``(tokens, rows)``; a stacked
        ``[*stack, out, in]`` weight multiplies as its flattened matrix."""
        if self.block_size != weight.block_size:
            raise ValueError(
                f"linear block_size {self.block_size} does not match gathered weight block_size {weight.block_size}"
            )
        if self.block_size != 128:
            raise AssertionError("the blockwise FP8 GEMM only supports block_size 128")
        if weight.fp8_data.dtype != torch.float8_e4m3fn:
            raise NotImplementedError(f"the FP8 GEMM reads float8_e4m3fn weights, not {weight.fp8_data.dtype}")
        if self.out_dtype != torch.bfloat16:
            raise NotImplementedError(f"the FP8 GEMM writes bf16, not {self.out_dtype}")
        if x_2d.ndim != 2:
            raise ValueError(f"expected a 2D activation, got {tuple(x_2d.shape)}")
        weight_matrix = weight.fp8_data.flatten(0, -2)
        logical_out_dim, in_dim = weight_matrix.shape
        if x_2d.shape[1] != in_dim:
            raise ValueError(f"input last dim {x_2d.shape[1]} does not match weight input dim {in_dim}")
        if x_2d.dtype != torch.bfloat16:
            x_2d = x_2d.to(torch.bfloat16)
        if x_2d.stride(1) != 1 or x_2d.stride(0) % 8 or x_2d.data_ptr() % 16:
            x_2d = x_2d.contiguous()
        if in_dim % 8:
            x_2d = _pad_last_dim_to(x_2d, -(-in_dim // 8) * 8)
        # The quantizer pads the activation to whole 128-element runs itself;
        # only a weight whose rows are not whole runs has to be copied.
        x_fp8, x_scale = hip_ops.act_quant_1x128(x_2d)
        padded_in_dim = x_fp8.shape[1]
        if weight_matrix.shape[1] != padded_in_dim or weight_matrix.stride(1) != 1 or weight_matrix.stride(0) % 16:
            weight_matrix = _pad_last_dim_to(weight_matrix.view(torch.uint8), padded_in_dim).view(torch.float8_e4m3fn)
        return hip_ops.fp8_gemm_1x128_128x128(x_fp8, x_scale, weight_matrix, weight.recip_scale)

    def backward(self, grad_output_2d, x_2d, weight, needs_x_grad, needs_weight_grad):
        raise NotImplementedError(
            "the backward products of the blockwise FP8 linear (1x128 x 128x128 for the input gradient, "
            "1x128 x 128x1 for the weight gradient) are not built yet"
        )


__all__ = ["Fp8BlockwiseGemms"]
