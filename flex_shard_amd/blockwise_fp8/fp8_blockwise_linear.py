"""Blockwise FP8 linear consumer for weights prequantized by the FP8 unshard.

Mirror of the reference's ``blockwise_fp8/fp8_blockwise_linear.py:42-91``
(``Fp8BlockwiseGemms.forward``): the activation is quantized in runs of 1x128
and multiplied with the gathered 128x128-scaled FP8 weight on the FP8 matrix
cores, both scale sets applied per k-block in fp32.  The reference takes both
kernels from torchao (``triton_fp8_blockwise_act_quant_lhs``,
``triton_fp8_gemm_1x128_128x128``); here they are ``fsh_act_quant_1x128`` and
``fsh_fp8_gemm_1x128_128x128`` of the HIP library.

``Fp8BlockwiseGemms.backward`` mirrors :93-162: the input gradient is the same
1x128 x 128x128 product against the transposed weight bytes
(``fsh_fp8_transpose`` + ``fsh_fp8_gemm_1x128_128x128_dgrad``), the weight
gradient a 1x128 x 128x1 product over the tokens, both operands quantized in
runs of 128 tokens and written transposed
(``fsh_act_quant_128x1_transposed``, ``fsh_fp8_gemm_1x128_128x1``).

``prequantized_linear`` / ``FlexShardFloat8BlockwiseLinear`` are the autograd
function and the ``nn.Linear`` replacement of the reference's
``blockwise_quant/linear.py:74-155`` and ``fp8_blockwise_linear.py:165-213``.
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any

import torch
import torch.nn as nn

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


class _SharedActivationQuantizer:
    """The last quantization of an activation in each of the two forms (runs
    along a row for the forward, runs of tokens for the weight gradient).

    Projections that read the same activation (q, k and v; gate and up)
    quantize it with the same arithmetic, so the second and third ask for the
    very bytes the first produced: the result is kept until another tensor is
    quantized in that form and handed out again when the request names the
    same memory (address, shape, strides), unchanged since (version counter),
    on the same stream.  The entry holds the activation itself, so its memory
    cannot have been handed to another tensor in the meantime; that keeps at
    most one activation per form alive a little longer.  Only the saving is
    new: the outputs are the ones the quantizer would write again."""

    def __init__(self) -> None:
        self._entries: dict[str, tuple] = {}
        self.enabled = True

    def quantize(self, form: str, x: torch.Tensor, quantizer) -> tuple[torch.Tensor, torch.Tensor]:
        if not self.enabled or torch.compiler.is_compiling():
            return quantizer(x)
        key = (x.data_ptr(), x._version, x.shape, x.stride(), x.dtype, hip_ops.stream_ptr(x.device))
        entry = self._entries.get(form)
        if entry is not None and entry[0] == key:
            return entry[2]
        result = quantizer(x)
        self._entries[form] = (key, x, result)
        return result

    def quantize_both(self, x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
        """Both forms of ``x`` from one pass over it (``hip_ops.act_quant_both``),
        kept and handed out like the single forms."""
        if not self.enabled or torch.compiler.is_compiling():
            return hip_ops.act_quant_both(x)
        key = (x.data_ptr(), x._version, x.shape, x.stride(), x.dtype, hip_ops.stream_ptr(x.device))
        rows, runs = self._entries.get("rows"), self._entries.get("token_runs")
        if rows is not None and runs is not None and rows[0] == key and runs[0] == key:
            return (*rows[2], *runs[2])
        result = hip_ops.act_quant_both(x)
        self._entries["rows"] = (key, x, result[:2])
        self._entries["token_runs"] = (key, x, result[2:])
        return result

    def clear(self) -> None:
        self._entries.clear()


#: shared by every ``Fp8BlockwiseGemms`` (the linears of a model create one per call)
shared_activation_quantizer = _SharedActivationQuantizer()


@dataclass(frozen=True)
class Fp8BlockwiseGemms:
    """1x128 activation / 128x128 weight blockwise FP8 GEMMs."""

    block_size: int
    out_dtype: torch.dtype = torch.bfloat16
    #: ``backward`` reads a gradient whose rows are strided (a slice of a wider
    #: matrix) in place; the autograd function then hands it over as it is
    accepts_strided_rows = True

    def forward(self, x_2d: torch.Tensor, weight: BlockwiseFp8Weight) -> torch.Tensor:
        """``x_2d @ weight_matrix.T`` with shape ``(tokens, rows)``; a stacked
        ``[*stack, out, in]`` weight multiplies as its flattened matrix."""
        return self._forward(x_2d, weight, False)[0]

    def forward_with_token_runs(
        self, x_2d: torch.Tensor, weight: BlockwiseFp8Weight
    ) -> tuple[torch.Tensor, tuple[torch.Tensor, torch.Tensor]]:
        """:meth:`forward`, and the activation quantized in runs of 128 tokens,
        transposed, with its scales: what :meth:`backward` needs of ``x_2d`` for
        the weight gradient (pass it as ``x_token_runs``).  The one pass over
        the activation that quantizes it for the product writes this form too,
        so the backward neither keeps nor re-reads the bf16 activation."""
        return self._forward(x_2d, weight, True)

    def _forward(self, x_2d: torch.Tensor, weight: BlockwiseFp8Weight, with_token_runs: bool):
        self._check(weight)
        if x_2d.ndim != 2:
            raise ValueError(f"expected a 2D activation, got {tuple(x_2d.shape)}")
        weight_matrix = weight.fp8_data.flatten(0, -2)
        logical_out_dim, in_dim = weight_matrix.shape
        if x_2d.shape[1] != in_dim:
            raise ValueError(f"input last dim {x_2d.shape[1]} does not match weight input dim {in_dim}")
        x_2d = _as_quantizer_input(x_2d)
        # The quantizer pads the activation to whole 128-element runs itself;
        # only a weight whose rows are not whole runs has to be copied.
        token_runs = None
        if with_token_runs:
            x_fp8, x_scale, *token_runs = shared_activation_quantizer.quantize_both(x_2d)
            token_runs = tuple(token_runs)
        else:
            x_fp8, x_scale = shared_activation_quantizer.quantize("rows", x_2d, hip_ops.act_quant_1x128)
        padded_in_dim = x_fp8.shape[1]
        if weight_matrix.shape[1] != padded_in_dim or weight_matrix.stride(1) != 1 or weight_matrix.stride(0) % 16:
            weight_matrix = _pad_last_dim_to(weight_matrix.view(torch.uint8), padded_in_dim).view(torch.float8_e4m3fn)
        return hip_ops.fp8_gemm_1x128_128x128(x_fp8, x_scale, weight_matrix, weight.recip_scale), token_runs

    def _check(self, weight: BlockwiseFp8Weight) -> None:
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

    def backward(
        self,
        grad_output_2d: torch.Tensor,
        x_2d: torch.Tensor | None,
        weight: BlockwiseFp8Weight,
        needs_x_grad: bool,
        needs_weight_grad: bool,
        *,
        x_token_runs: tuple[torch.Tensor, torch.Tensor] | None = None,
    ) -> tuple[torch.Tensor | None, torch.Tensor | None]:
        """``(grad_x_2d, grad_weight)``; ``grad_weight`` is contiguous, has the
        weight's shape and its original dtype.  With ``x_token_runs`` (from
        :meth:`forward_with_token_runs`) ``x_2d`` may be None."""
        self._check(weight)
        weight_matrix = weight.fp8_data.flatten(0, -2)
        out_dim, in_dim = weight_matrix.shape
        if grad_output_2d.ndim != 2 or grad_output_2d.shape[1] != out_dim:
            raise ValueError(f"grad_output {tuple(grad_output_2d.shape)} does not match weight output dim {out_dim}")
        tokens = grad_output_2d.shape[0]
        if x_token_runs is not None:
            runs_fp8, runs_scale = x_token_runs
            want = (-(-in_dim // 8) * 8, -(-tokens // 128) * 128)
            if tuple(runs_fp8.shape) != want or tuple(runs_scale.shape) != (want[1] // 128, want[0]):
                raise ValueError(
                    f"x_token_runs {tuple(runs_fp8.shape)} / {tuple(runs_scale.shape)} do not match {tokens} tokens "
                    f"and weight input dim {in_dim}"
                )
        elif x_2d is None:
            raise ValueError("backward needs the activation or its token-run form")
        if x_2d is not None and (x_2d.ndim != 2 or x_2d.shape != (tokens, in_dim)):
            raise ValueError(
                f"activation {tuple(x_2d.shape)} does not match grad_output {tuple(grad_output_2d.shape)} "
                f"and weight input dim {in_dim}"
            )
        grad_output_2d = _as_quantizer_input(grad_output_2d)
        grad_x = grad_weight = None
        grad_t_fp8 = grad_t_scale = None
        if needs_x_grad:
            # runs of 128 along the output index; the quantizer zero-pads it to whole runs.
            # When the weight gradient is wanted too, the same pass over grad_output
            # also writes its token-run form.
            if needs_weight_grad:
                grad_fp8, grad_scale, grad_t_fp8, grad_t_scale = hip_ops.act_quant_both(grad_output_2d)
            else:
                grad_fp8, grad_scale = hip_ops.act_quant_1x128(grad_output_2d)
            if in_dim % 16 or weight_matrix.stride(1) != 1 or weight_matrix.stride(0) % 16:
                weight_matrix = _pad_last_dim_to(weight_matrix.view(torch.uint8), -(-in_dim // 16) * 16).view(
                    torch.float8_e4m3fn
                )
            weight_t_fp8 = hip_ops.fp8_transpose(weight_matrix)  # [in, out rounded up to 128]
            grad_x = hip_ops.fp8_gemm_1x128_128x128_dgrad(
                grad_fp8, grad_scale, weight_t_fp8, weight.recip_scale, in_dim=in_dim
            )
        if needs_weight_grad:
            # runs of 128 tokens for both operands; the quantizer pads the token count itself
            if grad_t_fp8 is None:
                grad_t_fp8, grad_t_scale = hip_ops.act_quant_128x1_transposed(grad_output_2d)
            if x_token_runs is not None:
                x_t_fp8, x_t_scale = x_token_runs
            else:
                x_t_fp8, x_t_scale = shared_activation_quantizer.quantize(
                    "token_runs", _as_quantizer_input(x_2d), hip_ops.act_quant_128x1_transposed
                )
            grad_weight = hip_ops.fp8_gemm_1x128_128x1(grad_t_fp8, grad_t_scale, x_t_fp8, x_t_scale)
            grad_weight = grad_weight[:out_dim, :in_dim].to(weight.dtype).contiguous().view(weight.shape)
        return grad_x, grad_weight


def _as_quantizer_input(matrix: torch.Tensor) -> torch.Tensor:
    """bf16, contiguous rows on 16-byte boundaries, a multiple of 8 columns."""
    if matrix.dtype != torch.bfloat16:
        matrix = matrix.to(torch.bfloat16)
    if matrix.shape[1] % 8:
        return _pad_last_dim_to(matrix, -(-matrix.shape[1] // 8) * 8)
    if matrix.stride(1) != 1 or matrix.stride(0) % 8 or matrix.data_ptr() % 16:
        matrix = matrix.contiguous()
    return matrix


class _PrequantizedLinearFunction(torch.autograd.Function):
    """``x @ W.T (+ bias)`` on a prequantized weight, with both gradients
    (reference: blockwise_quant/linear.py:74-123)."""

    @staticmethod
    def forward(ctx: Any, x: torch.Tensor, weight: BlockwiseFp8Weight, bias: torch.Tensor | None, gemms):
        x_shape = x.shape
        x_2d = x.reshape(-1, x_shape[-1])
        if x_2d.shape[-1] != weight.shape[-1]:
            raise ValueError(f"input last dim {x_2d.shape[-1]} does not match weight input dim {weight.shape[-1]}")
        # With a weight gradient to come, the pass that quantizes x for the
        # product also writes the form the weight gradient contracts over, and
        # that (1 byte per element) is kept instead of x.
        keeps_token_runs = (
            ctx.needs_input_grad[1] and hasattr(gemms, "forward_with_token_runs") and not torch.compiler.is_compiling()
        )
        if keeps_token_runs:
            out, token_runs = gemms.forward_with_token_runs(x_2d, weight)
            ctx.save_for_backward(weight, *token_runs)
        else:
            out = gemms.forward(x_2d, weight)
            ctx.save_for_backward(weight, x)
        out = out.reshape(*x_shape[:-1], *weight.shape[:-1])
        if bias is not None:
            out = out + bias
        ctx.keeps_token_runs = keeps_token_runs
        ctx.x_shape = x_shape
        ctx.gemms = gemms
        ctx.has_bias = bias is not None
        return out

    @staticmethod
    def backward(ctx: Any, grad_output: torch.Tensor):
        weight, *kept = ctx.saved_tensors
        out_dim = math.prod(weight.shape[:-1])
        grad_output_2d = grad_output.reshape(-1, out_dim)
        if not getattr(ctx.gemms, "accepts_strided_rows", False):
            grad_output_2d = grad_output_2d.contiguous()
        needs_x_grad, needs_weight_grad, needs_bias_grad = ctx.needs_input_grad[:3]
        if ctx.keeps_token_runs:
            grad_x, grad_weight = ctx.gemms.backward(
                grad_output_2d, None, weight, needs_x_grad, needs_weight_grad, x_token_runs=tuple(kept)
            )
        else:
            (x,) = kept
            grad_x, grad_weight = ctx.gemms.backward(
                grad_output_2d, x.reshape(-1, x.shape[-1]), weight, needs_x_grad, needs_weight_grad
            )
        if grad_x is not None:
            grad_x = grad_x.reshape(ctx.x_shape)
        grad_bias = None
        if ctx.has_bias and needs_bias_grad:
            grad_bias = grad_output_2d.sum(dim=0).view(weight.shape[:-1])
        return grad_x, grad_weight, grad_bias, None


def prequantized_linear(
    x: torch.Tensor, weight: BlockwiseFp8Weight, bias: torch.Tensor | None = None, gemms: Fp8BlockwiseGemms | None = None
) -> torch.Tensor:
    """Differentiable ``x @ W.T + bias`` on a gathered blockwise FP8 weight; a
    stacked ``[*stack, out, in]`` weight returns ``[..., *stack, out]``."""
    if not isinstance(weight, BlockwiseFp8Weight):
        raise TypeError(
            f"prequantized_linear requires a BlockwiseFp8Weight produced by an FP8 unshard, got {type(weight).__name__}."
        )
    return _PrequantizedLinearFunction.apply(x, weight, bias, gemms or Fp8BlockwiseGemms(weight.block_size))


class FlexShardFloat8BlockwiseLinear(nn.Linear):
    """``nn.Linear`` whose weight is replaced, between unshard and reshard, by
    the ``BlockwiseFp8Weight`` of an FP8 unshard (reference:
    fp8_blockwise_linear.py:165-213).  ``block_size`` is fixed at 128."""

    weight_type = BlockwiseFp8Weight
    block_size = 128

    @classmethod
    def from_float(cls, mod: nn.Linear) -> "FlexShardFloat8BlockwiseLinear":
        with torch.device("meta"):
            new_mod = cls(mod.in_features, mod.out_features, bias=mod.bias is not None)
        new_mod.weight = mod.weight
        new_mod.bias = mod.bias
        new_mod.train(mod.training)
        return new_mod

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        weight = self.weight
        if not isinstance(weight, self.weight_type):
            raise TypeError(
                f"{type(self).__name__} requires a {self.weight_type.__name__} produced by a FlexShard quantized "
                f"all-gather, got {type(weight).__name__}."
            )
        return _PrequantizedLinearFunction.apply(input, weight, self.bias, Fp8BlockwiseGemms(self.block_size))


def convert_to_flex_shard_float8_blockwise_linear(module: nn.Module, filter_fn=None) -> nn.Module:
    """Swap every ``nn.Linear`` below ``module`` that ``filter_fn(fqn, child)``
    accepts (all, when it is None) for a ``FlexShardFloat8BlockwiseLinear``
    sharing its parameters (reference: blockwise_quant/linear.py:158-184)."""
    for name, child in list(module.named_children()):
        _convert_child(module, name, child, name, filter_fn)
    return module


def _convert_child(parent: nn.Module, name: str, child: nn.Module, fqn: str, filter_fn) -> None:
    if isinstance(child, FlexShardFloat8BlockwiseLinear):
        return
    if isinstance(child, nn.Linear) and (filter_fn is None or filter_fn(fqn, child)):
        setattr(parent, name, FlexShardFloat8BlockwiseLinear.from_float(child))
        return
    for sub_name, sub_child in list(child.named_children()):
        _convert_child(child, sub_name, sub_child, f"{fqn}.{sub_name}", filter_fn)


__all__ = [
    "FlexShardFloat8BlockwiseLinear", "Fp8BlockwiseGemms", "convert_to_flex_shard_float8_blockwise_linear",
    "prequantized_linear", "shared_activation_quantizer",
]
