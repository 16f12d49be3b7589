"""The hot path in eager torch CPU ops.  TEST INFRASTRUCTURE ONLY.

Each function spells the reference algorithm with the same torch operators
and dtypes the reference uses, so its results are what the reference's CPU
path produces; it doubles as the timed CPU baseline of ``bench.py``.
Citations are paths under the reference checkout (``src/flex_shard/...``).
"""

from __future__ import annotations

import math

import torch

FP8_MAX = 448.0
EPS = 1e-12


def _tile_view(matrix: torch.Tensor, block: int) -> tuple[torch.Tensor, int, int]:
    """Zero-pad to whole tiles and view as [tile_row, block, tile_col, block]."""
    rows, cols = matrix.shape
    tiles_r, tiles_c = -(-rows // block), -(-cols // block)
    if (rows, cols) == (tiles_r * block, tiles_c * block):
        padded = matrix.contiguous()
    else:
        padded = matrix.new_zeros((tiles_r * block, tiles_c * block))
        padded[:rows, :cols] = matrix
    return padded.view(tiles_r, block, tiles_c, block), tiles_r, tiles_c


def quantize_blockwise(
    weight: torch.Tensor, block: int, fp8_dtype: torch.dtype = torch.float8_e4m3fn
) -> tuple[torch.Tensor, torch.Tensor]:
    """tests/test_flex_shard_fp8_allgather.py:45-90 -- per-tile amax in the
    input dtype, floor 1e-12 in the input dtype, float64 division, float32
    scale, multiply, clamp, cast; returns (fp8 [rows, cols], recip fp32)."""
    if weight.ndim != 2 or 0 in weight.shape:
        raise ValueError(f"expects a non-empty 2D matrix, got {tuple(weight.shape)}")
    rows, cols = weight.shape
    tiles, tiles_r, tiles_c = _tile_view(weight, block)
    fp8_max = torch.finfo(fp8_dtype).max
    amax = tiles.abs().amax(dim=(1, 3), keepdim=True).clamp(min=EPS).to(torch.float64)
    scale = (fp8_max / amax).to(torch.float32)
    quant = (tiles.to(torch.float32) * scale).clamp(-fp8_max, fp8_max).to(fp8_dtype)
    recip = (1.0 / scale).reshape(tiles_r, tiles_c).to(torch.float32)
    quant = quant.reshape(tiles_r * block, tiles_c * block)[:rows, :cols]
    return quant.contiguous(), recip.contiguous()


def dequant_blockwise(
    quant: torch.Tensor, recip_scale: torch.Tensor, block: int, out_dtype: torch.dtype = torch.bfloat16
) -> torch.Tensor:
    """blockwise_fp8/blockwise_fp8_weight.py:25-54,121-127 -- fp32 product of
    the FP8 value and its tile's reciprocal scale, one cast to ``out_dtype``."""
    rows, cols = quant.shape
    tiles, tiles_r, tiles_c = _tile_view(quant, block)
    deq = tiles.to(torch.float32) * recip_scale.reshape(tiles_r, 1, tiles_c, 1).to(torch.float32)
    return deq.reshape(tiles_r * block, tiles_c * block)[:rows, :cols].to(out_dtype)


def act_quant_1x128(
    x: torch.Tensor, block: int = 128, fp8_dtype: torch.dtype = torch.float8_e4m3fn
) -> tuple[torch.Tensor, torch.Tensor]:
    """Activation quantizer of blockwise_fp8/fp8_blockwise_linear.py:66-71.  The
    kernel is torchao's ``triton_fp8_blockwise_act_quant_lhs``
    (torchao.prototype.blockwise_fp8_training.kernels, torchao >= 0.18, absent
    from the reference checkout and from this image); its published algorithm
    per 1 x block run of a row: amax floored at 1e-12 (fp32), float64 division
    448 / amax, float32 scale, ``x * scale`` clamped and cast, reciprocal scale
    stored.  PARITY UNPINNED against torchao itself; pinned here through the
    tile quantizer (a run is a 1-row tile) and closed forms.  Returns the FP8
    matrix padded with zero columns to whole runs and the reciprocal scales as
    ``[runs per row, rows]`` (torchao's column-major ``[rows, runs]``)."""
    if x.ndim != 2:
        raise ValueError(f"expects a 2D matrix, got {tuple(x.shape)}")
    rows, cols = x.shape
    runs = -(-cols // block)
    padded = x.new_zeros((rows, runs * block))
    padded[:, :cols] = x
    groups = padded.view(rows, runs, block)
    fp8_max = torch.finfo(fp8_dtype).max
    amax = groups.to(torch.float32).abs().amax(dim=2, keepdim=True).clamp(min=EPS).to(torch.float64)
    scale = (fp8_max / amax).to(torch.float32)
    quant = (groups.to(torch.float32) * scale).clamp(-fp8_max, fp8_max).to(fp8_dtype)
    recip = (1.0 / scale).reshape(rows, runs).to(torch.float32)
    return quant.reshape(rows, runs * block).contiguous(), recip.t().contiguous()


def fp8_gemm_1x128_128x128(
    xq: torch.Tensor, xs: torch.Tensor, wq: torch.Tensor, ws: torch.Tensor, block: int = 128,
    out_dtype: torch.dtype = torch.bfloat16,
) -> torch.Tensor:
    """Scaled product of blockwise_fp8/fp8_blockwise_linear.py:74-90 (torchao's
    ``triton_fp8_gemm_1x128_128x128``, same provenance and PARITY UNPINNED note
    as above): for every k-block the fp32 dot products of the FP8 operands are
    multiplied by the activation run's and the weight tile's reciprocal scales
    and added to an fp32 accumulator in k order; one cast at the end.
    ``xq`` [m, k], ``xs`` [k / block, m], ``wq`` [n, k], ``ws`` [ceil(n / block), k / block]."""
    m, k = xq.shape
    n = wq.shape[0]
    acc = torch.zeros((m, n), dtype=torch.float32)
    col_block = torch.arange(n) // block
    for kb in range(k // block):
        a = xq[:, kb * block : (kb + 1) * block].to(torch.float32)
        b = wq[:, kb * block : (kb + 1) * block].to(torch.float32)
        acc += (a @ b.t()) * xs[kb].to(torch.float32)[:, None] * ws[:, kb].to(torch.float32)[col_block][None, :]
    return acc.to(out_dtype)


def act_quant_128x1_transposed(
    x: torch.Tensor, block: int = 128, fp8_dtype: torch.dtype = torch.float8_e4m3fn
) -> tuple[torch.Tensor, torch.Tensor]:
    """Token-run quantizers of blockwise_fp8/fp8_blockwise_linear.py:134-143:
    torchao's ``triton_fp8_blockwise_act_quant_transposed_lhs`` (output
    ``[cols, rows]`` row-major, scales per column and run of ``block`` rows) and
    ``triton_fp8_blockwise_act_quant_rhs`` (output ``[rows, cols]`` column-major
    = the same bytes, scales ``[rows / block, cols]``).  Same provenance, same
    per-run arithmetic and the same PARITY UNPINNED note as
    ``act_quant_1x128``; pinned through the tile quantizer (a run is a
    one-column tile) and the identity with ``act_quant_1x128`` of the
    transposed matrix.  Returns the bytes transposed, ``[cols, rows padded to
    whole runs]`` (pad zero), and the reciprocal scales ``[runs, cols]``."""
    if x.ndim != 2:
        raise ValueError(f"expects a 2D matrix, got {tuple(x.shape)}")
    rows, cols = x.shape
    runs = -(-rows // block)
    fp8_max = torch.finfo(fp8_dtype).max
    quant = torch.zeros((cols, runs * block), dtype=fp8_dtype)
    recip = torch.empty((runs, cols), dtype=torch.float32)
    for run in range(runs):
        piece = x[run * block : (run + 1) * block].to(torch.float32)  # [<= block, cols]
        amax = piece.abs().amax(dim=0).clamp(min=EPS).to(torch.float64)
        scale = (fp8_max / amax).to(torch.float32)
        q = (piece * scale[None, :]).clamp(-fp8_max, fp8_max).to(fp8_dtype)
        quant[:, run * block : run * block + piece.shape[0]] = q.t()
        recip[run] = 1.0 / scale
    return quant, recip


def fp8_gemm_1x128_128x1(
    aq: torch.Tensor, a_scales: torch.Tensor, bq: torch.Tensor, b_scales: torch.Tensor, block: int = 128,
    out_dtype: torch.dtype = torch.bfloat16,
) -> torch.Tensor:
    """Scaled product of blockwise_fp8/fp8_blockwise_linear.py:144-155
    (torchao's ``triton_fp8_gemm_1x128_128x1``; PARITY UNPINNED against
    torchao, as above): both operands carry one scale per row and k-block.
    ``aq`` [m, k], ``bq`` [n, k], ``a_scales`` [k / block, m], ``b_scales``
    [k / block, n]; fp32 accumulation in k order, one cast."""
    m, k = aq.shape
    n = bq.shape[0]
    acc = torch.zeros((m, n), dtype=torch.float32)
    for kb in range(k // block):
        a = aq[:, kb * block : (kb + 1) * block].to(torch.float32)
        b = bq[:, kb * block : (kb + 1) * block].to(torch.float32)
        acc += (a @ b.t()) * a_scales[kb].to(torch.float32)[:, None] * b_scales[kb].to(torch.float32)[None, :]
    return acc.to(out_dtype)


def fp8_linear_backward(
    grad_out: torch.Tensor, x: torch.Tensor, wq: torch.Tensor, ws: torch.Tensor, block: int = 128,
    out_dtype: torch.dtype = torch.bfloat16,
) -> tuple[torch.Tensor, torch.Tensor]:
    """``Fp8BlockwiseGemms.backward`` (blockwise_fp8/fp8_blockwise_linear.py:93-162)
    for a 2D weight ``wq`` [out, in] with tile scales ``ws``: returns
    ``(grad_x [tokens, in], grad_weight [out, in])``.

    grad_x (:107-126): grad_out zero-padded to whole runs of the output index,
    quantized 1 x block, times the weight read as ``[out, in]`` with its scales
    (the column-major copies of :113-114 change layout, not values).
    grad_weight (:127-161): both operands zero-padded to whole runs of tokens
    and quantized along the tokens; 1 x block times block x 1 product."""
    out_dim, in_dim = wq.shape
    pad_out, pad_in = -(-out_dim // block) * block, -(-in_dim // block) * block
    wq_padded = torch.zeros((pad_out, pad_in), dtype=wq.dtype)
    wq_padded.view(torch.uint8)[:out_dim, :in_dim] = wq.view(torch.uint8)
    gq, gs = act_quant_1x128(grad_out, block, wq.dtype)  # pads the output index itself
    grad_x = fp8_gemm_1x128_128x128(gq, gs, wq_padded.t().contiguous(), ws.t().contiguous(), block, out_dtype)
    gtq, gts = act_quant_128x1_transposed(grad_out, block, wq.dtype)
    xtq, xts = act_quant_128x1_transposed(x, block, wq.dtype)
    grad_w = fp8_gemm_1x128_128x1(gtq, gts, xtq, xts, block, out_dtype)
    return grad_x[:, :in_dim].contiguous(), grad_w[:out_dim, :in_dim].contiguous()


def accumulate_microbatches(grads: list[torch.Tensor]) -> torch.Tensor:
    """flex_shard/bucket_runtime.py:931-933 -- each microbatch's bf16 grad is
    cast to the fp32 accumulation dtype and added in arrival order."""
    acc = torch.zeros(grads[0].shape, dtype=torch.float32)
    for grad in grads:
        acc += grad.to(torch.float32)
    return acc


def reduce_rank_contributions(
    contributions: list[torch.Tensor], offset: int, numel: int, *, divide: float | None = None,
    premultiply: float | None = None,
) -> torch.Tensor:
    """custom_placements/utils.py:157-172 on one GPU: a left fold over ranks
    0..W-1 of ``[offset, offset+numel)``; ``premultiply`` mirrors the
    premul-sum op (:134), ``divide`` the post-division (:172)."""
    total = None
    for contribution in contributions:
        piece = contribution[offset : offset + numel]
        if premultiply is not None:
            piece = piece * premultiply
        total = piece.clone() if total is None else total + piece
    if divide is not None:
        total = total / divide
    return total


def newton_schulz(
    update: torch.Tensor,
    coefficients: tuple[float, float, float] = (3.4445, -4.7750, 2.0315),
    steps: int = 5,
    eps: float = 1e-7,
) -> torch.Tensor:
    """dist_muon/optimizer.py:2120-2151 -- bf16 copy, transpose tall inputs,
    divide by the clamped Frobenius norm, then ``steps`` quintic iterations
    with every product in bf16; 3-D+ inputs take the batched branch."""
    a, b, c = coefficients
    x = update.to(dtype=torch.bfloat16, copy=True)
    tall = x.shape[-2] > x.shape[-1]
    if tall:
        x = x.transpose(-2, -1)
    x.div_(x.norm(dim=(-2, -1), keepdim=True).clamp_min(eps))
    if x.ndim == 2:
        for _ in range(steps):
            gram = x @ x.T
            poly = torch.addmm(gram, gram, gram, beta=b, alpha=c)
            x = torch.addmm(x, poly, x, beta=a)
    else:
        shape = x.shape
        batch = x.reshape(-1, *shape[-2:])
        for _ in range(steps):
            gram = batch @ batch.transpose(-2, -1)
            poly = torch.baddbmm(gram, gram, gram, beta=b, alpha=c)
            batch = torch.baddbmm(batch, poly, batch, beta=a)
        x = batch.reshape(shape)
    return x.transpose(-2, -1) if tall else x


def adjusted_lr(lr: float, adjust_lr_fn: str | None, shape) -> float:
    """dist_muon/optimizer.py:2031-2046."""
    rows, cols = shape[-2:]
    if adjust_lr_fn is None or adjust_lr_fn == "original":
        return lr * math.sqrt(max(1.0, rows / cols))
    if adjust_lr_fn == "match_rms_adamw":
        return lr * 0.2 * math.sqrt(max(rows, cols))
    if adjust_lr_fn == "spectral_unclamped":
        return lr * math.sqrt(rows / cols)
    raise ValueError(f"unsupported adjust_lr_fn {adjust_lr_fn!r}")


def muon_step(
    param: torch.Tensor,
    grad: torch.Tensor,
    momentum_buffer: torch.Tensor,
    *,
    lr: float = 1e-3,
    weight_decay: float = 0.1,
    momentum: float = 0.95,
    nesterov: bool = True,
    coefficients: tuple[float, float, float] = (3.4445, -4.7750, 2.0315),
    steps: int = 5,
    eps: float = 1e-7,
    adjust_lr_fn: str | None = None,
) -> None:
    """dist_muon/optimizer.py:2049-2117 for one whole matrix, in place:
    momentum lerp, Nesterov lerp, Newton-Schulz, decoupled weight decay and
    the scaled update, all in the parameter dtype."""
    momentum_buffer.lerp_(grad, 1 - momentum)
    update = torch.lerp(grad, momentum_buffer, momentum) if nesterov else momentum_buffer.clone()
    direction = newton_schulz(update, coefficients, steps, eps).to(param.dtype)
    param.mul_(1 - lr * weight_decay)
    param.add_(direction, alpha=-adjusted_lr(lr, adjust_lr_fn, param.shape))
