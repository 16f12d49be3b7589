"""FP8 (``float8_e4m3fn``) all-gather on bucketed block sharding.

``Fp8BucketedBlockShard`` keeps the reference's constructor, equality, repr and
format hooks (custom_placements/fp8_bucketed_block_shard.py:91-218):
``block_size`` is both the shard row unit and the quantization tile, each chunk
carries one fp32 reciprocal-scale tensor of shape ``(ceil(rows/block),
ceil(in_dim/block))``, and finish hands per-parameter views of the compact
buffer to the caller's ``weight_factory``.

The quantizer is the fused HIP kernel ``fsh_quantize_pack`` (bit-exact with the
reference's eager quantizer), and ``finish_prepared_unshard_with_dequant`` adds
a fused compaction + bf16 dequantization of the gathered rows.
"""

from __future__ import annotations

from typing import TYPE_CHECKING, Any, Protocol

import torch
import torch.nn as nn

from .. import hip_ops
from ..placement_contract import PlacementPreparedUnshard, PlacementUnshardResult
from ..profiling import record_copy_out
from . import quant_plan
from ._copy_kernels import _upload_i64
from .blockwise_quant_bucketed_block_shard import (
    BlockwiseQuantBucketedBlockShard,
    _callable_name,
    _ceil_div,
    _matrix_shape,
    _require_gpu_rows,
    _scale_shape,
    _validate_2d_non_empty,
    _validate_block_size,
)

if TYPE_CHECKING:
    from ..placement_contract import Placement


class BlockwiseFp8WeightFactory(Protocol):
    """Builds the consumer's tensor from gathered FP8 operands.  ``fp8_data``
    has the parameter's shape; ``recip_scale`` holds one scale per block of the
    ``(prod(shape[:-1]), shape[-1])`` matrix.  The result must *view* both:
    persistent unshards refill those buffers in place."""

    def __call__(
        self, fp8_data: torch.Tensor, recip_scale: torch.Tensor, block_size: int, *, orig_dtype: torch.dtype,
        requires_grad: bool,
    ) -> torch.Tensor: ...


def _quantize_dense_weight_to_blockwise_fp8(
    weight: torch.Tensor, block_size: int, fp8_dtype: torch.dtype, *, eps_mode: int = hip_ops.EPS_INPUT_DTYPE
) -> tuple[torch.Tensor, torch.Tensor]:
    """Quantize one dense 2-D GPU weight: FP8 data of the same shape and the
    ``[ceil(out/B), ceil(in/B)]`` fp32 reciprocal scales.  Same contract as the
    reference's function of this name (:66-88), served by the pack kernel with
    a one-chunk payload."""
    out_dim, in_dim = _validate_2d_non_empty(weight.shape, "dense blockwise fp8 weight")
    _validate_block_size(block_size)
    if fp8_dtype != torch.float8_e4m3fn:
        raise NotImplementedError(f"the HIP quantizer produces float8_e4m3fn, not {fp8_dtype}")
    _require_gpu_rows(weight, "Blockwise FP8 quantization")
    if weight.stride(-1) != 1:
        weight = weight.contiguous()
    kind = {torch.bfloat16: hip_ops.SRC_BF16, torch.float32: hip_ops.SRC_F32, torch.float16: hip_ops.SRC_F16}.get(
        weight.dtype
    )
    if kind is None:
        raise NotImplementedError(f"the HIP quantizer reads bf16, fp16 or fp32 weights, not {weight.dtype}")
    tiles_r, tiles_c = _scale_shape(weight.shape, block_size)
    data_nbytes = out_dim * in_dim
    scale_start = quant_plan.align_up(data_nbytes, quant_plan.VEC_ALIGN_BYTES)
    payload = torch.empty(scale_start + 4 * tiles_r * tiles_c, dtype=torch.uint8, device=weight.device)
    hip_ops.quantize_pack(
        [hip_ops.QuantChunkSpec(weight, 0, scale_start, kind)],
        payload,
        ((data_nbytes, scale_start), (payload.numel(), payload.numel())),
        block_size,
        eps_mode,
    )
    fp8 = payload[:data_nbytes].view(fp8_dtype).view(out_dim, in_dim)
    recip = payload[scale_start:].view(torch.float32).view(tiles_r, tiles_c)
    return fp8, recip


def make_fp8_bucketed_block_placement_fn(
    *, weight_factory: BlockwiseFp8WeightFactory, block_size: int = 128, fp8_dtype: torch.dtype = torch.float8_e4m3fn
):
    """A placement function giving every parameter of a bucket one FP8 bucketed
    block placement sized by the mesh."""

    def fp8_bucketed_block_placements(named_params: list[tuple[str, nn.Parameter]], mesh: Any) -> dict:
        placement = Fp8BucketedBlockShard(
            world_size=mesh.size(), weight_factory=weight_factory, block_size=block_size, fp8_dtype=fp8_dtype
        )
        return {fqn: (placement,) for fqn, _ in named_params}

    return fp8_bucketed_block_placements


class Fp8BucketedBlockShard(BlockwiseQuantBucketedBlockShard):
    """Bucketed block shard that all-gathers blockwise FP8 instead of bf16."""

    scale_dtype = torch.float32

    #: Floor of a tile's amax: 1e-12 rounded to the quantization dtype (what the
    #: reference's eager quantizer does on bf16 shards) or always to fp32.
    eps_mode: int = hip_ops.EPS_INPUT_DTYPE

    def __init__(
        self,
        *,
        world_size: int,
        weight_factory: BlockwiseFp8WeightFactory,
        block_size: int = 128,
        fp8_dtype: torch.dtype = torch.float8_e4m3fn,
    ) -> None:
        _validate_block_size(block_size)
        if not callable(weight_factory):
            raise TypeError("weight_factory must be callable.")
        self.block_size = block_size
        self.weight_factory = weight_factory
        super().__init__(world_size=world_size, shard_block_rows=block_size, qdata_dtype=fp8_dtype)

    def __eq__(self, other: object) -> bool:
        if type(other) is not type(self):
            return NotImplemented
        return (
            self.world_size == other.world_size
            and self.block_size == other.block_size
            and self.qdata_dtype == other.qdata_dtype
            and self.weight_factory is other.weight_factory
        )

    def __hash__(self) -> int:
        return hash((type(self), self.world_size, self.block_size, self.qdata_dtype, id(self.weight_factory)))

    def __repr__(self) -> str:
        return (
            f"Fp8BucketedBlockShard(world_size={self.world_size}, block_size={self.block_size}, "
            f"weight_factory={_callable_name(self.weight_factory)})"
        )

    # ------------------------------------------------------------ format hooks
    def _chunk_scale_numels(self, rows: int, in_dim: int) -> tuple[int, ...]:
        return (_ceil_div(rows, self.block_size) * _ceil_div(in_dim, self.block_size),)

    def _quantize_local_weight(self, tensor: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        return _quantize_dense_weight_to_blockwise_fp8(
            tensor, self.block_size, self.qdata_dtype, eps_mode=self.eps_mode
        )

    def _quantize_local_chunk(self, tensor: torch.Tensor) -> tuple[torch.Tensor, tuple[torch.Tensor, ...]]:
        quant, recip = self._quantize_local_weight(tensor)
        return quant, (recip,)

    def _param_scale_view(self, scale_index: int, scale: torch.Tensor, matrix_shape: torch.Size) -> torch.Tensor:
        return scale.view(_scale_shape(matrix_shape, self.block_size))

    def _make_quantized_weight(
        self, qdata: torch.Tensor, scales: tuple[torch.Tensor, ...], *, orig_dtype: torch.dtype, requires_grad: bool
    ) -> torch.Tensor:
        (recip,) = scales
        return self.weight_factory(qdata, recip, self.block_size, orig_dtype=orig_dtype, requires_grad=requires_grad)

    def _quantize_pack_source_kind(self, tensor_dtype: torch.dtype, quant_dtype: torch.dtype) -> int | None:
        if self.qdata_dtype != torch.float8_e4m3fn:
            raise NotImplementedError(f"the HIP quantizer produces float8_e4m3fn, not {self.qdata_dtype}")
        table = {
            (torch.bfloat16, torch.bfloat16): hip_ops.SRC_BF16,
            (torch.float32, torch.float32): hip_ops.SRC_F32,
            (torch.float32, torch.bfloat16): hip_ops.SRC_F32_AS_BF16,
            (torch.float16, torch.float16): hip_ops.SRC_F16,
            (torch.float32, torch.float16): hip_ops.SRC_F32_AS_F16,
        }
        if quant_dtype not in (torch.bfloat16, torch.float32, torch.float16):
            raise NotImplementedError(f"the HIP quantizer quantizes bf16, fp16 or fp32 values, not {quant_dtype}")
        return table.get((tensor_dtype, quant_dtype))

    def _make_quantize_pack_launch(self, specs, payload_nbytes, zero_ranges, device) -> hip_ops.QuantPackPlan:
        return hip_ops.QuantPackPlan(specs, payload_nbytes, zero_ranges, self.block_size, self.eps_mode, device=device)

    # --------------------------------------------- fused compaction + dequant
    def _unpack_table(
        self, state: "BlockwiseQuantBucketedBlockShard._QuantUnshardState", row_stride: int, device: torch.device
    ):
        """Device table of ``fsh_unpack_chunk`` records, one per (rank, chunk),
        built once per (bucket metadata, row stride, device)."""
        metadata = state.metadata
        key = (id(metadata), row_stride, device)
        cached = self._unpack_tables.get(key)
        if cached is not None and cached[0] is metadata:
            return cached[1:]
        block = self.block_size
        _, scale_start, _ = self._compact_sizes(metadata)
        scale_base: dict[str, int] = {}
        tiles_c_of: dict[str, int] = {}
        running = 0
        for info in state.infos:
            rows, in_dim = _matrix_shape(info.global_shape)
            scale_base[info.fqn] = running
            tiles_c_of[info.fqn] = _ceil_div(in_dim, block)
            running += _ceil_div(rows, block) * tiles_c_of[info.fqn]
        records: list[int] = []
        tile_starts = [0]
        located = iter(metadata.chunks)
        for rank, plan in enumerate(metadata.rank_pack_plans):
            scale_cursor = plan.scale_byte_offset
            for pack_chunk in plan.chunks:
                chunk = next(located)
                assert chunk.rank == rank and chunk.fqn == pack_chunk.fqn
                rows, in_dim = pack_chunk.local_shape
                first_scale = scale_base[chunk.fqn] + (chunk.row_start // block) * tiles_c_of[chunk.fqn]
                records += [
                    rank * row_stride + chunk.qdata_offset,
                    rank * row_stride + scale_cursor,
                    rows,
                    in_dim,
                    chunk.global_dense_offset,
                    scale_start + 4 * first_scale,
                    chunk.global_dense_offset,
                ]
                tile_starts.append(tile_starts[-1] + _ceil_div(rows, block) * tiles_c_of[chunk.fqn])
                scale_cursor += 4 * pack_chunk.scale_numels[0]
        table, table_host = _upload_i64(records, device)
        starts, starts_host = _upload_i64(tile_starts, device)
        table = table.view(-1, 7)
        self._unpack_tables[key] = (metadata, table, starts, tile_starts[-1], (table_host, starts_host))
        return table, starts, tile_starts[-1], (table_host, starts_host)

    def finish_prepared_unshard_with_dequant(
        self,
        prepared: PlacementPreparedUnshard,
        rank_rows: torch.Tensor | None = None,
        *,
        dequant_dtype: torch.dtype = torch.bfloat16,
        dequant_out: torch.Tensor | None = None,
        compact: bool = True,
    ) -> tuple[PlacementUnshardResult, list[torch.Tensor]]:
        """``finish_prepared_unshard`` plus dequantized weights from the same
        pass over the gathered FP8 bytes: returns the usual result (FP8 views
        through the weight factory; empty when ``compact`` is False) and one
        ``dequant_dtype`` tensor per parameter, each a view of one flat buffer
        in parameter order.  Values equal ``BlockwiseFp8Weight.dequantize()`` on
        the gathered weight: fp32 product of the FP8 value and its tile's scale,
        rounded once."""
        state = self._unshard_state(prepared)
        if rank_rows is None:
            rank_rows = prepared.buffers[1].view(len(state.metadata.rank_qdata_numels), prepared.buffers[0].numel())
        self._check_rank_rows(state, rank_rows)
        _require_gpu_rows(rank_rows, "The fused unpack")
        if rank_rows.stride(1) != 1:
            raise ValueError("gathered rank rows must have unit byte stride within a row")
        row_stride = rank_rows.stride(0) if rank_rows.size(0) > 1 else rank_rows.size(1)
        table, starts, total_tiles, _hosts = self._unpack_table(state, row_stride, rank_rows.device)
        total = sum(info.global_numel for info in state.infos)
        if dequant_out is None:
            dequant_out = torch.empty(total, dtype=dequant_dtype, device=rank_rows.device)
        elif dequant_out.numel() != total or dequant_out.dtype != dequant_dtype or not dequant_out.is_contiguous():
            raise ValueError(f"dequant_out must be a contiguous {dequant_dtype} tensor of {total} elements")
        compact_buf = self._compact_buffer(prepared, state.metadata, rank_rows.device) if compact else None
        with record_copy_out():
            hip_ops.unpack_dequant(rank_rows, table, starts, total_tiles, compact_buf, dequant_out.view(-1), self.block_size)
        dequant = [
            piece.view(info.global_shape)
            for piece, info in zip(torch.split(dequant_out.view(-1), [i.global_numel for i in state.infos]), state.infos)
        ]
        if compact_buf is None:
            return PlacementUnshardResult(full_params=[]), dequant
        result = PlacementUnshardResult(
            full_params=self._full_params_from_compact(state, compact_buf),
            persistent_buffers=[compact_buf] if prepared.persistent else [],
        )
        return result, dequant


__all__ = ["BlockwiseFp8WeightFactory", "Fp8BucketedBlockShard", "make_fp8_bucketed_block_placement_fn"]
