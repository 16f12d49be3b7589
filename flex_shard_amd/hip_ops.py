"""Tensor-level wrappers over the C ABI.

Each function checks on the host that operand shapes, dtypes, devices and
bounds match what the kernel assumes, then queues the kernel on the current
torch stream of the operands' device.  torch is used for memory and streams
only.  Nothing here synchronizes the host.
"""

from __future__ import annotations

import ctypes
from typing import Sequence

import torch

from . import _native
from ._native import (
    DT_BF16,
    DT_F16,
    DT_F32,
    EPS_FP32,
    EPS_INPUT_DTYPE,
    REDUCE_POSTDIV,
    REDUCE_POSTMUL,
    REDUCE_PREMUL,
    REDUCE_SUM,
    SRC_BF16,
    SRC_F16,
    SRC_F32,
    SRC_F32_AS_BF16,
    SRC_F32_AS_F16,
)

__all__ = [
    "DT_BF16", "DT_F16", "DT_F32", "EPS_FP32", "EPS_INPUT_DTYPE", "REDUCE_POSTDIV", "REDUCE_POSTMUL",
    "REDUCE_PREMUL", "REDUCE_SUM", "SRC_BF16", "SRC_F16", "SRC_F32", "SRC_F32_AS_BF16", "SRC_F32_AS_F16",
    "MuonStepPlan", "QuantChunkSpec", "QuantPackPlan", "accumulate_grad", "act_quant_128x1_transposed", "act_quant_1x128", "act_quant_both",
    "copy_segments", "fp8_gemm_1x128_128x1", "fp8_gemm_1x128_128x128", "fp8_gemm_1x128_128x128_dgrad",
    "fp8_transpose", "gemm_nt", "gemm_nt_group", "muon_apply", "muon_prepare", "newton_schulz_multi",
    "newton_schulz", "newton_schulz_noalloc", "newton_schulz_workspace_bytes", "pack_segments", "quantize_pack",
    "reduce_rows", "stream_ptr", "unpack_dequant", "zero_segments",
]


def _require_gpu(*tensors: torch.Tensor) -> torch.device:
    device = tensors[0].device
    for t in tensors:
        if t.device.type != "cuda":
            raise RuntimeError(
                "flex_shard_amd kernels run on the GPU only; got a tensor on "
                f"{t.device}. There is no CPU path."
            )
        if t.device != device:
            raise ValueError(f"tensors on different devices: {device} and {t.device}")
    return device


def stream_ptr(device: torch.device) -> int:
    """The raw hipStream_t of torch's current stream on ``device`` (torch's own
    accessor for kernel launchers: no Stream object is built)."""
    index = device.index
    return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device() if index is None else index)


def _dt(dtype: torch.dtype) -> int:
    if dtype == torch.bfloat16:
        return DT_BF16
    if dtype == torch.float32:
        return DT_F32
    raise NotImplementedError(f"dtype {dtype} is not supported by the HIP kernels (bf16 and fp32 are)")


class QuantChunkSpec:
    """One chunk of a quantize+pack launch: a 2-D row-major view (unit column
    stride) and where its FP8 bytes and scales go in the payload."""

    __slots__ = ("tensor", "qdata_offset", "scale_offset", "src_kind")

    def __init__(self, tensor: torch.Tensor, qdata_offset: int, scale_offset: int, src_kind: int) -> None:
        self.tensor = tensor
        self.qdata_offset = qdata_offset
        self.scale_offset = scale_offset
        self.src_kind = src_kind


class QuantPackPlan:
    """A validated, reusable launch of the fused quantize + pack kernel for
    fixed source shards (``fsh_quant_pack_plan_*``): the chunk table, the pad
    ranges and the launch geometry are checked and stored on the C side once,
    so a steady-state launch is one C call with three arguments.  The shards'
    data pointers are baked into the plan: the caller launches it only while
    tensors of the same shape live at those addresses (``keep_alive`` makes
    the plan hold them).  Any number of chunks."""

    __slots__ = ("_handle", "_payload_nbytes", "_device", "_keep", "_launch_fn", "_destroy_fn")

    def __init__(
        self,
        chunks: Sequence[QuantChunkSpec],
        payload_nbytes: int,
        zero_ranges: tuple[tuple[int, int], tuple[int, int]],
        block: int,
        eps_mode: int = EPS_INPUT_DTYPE,
        device: torch.device | None = None,
        keep_alive: bool = False,
    ) -> None:
        self._handle = None
        if chunks:
            device = _require_gpu(*[c.tensor for c in chunks])
        if device is None or device.type != "cuda":
            raise RuntimeError("flex_shard_amd kernels run on the GPU only; there is no CPU path.")
        self._device = device
        self._keep = [c.tensor for c in chunks] if keep_alive else None
        self._payload_nbytes = payload_nbytes
        table = (_native.QuantChunk * max(len(chunks), 1))()
        for slot, spec in zip(table, chunks):
            t = spec.tensor
            if t.ndim != 2 or t.stride(1) != 1 or t.shape[0] <= 0 or t.shape[1] <= 0:
                raise ValueError(
                    f"chunk must be a non-empty 2-D view with unit column stride, got {tuple(t.shape)} / {t.stride()}"
                )
            expected = {SRC_BF16: torch.bfloat16, SRC_F16: torch.float16}.get(spec.src_kind, torch.float32)
            if t.dtype != expected:
                raise ValueError(f"chunk dtype {t.dtype} does not match src_kind {spec.src_kind}")
            slot.src_dev = t.data_ptr()
            slot.rows, slot.in_dim = t.shape
            slot.src_row_stride = t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])
            slot.qdata_offset = spec.qdata_offset
            slot.scale_offset = spec.scale_offset
            slot.src_kind = spec.src_kind
        lib = _native.lib()
        self._launch_fn, self._destroy_fn = lib.fsh_quant_pack_plan_launch, lib.fsh_quant_pack_plan_destroy
        handle = ctypes.c_void_p()
        (z0, z1) = zero_ranges
        status = lib.fsh_quant_pack_plan_create(
            table, len(chunks), payload_nbytes, z0[0], z0[1], z1[0], z1[1], block, eps_mode, ctypes.byref(handle)
        )
        _native.check(status, "fsh_quant_pack_plan_create")
        self._handle = handle

    def __del__(self) -> None:
        if getattr(self, "_handle", None) is not None:
            self._destroy_fn(self._handle)
            self._handle = None

    @property
    def payload_nbytes(self) -> int:
        return self._payload_nbytes

    def raw_launch(self) -> tuple[object, object]:
        """``(function, handle)``: ``function(handle, payload_ptr, stream)`` is
        the C call of :meth:`launch_raw` (status 0 on success) for callers that
        count microseconds; the plan must outlive every such call."""
        return self._launch_fn, self._handle

    def launch_raw(self, payload_ptr: int, stream: int) -> None:
        """Queue the launch into ``payload_nbytes`` bytes at the device address
        ``payload_ptr`` (16-byte aligned) on the raw stream handle ``stream``.
        Nothing about the payload is checked beyond its alignment."""
        status = self._launch_fn(self._handle, payload_ptr, stream)
        if status != 0:
            _native.check(status, "fsh_quant_pack_plan_launch")

    def launch(self, payload: torch.Tensor, stream: torch.cuda.Stream | None = None) -> None:
        """Queue the launch on ``stream`` (default: the current stream of the
        plan's device); the caller orders the payload's allocation and the
        shards against that stream."""
        if payload.device != self._device or payload.dtype != torch.uint8 or payload.ndim != 1:
            raise ValueError("payload must be a 1-D uint8 tensor on the plan's device")
        if not payload.is_contiguous() or payload.numel() != self._payload_nbytes:
            raise ValueError(f"payload must be contiguous with {self._payload_nbytes} bytes")
        self.launch_raw(payload.data_ptr(), stream_ptr(self._device) if stream is None else stream.cuda_stream)


def quantize_pack(
    chunks: Sequence[QuantChunkSpec],
    payload: torch.Tensor,
    zero_ranges: tuple[tuple[int, int], tuple[int, int]],
    block: int,
    eps_mode: int = EPS_INPUT_DTYPE,
) -> None:
    """Fused tile quantize + pack of every chunk into ``payload`` (uint8,
    contiguous) and zeroing of the two pad ranges.  Launches are split when
    there are more than FSH_MAX_QUANT_CHUNKS chunks."""
    _require_gpu(payload)
    QuantPackPlan(chunks, payload.numel(), zero_ranges, block, eps_mode, device=payload.device).launch(payload)


def _check_i64_table(*tables: torch.Tensor) -> int:
    n = tables[0].numel()
    for t in tables:
        if t.dtype != torch.int64 or not t.is_contiguous() or t.numel() != n:
            raise ValueError("descriptor tables must be contiguous int64 tensors of equal length")
    return n


def copy_segments(
    source: torch.Tensor, output: torch.Tensor, src_offsets: torch.Tensor, numels: torch.Tensor,
    dst_offsets: torch.Tensor, max_segment_numel: int,
) -> None:
    """``output[dst+i] = source[src+i]`` per segment, in elements of the two
    tensors' common item size.  Only the data pointers are used, so ``source``
    may be a strided view whose offsets count from its first element."""
    _require_gpu(source, output, src_offsets, numels, dst_offsets)
    if source.element_size() != output.element_size():
        raise ValueError("source and output must have the same element size")
    n = _check_i64_table(src_offsets, numels, dst_offsets)
    status = _native.lib().fsh_copy_segments(
        source.data_ptr(), output.data_ptr(), src_offsets.data_ptr(), numels.data_ptr(), dst_offsets.data_ptr(),
        n, max_segment_numel, source.element_size(), stream_ptr(output.device),
    )
    _native.check(status, "fsh_copy_segments")


def zero_segments(output: torch.Tensor, numels: torch.Tensor, dst_offsets: torch.Tensor, max_segment_numel: int) -> None:
    _require_gpu(output, numels, dst_offsets)
    n = _check_i64_table(numels, dst_offsets)
    status = _native.lib().fsh_zero_segments(
        output.data_ptr(), numels.data_ptr(), dst_offsets.data_ptr(), n, max_segment_numel,
        output.element_size(), stream_ptr(output.device),
    )
    _native.check(status, "fsh_zero_segments")


def pack_segments(
    input_ptrs: torch.Tensor, tensor_indices: torch.Tensor, src_offsets: torch.Tensor, numels: torch.Tensor,
    dst_offsets: torch.Tensor, max_segment_numel: int, src_dtype: torch.dtype, output: torch.Tensor,
) -> None:
    _require_gpu(output, input_ptrs, tensor_indices, src_offsets, numels, dst_offsets)
    n = _check_i64_table(tensor_indices, src_offsets, numels, dst_offsets)
    status = _native.lib().fsh_pack_segments(
        input_ptrs.data_ptr(), tensor_indices.data_ptr(), src_offsets.data_ptr(), numels.data_ptr(),
        dst_offsets.data_ptr(), n, max_segment_numel, _dt(src_dtype), _dt(output.dtype), output.data_ptr(),
        stream_ptr(output.device),
    )
    _native.check(status, "fsh_pack_segments")


def unpack_dequant(
    rows: torch.Tensor,
    chunk_table: torch.Tensor,
    tile_starts: torch.Tensor,
    total_tiles: int,
    compact: torch.Tensor | None,
    dequant: torch.Tensor | None,
    block: int,
) -> None:
    """``rows``: uint8 tensor whose data pointer is the first gathered row
    (offsets in the table count from it).  ``chunk_table``: int64 [nchunks, 7]
    device tensor of ``fsh_unpack_chunk`` records; ``tile_starts``: int64
    [nchunks + 1].  ``compact`` (uint8) and ``dequant`` (bf16/fp32, flat) are
    optional outputs; the caller guarantees the table stays inside them."""
    present = [t for t in (compact, dequant) if t is not None]
    _require_gpu(rows, chunk_table, tile_starts, *present)
    if chunk_table.dtype != torch.int64 or chunk_table.ndim != 2 or chunk_table.shape[1] != _native.UNPACK_CHUNK_INT64S:
        raise ValueError("chunk_table must be int64 [nchunks, 7]")
    if not chunk_table.is_contiguous() or not tile_starts.is_contiguous() or tile_starts.dtype != torch.int64:
        raise ValueError("tables must be contiguous int64 tensors")
    nchunks = chunk_table.shape[0]
    if tile_starts.numel() != nchunks + 1:
        raise ValueError("tile_starts must have nchunks + 1 entries")
    if compact is not None and (compact.dtype != torch.uint8 or not compact.is_contiguous()):
        raise ValueError("compact must be contiguous uint8")
    dq_dtype = DT_BF16
    if dequant is not None:
        if not dequant.is_contiguous():
            raise ValueError("dequant must be contiguous")
        dq_dtype = DT_F16 if dequant.dtype == torch.float16 else _dt(dequant.dtype)
    status = _native.lib().fsh_unpack_dequant(
        rows.data_ptr(), chunk_table.data_ptr(), tile_starts.data_ptr(), nchunks, total_tiles,
        compact.data_ptr() if compact is not None else None,
        dequant.data_ptr() if dequant is not None else None,
        dq_dtype, block, stream_ptr(rows.device),
    )
    _native.check(status, "fsh_unpack_dequant")


def accumulate_grad(acc: torch.Tensor, grad: torch.Tensor, *, overwrite: bool = False) -> None:
    """``acc (+)= grad.float()`` over flat contiguous tensors of equal numel."""
    _require_gpu(acc, grad)
    if acc.dtype != torch.float32 or not acc.is_contiguous() or not grad.is_contiguous():
        raise ValueError("acc must be contiguous fp32 and grad contiguous")
    if acc.numel() != grad.numel():
        raise ValueError(f"numel mismatch: acc {acc.numel()} vs grad {grad.numel()}")
    status = _native.lib().fsh_accumulate_grad(
        acc.data_ptr(), grad.data_ptr(), _dt(grad.dtype), acc.numel(), int(overwrite), stream_ptr(acc.device)
    )
    _native.check(status, "fsh_accumulate_grad")


def reduce_rows(
    out: torch.Tensor, contributions: torch.Tensor, column_offset: int, *, mode: int = REDUCE_SUM, factor: float = 1.0
) -> None:
    """``out[i] = fold_r contributions[r, column_offset + i]`` in rank order;
    ``contributions`` is [W, row] with unit column stride, fp32 or bf16 like
    ``out`` (bf16 terms are added in fp32 and the sum rounded once)."""
    _require_gpu(out, contributions)
    if out.dtype != contributions.dtype or out.dtype not in (torch.float32, torch.bfloat16):
        raise NotImplementedError(
            f"the fixed-order reduction takes fp32 or bf16 contributions and an output of the same dtype, got "
            f"{contributions.dtype} -> {out.dtype}"
        )
    if contributions.ndim != 2 or contributions.stride(1) != 1 or not out.is_contiguous():
        raise ValueError("contributions must be [W, row] with unit column stride and out contiguous")
    world, row = contributions.shape
    if column_offset < 0 or column_offset + out.numel() > row:
        raise ValueError(f"range [{column_offset}, {column_offset + out.numel()}) outside rows of {row} elements")
    stride = contributions.stride(0) if world > 1 else row
    entry = "fsh_reduce_rows_f32" if out.dtype == torch.float32 else "fsh_reduce_rows_bf16"
    status = getattr(_native.lib(), entry)(
        out.data_ptr(), contributions.data_ptr(), stride, world, column_offset, out.numel(), mode, factor,
        stream_ptr(out.device),
    )
    _native.check(status, entry)


def newton_schulz_workspace_bytes(batch: int, rows: int, cols: int) -> int:
    """Workspace of ``newton_schulz`` for ``batch`` matrices; rows and columns
    count as rounded up to multiples of 8, which is how they are processed."""
    return int(_native.lib().fsh_newton_schulz_workspace_bytes(batch, -(-rows // 8) * 8, -(-cols // 8) * 8))


def newton_schulz(
    x: torch.Tensor,
    coefficients: tuple[float, float, float],
    steps: int,
    eps: float,
    workspace: torch.Tensor | None = None,
) -> torch.Tensor:
    """In-place Newton-Schulz of a contiguous bf16 [batch, rows, cols] (or
    [rows, cols]) tensor.  ``workspace`` (uint8) is allocated when not given."""
    _require_gpu(x)
    if x.dtype != torch.bfloat16 or not x.is_contiguous() or x.ndim not in (2, 3):
        raise ValueError("x must be a contiguous bf16 matrix or batch of matrices")
    batch = 1 if x.ndim == 2 else x.shape[0]
    rows, cols = x.shape[-2:]
    if (rows % 8 or cols % 8) and x.numel():
        # The kernels move 16-byte rows.  Zero rows and columns change nothing:
        # the Frobenius norm is the same, X X^T and the polynomial keep them
        # zero in every iteration, and the other entries see the same products.
        padded = x.new_zeros((batch, -(-rows // 8) * 8, -(-cols // 8) * 8))
        padded[:, :rows, :cols] = x.view(batch, rows, cols)
        need = newton_schulz_workspace_bytes(batch, padded.shape[1], padded.shape[2])
        if workspace is not None and (workspace.dtype != torch.uint8 or workspace.numel() < need):
            workspace = None  # sized for the unpadded shape
        newton_schulz(padded, coefficients, steps, eps, workspace)
        x.view(batch, rows, cols).copy_(padded[:, :rows, :cols])
        return x
    need = newton_schulz_workspace_bytes(batch, rows, cols)
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
    _require_gpu(x, workspace)
    if workspace.dtype != torch.uint8 or not workspace.is_contiguous() or workspace.numel() < need:
        raise ValueError(f"workspace must be contiguous uint8 with at least {need} bytes")
    a, b, c = coefficients
    status = _native.lib().fsh_newton_schulz(
        x.data_ptr(), batch, rows, cols, a, b, c, steps, eps, workspace.data_ptr(), workspace.numel(),
        stream_ptr(x.device),
    )
    _native.check(status, "fsh_newton_schulz")
    return x


def newton_schulz_noalloc(
    x: torch.Tensor, coefficients: tuple[float, float, float], steps: int, eps: float
) -> torch.Tensor:
    """``newton_schulz`` on the library's static device scratch: nothing is
    allocated, by this wrapper or by the library.  The batch must fit the
    scratch (``_native.NS_STATIC_SCRATCH_BYTES``); calls on one GPU share it,
    so calls that overlap on different streams race."""
    _require_gpu(x)
    if x.dtype != torch.bfloat16 or not x.is_contiguous() or x.ndim not in (2, 3):
        raise ValueError("x must be a contiguous bf16 matrix or batch of matrices")
    batch = 1 if x.ndim == 2 else x.shape[0]
    rows, cols = x.shape[-2:]
    a, b, c = coefficients
    status = _native.lib().fsh_newton_schulz_noalloc(
        x.data_ptr(), batch, rows, cols, a, b, c, steps, eps, stream_ptr(x.device)
    )
    _native.check(status, "fsh_newton_schulz_noalloc")
    return x


def newton_schulz_multi(
    problems: Sequence[tuple[torch.Tensor, torch.Tensor | None]],
    coefficients: tuple[float, float, float],
    steps: int,
    eps: float,
) -> None:
    """In-place Newton-Schulz of several contiguous bf16 [batch, rows, cols]
    tensors of different shapes, each with its workspace (allocated when
    ``None``).  Same results as one ``newton_schulz`` call per tensor."""
    if not problems:
        return
    if len(problems) > _native.MAX_NS_PROBLEMS:
        for begin in range(0, len(problems), _native.MAX_NS_PROBLEMS):
            newton_schulz_multi(problems[begin : begin + _native.MAX_NS_PROBLEMS], coefficients, steps, eps)
        return
    table = (_native.NsProblem * len(problems))()
    keep = []
    device = problems[0][0].device
    for i, (x, workspace) in enumerate(problems):
        _require_gpu(x)
        if x.device != device:
            raise ValueError("all problems of a call must live on one device")
        if x.dtype != torch.bfloat16 or not x.is_contiguous() or x.ndim not in (2, 3):
            raise ValueError("x must be a contiguous bf16 matrix or batch of matrices")
        batch = 1 if x.ndim == 2 else x.shape[0]
        rows, cols = x.shape[-2:]
        need = newton_schulz_workspace_bytes(batch, rows, cols)
        if workspace is None:
            workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
        _require_gpu(x, workspace)
        if workspace.dtype != torch.uint8 or not workspace.is_contiguous() or workspace.numel() < need:
            raise ValueError(f"workspace must be contiguous uint8 with at least {need} bytes")
        keep.append(workspace)
        table[i].x_dev, table[i].batch, table[i].rows, table[i].cols = x.data_ptr(), batch, rows, cols
        table[i].workspace_dev, table[i].workspace_nbytes = workspace.data_ptr(), workspace.numel()
    a, b, c = coefficients
    status = _native.lib().fsh_newton_schulz_multi(table, len(problems), a, b, c, steps, eps, stream_ptr(device))
    _native.check(status, "fsh_newton_schulz_multi")


def _gemm_desc(
    a: torch.Tensor, b: torch.Tensor, d: torch.Tensor | None, alpha: float, beta: float,
    out: torch.Tensor | None, out_t: torch.Tensor | None, symmetric: bool, diag_add: float = 0.0,
    k_major: bool = False,
) -> tuple["_native.GemmDesc", torch.Tensor]:
    _require_gpu(a, b)
    if a.dtype != torch.bfloat16 or b.dtype != torch.bfloat16 or not a.is_contiguous() or not b.is_contiguous():
        raise ValueError("a and b must be contiguous bf16")
    a3 = a if a.ndim == 3 else a.unsqueeze(0)
    b3 = b if b.ndim == 3 else b.unsqueeze(0)
    if k_major:  # [batch, k, m] and [batch, k, n]
        batch, k, m = a3.shape
        if b3.shape[0] != batch or b3.shape[1] != k:
            raise ValueError(f"shape mismatch: a {tuple(a.shape)} vs b {tuple(b.shape)}")
        n = b3.shape[2]
    else:
        batch, m, k = a3.shape
        if b3.shape[0] != batch or b3.shape[2] != k:
            raise ValueError(f"shape mismatch: a {tuple(a.shape)} vs b {tuple(b.shape)}")
        n = b3.shape[1]
    if out is None:
        out = torch.empty((batch, m, n) if a.ndim == 3 else (m, n), dtype=torch.bfloat16, device=a.device)
    for name, t, shape in (("d", d, (m, n)), ("out", out, (m, n)), ("out_t", out_t, (n, m))):
        if t is None:
            continue
        _require_gpu(a, t)
        if t.dtype != torch.bfloat16 or not t.is_contiguous() or tuple(t.shape[-2:]) != shape or t.numel() != batch * m * n:
            raise ValueError(f"{name} must be contiguous bf16 with trailing shape {shape}")
    desc = _native.GemmDesc()
    desc.a_dev, desc.b_dev = a.data_ptr(), b.data_ptr()
    desc.d_dev = d.data_ptr() if d is not None else None
    desc.c_dev = out.data_ptr()
    desc.ct_dev = out_t.data_ptr() if out_t is not None else None
    desc.m, desc.n, desc.k = m, n, k
    desc.lda, desc.ldb = (m, n) if k_major else (k, k)
    desc.ldd, desc.ldc, desc.ldct = n, n, m
    desc.batch = batch
    desc.stride_a, desc.stride_b = m * k, n * k
    desc.stride_d = desc.stride_c = desc.stride_ct = m * n
    desc.alpha, desc.beta = alpha, beta
    desc.symmetric = 1 if symmetric else 0
    desc.diag_add = diag_add
    desc.k_major = 1 if k_major else 0
    return desc, out


def gemm_nt(
    a: torch.Tensor, b: torch.Tensor, *, d: torch.Tensor | None = None, alpha: float = 1.0, beta: float = 0.0,
    out: torch.Tensor | None = None, out_t: torch.Tensor | None = None, symmetric: bool = False,
    diag_add: float = 0.0, k_major: bool = False,
) -> torch.Tensor:
    """``bf16(alpha * a @ b^T + beta * d + diag_add * I)`` for contiguous bf16
    [batch, m, k] / [batch, n, k] (or 2-D) operands; optionally also the
    transpose.  With ``symmetric`` the caller guarantees a symmetric result
    (m == n); only the upper triangle of tiles is computed and mirrored.  With
    ``k_major`` the operands are [batch, k, m] / [batch, k, n] and the product
    is ``a^T @ b`` (large whole-tile problems only)."""
    desc, out = _gemm_desc(a, b, d, alpha, beta, out, out_t, symmetric, diag_add, k_major)
    status = _native.lib().fsh_gemm_bf16_nt(ctypes.byref(desc), stream_ptr(a.device))
    _native.check(status, "fsh_gemm_bf16_nt")
    return out


def gemm_nt_group(problems: Sequence[dict]) -> list[torch.Tensor]:
    """Independent ``gemm_nt`` problems (dicts of its arguments) issued in one
    call; the ones that take the large-tile kernel share launches."""
    if not problems:
        return []
    descs = (_native.GemmDesc * len(problems))()
    outs = []
    for i, q in enumerate(problems):
        desc, out = _gemm_desc(
            q["a"], q["b"], q.get("d"), q.get("alpha", 1.0), q.get("beta", 0.0), q.get("out"), q.get("out_t"),
            q.get("symmetric", False), q.get("diag_add", 0.0), q.get("k_major", False),
        )
        descs[i] = desc
        outs.append(out)
        if out.device != outs[0].device:
            raise ValueError("all problems of a group must live on one device")
    status = _native.lib().fsh_gemm_bf16_nt_group(descs, len(problems), stream_ptr(outs[0].device))
    _native.check(status, "fsh_gemm_bf16_nt_group")
    return outs


def act_quant_1x128(x: torch.Tensor, *, eps_fp32: bool = True) -> tuple[torch.Tensor, torch.Tensor]:
    """Quantize every run of 128 consecutive elements of each row of the bf16
    matrix ``x`` to float8_e4m3fn.  Returns the bytes as ``[rows, cols rounded
    up to 128]`` (pad columns zero) and the reciprocal scales as a
    ``[cols / 128, rows]`` fp32 table.  ``eps_fp32`` floors an all-zero run's
    amax at fp32 1e-12 (the activation quantizer's rule); ``False`` rounds the
    floor to bf16 like the weight quantizer."""
    _require_gpu(x)
    if x.dtype != torch.bfloat16 or x.ndim != 2 or x.stride(1) != 1:
        raise ValueError("x must be a bf16 matrix with contiguous rows")
    rows, cols = x.shape
    padded = -(-cols // 128) * 128
    q = torch.empty((rows, padded), dtype=torch.float8_e4m3fn, device=x.device)
    scales = torch.empty((padded // 128, rows), dtype=torch.float32, device=x.device)
    if rows == 0 or cols == 0:
        return q, scales
    status = _native.lib().fsh_act_quant_1x128(
        x.data_ptr(), rows, cols, x.stride(0), q.data_ptr(), padded, scales.data_ptr(),
        EPS_FP32 if eps_fp32 else EPS_INPUT_DTYPE, stream_ptr(x.device),
    )
    _native.check(status, "fsh_act_quant_1x128")
    return q, scales


def fp8_gemm_1x128_128x128(
    xq: torch.Tensor, xs: torch.Tensor, wq: torch.Tensor, ws: torch.Tensor, out: torch.Tensor | None = None
) -> torch.Tensor:
    """``out[i, j] = bf16(sum_kb dot(xq[i, kb], wq[j, kb]) * xs[kb, i] * ws[j // 128, kb])``
    for float8_e4m3fn ``xq`` [m, k], ``wq`` [n, k] (rows contiguous, k a
    multiple of 128), ``xs`` [k / 128, m] and ``ws`` [ceil(n / 128), >= k / 128]."""
    _require_gpu(xq, xs, wq, ws)
    for name, t in (("xq", xq), ("wq", wq)):
        if t.dtype not in (torch.float8_e4m3fn, torch.uint8) or t.ndim != 2 or t.stride(1) != 1:
            raise ValueError(f"{name} must be a float8_e4m3fn matrix with contiguous rows")
    m, k = xq.shape
    n = wq.shape[0]
    if wq.shape[1] != k:
        raise ValueError(f"inner dimensions differ: xq {tuple(xq.shape)} vs wq {tuple(wq.shape)}")
    blocks = k // 128
    if xs.dtype != torch.float32 or not xs.is_contiguous() or tuple(xs.shape) != (blocks, m):
        raise ValueError(f"xs must be contiguous fp32 of shape {(blocks, m)}, got {tuple(xs.shape)}")
    if ws.dtype != torch.float32 or ws.ndim != 2 or not _unit_column_stride(ws) or ws.shape[0] != -(-n // 128) or ws.shape[1] < blocks:
        raise ValueError(f"ws must be fp32 [{-(-n // 128)}, >= {blocks}] with contiguous rows, got {tuple(ws.shape)}")
    if out is None:
        out = torch.empty((m, n), dtype=torch.bfloat16, device=xq.device)
    _require_gpu(xq, out)
    if out.dtype != torch.bfloat16 or tuple(out.shape) != (m, n) or out.stride(1) != 1:
        raise ValueError(f"out must be bf16 [{m}, {n}] with contiguous rows")
    status = _native.lib().fsh_fp8_gemm_1x128_128x128(
        xq.data_ptr(), xs.data_ptr(), wq.data_ptr(), ws.data_ptr(), out.data_ptr(), m, n, k, xq.stride(0),
        wq.stride(0), out.stride(0), ws.stride(0), stream_ptr(xq.device),
    )
    _native.check(status, "fsh_fp8_gemm_1x128_128x128")
    return out


def _unit_column_stride(t: torch.Tensor) -> bool:
    return t.shape[1] <= 1 or t.stride(1) == 1  # the stride of a single column is arbitrary


def _fp8_matrix(name: str, t: torch.Tensor) -> None:
    if t.dtype not in (torch.float8_e4m3fn, torch.uint8) or t.ndim != 2 or t.stride(1) != 1:
        raise ValueError(f"{name} must be a float8_e4m3fn matrix with contiguous rows")


def fp8_transpose(src: torch.Tensor) -> torch.Tensor:
    """Transposed copy of a float8_e4m3fn (byte) matrix ``[rows, cols]``: returns
    ``[cols, rows rounded up to 128]`` whose pad columns are zero.  ``cols`` and
    the row stride must be multiples of 16."""
    _require_gpu(src)
    _fp8_matrix("src", src)
    rows, cols = src.shape
    ld_dst = -(-rows // 128) * 128
    dst = torch.empty((cols, ld_dst), dtype=src.dtype, device=src.device)
    if rows == 0 or cols == 0:
        return dst
    status = _native.lib().fsh_fp8_transpose(
        src.data_ptr(), rows, cols, src.stride(0), dst.data_ptr(), ld_dst, stream_ptr(src.device)
    )
    _native.check(status, "fsh_fp8_transpose")
    return dst


def act_quant_128x1_transposed(x: torch.Tensor, *, eps_fp32: bool = True) -> tuple[torch.Tensor, torch.Tensor]:
    """Quantize every run of 128 consecutive rows of each column of the bf16
    matrix ``x`` to float8_e4m3fn and return the bytes transposed: ``q`` is
    ``[cols, rows rounded up to 128]`` (pad zero), the reciprocal scales are a
    ``[rows / 128, cols]`` fp32 table.  Same arithmetic and ``eps_fp32`` rule as
    :func:`act_quant_1x128`."""
    _require_gpu(x)
    if x.dtype != torch.bfloat16 or x.ndim != 2 or x.stride(1) != 1:
        raise ValueError("x must be a bf16 matrix with contiguous rows")
    rows, cols = x.shape
    padded = -(-rows // 128) * 128
    q = torch.empty((cols, padded), dtype=torch.float8_e4m3fn, device=x.device)
    scales = torch.empty((padded // 128, cols), dtype=torch.float32, device=x.device)
    if rows == 0 or cols == 0:
        return q, scales
    status = _native.lib().fsh_act_quant_128x1_transposed(
        x.data_ptr(), rows, cols, x.stride(0), q.data_ptr(), padded, scales.data_ptr(),
        EPS_FP32 if eps_fp32 else EPS_INPUT_DTYPE, stream_ptr(x.device),
    )
    _native.check(status, "fsh_act_quant_128x1_transposed")
    return q, scales


def act_quant_both(
    x: torch.Tensor, *, eps_fp32: bool = True
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """:func:`act_quant_1x128` and :func:`act_quant_128x1_transposed` of the same
    bf16 matrix in one pass over it: returns ``(q_rows, scales_rows, q_cols,
    scales_cols)``, each pair bit for bit what the respective function returns."""
    _require_gpu(x)
    if x.dtype != torch.bfloat16 or x.ndim != 2 or x.stride(1) != 1:
        raise ValueError("x must be a bf16 matrix with contiguous rows")
    rows, cols = x.shape
    padded_rows, padded_cols = -(-rows // 128) * 128, -(-cols // 128) * 128
    q_rows = torch.empty((rows, padded_cols), dtype=torch.float8_e4m3fn, device=x.device)
    scales_rows = torch.empty((padded_cols // 128, rows), dtype=torch.float32, device=x.device)
    q_cols = torch.empty((cols, padded_rows), dtype=torch.float8_e4m3fn, device=x.device)
    scales_cols = torch.empty((padded_rows // 128, cols), dtype=torch.float32, device=x.device)
    if rows == 0 or cols == 0:
        return q_rows, scales_rows, q_cols, scales_cols
    status = _native.lib().fsh_act_quant_both(
        x.data_ptr(), rows, cols, x.stride(0), q_rows.data_ptr(), padded_cols, scales_rows.data_ptr(),
        q_cols.data_ptr(), padded_rows, scales_cols.data_ptr(), EPS_FP32 if eps_fp32 else EPS_INPUT_DTYPE,
        stream_ptr(x.device),
    )
    _native.check(status, "fsh_act_quant_both")
    return q_rows, scales_rows, q_cols, scales_cols


def fp8_gemm_1x128_128x128_dgrad(
    gq: torch.Tensor, gs: torch.Tensor, wtq: torch.Tensor, ws: torch.Tensor, in_dim: int | None = None
) -> torch.Tensor:
    """``out[i, j] = bf16(sum_ob dot(gq[i, ob], wtq[j, ob]) * gs[ob, i] * ws[ob, j // 128])``:
    the input gradient of a linear whose weight has scales ``ws`` ``[out / 128,
    >= in / 128]``.  ``gq`` [m, out] with ``gs`` [out / 128, m] from
    :func:`act_quant_1x128`, ``wtq`` [in, out] from :func:`fp8_transpose`; ``out``
    (the contraction) a multiple of 128.  Returns ``[m, in_dim]``."""
    _require_gpu(gq, gs, wtq, ws)
    _fp8_matrix("gq", gq)
    _fp8_matrix("wtq", wtq)
    m, out_dim = gq.shape
    in_dim = wtq.shape[0] if in_dim is None else in_dim
    if wtq.shape[1] != out_dim or in_dim > wtq.shape[0]:
        raise ValueError(f"shapes do not match: gq {tuple(gq.shape)}, wtq {tuple(wtq.shape)}, in_dim {in_dim}")
    blocks = out_dim // 128
    if gs.dtype != torch.float32 or not gs.is_contiguous() or tuple(gs.shape) != (blocks, m):
        raise ValueError(f"gs must be contiguous fp32 of shape {(blocks, m)}, got {tuple(gs.shape)}")
    if ws.dtype != torch.float32 or ws.ndim != 2 or not _unit_column_stride(ws) or ws.shape[0] < blocks or ws.shape[1] < -(-in_dim // 128):
        raise ValueError(f"ws must be fp32 [>= {blocks}, >= {-(-in_dim // 128)}] with contiguous rows, got {tuple(ws.shape)}")
    out = torch.empty((m, in_dim), dtype=torch.bfloat16, device=gq.device)
    status = _native.lib().fsh_fp8_gemm_1x128_128x128_dgrad(
        gq.data_ptr(), gs.data_ptr(), wtq.data_ptr(), ws.data_ptr(), out.data_ptr(), m, in_dim, out_dim,
        gq.stride(0), wtq.stride(0), out.stride(0), ws.stride(0), stream_ptr(gq.device),
    )
    _native.check(status, "fsh_fp8_gemm_1x128_128x128_dgrad")
    return out


def fp8_gemm_1x128_128x1(
    aq: torch.Tensor, a_scales: torch.Tensor, bq: torch.Tensor, b_scales: torch.Tensor
) -> torch.Tensor:
    """``out[i, j] = bf16(sum_kb dot(aq[i, kb], bq[j, kb]) * a_scales[kb, i] * b_scales[kb, j])``
    for two operands quantized in runs of 128 along the contraction
    (:func:`act_quant_128x1_transposed`)."""
    _require_gpu(aq, a_scales, bq, b_scales)
    _fp8_matrix("aq", aq)
    _fp8_matrix("bq", bq)
    k = aq.shape[1]
    if bq.shape[1] != k:
        raise ValueError(f"inner dimensions differ: aq {tuple(aq.shape)} vs bq {tuple(bq.shape)}")
    m, n = aq.shape[0], bq.shape[0]
    blocks = k // 128
    for name, t, size in (("a_scales", a_scales, aq.shape[0]), ("b_scales", b_scales, bq.shape[0])):
        if t.dtype != torch.float32 or not t.is_contiguous() or tuple(t.shape) != (blocks, size):
            raise ValueError(f"{name} must be contiguous fp32 of shape {(blocks, size)}, got {tuple(t.shape)}")
    out = torch.empty((m, n), dtype=torch.bfloat16, device=aq.device)
    status = _native.lib().fsh_fp8_gemm_1x128_128x1(
        aq.data_ptr(), a_scales.data_ptr(), bq.data_ptr(), b_scales.data_ptr(), out.data_ptr(), m, n, k,
        aq.stride(0), bq.stride(0), out.stride(0), stream_ptr(aq.device),
    )
    _native.check(status, "fsh_fp8_gemm_1x128_128x1")
    return out


def _muon_master_dtype(who: str, masters: Sequence[torch.Tensor], bf16: Sequence[torch.Tensor]) -> torch.dtype:
    """The dtype of the master tensors of a Muon elementwise step (all bf16 or
    all fp32, contiguous, of equal numel with the bf16 operands)."""
    dtype, numel = masters[0].dtype, masters[0].numel()
    if dtype not in (torch.bfloat16, torch.float32):
        raise NotImplementedError(f"{who} takes bf16 or fp32 master tensors, got {dtype}")
    for t in masters:
        if t.dtype != dtype or not t.is_contiguous() or t.numel() != numel:
            raise ValueError(f"{who} needs contiguous tensors of one dtype and equal numel")
    for t in bf16:
        if t.dtype != torch.bfloat16 or not t.is_contiguous() or t.numel() != numel:
            raise ValueError(f"{who} needs a contiguous bf16 Newton-Schulz operand of the same numel")
    return dtype


def muon_prepare(
    momentum_buffer: torch.Tensor, grad: torch.Tensor, out: torch.Tensor, *, momentum: float, nesterov: bool
) -> None:
    """Momentum update and the input of the orthogonalization.  ``momentum_buffer``
    and ``grad`` are both bf16 or both fp32; ``out`` is bf16."""
    _require_gpu(momentum_buffer, grad, out)
    dtype = _muon_master_dtype("muon_prepare", (momentum_buffer, grad), (out,))
    entry = "fsh_muon_prepare" if dtype == torch.bfloat16 else "fsh_muon_prepare_f32"
    status = getattr(_native.lib(), entry)(
        momentum_buffer.data_ptr(), grad.data_ptr(), out.data_ptr(), grad.numel(), 1 - momentum, momentum,
        int(nesterov), stream_ptr(grad.device),
    )
    _native.check(status, entry)


def muon_apply(
    param: torch.Tensor, direction: torch.Tensor, *, decay_factor: float, neg_adjusted_lr: float,
    direction_scale: float = 1.0,
) -> None:
    """Decayed update of a bf16 or fp32 ``param`` by the bf16 ``direction``."""
    _require_gpu(param, direction)
    dtype = _muon_master_dtype("muon_apply", (param,), (direction,))
    entry = "fsh_muon_apply" if dtype == torch.bfloat16 else "fsh_muon_apply_f32"
    status = getattr(_native.lib(), entry)(
        param.data_ptr(), direction.data_ptr(), param.numel(), decay_factor, neg_adjusted_lr, direction_scale,
        stream_ptr(param.device),
    )
    _native.check(status, entry)


class MuonStepPlan:
    """The launch tables of ``fsh_muon_step`` for the whole matrices of an
    optimizer: per shape group three device tables of addresses (parameters,
    momentum buffers, gradients), a contiguous batch buffer and the
    Newton-Schulz workspace.  The address tables are checked on every step and
    re-uploaded only when a tensor moved (gradients usually do, parameters and
    momentum buffers usually do not)."""

    def __init__(self, groups: Sequence[tuple], device: torch.device) -> None:
        """``groups``: per group (shape, matrix count, neg_adjusted_lr,
        direction_scale[, master dtype]); the master dtype (of parameters,
        gradients and momentum buffers) is bf16 when left out, or fp32."""
        if not groups:
            raise ValueError("a Muon step needs at least one group")
        if len(groups) > _native.MAX_NS_PROBLEMS:
            raise NotImplementedError(f"at most {_native.MAX_NS_PROBLEMS} shape groups per step")
        if device.type != "cuda":
            raise RuntimeError("flex_shard_amd kernels run on the GPU only; there is no CPU path.")
        self._device = device
        self._table = (_native.MuonGroup * len(groups))()
        self._shapes: list[tuple[int, int]] = []
        self._dtypes: list[torch.dtype] = []
        self._address_tables: list[list[tuple[torch.Tensor, list[int]]]] = []
        self.batches: list[torch.Tensor] = []
        self.workspaces: list[torch.Tensor] = []
        for slot, (shape, n, neg_lr, scale, *rest) in zip(self._table, groups):
            master = rest[0] if rest else torch.bfloat16
            if master not in (torch.bfloat16, torch.float32):
                raise NotImplementedError(f"Muon master tensors are bf16 or fp32, got {master}")
            if len(shape) != 2 or shape[0] % 8 or shape[1] % 8 or n <= 0:
                raise NotImplementedError(f"whole matrices with rows and cols multiples of 8, got {n} x {tuple(shape)}")
            batch = torch.empty((n, *shape), dtype=torch.bfloat16, device=device)
            workspace = torch.empty(newton_schulz_workspace_bytes(n, *shape), dtype=torch.uint8, device=device)
            tables = [(torch.zeros(n, dtype=torch.int64, device=device), [0] * n) for _ in range(3)]
            self.batches.append(batch)
            self.workspaces.append(workspace)
            self._shapes.append(tuple(shape))
            self._dtypes.append(master)
            slot.master_dtype = DT_BF16 if master == torch.bfloat16 else DT_F32
            self._address_tables.append(tables)
            slot.param_ptrs_dev, slot.momentum_ptrs_dev, slot.grad_ptrs_dev = (t.data_ptr() for t, _ in tables)
            slot.batch_dev, slot.batch, slot.rows, slot.cols = batch.data_ptr(), n, shape[0], shape[1]
            slot.workspace_dev, slot.workspace_nbytes = workspace.data_ptr(), workspace.numel()
            slot.neg_adjusted_lr, slot.direction_scale = neg_lr, scale

    def _refresh(self, table: torch.Tensor, current: list[int], tensors: Sequence[torch.Tensor], shape, dtype) -> None:
        if len(tensors) != len(current):
            raise ValueError(f"expected {len(current)} matrices of shape {shape}, got {len(tensors)}")
        addresses = []
        for t in tensors:
            if t.device != self._device:
                raise ValueError(f"all matrices of a Muon step must live on {self._device}, got {t.device}")
            if t.dtype != dtype or not t.is_contiguous() or tuple(t.shape) != shape:
                raise ValueError(f"the Muon step kernels need contiguous {dtype} matrices of shape {shape}")
            if t.data_ptr() % 16:
                raise ValueError("the Muon step kernels need 16-byte aligned matrices")
            addresses.append(t.data_ptr())
        if addresses != current:
            # A fresh pinned staging tensor per change: torch's host allocator
            # keeps its block from reuse until the queued copy has read it, so
            # nothing here waits for the GPU.
            table.copy_(torch.tensor(addresses, dtype=torch.int64, pin_memory=True), non_blocking=True)
            current[:] = addresses

    def step(
        self, params: Sequence[Sequence[torch.Tensor]], momenta: Sequence[Sequence[torch.Tensor]],
        grads: Sequence[Sequence[torch.Tensor]], *, lerp_weight: float, nesterov_weight: float, nesterov: bool,
        decay_factor: float, coefficients: tuple[float, float, float], steps: int, eps: float,
        neg_adjusted_lrs: Sequence[float] | None = None, direction_scales: Sequence[float] | None = None,
    ) -> None:
        """Per group: the parameters, their momentum buffers and their
        gradients, one of each per matrix, in the same order.  All three are
        read (and the first two written) by kernels queued on the current
        stream, and so are the plan's address tables, batch buffers and
        workspaces: steps of one plan belong on one stream (or on streams
        ordered one behind the other).  ``neg_adjusted_lrs`` / ``direction_scales`` (one per group)
        replace the step sizes and direction scales the plan was built with:
        the C call reads them from the host table at launch time, so a
        learning-rate schedule passes the current values on every step."""
        for name, values in (("neg_adjusted_lr", neg_adjusted_lrs), ("direction_scale", direction_scales)):
            if values is None:
                continue
            if len(values) != len(self._shapes):
                raise ValueError(f"expected one {name} per group ({len(self._shapes)}), got {len(values)}")
            for slot, value in zip(self._table, values):
                setattr(slot, name, float(value))
        for name, lists in (("parameter", params), ("momentum", momenta), ("gradient", grads)):
            if len(lists) != len(self._shapes):
                raise ValueError(f"expected {name} lists for {len(self._shapes)} groups, got {len(lists)}")
        for tables, shape, dtype, p, m, g in zip(self._address_tables, self._shapes, self._dtypes, params, momenta, grads):
            for (table, current), tensors in zip(tables, (p, m, g)):
                self._refresh(table, current, tensors, shape, dtype)
        a, b, c = coefficients
        status = _native.lib().fsh_muon_step(
            self._table, len(self._shapes), lerp_weight, nesterov_weight, 1 if nesterov else 0, decay_factor, a, b, c,
            steps, eps, stream_ptr(self._device),
        )
        _native.check(status, "fsh_muon_step")
