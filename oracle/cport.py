"""ctypes bindings of ``flexshard_oracle.c``.  TEST INFRASTRUCTURE ONLY.

Tensors are CPU torch tensors (torch is used here only as a typed byte
container: numpy has no bfloat16).
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libflexshard_oracle.so")
_LIB: ctypes.CDLL | None = None

SRC_BF16, SRC_F32, SRC_F32_AS_BF16 = 0, 1, 2
EPS_INPUT_DTYPE, EPS_FP32 = 0, 1
REDUCE_SUM, REDUCE_PREMUL, REDUCE_POSTMUL, REDUCE_POSTDIV = 0, 1, 2, 3


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (seconds).  Returns the library path."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s"], check=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _LIB
    if _LIB is None:
        build()
        handle = ctypes.CDLL(_LIB_PATH)
        i64, vp, f32 = ctypes.c_int64, ctypes.c_void_p, ctypes.c_float
        handle.fso_quantize_blockwise.argtypes = [vp, ctypes.c_int, i64, i64, i64, i64, ctypes.c_int, vp, vp]
        handle.fso_quantize_blockwise.restype = ctypes.c_int
        handle.fso_dequant_blockwise.argtypes = [vp, vp, i64, i64, i64, ctypes.c_int, vp]
        handle.fso_dequant_blockwise.restype = ctypes.c_int
        handle.fso_copy_segments.argtypes = [vp, vp, vp, vp, vp, i64]
        handle.fso_zero_segments.argtypes = [vp, vp, vp, i64]
        handle.fso_accumulate_bf16.argtypes = [vp, vp, i64]
        handle.fso_reduce_rows_f32.argtypes = [vp, vp, i64, i64, ctypes.c_int, f32]
        handle.fso_newton_schulz_bf16.argtypes = [vp, i64, i64, f32, f32, f32, ctypes.c_int, f32]
        handle.fso_newton_schulz_bf16.restype = ctypes.c_int
        handle.fso_scalar_f32_to_e4m3fn.argtypes = [f32]
        handle.fso_scalar_f32_to_e4m3fn.restype = ctypes.c_uint8
        handle.fso_scalar_e4m3fn_to_f32.argtypes = [ctypes.c_uint8]
        handle.fso_scalar_e4m3fn_to_f32.restype = f32
        handle.fso_scalar_f32_to_bf16.argtypes = [f32]
        handle.fso_scalar_f32_to_bf16.restype = ctypes.c_uint16
        _LIB = handle
    return _LIB


def _cpu(t: torch.Tensor) -> torch.Tensor:
    if t.device.type != "cpu":
        raise ValueError("the oracle works on CPU tensors")
    return t


def f32_to_e4m3fn(x: float) -> int:
    return int(lib().fso_scalar_f32_to_e4m3fn(x))


def e4m3fn_to_f32(b: int) -> float:
    return float(lib().fso_scalar_e4m3fn_to_f32(b))


def quantize_blockwise(
    weight: torch.Tensor,
    block: int,
    *,
    cast_to_bf16: bool = False,
    eps_mode: int = EPS_INPUT_DTYPE,
) -> tuple[torch.Tensor, torch.Tensor]:
    """FP8 bytes ``[rows, in_dim]`` (uint8) and reciprocal scales (fp32) of a
    2-D row-major matrix; rows may be strided.  ``cast_to_bf16`` quantizes an
    fp32 master weight as its bf16 rounding."""
    weight = _cpu(weight)
    if weight.ndim != 2 or weight.stride(1) != 1:
        raise ValueError("expects a 2-D matrix with unit column stride")
    rows, in_dim = weight.shape
    if weight.dtype == torch.bfloat16:
        kind = SRC_BF16
    elif weight.dtype == torch.float32:
        kind = SRC_F32_AS_BF16 if cast_to_bf16 else SRC_F32
    else:
        raise ValueError(f"unsupported dtype {weight.dtype}")
    qdata = torch.empty((rows, in_dim), dtype=torch.uint8)
    scales = torch.empty((-(-rows // block), -(-in_dim // block)), dtype=torch.float32)
    rc = lib().fso_quantize_blockwise(
        weight.data_ptr(), kind, rows, in_dim, weight.stride(0), block, eps_mode,
        qdata.data_ptr(), scales.data_ptr(),
    )
    if rc != 0:
        raise ValueError(f"fso_quantize_blockwise failed with {rc}")
    return qdata, scales


def dequant_blockwise(
    qdata: torch.Tensor, scales: torch.Tensor, block: int, out_dtype: torch.dtype = torch.bfloat16
) -> torch.Tensor:
    qdata = _cpu(qdata).contiguous().view(torch.uint8)
    scales = _cpu(scales).contiguous()
    rows, in_dim = qdata.shape
    out = torch.empty((rows, in_dim), dtype=out_dtype)
    kind = {torch.bfloat16: 0, torch.float32: 1}[out_dtype]
    rc = lib().fso_dequant_blockwise(
        qdata.data_ptr(), scales.data_ptr(), rows, in_dim, block, kind, out.data_ptr()
    )
    if rc != 0:
        raise ValueError(f"fso_dequant_blockwise failed with {rc}")
    return out


def _i64(values) -> torch.Tensor:
    return torch.tensor(list(values), dtype=torch.int64)


def copy_segments(src: torch.Tensor, out: torch.Tensor, src_off, nbytes, dst_off) -> None:
    """Byte segment copy; ``src``/``out`` are contiguous uint8."""
    so, nb, do = _i64(src_off), _i64(nbytes), _i64(dst_off)
    lib().fso_copy_segments(src.data_ptr(), out.data_ptr(), so.data_ptr(), nb.data_ptr(), do.data_ptr(), so.numel())


def zero_segments(out: torch.Tensor, nbytes, dst_off) -> None:
    nb, do = _i64(nbytes), _i64(dst_off)
    lib().fso_zero_segments(out.data_ptr(), nb.data_ptr(), do.data_ptr(), nb.numel())


def accumulate_bf16(acc: torch.Tensor, grad: torch.Tensor) -> None:
    assert acc.dtype == torch.float32 and grad.dtype == torch.bfloat16
    assert acc.is_contiguous() and grad.is_contiguous() and acc.numel() == grad.numel()
    lib().fso_accumulate_bf16(acc.data_ptr(), grad.data_ptr(), acc.numel())


def reduce_rows(rows: list[torch.Tensor], mode: int = REDUCE_SUM, factor: float = 1.0) -> torch.Tensor:
    """Left fold of equally long contiguous fp32 vectors in list order."""
    n = rows[0].numel()
    assert all(r.dtype == torch.float32 and r.is_contiguous() and r.numel() == n for r in rows)
    ptrs = (ctypes.c_void_p * len(rows))(*[r.data_ptr() for r in rows])
    out = torch.empty(n, dtype=torch.float32)
    lib().fso_reduce_rows_f32(out.data_ptr(), ptrs, len(rows), n, mode, factor)
    return out


def newton_schulz(
    x: torch.Tensor,
    coefficients: tuple[float, float, float] = (3.4445, -4.7750, 2.0315),
    steps: int = 5,
    eps: float = 1e-7,
) -> torch.Tensor:
    """Newton-Schulz of one 2-D matrix in bf16 (small sizes: O(n^3) scalar C)."""
    x = _cpu(x).to(torch.bfloat16)
    transposed = x.shape[0] > x.shape[1]
    work = (x.t() if transposed else x).contiguous().clone()
    a, b, c = coefficients
    rc = lib().fso_newton_schulz_bf16(work.data_ptr(), work.shape[0], work.shape[1], a, b, c, steps, eps)
    if rc != 0:
        raise ValueError(f"fso_newton_schulz_bf16 failed with {rc}")
    return work.t() if transposed else work
