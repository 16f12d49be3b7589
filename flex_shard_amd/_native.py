"""ctypes binding of ``libflexshard_hip.so`` (the C ABI in ``include/flexshard_hip.h``).

The library is the only compute path of this package.  If it is missing or
does not export a declared symbol, :func:`lib` raises ``RuntimeError``; there
is no eager or CPU substitute.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, Structure, c_char_p, c_float, c_int, c_int32, c_int64, c_void_p

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libflexshard_hip.so")

FSH_OK = 0
FSH_MAX_QUANT_CHUNKS = 24

SRC_BF16, SRC_F32, SRC_F32_AS_BF16, SRC_F16, SRC_F32_AS_F16 = 0, 1, 2, 3, 4
EPS_INPUT_DTYPE, EPS_FP32 = 0, 1
DT_BF16, DT_F32, DT_F16 = 0, 1, 2
REDUCE_SUM, REDUCE_PREMUL, REDUCE_POSTMUL, REDUCE_POSTDIV = 0, 1, 2, 3


class QuantChunk(Structure):
    """``fsh_quant_chunk``."""

    _fields_ = [
        ("src_dev", c_void_p),
        ("rows", c_int64),
        ("in_dim", c_int64),
        ("src_row_stride", c_int64),
        ("qdata_offset", c_int64),
        ("scale_offset", c_int64),
        ("src_kind", c_int32),
        ("reserved", c_int32),
    ]


class UnpackChunk(Structure):
    """``fsh_unpack_chunk`` (seven int64 fields, 56 bytes)."""

    _fields_ = [
        ("src_qdata_offset", c_int64),
        ("src_scale_offset", c_int64),
        ("rows", c_int64),
        ("in_dim", c_int64),
        ("dst_qdata_offset", c_int64),
        ("dst_scale_offset", c_int64),
        ("dst_dequant_offset", c_int64),
    ]


UNPACK_CHUNK_INT64S = 7


class GemmDesc(Structure):
    """``fsh_gemm_desc``."""

    _fields_ = [
        ("a_dev", c_void_p),
        ("b_dev", c_void_p),
        ("d_dev", c_void_p),
        ("c_dev", c_void_p),
        ("ct_dev", c_void_p),
        ("m", c_int64),
        ("n", c_int64),
        ("k", c_int64),
        ("lda", c_int64),
        ("ldb", c_int64),
        ("ldd", c_int64),
        ("ldc", c_int64),
        ("ldct", c_int64),
        ("batch", c_int64),
        ("stride_a", c_int64),
        ("stride_b", c_int64),
        ("stride_d", c_int64),
        ("stride_c", c_int64),
        ("stride_ct", c_int64),
        ("alpha", c_float),
        ("beta", c_float),
        ("symmetric", c_int32),
        ("diag_add", c_float),
        ("k_major", c_int32),
        ("reserved", c_int32),
    ]


class NsProblem(Structure):
    """``fsh_ns_problem``."""

    _fields_ = [
        ("x_dev", c_void_p),
        ("batch", c_int64),
        ("rows", c_int64),
        ("cols", c_int64),
        ("workspace_dev", c_void_p),
        ("workspace_nbytes", c_int64),
    ]


class MuonGroup(Structure):
    """``fsh_muon_group``."""

    _fields_ = [
        ("param_ptrs_dev", c_void_p),
        ("grad_ptrs_dev", c_void_p),
        ("momentum_ptrs_dev", c_void_p),
        ("batch_dev", c_void_p),
        ("batch", c_int64),
        ("rows", c_int64),
        ("cols", c_int64),
        ("workspace_dev", c_void_p),
        ("workspace_nbytes", c_int64),
        ("neg_adjusted_lr", c_float),
        ("direction_scale", c_float),
        ("master_dtype", c_int32),
        ("reserved", c_int32),
    ]


MAX_NS_PROBLEMS = 16
NS_STATIC_SCRATCH_BYTES = 128 << 20


# name -> (restype, argtypes); every symbol include/flexshard_hip.h declares.
SIGNATURES: dict[str, tuple[object, list[object]]] = {
    "fsh_version": (c_int32, []),
    "fsh_last_error": (c_char_p, []),
    "fsh_quantize_pack": (
        c_int,
        [POINTER(QuantChunk), c_int32, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_int32, c_int32, c_void_p],
    ),
    "fsh_quant_pack_plan_create": (
        c_int,
        [POINTER(QuantChunk), c_int32, c_int64, c_int64, c_int64, c_int64, c_int64, c_int32, c_int32, POINTER(c_void_p)],
    ),
    "fsh_quant_pack_plan_launch": (c_int, [c_void_p, c_void_p, c_void_p]),
    "fsh_quant_pack_plan_destroy": (None, [c_void_p]),
    "fsh_copy_segments": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int32, c_void_p]),
    "fsh_zero_segments": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int32, c_void_p]),
    "fsh_pack_segments": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int32, c_int32, c_void_p, c_void_p],
    ),
    "fsh_unpack_dequant": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_void_p, c_void_p, c_int32, c_int32, c_void_p],
    ),
    "fsh_accumulate_grad": (c_int, [c_void_p, c_void_p, c_int32, c_int64, c_int32, c_void_p]),
    "fsh_reduce_rows_f32": (c_int, [c_void_p, c_void_p, c_int64, c_int32, c_int64, c_int64, c_int32, c_float, c_void_p]),
    "fsh_reduce_rows_bf16": (c_int, [c_void_p, c_void_p, c_int64, c_int32, c_int64, c_int64, c_int32, c_float, c_void_p]),
    "fsh_newton_schulz_workspace_bytes": (c_int64, [c_int64, c_int64, c_int64]),
    "fsh_newton_schulz": (
        c_int,
        [c_void_p, c_int64, c_int64, c_int64, c_float, c_float, c_float, c_int32, c_float, c_void_p, c_int64, c_void_p],
    ),
    "fsh_newton_schulz_noalloc": (
        c_int, [c_void_p, c_int64, c_int64, c_int64, c_float, c_float, c_float, c_int32, c_float, c_void_p],
    ),
    "fsh_newton_schulz_multi": (
        c_int, [POINTER(NsProblem), c_int32, c_float, c_float, c_float, c_int32, c_float, c_void_p],
    ),
    "fsh_gemm_bf16_nt": (c_int, [POINTER(GemmDesc), c_void_p]),
    "fsh_gemm_bf16_nt_group": (c_int, [POINTER(GemmDesc), c_int32, c_void_p]),
    "fsh_act_quant_1x128": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_int32, c_void_p]),
    "fsh_fp8_gemm_1x128_128x128": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
         c_void_p],
    ),
    "fsh_fp8_transpose": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p]),
    "fsh_act_quant_128x1_transposed": (
        c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_int32, c_void_p],
    ),
    "fsh_act_quant_both": (
        c_int,
        [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_void_p, c_int32, c_void_p],
    ),
    "fsh_fp8_gemm_1x128_128x128_dgrad": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
         c_void_p],
    ),
    "fsh_fp8_gemm_1x128_128x1": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p],
    ),
    "fsh_muon_prepare": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_float, c_float, c_int32, c_void_p]),
    "fsh_muon_apply": (c_int, [c_void_p, c_void_p, c_int64, c_float, c_float, c_float, c_void_p]),
    "fsh_muon_prepare_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_float, c_float, c_int32, c_void_p]),
    "fsh_muon_apply_f32": (c_int, [c_void_p, c_void_p, c_int64, c_float, c_float, c_float, c_void_p]),
    "fsh_muon_step": (
        c_int,
        [POINTER(MuonGroup), c_int32, c_float, c_float, c_int32, c_float, c_float, c_float, c_float, c_int32, c_float,
         c_void_p],
    ),
}

_LIB: ctypes.CDLL | None = None


class NativeError(RuntimeError):
    """A C-ABI call returned a negative status."""


def lib() -> ctypes.CDLL:
    """Load the shared library once and bind every declared symbol."""
    global _LIB
    if _LIB is not None:
        return _LIB
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `make -C flex_shard_amd/csrc` "
            "(or __graft_entry__.build()). flex_shard_amd has no fallback compute path."
        )
    handle = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        try:
            fn = getattr(handle, name)
        except AttributeError as exc:
            raise RuntimeError(f"{LIB_PATH} does not export {name}") from exc
        fn.restype = restype
        fn.argtypes = argtypes
    _LIB = handle
    return handle


def check(status: int, what: str) -> None:
    if status != FSH_OK:
        message = lib().fsh_last_error().decode("utf-8", "replace")
        raise NativeError(f"{what} failed with status {status}: {message}")
