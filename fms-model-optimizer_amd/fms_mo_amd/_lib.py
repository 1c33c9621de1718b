"""ctypes binding of libfmsmo_hip.so, the C-ABI library of hand-written gfx950 kernels.

There is no CPU fallback: every operator of this package ends in one of these entry points, and
loading fails loudly when the library has not been built
(``make -C fms-model-optimizer_amd/csrc`` or ``python -c 'import __graft_entry__ as g; g.build()'``).
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
# FMSMO_LIB names another build of the library (A/B measurements of kernel variants)
LIB_PATH = os.environ.get("FMSMO_LIB") or os.path.normpath(os.path.join(_HERE, "..", "lib", "libfmsmo_hip.so"))

# dtype / enum codes of include/fmsmo_hip.h
F16, BF16, F32 = 0, 1, 2
OP_I8, OP_E4M3, OP_F16, OP_BF16, OP_F32 = 0, 1, 2, 3, 4
EPI_REF_F16, EPI_F32, EPI_F32_MULADD, EPI_SEQ_OUT = 0, 1, 2, 3
SQ_RAW, SQ_FMO, SQ_U8_SHIFT, SQ_S8_NARROW = 0, 1, 2, 3
DQ_PER_TENSOR, DQ_PER_COLUMN = 0, 1
F8E_SAT, F8E_PER_TENSOR, F8E_PER_ROW = 0, 1, 2
FP8_LINEAR, FP8_FPXACC, FP8_FPXACC_DL8 = 0, 1, 2
WQ_MUL, WQ_DIV = 0, 1
MS_PER_TOKEN, MS_SYMM, MS_ASYMM = 0, 1, 2
ABI_VERSION = 2
PLAN_DECODE, PLAN_TILE_REGISTER_STAGED, PLAN_TILE_LDS_DMA, PLAN_GENERIC = 0, 1, 2, 3

_P, _I, _L, _F = c_void_p, c_int, c_int64, c_float

# name -> argument types (all functions return int except the three below)
SIGNATURES = {
    "fmsmo_quant_act_i8_pertoken": [_P, _I, _L, _P, _I, _I, _I, _P, _L, _P, _L, _L, _P],
    "fmsmo_quant_act_i8_static": [_P, _I, _L, _F, _I, _I, _P, _L, _L, _L, _P],
    "fmsmo_quant_act_i8_static_t": [_P, _I, _L, _I, _I, _F, _F, _I, _F, _F, _P, _L, _L, _L, _P],
    "fmsmo_quant_act_i8_dynamic": [_P, _I, _L, _P, _I, _I, _I, _P, _L, _P, _L, _L, _P],
    "fmsmo_fake_quant_fp8": [_P, _I, _L, _I, _P, _P, _L, _P, _L, _P, _P, _L, _L, _P],
    "fmsmo_quant_act_i8_mulscale": [_P, _I, _L, _P, _P, _I, _I, _I, _P, _L, _P, _L, _L, _P],
    "fmsmo_quant_act_fp8_pertoken": [_P, _I, _L, _I, _I, _P, _L, _P, _L, _L, _P],
    "fmsmo_quant_act_fp8_dynamic": [_P, _I, _L, _I, _I, _P, _F, _I, _P, _L, _P, _L, _L, _P],
    "fmsmo_gemm_i8_i32": [_P, _L, _P, _L, _P, _L, _L, _L, _L, _P],
    "fmsmo_gemm_i8_i32_ws": [_P, _L, _P, _L, _P, _L, _L, _L, _L, _P, _L, _P],
    "fmsmo_gemm_i8_dq": [_P, _L, _P, _L, _P, _L, _P, _L, _P, _I, _I, _P, _I, _L, _L, _L, _L, _P],
    "fmsmo_gemm_fp8_dq": [_P, _L, _P, _L, _P, _L, _P, _L, _P, _I, _P, _I, _L, _L, _L, _L, _P],
    "fmsmo_gemm_i8_dq_ws": [_P, _L, _P, _L, _P, _L, _P, _L, _P, _I, _I, _P, _I, _L, _L, _L, _L, _P, _L, _P],
    "fmsmo_gemm_i8_dq_noalloc": [_P, _L, _P, _L, _P, _L, _P, _L, _P, _I, _I, _P, _I, _L, _L, _L, _L, _P],
    "fmsmo_gemm_fp8_dq_ws": [_P, _L, _P, _L, _P, _L, _P, _L, _P, _I, _P, _I, _L, _L, _L, _L, _P, _L, _P],
    "fmsmo_gemv_i8_dq": [_P, _L, _P, _L, _P, _L, _P, _L, _P, _I, _I, _P, _I, _L, _L, _L, _L, _P],
    "fmsmo_gemv_fp8_dq": [_P, _L, _P, _L, _P, _L, _P, _L, _P, _I, _P, _I, _L, _L, _L, _L, _P],
    "fmsmo_decode_linear_i8": [_P, _I, _L, _P, _I, _I, _P, _L, _P, _L, _P, _I, _I, _P, _I, _L, _P, _L, _L, _L, _P],
    "fmsmo_decode_linear_fp8": [_P, _I, _L, _P, _L, _P, _L, _P, _I, _P, _I, _L, _P, _L, _L, _L, _P],
    "fmsmo_matmul_chunk_i8": [_P, _L, _P, _L, _P, _P, _L, _L, _L, _L, _I, _I, _I, _I, _P],
    "fmsmo_matmul_chunk_fp": [_P, _L, _P, _L, _I, _P, _P, _L, _L, _L, _L, _I, _I, _I, _I, _P],
    "fmsmo_matmul_chunk_i8_dq": [_P, _L, _P, _L, _P, _L, _P, _L, _P, _I, _I, _P, _I, _L, _L, _L, _L,
                                 _I, _I, _I, _I, _P],
    "fmsmo_matmul_chunk_fp_dq": [_P, _L, _P, _L, _I, _P, _L, _P, _L, _P, _I, _I, _P, _I, _L, _L, _L, _L,
                                 _I, _I, _I, _I, _P],
    "fmsmo_grouped_gemm_i8_dq": [_P, _L, _P, _L, _L, _P, _I, _L, _P, _P, _P, _I, _I, _P, _I, _L,
                                 _L, _L, _P],
    "fmsmo_quant_weight_i8": [_P, _I, _L, _P, _I, _P, _I, _L, _I, _P, _L, _P, _L, _L, _P],
    "fmsmo_absmax_cols": [_P, _I, _L, _L, _L, _P, _P],
    "fmsmo_quant_i8_affine": [_P, _I, _L, _L, _F, _F, _I, _I, _P, _L, _L, _L, _L, _L, _P],
    "fmsmo_bmm_i8_dq": [_P, _L, _P, _L, _L, _P, _P, _P, _P, _I, _L, _L, _L, _L, _L, _P],
    "fmsmo_bmm_fp8_dq": [_P, _L, _P, _L, _L, _P, _P, _P, _P, _I, _L, _L, _L, _L, _L, _P],
    "fmsmo_zero_shift_bias": [_P, _L, _P, _L, _P, _F, _P, _I, _P, _L, _L, _P],
    "fmsmo_debug_clock_probe": [_P],
    "fmsmo_debug_stream_read": [_P, _L, _P, _P],
    "fmsmo_debug_mfma_loop": [_I, _P, _L, _I, _P, _P, _P],
    "fmsmo_gemm_plan": [_L, _L, _L, _I, _P, _P, _P, _P],
}
OTHER = {
    "fmsmo_abi_version": ([], c_int),
    "fmsmo_status_str": ([c_int], c_char_p),
    "fmsmo_last_error": ([], c_char_p),
    "fmsmo_gemm_workspace_bytes": ([c_int64, c_int64, c_int64], c_int64),
    "fmsmo_decode_linear_ok": ([c_int64, c_int64], c_int),
    "fmsmo_decode_linear_f32s_ok": ([c_int64, c_int64], c_int),
    "fmsmo_gemm_tail_columns": ([c_int64, c_int64, c_int64], c_int64),
}

_lib = None


class FmsMoHipError(RuntimeError):
    """A C-ABI entry point returned a non-zero status (the reference raises RuntimeError from
    TORCH_CHECK in the same situations, fms_mo/custom_ext_kernels/cutlass_i8i32gemm.cu:118)."""


def load() -> ctypes.CDLL:
    """Load the shared library once and attach argument / return types."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FmsMoHipError(
            f"{LIB_PATH} is missing: build the HIP kernels first "
            "(make -C fms-model-optimizer_amd/csrc). There is no fallback path."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = c_int
    for name, (argtypes, restype) in OTHER.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = restype
    if lib.fmsmo_abi_version() != ABI_VERSION:
        raise FmsMoHipError("libfmsmo_hip.so ABI version mismatch; rebuild the library")
    _lib = lib
    return lib


def raise_status(name: str, rc: int) -> None:
    lib = load()
    msg = lib.fmsmo_status_str(rc).decode()
    if rc in (5, 6):
        msg += ": " + lib.fmsmo_last_error().decode()
    raise FmsMoHipError(f"{name} failed with status {rc} ({msg})")


def call(name: str, *args) -> None:
    """Invoke an entry point and raise on a non-zero status."""
    rc = getattr(load(), name)(*args)
    if rc != 0:
        raise_status(name, rc)


def entry(name: str):
    """The bound entry point itself (returns the status), for callers that keep it."""
    return getattr(load(), name)
