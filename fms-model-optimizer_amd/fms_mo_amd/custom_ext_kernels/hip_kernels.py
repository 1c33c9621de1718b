"""HIP replacement of the reference's Triton kernel module
(fms_mo/custom_ext_kernels/triton_kernels.py): same public function, same arguments."""
from __future__ import annotations

import torch

from .. import kernels

DTYPE_I8 = [torch.int8]
DTYPE_F8 = [torch.float8_e4m3fn]
DTYPE_8BIT = DTYPE_I8 + DTYPE_F8


def matmul_chunk_truncate(a, b, c=None, activation="", chunk_trun_bits=0, chunk_size=16,
                          max_acc_bits=32, truncate_then_accumulate=True,
                          cast_output_to_input_dtype=None, clamp_acc_to_dl16=False):
    """D = A.B (+C) with per-K-chunk LSB rounding / MSB clamping of the accumulator.

    a: [M,K] contiguous; b: [K,N] with any strides (a ``W.t()`` view costs nothing);
    dtypes float32/16, bfloat16, float8_e4m3fn or int8.  Argument meaning, chunk-size rules
    (minimum 32 for 8-bit operands else 16, non powers of two fall back to the minimum, chunk 8
    emulated by interleaving zeros) and the output dtype rule follow tl_matmul_chunk_truncate
    (fms_mo/custom_ext_kernels/triton_kernels.py:468-621)."""
    assert a.shape[1] == b.shape[0], "Incompatible dimensions"
    assert a.is_contiguous(), "Matrix A must be contiguous"
    assert a.dtype == b.dtype, "Input dtypes inconsistent"
    allowed = [torch.float, torch.bfloat16, torch.float16] + DTYPE_8BIT
    assert a.dtype in allowed, "Input dtype is not supported"
    if activation not in ("", None):
        raise NotImplementedError("fused activations are not part of the quantized-linear path")
    if cast_output_to_input_dtype is None:
        cast_output_to_input_dtype = a.dtype not in DTYPE_8BIT
    min_chunk = 32 if a.dtype in DTYPE_8BIT else 16
    if chunk_size == 8 and a.dtype in (torch.float8_e4m3fn, torch.int8, torch.float16, torch.bfloat16):
        ratio = min_chunk // chunk_size
        a_p = torch.zeros(a.shape[0], a.shape[1] * ratio, dtype=torch.float32, device=a.device).to(a.dtype)
        a_p[:, ::ratio] = a
        b_p = torch.zeros(b.shape[0] * ratio, b.shape[1], dtype=torch.float32, device=b.device).to(b.dtype)
        b_p[::ratio, :] = b
        a, b, chunk_size = a_p, b_p, min_chunk
    else:
        pow2 = (chunk_size & (chunk_size - 1)) == 0
        chunk_size = max(chunk_size, min_chunk) if pow2 else min_chunk
    if a.dtype not in DTYPE_I8:
        assert chunk_trun_bits < 23, "FP32 accumulator only has 23 mantissa bits"
    c_org_dtype = a.dtype if c is None else c.dtype
    w = b.t()  # [N,K]; row-major already when b is a transposed weight view
    d = kernels.matmul_chunk(a, w, c, chunk_size=chunk_size, chunk_trun_bits=chunk_trun_bits,
                             max_acc_bits=max_acc_bits,
                             truncate_then_accumulate=truncate_then_accumulate,
                             clamp_acc_to_dl16=clamp_acc_to_dl16)
    return d.to(c_org_dtype) if cast_output_to_input_dtype else d


# the name the reference exports
tl_matmul_chunk_truncate = matmul_chunk_truncate
