"""``torch.ops.spyre.scaled_bmm`` on the MI355X: the batched per-tensor-scaled FP8 matmul of the
reference's FP8 attention (fms_mo/aiu_addons/fp8/fp8_spyre_op.py:102-155), same name and schema.
The reference loops over the batch calling its CPU ``_scaled_mm`` (dequantize both operands, then
a floating-point matmul); here the e4m3 operands go to the MFMA units in one batched launch with
fp32 accumulation, and ``scale1 * scale2`` is applied in the epilogue."""
from __future__ import annotations

from typing import Optional

import torch

from ... import kernels

_LIB = None


def _pad_last(t, to):
    k = t.shape[-1]
    if k % to == 0:
        return t
    return torch.nn.functional.pad(t.view(torch.uint8), (0, to - k % to)).view(torch.float8_e4m3fn)


def scaled_bmm(mat1, mat2, scale1, scale2, out_dtype: Optional[torch.dtype] = None,
               use_fast_accum: bool = False):
    """mat1 [..., M, K] e4m3, mat2 [..., K, N] e4m3, one scale each -> [..., M, N] of out_dtype
    (fp32 when None, as the reference's CPU kernel).  ``use_fast_accum`` is accepted and ignored:
    accumulation is always fp32."""
    assert mat1.shape[:-2] == mat2.shape[:-2], "batch dimensions must match for mat1 and mat2"
    assert scale1.numel() == 1, "only per-tensor scales supported"
    assert scale2.numel() == 1, "only per-tensor scales supported"
    if mat1.dtype != torch.float8_e4m3fn or mat2.dtype != torch.float8_e4m3fn:
        raise TypeError("scaled_bmm operands must be float8_e4m3fn")
    od = torch.float32 if out_dtype is None else out_dtype
    M, K = mat1.shape[-2:]
    N = mat2.shape[-1]
    a = mat1.reshape(-1, M, K)
    # [.., K, N] -> [batch, N, K] with K contiguous: free for a transposed view of [N, K] storage
    # (Q.K^T), one byte transposition otherwise (P.V)
    b = mat2.transpose(-1, -2).reshape(-1, N, K)
    if b.stride(2) != 1:
        b = b.contiguous()
    a, b = _pad_last(a.contiguous(), 64), _pad_last(b, 64)  # zero bytes are +0.0 in e4m3
    y = kernels.bmm_fp8_dq(a, b, scale1, scale2, bias=None, out_dtype=od)
    return y.reshape(*mat1.shape[:-2], M, N)


def _scaled_bmm_fake(mat1, mat2, scale1, scale2, out_dtype=None, use_fast_accum=False):
    return torch.empty((*mat1.shape[:-2], mat1.shape[-2], mat2.shape[-1]),
                       dtype=torch.float32 if out_dtype is None else out_dtype, device=mat1.device)


def register_spyre_scaled_bmm():
    """Register ``spyre::scaled_bmm`` for GPU tensors with its shape-only twin (no-op when an op of
    that name exists already)."""
    global _LIB
    if hasattr(torch.ops, "spyre") and hasattr(torch.ops.spyre, "scaled_bmm"):
        return
    _LIB = torch.library.Library("spyre", "FRAGMENT")
    _LIB.define("scaled_bmm(Tensor mat1, Tensor mat2, Tensor scale1, Tensor scale2, "
                "ScalarType? out_dtype=None, bool use_fast_accum=False) -> Tensor")
    _LIB.impl("scaled_bmm", scaled_bmm, "CUDA")
    torch.library.register_fake("spyre::scaled_bmm")(_scaled_bmm_fake)
