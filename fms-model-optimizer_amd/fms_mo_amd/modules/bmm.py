"""Quantized batched matmul of attention on the MI355X: ``QBmmINT8Deploy`` with the reference's
class name, ``from_fms_mo`` signature and buffers (fms_mo/modules/bmm.py:607-748).

The reference's forward still *simulates* the integer product (``torch.matmul`` on the int8 codes
cast to fp16, "haven't implemented any batched CUTLASS matmul").  Here both operands are quantized
by one HIP kernel each (m2, stored ``[k, n]``, is written transposed so that its reduction
dimension becomes contiguous), multiplied on the MFMA units with exact int32 accumulation, and
dequantized in the GEMM epilogue together with the zero-point correction of the asymmetric m1.
The correction is summed over the reduction dimension of every batch entry; the reference's
``m2_i8.sum(dim=0)`` is that sum only for a 2-D m2.
"""
from __future__ import annotations

import torch
from torch import nn

from .. import kernels


class QBmmINT8Deploy(nn.Module):
    """m1 is treated as activations (asymmetric), m2 as weights (symmetric)."""

    @classmethod
    def from_fms_mo(cls, fms_mo_qbmm, **kwargs):
        """Build from a trained QBmm-like module: needs ``num_bits_m1`` (7 or 8), ``num_bits_m2``
        (8), ``qm1_mode``, ``quantize_m1`` / ``quantize_m2`` with ``clip_val`` (``clip_valn``) and
        ``num_bits``, optionally ``qcfg`` (bmm.py:619-675)."""
        assert fms_mo_qbmm.num_bits_m1 in [7, 8] and fms_mo_qbmm.num_bits_m2 == 8, \
            "Only support 8bit QBmm!"
        target_device = kwargs.get("target_device", kwargs.get("device", None))
        if target_device is None:
            target_device = next(fms_mo_qbmm.parameters()).device
        qbmm_int = cls()
        qbmm_int.num_bits_m1 = fms_mo_qbmm.num_bits_m1
        qbmm_int.num_bits_m2 = fms_mo_qbmm.num_bits_m2
        qcfg = getattr(fms_mo_qbmm, "qcfg", None)
        qbmm_int.use_int_kernel = True  # the integer kernel is the only path here
        qbmm_int.use_PT_native_Qfunc = qcfg["use_PT_native_Qfunc"] if qcfg else False
        with torch.no_grad():
            Qa, Qw = fms_mo_qbmm.quantize_m1, fms_mo_qbmm.quantize_m2
            cvn_ext_ratio = 128 / 127
            if qbmm_int.num_bits_m1 == 7 or "sym" in fms_mo_qbmm.qm1_mode:
                Qa_cvn = -Qa.clip_val
            else:
                Qa_cvn = getattr(Qa, "clip_valn", torch.zeros_like(Qa.clip_val))
            m1_scale = (Qa.clip_val - Qa_cvn) / (2 ** Qa.num_bits - 1)
            m2_scale = Qw.clip_val * 2 / (2 ** Qw.num_bits - 2)
            qbmm_int.register_buffer("m1_scale", m1_scale.detach().clone())
            qbmm_int.register_buffer("m1_zp", torch.round(-Qa_cvn / m1_scale).to(torch.int))
            qbmm_int.register_buffer("m2_scale", m2_scale.detach().clone())
            qbmm_int.register_buffer("m2_zp", torch.zeros_like(m2_scale, dtype=torch.int))
            qbmm_int.register_buffer("m1_clip_val", Qa.clip_val.detach().clone())
            qbmm_int.register_buffer("m1_clip_valn", Qa_cvn.detach() * cvn_ext_ratio)
            qbmm_int.register_buffer("m2_clip_val", Qw.clip_val.detach().clone())
            qbmm_int.register_buffer("m2_clip_valn", -Qw.clip_val.detach() * cvn_ext_ratio)
        return qbmm_int.to(target_device)

    # host copies of the four scalars and the device metadata of the correction kernel are made
    # once (and again when the buffers change dtype or device), so forward never synchronizes
    def _scalars(self):
        key = (self.m1_scale.dtype, self.m1_scale.device)
        if getattr(self, "_cache_key", None) != key:
            s1, s2 = float(self.m1_scale), float(self.m2_scale)
            z1, z2 = int(self.m1_zp) - 128, int(self.m2_zp)
            dev = self.m1_scale.device
            self._host = (s1, z1, s2, z2)
            self._s1 = torch.tensor([s1], dtype=torch.float32, device=dev)
            self._s2 = torch.tensor([s2], dtype=torch.float32, device=dev)
            self._meta = torch.tensor([s1, -float(z1)], dtype=torch.float32, device=dev)
            self._cache_key = key
        return self._host

    def _get_name(self):
        return "QBmmINT8Deploy"

    def extra_repr(self) -> str:
        return (f"nbits_m1,m2={self.num_bits_m1},{self.num_bits_m2}, "
                f"use_int_kernel={self.use_int_kernel}")

    def quantize_operands(self, m1, m2):
        """int8 codes ready for the batched kernel: m1 as [batch, M, Kp], m2 as [batch, N, Kp]
        (Kp = K rounded up to 64, zero-filled)."""
        s1, z1, s2, z2 = self._scalars()
        sc = self.m1_scale
        T = torch.promote_types(m1.dtype, sc.dtype) if sc.dim() > 0 else m1.dtype
        q1 = kernels.quant_i8_affine(m1, s1, z1, T, transpose=False)
        if m2.stride(-2) == 1 and m2.shape[-2] > 1:  # a transposed view of a [n, k] tensor
            q2 = kernels.quant_i8_affine(m2.transpose(-1, -2), s2, z2, T, transpose=False)
        else:
            q2 = kernels.quant_i8_affine(m2, s2, z2, T, transpose=True)
        return q1, q2

    def forward(self, m1: torch.Tensor, m2: torch.Tensor) -> torch.Tensor:
        """[*, m, k] @ [*, k, n] -> [*, m, n]."""
        if m2.dim() < m1.dim():
            m2 = m2.expand(*m1.shape[:-2], *m2.shape[-2:])
        if m1.shape[:-2] != m2.shape[:-2] or m1.shape[-1] != m2.shape[-2]:
            raise ValueError(f"incompatible operands {tuple(m1.shape)} @ {tuple(m2.shape)}")
        with torch.no_grad():
            q1, q2 = self.quantize_operands(m1, m2)
            B, N, Kp = q2.shape
            corr = kernels.zero_shift_bias(q2.view(B * N, Kp), self._s2, self._meta, bias=None,
                                           offset=0.0)
            y = kernels.bmm_i8_dq(q1, q2, self._s1, self._s2, bias=corr, out_dtype=m1.dtype)
        return y.reshape(*m1.shape[:-1], m2.shape[-1])


QBmm_modules = (QBmmINT8Deploy,)
