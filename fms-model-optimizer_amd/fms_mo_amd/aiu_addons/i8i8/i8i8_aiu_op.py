"""``torch.ops.fms_mo.i8i8_aiu`` on the MI355X: the W8A8 linear node of the reference's
accelerator flow (fms_mo/aiu_addons/i8i8/i8i8_aiu_op.py:60-231), same name, schema and argument
meaning, with the arithmetic done by the HIP kernels.

The reference *simulates* the node on CPU/GPU: activations are quantized and dequantized, the
integer weights are dequantized, and a floating-point ``F.linear`` runs on the results.  Here the
node is executed the way the integer hardware it stands for would: the activation codes are
produced by one fused kernel (identical integers to the reference's ``x_int``), multiplied with
the int8 weights on the MFMA units with exact int32 accumulation, and dequantized in the GEMM
epilogue::

    y[m,n] = (sum_k q[m,k] w[n,k] [+ (128 + zp) sum_k w[n,k]]) * (1/scale_x[m]) * (w_cv[n]/127) + b[n]

The SmoothQuant factor cancels between ``x_dq`` and ``w_dq`` and only enters the quantizer.  The
result differs from the simulated one by the fp16/bf16 roundings the simulation applies to
``x_dq`` and ``w_dq`` element by element (about 2^-11 relative per operand).
"""
from __future__ import annotations

import logging

import torch

from ... import _lib as L
from ... import kernels

logger = logging.getLogger(__name__)

_ACT_MODES = {"per_token": L.MS_PER_TOKEN, "per_tensor_symm": L.MS_SYMM,
              "per_tensor_asymm": L.MS_ASYMM}
_LIB = None


def qdata_offsets(weight_quant_type: str, activ_quant_type: str, w_in_feat: int, w_out_feat: int,
                  smoothquant: bool):
    """End offsets of the six pieces of ``qdata`` (w_clip_val, w_clip_valn, a_clip_val,
    a_clip_valn, zero_shift, smoothquant_scale) -- extract_qdata of the reference
    (i8i8_aiu_op.py:128-177)."""
    if weight_quant_type == "per_tensor":
        idx1 = 1
    elif weight_quant_type == "per_channel":
        idx1 = w_out_feat
    else:
        raise NotImplementedError(f"weight quantizantion type {weight_quant_type} is not supported")
    idx2 = 2 * idx1
    idx3, idx4 = idx2 + 1, idx2 + 2
    idx5 = idx4 + (w_out_feat if activ_quant_type == "per_tensor_asymm" else 1)
    idx6 = idx5 + (w_in_feat if smoothquant else 1)
    return idx1, idx2, idx3, idx4, idx5, idx6


def extract_qdata(qdata, weight_quant_type, activ_quant_type, w_in_feat, w_out_feat, smoothquant):
    idx = qdata_offsets(weight_quant_type, activ_quant_type, w_in_feat, w_out_feat, smoothquant)
    if len(qdata) != idx[5]:
        raise ValueError(
            f"qdata length ({len(qdata)}) does not match series of indices for split:{list(idx)}"
        )
    return torch.tensor_split(qdata, idx[:5])


def _pad_k(t: torch.Tensor, k_to: int, value=0):
    return torch.nn.functional.pad(t, (0, k_to - t.shape[-1]), value=value)


def i8i8_aiu(x, weight, bias, qdata, weight_quant_type, activ_quant_type, smoothquant):
    """X -> int8 codes; Y = dequant(X_int . W_int^T) + B.  ``weight`` holds integers (int8, or a
    floating dtype with integer values as in the reference's stored test vectors).  When
    ``smoothquant`` is False the single smoothquant_scale entry of ``qdata`` is taken to be 1, the
    value the reference's module registers for that case (i8i8_aiu_linear.py:139-145)."""
    if activ_quant_type not in _ACT_MODES:
        raise NotImplementedError(
            f"activation quantizantion type {activ_quant_type} is not supported")
    out_feat, in_feat = weight.shape
    idx = qdata_offsets(weight_quant_type, activ_quant_type, in_feat, out_feat, smoothquant)
    if len(qdata) != idx[5]:
        raise ValueError(
            f"qdata length ({len(qdata)}) does not match series of indices for split:{list(idx)}"
        )
    w_cv, sq = qdata[: idx[0]], qdata[idx[4]:]
    x2 = x.reshape(-1, in_feat)
    w8 = weight if weight.dtype == torch.int8 else weight.to(torch.int8)
    smooth = sq if smoothquant else None
    if in_feat % 16:  # the kernels read whole 16-byte groups: zero columns change nothing
        k_to = (in_feat + 15) // 16 * 16
        x2, w8 = _pad_k(x2, k_to), _pad_k(w8, k_to)
        if smooth is not None:
            smooth = _pad_k(smooth, k_to, value=1.0)
    mode = _ACT_MODES[activ_quant_type]
    clip = None if mode == L.MS_PER_TOKEN else qdata[idx[1]:idx[3]]  # {a_clip_val, a_clip_valn}
    q, a_meta = kernels.quant_act_i8_mulscale(x2, mode, clip=clip, smooth=smooth,
                                              meta_dtype=qdata.dtype)
    w_scale = w_cv.to(torch.float32) / 127
    b = bias.to(x.dtype).reshape(-1)
    if b.numel() == 1 and out_feat > 1:
        b = b.expand(out_feat)
    if mode == L.MS_ASYMM:
        b = kernels.zero_shift_bias(w8, w_scale, a_meta, bias=b.contiguous())
        a_scale = a_meta[:1]
    elif mode == L.MS_SYMM:
        a_scale = a_meta[:1]
    else:
        a_scale = a_meta
    y = kernels.gemm_i8_dq(q, w8, a_scale, w_scale, bias=b, out_dtype=x.dtype, exact_ref=False)
    return y.reshape(tuple(x.shape[:-1]) + (out_feat,))


def _i8i8_aiu_fake(x, weight, bias, qdata, weight_quant_type, activ_quant_type, smoothquant):
    outshape = tuple(x.size()[:-1]) + (weight.size(0),)
    return torch.empty(outshape, dtype=x.dtype, device=x.device, requires_grad=False)


def register_aiu_i8i8_op():
    """Register ``fms_mo::i8i8_aiu`` (schema of i8i8_aiu_op.py:74-80) with its shape-only twin,
    so that ``torch.compile`` traces the node without a graph break.  A second call is a no-op
    with a warning, as in the reference (:69-71)."""
    global _LIB
    if hasattr(torch.ops, "fms_mo") and hasattr(torch.ops.fms_mo, "i8i8_aiu"):
        logger.warning("AIU op has already been registered")
        return
    _LIB = torch.library.Library("fms_mo", "FRAGMENT")
    _LIB.define("i8i8_aiu(Tensor x, Tensor weight, Tensor bias, Tensor qdata, "
                "str weight_quant_type, str activ_quant_type, bool smoothquant) -> Tensor")
    _LIB.impl("i8i8_aiu", i8i8_aiu, "CUDA")
    torch.library.register_fake("fms_mo::i8i8_aiu")(_i8i8_aiu_fake)
    logger.info("W8A8 op `i8i8_aiu` has been registered under the `fms_mo` namespace")
