"""Quantized-linear modules of the inference path, running on hand-written gfx950 kernels.

Class names, constructor / classmethod signatures, keyword arguments, buffer names and
``_get_name`` strings follow fms_mo/modules/linear.py so that model-surgery code
(``qcfg["mapping"]``, lowering loops, checkpoint code reading ``clip_val`` / ``w_scale`` ...)
keeps working when this package is imported in place of the reference:

  QLinear                 linear.py:51-393     fake-quant training/calibration wrapper; its eval
                                               forward runs as act-quant -> int8 GEMM -> dequant
  QLinearINT8Deploy       linear.py:708-1338   Q -> int8 matmul -> dQ deploy module
  LinearFPxAcc            linear.py:2048-2124  chunked reduced-precision FP accumulation
  QLinearINT8Train        linear.py:2227-2285  chunked int8 forward (forward only here)

There is no CPU path: a forward on CPU tensors raises.
"""
from __future__ import annotations

import json
import logging

import torch
import torch.nn.functional as F
from torch import nn

from .. import _lib as L
from .. import kernels
from ..custom_ext_kernels.hip_kernels import matmul_chunk_truncate as tl_matmul
from ..quant.quantizers import (
    Qbypass,
    QMaxDynamic,
    Qmax,
    SAWB,
    get_activation_quantizer,
    get_weight_quantizer,
    to_fp8,
)

logger = logging.getLogger(__name__)


def prepare_deploy_weights(weight, smoothq_act_scale=None, smoothq_alpha=0.5, w_clip_val=None):
    """Offline weight preparation of the deploy module (from_fms_mo, linear.py:800-871):

    smoothq_scale = clamp(a^alpha / clamp(max_n |W|, 1e-5)^(1-alpha), 1e-5)   if every a_k != 0
    w_scale       = clip_val * 2 / 254          (clip_val defaults to the per-channel abs-max of W*s)
    w_int8        = clamp(round((W * s).t() / w_scale), -127, 127).t()

    Returns (w_int8 [N,K], w_scale [N], smoothq_scale [1,K] or [1])."""
    with torch.no_grad():
        sq = torch.tensor([1.0], device=weight.device, dtype=weight.dtype)
        if smoothq_act_scale is not None and torch.all(smoothq_act_scale != 0).item():
            a = smoothq_act_scale.to(weight.device)
            wmax = weight.abs().max(dim=0, keepdim=True)[0].clamp(min=1e-5)
            alpha = torch.as_tensor(smoothq_alpha, dtype=torch.float32, device=weight.device)
            sq = (a**alpha / wmax ** (1.0 - alpha)).clamp(min=1e-5).to(a.dtype)
        ws = weight * sq
        if w_clip_val is None:
            w_clip_val = ws.abs().amax(dim=1).float()
        # divide by a tensor, not a Python scalar: on the GPU torch turns "/ scalar" into a multiply
        # by the reciprocal, which is one ulp off the IEEE quotient the CPU evaluation gives
        w_scale = w_clip_val * 2 / torch.tensor(254.0, device=w_clip_val.device, dtype=w_clip_val.dtype)
        w_int8 = _quantize_weight_rows(weight, sq, w_scale)
    return w_int8.contiguous(), w_scale, sq


def _quantize_weight_rows(weight, smoothq_scale, w_scale):
    """clamp(round((W * s).t() / w_scale), -127, 127).t() as int8 (from_fms_mo, linear.py:861-866).
    On the GPU this is one pass of the HIP weight quantizer (bit-identical to the torch expression
    for the same operands); weights still on the CPU are converted with the torch expression."""
    N, Kd = weight.shape
    if weight.is_cuda and Kd % 8 == 0 and weight.dtype in (torch.float16, torch.bfloat16, torch.float32):
        sq = smoothq_scale.to(weight.device).reshape(-1)
        smooth = None if sq.numel() == 1 and float(sq[0]) == 1.0 else sq.expand(Kd).contiguous()
        ws = torch.as_tensor(w_scale, device=weight.device).reshape(-1)
        if not ws.is_floating_point():
            ws = ws.float()
        return kernels.quant_weight_i8(weight.detach(), ws, smooth, mode="div")
    w = torch.round((weight * smoothq_scale).t() / w_scale).clamp(-127, 127).t()
    return w.to(torch.int).to(torch.int8)


def _compute_dtype(x_dtype, smooth):
    return x_dtype if smooth is None else torch.promote_types(x_dtype, smooth.dtype)


class QLinear(nn.Linear):
    """Quantized linear wrapper (weights and activations to int8 / fp8 levels, bias untouched).

    Training-mode and calibration forwards evaluate the quantizers with torch ops exactly like
    the reference (they also update ``clip_val`` buffers).  The eval-mode forward of the W8A8
    configuration (``qa_mode`` per-token max, ``qw_mode`` max / maxperCh, 8 bits) computes the same
    fake-quant result as integer arithmetic on the GPU: fused SmoothQuant divide + per-token
    quantizer, int8 MFMA GEMM against the (cached) integer weights, dequantizing epilogue."""

    def __init__(self, in_features, out_features, bias=True, num_bits_feature=32, qa_mode=None,
                 num_bits_weight=32, qw_mode=None, **kwargs):
        super().__init__(in_features, out_features, bias, device=kwargs.get("device", "cuda"))
        qcfg = kwargs.pop("qcfg")
        self.num_bits_feature = num_bits_feature
        self.num_bits_weight = num_bits_weight
        self.qa_mode = qa_mode
        self.qw_mode = qw_mode
        default_calib = "max" if num_bits_feature == 8 else "percentile"
        self.qa_mode_calib = kwargs.get("qa_mode_calib", qcfg.get("qa_mode_calib", default_calib))
        self.qw_mode_calib = kwargs.get("qw_mode_calib", qcfg.get("qw_mode_calib", default_calib))
        self.act_clip_init_val = kwargs.get("act_clip_init_val", qcfg.get("act_clip_init_val", 8.0))
        self.act_clip_init_valn = kwargs.get("act_clip_init_valn", qcfg.get("act_clip_init_valn", -8.0))
        self.w_clip_init_val = kwargs.get("w_clip_init_val", qcfg.get("w_clip_init_val", 1.0))
        self.w_clip_init_valn = kwargs.get("w_clip_init_valn", qcfg.get("w_clip_init_valn", -1.0))
        self.non_neg = kwargs.get("non_neg", qcfg.get("non_neg", False))
        self.align_zero = kwargs.get("align_zero", qcfg.get("align_zero", True))
        self.extend_act_range = kwargs.get("extend_act_range", qcfg.get("extend_act_range", False))
        self.fp8_use_subnormal = kwargs.get("fp8_use_subnormal", qcfg.get("fp8_use_subnormal", False))
        self.register_buffer("calib_counter", torch.tensor(qcfg.get("qmodel_calibration_new", 0)))
        self.register_buffer("num_module_called", torch.tensor(0))
        self.ptqmode = "qout"
        self.W_fp = None
        self.use_PT_native_Qfunc = kwargs.get("use_PT_native_Qfunc", qcfg.get("use_PT_native_Qfunc", False))
        self.perGp = kwargs.get("qgroup", qcfg.get("qgroup", None))
        self.qcfg = qcfg
        self.calib_iterator = []
        self.quantize_feature = Qbypass()
        self.quantize_calib_feature = Qbypass()
        if self.num_bits_feature not in [32, 16]:
            self.quantize_feature = get_activation_quantizer(
                self.qa_mode, nbits=self.num_bits_feature, clip_val=self.act_clip_init_val,
                clip_valn=self.act_clip_init_valn, non_neg=self.non_neg, align_zero=self.align_zero,
                extend_act_range=bool(self.extend_act_range),
                use_PT_native_Qfunc=self.use_PT_native_Qfunc, use_subnormal=self.fp8_use_subnormal)
            if self.calib_counter > 0:
                self.quantize_calib_feature = self.quantize_feature
        self.quantize_weight = Qbypass()
        self.quantize_calib_weight = Qbypass()
        if self.num_bits_weight not in [32, 16]:
            self.quantize_weight = get_weight_quantizer(
                self.qw_mode, nbits=self.num_bits_weight, clip_val=self.w_clip_init_val,
                clip_valn=self.w_clip_init_valn, align_zero=self.align_zero,
                w_shape=self.weight.shape, perGp=self.perGp, use_subnormal=self.fp8_use_subnormal)
            if self.calib_counter > 0:
                self.quantize_calib_weight = self.quantize_weight
        self.mask = None
        self.smoothq = qcfg.get("smoothq", False)
        if self.smoothq:
            self.register_buffer("smoothq_act_scale", torch.zeros(self.weight.shape[1]))
            self.register_buffer("smoothq_alpha",
                                 torch.tensor([qcfg.get("smoothq_alpha", 0.5)], dtype=torch.float32))
        self._wcache = None   # (key, quantized weights, weight scales) of the eval-mode kernel paths
        self._sqcache = None  # (key, SmoothQuant scale or None)
        self._sq_gen = 0

    # -- SmoothQuant ------------------------------------------------------------------------
    def set_act_scale(self, act_scale):
        assert act_scale.shape[0] == self.weight.shape[1], "scale applies to per-channel"
        self.smoothq_act_scale.copy_(act_scale)

    def get_smoothq_scale(self, x):
        if self.smoothq_act_scale.sum().item() == 0.0:
            return torch.tensor([1.0]).to(x.dtype).to(x.device)
        wmax = self.weight.abs().max(dim=0, keepdim=True)[0].clamp(min=1e-5)
        alpha = self.smoothq_alpha.item() if isinstance(self.smoothq_alpha, torch.Tensor) else self.smoothq_alpha
        return (self.smoothq_act_scale.pow(alpha) / wmax.pow(1.0 - alpha)).clamp(min=1e-5).to(x.dtype)

    def _cached_smoothq_scale(self, x):
        """get_smoothq_scale(x), recomputed only when the activation statistics, alpha or the
        weights change: the reference re-reads all of W for a column maximum and synchronizes with
        the host (``.sum().item()``) on every forward (linear.py:345-368)."""
        if not self.smoothq:
            return None
        a, al, w = self.smoothq_act_scale, self.smoothq_alpha, self.weight
        key = (a.data_ptr(), a._version, w.data_ptr(), w._version, x.dtype, x.device,
               (al.data_ptr(), al._version) if torch.is_tensor(al) else al)
        if self._sqcache is None or self._sqcache[0] != key:
            # detached and built outside autograd: the cached tensor serves the kernel paths and
            # no-grad evaluation only (forward() recomputes the scale inside the graph whenever a
            # gradient can flow through it, as the reference does on every call)
            with torch.no_grad():
                scale = self.get_smoothq_scale(x).detach()
            self._sq_gen += 1  # names this scale in the keys of the weight caches
            self._sqcache = (key, scale if scale.numel() > 1 else None)
        return self._sqcache[1]

    # -- forward ----------------------------------------------------------------------------
    def _eval_path_ok(self, x):
        return (not self.training and self.calib_counter <= 0 and self.ptqmode != "fp32_out"
                and self.mask is None and x.is_cuda
                and self.num_bits_feature == 8 and self.num_bits_weight == 8)

    def _int_path_ok(self, x):
        return (self._eval_path_ok(x)
                and isinstance(self.quantize_feature, QMaxDynamic)
                and self.quantize_feature.reduce_dim == -1
                and isinstance(self.quantize_weight, Qmax))

    @staticmethod
    def _fp8_quantizer_ok(q):
        # a q_mode with neither "_sat" nor "_scale" (and no per-channel / per-token flag) makes the
        # reference's quantizer return None (quantizers.py:5423-5488): not a mode to accelerate
        return (isinstance(q, to_fp8) and q.emulate
                and bool(q.perCh or q.perToken or "_sat" in q.q_mode or "_scale" in q.q_mode))

    def _fp8_path_ok(self, x):
        return (self._eval_path_ok(x) and x.shape[-1] % 16 == 0
                and x.dtype in (torch.float16, torch.bfloat16, torch.float32)
                and self._fp8_quantizer_ok(self.quantize_feature)
                and self._fp8_quantizer_ok(self.quantize_weight))

    def _weights_key(self, scale):
        w = self.weight
        return (w._version, w.data_ptr(), w.dtype, None if scale is None else self._sq_gen)

    def _int_weights(self, scale):
        """Integer weights of the fake-quantized W*scale, cached until W, the clip values or the
        SmoothQuant scale change (``scale`` is the cached tensor of _cached_smoothq_scale, so its
        identity stands for the statistics it was computed from).  Levels:
        fake_quantize_per_channel_affine / QmaxSTE, i.e. the stored ``clip_val`` of the weight
        quantizer defines the grid (eval-mode semantics)."""
        qw = self.quantize_weight
        key = self._weights_key(scale) + (qw.clip_val._version, qw.clip_val.data_ptr())
        if self._wcache is not None and self._wcache[0] == key:
            return self._wcache[1], self._wcache[2]
        with torch.no_grad():
            cv = qw.clip_val.to(self.weight.device).float()
            w_scale = cv * 2 / 254
            Kd = self.weight.shape[1]
            if qw.perCh and Kd % 8 == 0 and self.weight.dtype in (torch.float16, torch.bfloat16, torch.float32):
                # torch.fake_quantize_per_channel_affine rounds W.float() * (1 / scale): one pass of
                # the weight-quantizer kernel (SmoothQuant folding W * s in W's dtype included)
                smooth = None if scale is None else scale.reshape(-1).to(self.weight.dtype).contiguous()
                w_int8 = kernels.quant_weight_i8(self.weight.detach(), 1.0 / w_scale, smooth, mode="mul")
            elif qw.perCh:
                ws = self.weight if scale is None else self.weight * scale
                w_int8 = torch.clamp(torch.round(ws.float() * (1.0 / w_scale)[:, None]), -127, 127).to(torch.int8)
            else:
                ws = self.weight if scale is None else self.weight * scale
                u = ws.mul(1 / cv.to(ws.dtype)).clamp(-1, 1).mul(0.5).add(0.5)
                w_int8 = (torch.round(254 * u) - 127).to(torch.int8).contiguous()
        self._wcache = (key, w_int8, w_scale.float().reshape(-1))
        return w_int8, self._wcache[2]

    @staticmethod
    def _fp8_mode(q):
        if q.perCh or q.perToken:
            return L.F8E_PER_ROW
        return L.F8E_SAT if "_sat" in q.q_mode else L.F8E_PER_TENSOR

    def _fp8_weights(self, scale):
        """e4m3 codes of the emulation quantizer's W*scale and their dequantizing factors, cached
        like the integer weights."""
        key = self._weights_key(scale) + ("fp8", self.quantize_weight.q_mode)
        if self._wcache is not None and self._wcache[0] == key:
            return self._wcache[1], self._wcache[2]
        with torch.no_grad():
            ws = self.weight.detach() if scale is None else self.weight.detach() * scale
            _, q, _, inv = kernels.fake_quant_fp8(ws, self._fp8_mode(self.quantize_weight),
                                                  want_values=False, want_codes=True)
            if inv is None:
                inv = torch.ones(1, dtype=torch.float32, device=ws.device)
        self._wcache = (key, q, inv)
        return q, inv

    def forward(self, x):
        scale = self._cached_smoothq_scale(x) if x.is_cuda else None
        if self._int_path_ok(x):
            x2 = x.reshape(-1, x.shape[-1])
            smooth = None if scale is None else scale.reshape(-1)
            q, s = kernels.quant_act_i8_pertoken(x2, smooth, compute_dtype=x.dtype)
            w_int8, w_scale = self._int_weights(scale)
            y = kernels.gemm_i8_dq(q, w_int8, s, w_scale, self.bias, out_dtype=x.dtype, exact_ref=False)
            self.num_module_called += 1
            return y.reshape(tuple(x.shape[:-1]) + (self.out_features,))
        if self._fp8_path_ok(x):
            # FP8 emulation modes: the reference multiplies the fake-quantized tensors with F.linear;
            # here the e4m3 codes go through the FP8 MFMA GEMM and the two reciprocal scales are
            # applied to the fp32 accumulator
            x2 = x.reshape(-1, x.shape[-1])
            if scale is not None:
                x2 = x2 / scale
            _, q, _, inv = kernels.fake_quant_fp8(x2, self._fp8_mode(self.quantize_feature),
                                                  want_values=False, want_codes=True)
            if inv is None:
                inv = torch.ones(1, dtype=torch.float32, device=x.device)
            wq, w_inv = self._fp8_weights(scale)
            y = kernels.gemm_fp8_dq(q, wq, inv, w_inv, self.bias, out_dtype=x.dtype)
            self.num_module_called += 1
            return y.reshape(tuple(x.shape[:-1]) + (self.out_features,))
        if not x.is_cuda:
            raise RuntimeError("fms_mo_amd.QLinear runs on an AMD GPU only; there is no CPU path")
        if self.smoothq and torch.is_grad_enabled() and (self.training or self.weight.requires_grad):
            # a gradient can reach the weights through the scale: build it in this call's graph
            # (a cached tensor would be backpropagated through twice under gradient accumulation)
            scale = self.get_smoothq_scale(x)
        elif scale is None:
            scale = torch.tensor([1.0]).to(x.dtype).to(x.device)
        # training / calibration / other quantizer modes: quantizer modules evaluated with torch ops
        if self.calib_counter > 0:
            with torch.no_grad():
                qinput = self.quantize_calib_feature(x / scale)
                qweight = self.quantize_calib_weight(self.weight * scale)
            self.calib_counter -= 1
            if self.calib_counter == 0:
                self.quantize_calib_feature = None
                self.quantize_calib_weight = None
        elif self.ptqmode == "fp32_out":
            if self.W_fp is None:
                self.W_fp = self.weight.detach().clone()
                self.weight.requires_grad = True
            return F.linear(x, self.W_fp, self.bias)
        else:
            qinput = self.quantize_feature(x / scale).to(x.dtype)
            qweight = self.quantize_weight(self.weight * scale).to(self.weight.dtype)
        output = F.linear(qinput, qweight, self.bias)
        self.num_module_called += 1
        return output

    def __repr__(self):
        s = ",QntzerW,A="
        s += "" if self.num_bits_weight == 32 else f"{self.quantize_weight.__repr__().split('(')[0]},"
        s += "" if self.num_bits_feature == 32 else f"{self.quantize_feature.__repr__().split('(')[0]}"
        return (f"{self.__class__.__name__}({self.in_features},{self.out_features}, "
                f"Nbits_W,A={self.num_bits_weight},{self.num_bits_feature}{s})")


class QLinearINT8Deploy(nn.Linear):
    """Deploy-time W8A8 linear: quantize -> int8 matmul (int32 accumulate) -> dequantize.

    Buffers: ``weight`` (int8 [N,K]), ``input_scale``, ``input_zp``, ``w_scale``, ``w_zp``,
    ``smoothq_scale``, ``corr_term``, ``bias`` -- the names the reference registers
    (linear.py:843-911)."""

    @classmethod
    def from_fms_mo(cls, fms_mo_qlinear, **kwargs):
        """Convert a QLinear.  Keyword arguments as in the reference: use_int_kernel
        ('cutlass' | 'triton' | True all select the HIP kernels, False the FP emulation),
        use_PT_native_Qfunc, use_dynamic_max_act_Qfunc (-1 | -2 | 1..64 | False), max_acc_bits,
        truncate_lsb, chunk_size, recalc_clipvals, target_device."""
        assert all(getattr(fms_mo_qlinear, a) in [4, 8] for a in ["num_bits_feature", "num_bits_weight"]), \
            "Please check nbits setting!"
        tar_dev = kwargs.get("target_device", kwargs.get("device", next(fms_mo_qlinear.parameters()).device))
        w_dtype = fms_mo_qlinear.weight.dtype
        # All offline arithmetic runs where the source module lives (the reference requires source
        # and target on one device; converting a CPU module for a GPU target also works here and
        # gives the CPU roundings of pow / division for the offline scales).
        src_dev = fms_mo_qlinear.weight.device
        m = cls(fms_mo_qlinear.in_features, fms_mo_qlinear.out_features,
                bias=fms_mo_qlinear.bias is not None, device="meta")
        qcfg = getattr(fms_mo_qlinear, "qcfg", {})
        m.use_int_kernel = kwargs.get("use_int_kernel", qcfg.get("use_int_kernel", "cutlass"))
        m.usePTnativeQfunc = kwargs.get("use_PT_native_Qfunc", False)
        m.useDynMaxQfunc = kwargs.get("use_dynamic_max_act_Qfunc", False)
        m.useSymAct = "sym" in fms_mo_qlinear.qa_mode or fms_mo_qlinear.qa_mode in ["pertokenmax", "max"]
        m.max_acc_bits = kwargs.get("max_acc_bits", 32)
        m.accminmax = (-(1 << (m.max_acc_bits - 1)), (1 << (m.max_acc_bits - 1)) - 1)
        m.truncate_lsb = kwargs.get("truncate_lsb", 0)
        m.chunk_size = kwargs.get("chunk_size", 100000)
        m.acc_dtype = torch.float16
        m.nbits_a = fms_mo_qlinear.num_bits_feature
        m.nbits_w = fms_mo_qlinear.num_bits_weight
        w_levels = 2**m.nbits_w - 2
        a_levels = 2**m.nbits_a - 1 - m.useSymAct
        with torch.no_grad():
            Qa, Qw = fms_mo_qlinear.quantize_feature, fms_mo_qlinear.quantize_weight
            if kwargs.get("recalc_clipvals", True):
                Qw(fms_mo_qlinear.weight)
            w_cv = Qw.clip_val
            a_cv = getattr(Qa, "clip_val", torch.tensor(8.0, device=src_dev))
            a_cvn = getattr(Qa, "clip_valn", torch.tensor(-8.0, device=src_dev))
            m.cvs = [a_cv, a_cvn, w_cv]
            smoothq_scale = torch.tensor([1.0], device=src_dev, dtype=w_dtype)
            if getattr(fms_mo_qlinear, "smoothq", False):
                a_s = fms_mo_qlinear.smoothq_act_scale
                w_s = fms_mo_qlinear.weight.abs().max(dim=0, keepdim=True)[0].clamp(min=1e-5)
                alpha = fms_mo_qlinear.smoothq_alpha
                if torch.all(a_s != 0).item():
                    smoothq_scale = (a_s**alpha / w_s ** (1.0 - alpha)).clamp(min=1e-5).to(a_s.dtype)
            input_scale = torch.tensor(1.0, device=src_dev)
            # tensor divisor: keeps the IEEE quotient on the GPU as well (see prepare_deploy_weights)
            w_scale = w_cv * 2 / torch.tensor(float(w_levels), device=w_cv.device, dtype=w_cv.dtype)
            m.use_fake_zero_shift = False
            if m.useDynMaxQfunc in [-1, -2]:
                input_zero_point = torch.tensor(128 - m.useSymAct, device=src_dev)
            elif 0 < m.useDynMaxQfunc < 65:
                m.use_fake_zero_shift = True
                input_zero_point = torch.tensor(m.useDynMaxQfunc, device=src_dev)
            elif m.usePTnativeQfunc:
                input_scale = torch.tensor([(a_cv - a_cvn) / a_levels], device=src_dev)
                input_zero_point = torch.round(-a_cvn / input_scale)
            else:
                quant_scale = a_levels / torch.tensor([a_cv - a_cvn], device=src_dev)
                quant_stepsize = 1.0 / quant_scale
                quant_zero_point = torch.round(a_cvn * quant_scale)
                input_scale = quant_stepsize
                input_zero_point = -quant_zero_point
                w_scale = 1.0 / (w_levels / (w_cv * 2))
                m.register_buffer("quant_scale", quant_scale)
                m.register_buffer("quant_stepsize", quant_stepsize)
                m.register_buffer("quant_zero_point", quant_zero_point)
            w_zp = torch.zeros_like(w_scale, dtype=torch.int)
            input_zero_point = input_zero_point.to(torch.int)
            m.register_buffer("input_scale", input_scale)
            m.register_buffer("input_zp", input_zero_point)
            m.register_buffer("w_scale", w_scale)
            m.register_buffer("w_zp", w_zp)
            m.register_buffer("smoothq_scale", smoothq_scale)
            if isinstance(Qw, SAWB):
                # the quantizer's own integer output (linear.py:859-861); it stays switched to codes
                Qw.dequantize = False
                w_int8 = Qw(fms_mo_qlinear.weight.float() * smoothq_scale).to(torch.int)
            else:
                w_int8 = _quantize_weight_rows(fms_mo_qlinear.weight, smoothq_scale, w_scale).to(torch.int)
            m.weight = nn.Parameter(w_int8.to(torch.int8), requires_grad=False)
            if m.useSymAct:
                corr_term_int = 0
                if m.use_fake_zero_shift:
                    corr_term_int = input_zero_point * (w_int8.sum(dim=1))
            else:
                corr_term_int = (input_zero_point - 128) * (w_int8.sum(dim=1))
            m.register_buffer("corr_term", corr_term_int * w_scale.float() * input_scale.float())
            m.org_model_has_bias = fms_mo_qlinear.bias is not None
            new_bias = (fms_mo_qlinear.bias.float() - m.corr_term) if m.org_model_has_bias else -m.corr_term
            if m.use_fake_zero_shift:
                new_bias += m.corr_term
            delattr(m, "bias")
            m.register_buffer("bias", new_bias.to(w_dtype))
        m.set_matmul_op()
        return m.to(tar_dev)

    @classmethod
    def from_torch_iW(cls, nnlin_iW, prec, a_cv, a_cvn, w_cv, zero_shift, **kwargs):
        """Build the module from an nn.Linear that already holds integer weights (linear.py:923-1023)."""
        assert prec == "int8", "Only support INT8 for now."
        target_device = kwargs.get("target_device", kwargs.get("device", next(nnlin_iW.parameters()).device))
        m = cls(nnlin_iW.in_features, nnlin_iW.out_features, bias=nnlin_iW.bias is not None, device=target_device)
        m.nbits_a = m.nbits_w = 8
        m.acc_dtype = kwargs.get("acc_dtype", torch.float)
        m.usePTnativeQfunc = kwargs.get("use_PT_native_Qfunc", True)
        m.use_int_kernel = kwargs.get("use_int_kernel", "triton")
        m.useDynMaxQfunc = False
        m.useSymAct = False
        m.use_fake_zero_shift = False
        m.weight = nn.Parameter(nnlin_iW.weight.to(torch.int8), requires_grad=False)
        m.max_acc_bits = kwargs.get("max_acc_bits", 32)
        m.accminmax = (-(1 << (m.max_acc_bits - 1)), (1 << (m.max_acc_bits - 1)) - 1)
        m.truncate_lsb = kwargs.get("truncate_lsb", False)
        m.chunk_size = kwargs.get("chunk_size", 100000)
        with torch.no_grad():
            if m.usePTnativeQfunc:
                input_scale = torch.Tensor([(a_cv - a_cvn) / (2**m.nbits_a - 1)])
                input_zero_point = torch.round(-a_cvn / input_scale).to(torch.int)
                w_scale = torch.Tensor([w_cv * 2 / (2**m.nbits_w - 2)])
            else:
                quant_scale = (2**m.nbits_a - 1) / torch.Tensor([a_cv - a_cvn])
                quant_stepsize = 1.0 / quant_scale
                quant_zero_point = torch.round(a_cvn * quant_scale)
                input_scale = quant_stepsize
                input_zero_point = -quant_zero_point
                w_scale = 1.0 / ((2**m.nbits_a - 2) / torch.Tensor([w_cv * 2]))
                m.register_buffer("quant_scale", quant_scale)
                m.register_buffer("quant_stepsize", quant_stepsize)
                m.register_buffer("quant_zero_point", quant_zero_point)
            m.register_buffer("input_scale", input_scale)
            m.register_buffer("input_zp", input_zero_point)
            m.register_buffer("w_scale", w_scale)
            m.register_buffer("w_zp", torch.zeros_like(w_scale, dtype=torch.int))
            m.register_buffer("smoothq_scale", torch.tensor([1.0]))
            m.cvs = [a_cv, a_cvn, w_cv]
            zero_s = torch.Tensor(json.loads(zero_shift)) if isinstance(zero_shift, str) else torch.Tensor([zero_shift])
            corr_term = (input_zero_point - 128) * zero_s * w_scale * input_scale
            m.register_buffer("corr_term", corr_term)
            m.register_buffer("zero_shift", zero_s)
            if nnlin_iW.bias is not None:
                m.bias = nn.Parameter((nnlin_iW.bias - corr_term.to(nnlin_iW.bias.device)).to(m.acc_dtype),
                                      requires_grad=False)
                m.org_mod_has_bias = True
            else:
                delattr(m, "bias")
                m.register_buffer("bias", -corr_term.to(m.acc_dtype))
                m.org_mod_has_bias = False
        m.set_matmul_op()
        return m.to(target_device)

    # -- activation quantizers (device kernels) ----------------------------------------------
    def _static_params(self, x_dtype):
        """Host copies of the static quantizer's parameters and the dtype torch would evaluate the
        formula in, refreshed when a buffer changes (reading them costs a host sync)."""
        tensors = [self.input_scale, self.input_zp]
        fmo = not self.usePTnativeQfunc and hasattr(self, "quant_stepsize")
        if fmo:
            tensors += [self.quant_stepsize, self.quant_zero_point]
            tensors += [t for t in self.cvs[:2] if torch.is_tensor(t)]
        key = (x_dtype,) + tuple((t.data_ptr(), t._version, t.dtype) for t in tensors)
        if getattr(self, "_sp_key", None) != key:
            probe = torch.empty((1, 1), dtype=x_dtype)
            p = {"scale": float(self.input_scale.reshape(-1)[0]), "zp": int(self.input_zp.reshape(-1)[0]),
                 "T": torch.result_type(probe, self.input_scale.cpu())}
            if fmo:
                cvn, cv = (t.detach().cpu() if torch.is_tensor(t) else torch.tensor(float(t)) for t in
                           (self.cvs[1], self.cvs[0]))
                clamped = probe.clamp(cvn, cv)                     # torch's own promotion rules
                quot = clamped / self.quant_stepsize.cpu() - self.quant_zero_point.cpu()
                p.update(T=quot.dtype, lo=float(cvn.to(clamped.dtype).reshape(-1)[0]),
                         hi=float(cv.to(clamped.dtype).reshape(-1)[0]),
                         step=float(self.quant_stepsize.reshape(-1)[0]),
                         qzp=float(self.quant_zero_point.reshape(-1)[0]))
            self._sp_key, self._sp = key, p
        return self._sp

    def qa_raw_qfunc(self, x):
        """clamp(round(x / input_scale + input_zp - 128 + sym), -128, 127) in the dtype torch
        promotes x and ``input_scale`` to (linear.py:1061-1071)."""
        p = self._static_params(x.dtype)
        if p["T"] == torch.float32:
            return kernels.quant_act_i8_static(x, p["scale"], p["zp"], int(self.useSymAct))
        return kernels.quant_act_i8_static_t(x, L.SQ_RAW, p["T"], p["scale"], p["zp"], int(self.useSymAct))

    def qa_pt_quant_func(self, x):
        """torch.quantize_per_tensor(x.float(), scale, zp - 128 + sym) arithmetic (linear.py:1043-1059)."""
        p = self._static_params(x.dtype)
        return kernels.quant_act_i8_static(x, p["scale"], p["zp"], int(self.useSymAct) | 2)

    qa_pt_qfunc_wrapped = qa_pt_quant_func

    def qa_fmo_mo_qfunc(self, x):
        """round(clamp(x, cvn, cv) / stepsize - zero_point) - (128 - sym): clamp-then-round with the
        fms_mo formula (linear.py:1073-1083), in the dtype torch's promotion gives the chain."""
        p = self._static_params(x.dtype)
        return kernels.quant_act_i8_static_t(x, L.SQ_FMO, p["T"], p["step"], p["qzp"], int(self.useSymAct),
                                             p["lo"], p["hi"])

    def qa_dynamic_max_qfunc(self, x):
        """Dynamic abs-max quantizer per token (dim -1) or per input channel over the tokens
        (dim -2); stores ``input_scale`` ([M,1] / [1,K]) and ``cvs[0:2]`` like the reference
        (linear.py:1085-1100)."""
        if self.useDynMaxQfunc == -2:
            q, s, col_amax = kernels.quant_act_i8_dynamic(x, True, 2 ** (self.nbits_a - 1) - 1,
                                                          want_amax=True)
            s = s.reshape(1, -1).to(x.dtype)
            amax = col_amax.reshape(1, -1).to(x.dtype)      # the abs-max itself, as the reference stores
        else:
            q, s = kernels.quant_act_i8_pertoken(x, None, compute_dtype=x.dtype)
            s = s.reshape(-1, 1)
            # the per-token kernel hands over scales only: scale * 127 is the row maximum up to the
            # scale's rounding (and 1e-5 where the clamp of a tiny row acted)
            amax = s * 127
        self.input_scale = s
        self.cvs[0], self.cvs[1] = amax, -amax
        return q

    def qa_dyn_max_fake_zero_shift(self, x):
        """One dynamic scale amax / (127 - zp) for the whole tensor, codes shifted by zp
        (linear.py:1102-1113).  The zero point is a construction-time constant."""
        zp = self.input_zp
        key = (zp.data_ptr(), zp._version)
        if getattr(self, "_fzs_key", None) != key:      # reading the buffer costs a host sync
            self._fzs_key, self._fzs_zp = key, int(zp)
        levels = 2 ** (self.nbits_a - 1) - 1 - self._fzs_zp
        q, s, col_amax = kernels.quant_act_i8_dynamic(x, False, levels, self._fzs_zp, want_amax=True)
        self.input_scale = s.reshape(()).to(x.dtype)
        amax = col_amax.max().to(x.dtype)
        self.cvs[0], self.cvs[1] = amax, -amax
        return q

    # -- matmul + dequant ----------------------------------------------------------------------
    def _quantize(self, m1):
        if self.useDynMaxQfunc in [-1, -2]:
            return self.qa_dynamic_max_qfunc(m1)
        if self.use_fake_zero_shift:
            return self.qa_dyn_max_fake_zero_shift(m1)
        if self.usePTnativeQfunc:
            return self.qa_raw_qfunc(m1)
        return self.qa_fmo_mo_qfunc(m1)

    def iaddmm_int(self, bias, m1, m2):
        """Q(m1) -> int matmul -> dQ (+bias).  m2 is ``W.t()`` ([K,N] view of the [N,K] weight).

        Three cases, as in the reference (linear.py:1115-1188):
          * K > chunk_size and kernel != 'triton': its serial PyTorch chunk loop (clamp to
            max_acc_bits, (p + 2^(t-1)) >> t, int32 accumulate, fp32 scales) -- one launch of
            the chunked int8 kernel here;
          * kernel == 'triton' with LSB truncation: imatmul is the chunked kernel (chunk_size /
            truncate_lsb only, max_acc_bits is not forwarded there either), then the fp16-scale
            epilogue;
          * otherwise the int8 MFMA GEMM with the fused fp16-scale epilogue."""
        w = m2.t()
        m1 = self._quantize(m1)
        K = m1.shape[1]
        if K > self.chunk_size and self.use_int_kernel != "triton":
            cs = int(self.chunk_size)
            if cs >= 32 and not cs & (cs - 1):
                # the accumulator is 2^t * (the reference's shifted one); (2^t a) * s == a * (2^t s) exactly
                if (torch.result_type(self.input_scale, self.w_scale) == torch.float32
                        and self.acc_dtype in (torch.float16, torch.bfloat16, torch.float32)):
                    # fp32 scale product, multiply and add rounded separately, cast to acc_dtype: the
                    # final expression of the reference's loop inside the kernel's epilogue (one launch)
                    a_scale, w_scale = self.input_scale.float().reshape(-1), self._w_scale_f32()
                    if self.useDynMaxQfunc == -2:      # [1,K] scales against [M,N] (K == N): a column scale
                        if a_scale.numel() != w.shape[0]:
                            raise RuntimeError("per-channel activation scales need in_features == out_features "
                                               "(the reference's [1,K] scale broadcasts against [M,N])")
                        w_scale = a_scale * w_scale
                        a_scale = torch.ones(1, dtype=torch.float32, device=m1.device)
                    return kernels.matmul_chunk_dq(m1, w, a_scale, w_scale, bias, L.EPI_F32_MULADD, self.acc_dtype,
                                                   chunk_size=cs, chunk_trun_bits=int(self.truncate_lsb),
                                                   max_acc_bits=self.max_acc_bits)
                # 16-bit scale buffers on both sides: torch evaluates the chain in that dtype
                acc = kernels.matmul_chunk(m1, w, None, chunk_size=cs, chunk_trun_bits=int(self.truncate_lsb),
                                           max_acc_bits=self.max_acc_bits)
                return (acc * (self.input_scale * self.w_scale) + bias).to(self.acc_dtype)
            # any other chunk size (ragged last chunk included): the reference's serial loop, one
            # exact int32 GEMM per chunk
            acc = torch.zeros((m1.shape[0], w.shape[0]), dtype=torch.int, device=m1.device)
            t = int(self.truncate_lsb)
            for k0 in range(0, K, cs):
                a_c, w_c = m1[:, k0:k0 + cs], w[:, k0:k0 + cs]
                # the GEMM wants 16-byte aligned rows: copy the slices out, zero-padded
                pad = (-a_c.shape[1]) % 16
                a_c, w_c = F.pad(a_c, (0, pad)).contiguous(), F.pad(w_c, (0, pad)).contiguous()
                p = kernels.gemm_i8_i32(a_c, w_c)
                if self.max_acc_bits < 32:
                    p = p.clamp(self.accminmax[0], self.accminmax[1])
                if t > 0:
                    p = torch.bitwise_right_shift(p + (1 << (t - 1)), t)
                acc += p
            return (acc * ((1 << t) * self.input_scale * self.w_scale) + bias).to(self.acc_dtype)
        updated_bias = bias
        if self.use_fake_zero_shift:
            updated_bias = bias - self.input_scale * self.corr_term
        if self.use_int_kernel == "triton" and self.truncate_lsb > 0:
            cs = int(self.chunk_size)
            cs = max(cs, 32) if cs & (cs - 1) == 0 else 32          # tl_matmul's chunk-size rule for int8
            if self.useDynMaxQfunc != -2 and self.acc_dtype in (torch.float16, torch.float32) and cs >= 32:
                # imatmul = the chunked kernel, then the fp16-scale epilogue: one launch
                return kernels.matmul_chunk_dq(m1, w, self.input_scale.float().reshape(-1), self._w_scale_f32(),
                                               updated_bias, L.EPI_REF_F16, self.acc_dtype, chunk_size=cs,
                                               chunk_trun_bits=int(self.truncate_lsb))
            imm_out = tl_matmul(m1, m2, chunk_trun_bits=int(self.truncate_lsb), chunk_size=int(self.chunk_size))
            return (imm_out.float() * (self.input_scale * self.w_scale).to(torch.float16)
                    + updated_bias).to(self.acc_dtype)
        # fused epilogue: acc.float() * f16(input_scale * w_scale) + bias, rounded once to the fp16
        # accumulator dtype of from_fms_mo or left in fp32 for any other (from_torch_iW: fp32)
        ref16 = self.acc_dtype == torch.float16
        a_scale = self.input_scale.float().reshape(-1)
        w_scale = self._w_scale_f32()
        if self.useDynMaxQfunc == -2:
            # per-input-channel scales [1,K] broadcast against the [M,N] accumulator (K == N): the
            # product input_scale[n] * w_scale[n] goes in as the column scale
            if a_scale.numel() != w.shape[0]:
                raise RuntimeError("per-channel activation scales need in_features == out_features "
                                   "(the reference's [1,K] scale broadcasts against [M,N])")
            w_scale = a_scale * w_scale
            a_scale = torch.ones(1, dtype=torch.float32, device=m1.device)
        y = kernels.gemm_i8_dq(m1, w, a_scale, w_scale, updated_bias,
                               out_dtype=torch.float16 if ref16 else torch.float32, exact_ref=True)
        return y if ref16 else y.to(self.acc_dtype)

    def iaddmm_FP(self, bias, m1, m2):
        """The reference's non-integer emulation (torch.matmul on dequantized operands)."""
        x_dtype = m1.dtype
        if self.useDynMaxQfunc in [-1, -2]:
            m1 = self.qa_dynamic_max_qfunc(m1)
        elif self.usePTnativeQfunc:
            m1 = self.qa_raw_qfunc(m1)
        else:
            m1 = self.qa_fmo_mo_qfunc(m1)
        # the kernels hand the dynamic scale over as fp32 holding a value of x's dtype
        return torch.matmul(m1 * self.input_scale.to(x_dtype), m2 * self.w_scale) + bias

    def set_matmul_op(self):
        from ..custom_ext_kernels.utils import imatmul_ops_reg

        imatmul_ops_reg(self.use_int_kernel)
        self.imatmul = torch.ops.fms_mo.imatmul
        self.iaddmm = self.iaddmm_int if self.use_int_kernel else self.iaddmm_FP

    def _get_name(self):
        return "QLinear_INT8"

    def extra_repr(self) -> str:
        s = (f"in={self.in_features}, out={self.out_features}, bias={self.bias is not None}, "
             f"int_kernel={self.use_int_kernel}")
        if self.truncate_lsb > 0 or self.max_acc_bits < 32:
            s += f", acc_bits={self.max_acc_bits}, trun_lsb={self.truncate_lsb}"
        return s

    def __getstate__(self):
        state = self.__dict__.copy()
        state.pop("imatmul", None)
        state.pop("iaddmm", None)
        return state

    def __setstate__(self, state):
        self.__dict__.update(state)
        self.set_matmul_op()

    def _smoothq_active(self):
        """The reference divides by ``smoothq_scale`` only if EVERY element differs from 1
        (linear.py:1331); the answer is cached until the buffer changes (it costs a host sync)."""
        sq = self.smoothq_scale
        if torch.compiler.is_compiling():
            # the answer of the last eager call (the module has to run eagerly once before it is
            # compiled, as it has to before it is captured in a graph)
            return self._sq_on
        key = (sq.data_ptr(), sq._version)
        if getattr(self, "_sq_key", None) != key:
            self._sq_key = key
            self._sq_on = bool(torch.all(sq != 1).item())
        return self._sq_on

    def _w_scale_f32(self):
        """``w_scale`` as the contiguous fp32 vector the kernels read, converted once (the buffer
        is fp16 in a deployed ``.half()`` module; converting it in every forward costs a launch)."""
        ws = self.w_scale
        if torch.compiler.is_compiling():
            return ws.float().reshape(-1)
        key = (ws.data_ptr(), ws._version, ws.dtype)
        if getattr(self, "_ws_key", None) != key:
            self._ws_key = key
            self._ws_f32 = ws.detach().float().reshape(-1).contiguous()
        return self._ws_f32

    def _set_input_scale(self, s):
        """Replace the ``input_scale`` buffer (the reference assigns it in every dynamic forward,
        linear.py:1074-1082).  Eagerly the entry of the buffer table is swapped directly:
        ``Module.__setattr__`` spends several microseconds per call on its checks, as much as a
        decode kernel runs."""
        if torch.compiler.is_compiling() or "input_scale" not in self._buffers:
            self.input_scale = s
        else:
            self._buffers["input_scale"] = s

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        # (the reference runs this forward under torch.no_grad; the kernel paths below create their
        # outputs outside autograd anyway, and the torch-op branch enters no_grad itself -- an eager
        # decode step is bound by what the host does per call, so nothing is done twice here)
        org_dtype = x.dtype
        K = x.shape[-1]
        two_d = x.dim() == 2
        x2 = x if two_d else x.reshape(-1, K)
        if not x2.is_cuda:
            raise RuntimeError("fms_mo_amd.QLinearINT8Deploy runs on an AMD GPU only; there is no CPU path")
        use_sq = self._smoothq_active()
        plain = (self.useDynMaxQfunc == -1 and self.use_int_kernel
                 and not (K > self.chunk_size or self.truncate_lsb > 0)
                 and not getattr(self, "use_fake_zero_shift", False))
        sq = self.smoothq_scale.reshape(-1) if use_sq else None
        if plain and (sq is None or sq.numel() == K) and kernels.decode_linear_ok(x2, sq, K):
            # decode step of a few tokens: quantizer and weight-streaming matmul in one launch
            y, s = kernels.decode_linear_i8(x2, self.weight, self._w_scale_f32(), self.bias, sq,
                                            out_dtype=torch.float16, exact_ref=True)
            self._set_input_scale(s.reshape(-1, 1))
        elif plain and use_sq and sq.numel() == K:
            # SmoothQuant divide inside the quantizer kernel
            q, s = kernels.quant_act_i8_pertoken(x2, sq, compute_dtype=_compute_dtype(x2.dtype, sq))
            self._set_input_scale(s.reshape(-1, 1))
            y = kernels.gemm_i8_dq(q, self.weight, s, self._w_scale_f32(), self.bias,
                                   out_dtype=torch.float16, exact_ref=True)
        else:
            with torch.no_grad():
                if use_sq:
                    x2 = x2 / self.smoothq_scale
                y = self.iaddmm(self.bias, x2, self.weight.t())
        if y.dtype != self.acc_dtype:
            y = y.to(self.acc_dtype)
        if not two_d:
            y = y.reshape(tuple(x.shape[:-1]) + (y.shape[-1],))
        return y if y.dtype == org_dtype else y.to(org_dtype)


class LinearFPxAcc(torch.nn.Linear):
    """Linear layer whose FP32 accumulator is LSB-rounded after every K-chunk (forward only)."""

    @classmethod
    def from_nn(cls, nnlin, trun_bits=0, **kwargs):
        target_device = kwargs.get("target_device", kwargs.get("device", next(nnlin.parameters()).device))
        m = cls(nnlin.in_features, nnlin.out_features, bias=nnlin.bias is not None, device="meta")
        m.weight = nnlin.weight
        m.trun_bits = trun_bits
        m.chunk_size = kwargs.get("chunk_size", False)
        m.fp8_dyn = kwargs.get("dynamic_fp8", False)
        m.clamp_acc_to_dl16 = kwargs.get("clamp_acc_to_dl16", False)
        if nnlin.bias is not None:
            m.bias = nnlin.bias
        return m.to(target_device)

    def forward(self, inputs):
        x = inputs
        assert x.dtype in [torch.float, torch.bfloat16, torch.float16]
        org_dtype = x.dtype
        out_shape = x.shape[:-1] + (self.weight.shape[0],)
        x = x.reshape(-1, x.shape[-1])
        weight = self.weight.detach()
        # tl_matmul's chunk-size rule for the tensors the reference hands it: the FP8 codes travel as
        # fp32 tensors there (minimum chunk 16, like 16-bit and fp32 operands)
        cs = int(self.chunk_size)
        # (a chunk of 8 sixteen-bit elements is emulated by the reference with interleaved zeros)
        pad8 = cs == 8 and not self.fp8_dyn and x.dtype in (torch.float16, torch.bfloat16)
        if not pad8:
            cs = max(cs, 16) if cs & (cs - 1) == 0 else 16
        with torch.no_grad():
            if self.fp8_dyn:
                variant = L.FP8_FPXACC_DL8 if self.clamp_acc_to_dl16 else L.FP8_FPXACC
                per_tensor = self.fp8_dyn == "per_tensor"
                # scales in the original dtype like the reference (the kernels hand them over as fp32
                # holding those values); per tensor: column abs-max and quantizer, nothing read back
                xq, xs = kernels.quant_act_fp8_dynamic(x, variant, per_tensor, 1e-5, True)
                wq, wsc = kernels.quant_act_fp8_dynamic(weight, variant, per_tensor, 1e-5, True)
                if cs < 32:
                    # a chunk of 16 FP8-valued elements: every e4m3 value is an fp16 value, and the
                    # fp16 matrix instructions take 16 elements per step
                    xq, wq = xq.to(torch.float16), wq.to(torch.float16)
                a_op, w_op = xq, wq
            else:
                xs = wsc = torch.ones(1, dtype=torch.float32, device=x.device)
                a_op, w_op = x.contiguous(), weight.to(x.dtype)
            if pad8:
                out = tl_matmul(a_op, w_op.t(), chunk_trun_bits=self.trun_bits, chunk_size=8,
                                clamp_acc_to_dl16=self.clamp_acc_to_dl16).to(org_dtype).reshape(out_shape)
                if self.bias is not None:
                    out = out + self.bias.to(org_dtype)
                return out
            # descale, cast to the original dtype, add the bias there: the kernel's epilogue
            out = kernels.matmul_chunk_dq(a_op, w_op, xs, wsc, self.bias, L.EPI_SEQ_OUT, org_dtype, chunk_size=cs,
                                          chunk_trun_bits=self.trun_bits, clamp_acc_to_dl16=self.clamp_acc_to_dl16)
        return out.reshape(out_shape)

    def extra_repr(self) -> str:
        s = f"{self.in_features},{self.out_features}"
        if self.bias is not None:
            s += f",bias={self.bias is not None}"
        if self.trun_bits > 0:
            s += f",trun_bits={self.trun_bits}"
        if self.fp8_dyn:
            s += f",fp8_dyn={self.fp8_dyn}"
        if self.clamp_acc_to_dl16:
            s += ",use_DL16_acc"
        return s + f",chunk_size={self.chunk_size}"


class QLinearINT8Train(torch.nn.Linear):
    """INT8 forward with chunked accumulation (MSB clamp / LSB rounding), dynamic per-token
    activation and per-channel weight scales (linear.py:2141-2189).  Forward only."""

    @classmethod
    def from_fms_mo(cls, nnlin, lsb_trun_bits=0, **kwargs):
        target_device = kwargs.get("target_device", kwargs.get("device", next(nnlin.parameters()).device))
        m = cls(nnlin.in_features, nnlin.out_features, bias=nnlin.bias is not None, device="meta")
        m.weight = nnlin.weight
        m.lsb_trun_bits = lsb_trun_bits
        m.chunk_size = kwargs.get("chunk_size", 64)
        m.max_acc_bits = kwargs.get("max_acc_bits", 32)
        if nnlin.bias is not None:
            m.bias = nnlin.bias
        return m.to(target_device)

    def forward(self, inputs):
        x = inputs
        assert x.dtype in [torch.float, torch.bfloat16, torch.float16]
        org_dtype = x.dtype
        out_shape = x.shape[:-1] + (self.weight.shape[0],)
        x = x.reshape(-1, x.shape[-1])
        with torch.no_grad():
            # amax/127 scales; all-zero rows give scale 1e-5/127 here where the reference divides
            # 0/0 (its int8 result is undefined there)
            x_i8, x_scale = kernels.quant_act_i8_pertoken(x, None, compute_dtype=x.dtype)
            w = self.weight.detach()
            w_i8, w_scale = kernels.quant_act_i8_pertoken(w, None, compute_dtype=w.dtype)
            cs = int(self.chunk_size)
            if cs == 8:     # emulated by the reference with interleaved zeros: its wrapper's business
                acc = tl_matmul(x_i8, w_i8.t(), chunk_trun_bits=self.lsb_trun_bits, chunk_size=8,
                                max_acc_bits=self.max_acc_bits)
                out = (acc.to(torch.float) * x_scale.reshape(-1, 1).to(org_dtype)
                       * w_scale.reshape(1, -1).to(w.dtype)).reshape(out_shape).to(org_dtype)
                return out if self.bias is None else out + self.bias.to(org_dtype)
            cs = max(cs, 32) if cs & (cs - 1) == 0 else 32      # tl_matmul's rule for int8
            # (acc.float() * x_scale * w_scale.t()).to(org_dtype) + bias.to(org_dtype) in the epilogue
            out = kernels.matmul_chunk_dq(x_i8, w_i8, x_scale, w_scale, self.bias, L.EPI_SEQ_OUT, org_dtype,
                                          chunk_size=cs, chunk_trun_bits=self.lsb_trun_bits,
                                          max_acc_bits=self.max_acc_bits)
        return out.reshape(out_shape)

    def extra_repr(self) -> str:
        s = f"{self.in_features},{self.out_features},bias={self.bias is not None},chunk_size={self.chunk_size}"
        if self.lsb_trun_bits > 0:
            s += f",lsb_trun={self.lsb_trun_bits}"
        if self.max_acc_bits < 32:
            s += f",max_acc_bits={self.max_acc_bits}"
        return s


class QLinearCublasI8I32NT(nn.Linear):
    """Deploy linear with a STATIC activation quantizer, int8 x int8 -> int32 GEMM and an fp32
    dequantization ``input_scale * w_scale * acc + bias`` (linear.py:1341-1535).  Asymmetric
    activations are quantized to uint8 codes stored minus 128 with the zero-point correction
    folded into the bias.  Here the quantizer is one HIP launch and the GEMM carries the
    dequantization in its epilogue (``torch.ops.mygemm.gemm_nt_i8i32`` stays registered for callers
    that want the raw int32 product)."""

    @classmethod
    def from_reference(cls, ref_qlinear, input_scale, input_zero_point, input_dtype, forceSymA=False):
        """From a torch.ao reference quantized linear (per-channel weights), linear.py:1349-1427."""
        m = cls(ref_qlinear.in_features, ref_qlinear.out_features, device="meta")
        m.forceSymA = forceSymA
        m.input_dtype = input_dtype
        m.register_buffer("input_scale", input_scale.clone())
        m.register_buffer("input_zp", input_zero_point.clone())
        qweight = ref_qlinear.float().get_quantized_weight()
        if ref_qlinear.weight_qscheme not in [torch.per_channel_symmetric, torch.per_channel_affine]:
            raise RuntimeError("QLinear_cublas only supports perCh for now. ")
        m.register_buffer("w_scale", qweight.q_per_channel_scales().float())
        m.register_buffer("w_zp", qweight.q_per_channel_zero_points())
        m.weight = nn.Parameter(qweight.int_repr(), requires_grad=False)
        m.bias = nn.Parameter(ref_qlinear.bias, requires_grad=False)
        if input_dtype == torch.quint8:
            if forceSymA:
                a_min = -input_zero_point * input_scale
                a_max = (255 - input_zero_point) * input_scale
                a_max_new = max(abs(a_min), abs(a_max))
                m.input_scale.copy_((2 * a_max_new) / (255 - 2))
                m.input_zp.copy_(0)
                m.input_dtype = torch.qint8
            else:
                corr_term = m.w_scale * input_scale * (input_zero_point - 128) * m.weight.sum(dim=1)
                corr_term = corr_term.to(ref_qlinear.bias.dtype)
                m.bias = nn.Parameter(ref_qlinear.bias - corr_term, requires_grad=False)
        return m

    @classmethod
    def from_fms_mo(cls, fms_mo_qlinear, **kwargs):
        """From a QLinear with static (clip_val / clip_valn) activation quantizer and a max weight
        quantizer (linear.py:1429-1489).  The activation is taken as asymmetric (quint8)."""
        assert fms_mo_qlinear.num_bits_feature in [4, 8] and fms_mo_qlinear.num_bits_weight in [4, 8], \
            "Please check nbits setting!"
        target_device = kwargs.get("target_device", next(fms_mo_qlinear.parameters()).device)
        m = cls(fms_mo_qlinear.in_features, fms_mo_qlinear.out_features, device="meta")
        m.input_dtype = torch.quint8
        with torch.no_grad():
            Qa = fms_mo_qlinear.quantize_feature
            input_scale = (Qa.clip_val - Qa.clip_valn) / (2**Qa.num_bits - 1)
            input_zero_point = torch.round(-Qa.clip_valn / input_scale).to(torch.int)
            m.register_buffer("input_scale", input_scale)
            m.register_buffer("input_zp", input_zero_point)
            Qw = fms_mo_qlinear.quantize_weight
            w_scale = Qw.clip_val * 2 / (2**Qw.num_bits - 2)
            m.register_buffer("w_scale", w_scale.float())
            m.register_buffer("w_zp", torch.zeros_like(w_scale, dtype=torch.int))
            # the weight quantizer's integer output, cast (truncated) to int8 like the reference
            Qw.dequantize = False
            m.weight = nn.Parameter(Qw(fms_mo_qlinear.weight.float()).to(torch.int8), requires_grad=False)
            corr_term = m.w_scale * input_scale * (input_zero_point - 128) * m.weight.sum(dim=1)
            corr_term = corr_term.to(fms_mo_qlinear.bias.dtype)
            m.bias = nn.Parameter(fms_mo_qlinear.bias - corr_term, requires_grad=False)
        return m.to(target_device)

    def _get_name(self):
        return "QuantizedLinear_cublasi8i32"

    def _params(self, x_dtype):
        """Host copies of scale and zero point and the dtype torch evaluates the quantizer in."""
        key = (x_dtype, self.input_scale.data_ptr(), self.input_scale._version, self.input_scale.dtype,
               self.input_zp.data_ptr(), self.input_zp._version)
        if getattr(self, "_p_key", None) != key:
            probe = torch.empty((1, 1), dtype=x_dtype)
            T = (probe / self.input_scale.cpu() + self.input_zp.cpu()).dtype
            self._p_key = key
            self._p = (float(self.input_scale.reshape(-1)[0]), float(self.input_zp.reshape(-1)[0]), T)
        return self._p

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        with torch.no_grad():
            if not x.is_cuda:
                raise RuntimeError("fms_mo_amd quantized linears run on an AMD GPU only; there is no CPU path")
            if x.dim() not in (2, 3) and type(self) is QLinearCublasI8I32NT:
                raise RuntimeError("Input dimension to QLinear is not 2D or batched 2D")
            in_dtype = x.dtype
            scale, zp, T = self._params(in_dtype)
            x2 = x.reshape(-1, x.shape[-1])
            mode = L.SQ_U8_SHIFT if self.input_dtype == torch.quint8 else L.SQ_S8_NARROW
            q = kernels.quant_act_i8_static_t(x2, mode, T, scale, zp)
            # input_scale * w_scale * acc + bias in fp32, product and sum rounded separately
            y = kernels.gemm_i8_dq(q, self.weight, self.input_scale.float().reshape(-1),
                                   self.w_scale.float().reshape(-1), self.bias, out_dtype=in_dtype,
                                   epilogue=L.EPI_F32_MULADD)
            return y.reshape(tuple(x.shape[:-1]) + (self.weight.shape[0],))


class QLinearCutlassI8I32NT(QLinearCublasI8I32NT):
    """The same module under the name of the CUTLASS variant (linear.py:1538-1583): any number of
    leading dimensions is accepted."""

    def _get_name(self):
        return "QuantizedLinear_cutlassi8i32"


QLinear_modules = (QLinear, QLinearINT8Deploy, QLinearCublasI8I32NT, QLinearCutlassI8I32NT,
                   LinearFPxAcc, QLinearINT8Train)


def isinstance_qlinear(module):
    return isinstance(module, QLinear_modules)
