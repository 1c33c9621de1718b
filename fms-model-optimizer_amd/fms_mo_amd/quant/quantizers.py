"""The quantizer subset that the quantized-linear inference path needs.

These are small host-side ``nn.Module``s with the reference's names, constructor arguments and
buffers (``clip_val`` / ``clip_valn``), so that ``QLinear`` keeps exposing ``quantize_feature`` /
``quantize_weight`` objects that calibration, checkpointing and lowering code can read.  They are
evaluated with torch ops when called directly (offline weight preparation, calibration); the
inference forward of the modules in ``fms_mo_amd.modules.linear`` does not call them -- it goes
to the HIP kernels.

Reference: fms_mo/quant/quantizers.py (factories :46-373, Qmax :2990-3141, QmaxSTE :3159,
QmaxPerChSTE :3190, QMaxDynamic :3504-3537, to_fp8* :5309-5488, Qbypass, SAWB :377-452 with its
zero-aligned forward functions :455-630 and the clip rule :633-672 -- forward only, as
QLinearINT8Deploy.from_fms_mo uses it).  Training-time learnable quantizers (PACT, LSQ, AdaRound,
...) are outside the inference path and raise NotImplementedError here.
"""
from __future__ import annotations

import torch
from torch import nn

E4M3_MAX_POS = torch.finfo(torch.float8_e4m3fn).max
EPS = 1e-12


class Qbypass(nn.Module):
    """Identity quantizer (num_bits in {16, 32})."""

    def forward(self, x):
        return x


class QMaxDynamic(nn.Module):
    """Dynamic symmetric abs-max quantize/dequantize along ``dim`` (-1 per token, -2 per channel).
    All arithmetic stays in the input dtype; round half to even; no clamp."""

    def __init__(self, num_bits, dim=-1):
        super().__init__()
        self.num_bits = num_bits
        self.levels = 2 ** (num_bits - 1) - 1
        if isinstance(dim, str):
            if "perCh" in dim or "per_channel" in dim:
                dim = -2
            elif "perToken" in dim or "per_token" in dim or "per_Token" in dim:
                dim = -1
        if dim not in (-1, -2):
            raise ValueError(f"Reduce dim can only be [-1, -2] or ['perCh', 'perToken'] but found {dim}")
        self.reduce_dim = dim

    def forward(self, input_tensor):
        amax = input_tensor.abs().max(dim=self.reduce_dim, keepdim=True)[0]
        scales = amax.clamp(min=1e-5).div(self.levels)
        return input_tensor.div(scales).round().mul(scales)

    def __repr__(self):
        return f"{self.__class__.__name__}(num_bits={self.num_bits}, quantizer=)"


class _PassThrough(torch.autograd.Function):
    """Straight-through wrapper: forward = quantizer, backward = identity."""

    @staticmethod
    def forward(ctx, x, fn):
        return fn(x)

    @staticmethod
    def backward(ctx, g):
        return g, None


def _qmax_per_tensor(x, num_bits, dequantize, cv, align_zero):
    levels = (2**num_bits - 2) if align_zero else (2**num_bits - 1)
    cv = cv.to(x.dtype)
    u = x.mul(1 / cv).clamp(-1, 1).mul(0.5).add(0.5)
    q = torch.round(levels * u)
    if dequantize:
        return (2 * (q / levels) - 1) * cv
    if not align_zero:
        raise ValueError("Dequantize=False in QmaxSTE requires zero alignment")
    return q - levels / 2


def _qminmax_per_tensor(x, num_bits, cv, cvn, align_zero):
    """QminmaxSTE.forward (fms_mo/quant/quantizers.py:3270-3287): asymmetric, always dequantized."""
    cv, cvn = cv.to(x.dtype), cvn.to(x.dtype)
    scale = (2**num_bits - 1) / (cv - cvn)
    zero_point = cvn * scale
    if align_zero:
        zero_point = torch.round(zero_point)
    out = (x.clamp(cvn.item(), cv.item()) - cvn) * scale
    return (torch.round(out) + zero_point) / scale


def _qmax_per_channel(x, num_bits, dequantize, cv):
    nspace = 2**num_bits - 2
    lo = -(2 ** (num_bits - 1)) + 1
    scale = cv * 2 / nspace
    out = torch.fake_quantize_per_channel_affine(
        x.float(), scale.float(), torch.zeros_like(scale).float(), axis=0, quant_min=lo,
        quant_max=-lo,
    ).to(x.dtype)
    if not dequantize:
        return (out.t() / scale).t()
    return out


class Qmax(nn.Module):
    """Symmetric abs-max quantizer for weights (per tensor or per output channel) or activations.

    Same state machine as the reference: in training mode the clip values of the current tensor
    are used for quantization and folded into ``clip_val`` with a 0.1 moving average (the first
    call copies them); in eval mode the stored ``clip_val`` is used."""

    def __init__(self, num_bits, dequantize=True, inplace=False, align_zero=False, clipSTE=True,
                 minmax=False, perCh=None, perGp=None, extend_act_range=False):
        super().__init__()
        if perGp or extend_act_range or (minmax and perCh):
            raise NotImplementedError(
                "Qmax variants perGp / extend_act_range / per-channel minmax are outside the W8A8 "
                "inference path"
            )
        self.num_bits = num_bits
        self.dequantize = dequantize
        self.inplace = inplace
        self.align_zero = align_zero
        self.clipSTE = clipSTE
        self.minmax = minmax
        self.perCh = perCh
        self.perGp = None
        self.extend_act_range = False
        self.quantizer_name = "Qminmax" if minmax else "Qmax"
        self.movAvgFac = 0.1
        self.Niter = 0
        n = perCh if perCh else 1
        self.register_buffer("clip_val", torch.zeros(n))
        self.register_buffer("clip_valn", torch.zeros(n))

    def _quantize(self, x, cv, cvn=None):
        if self.minmax:
            return _PassThrough.apply(x, lambda t: _qminmax_per_tensor(t, self.num_bits, cv, cvn, self.align_zero))
        if self.perCh:
            return _PassThrough.apply(x, lambda t: _qmax_per_channel(t, self.num_bits, self.dequantize, cv))
        return _PassThrough.apply(
            x, lambda t: _qmax_per_tensor(t, self.num_bits, self.dequantize, cv, self.align_zero)
        )

    def forward(self, input_tensor):
        if self.perCh:
            cv_new = torch.max(input_tensor.abs().reshape([self.perCh, -1]), dim=1).values
            assert len(cv_new) == input_tensor.shape[0], "dimension error"
        elif self.minmax:  # asymmetric
            cv_new = input_tensor.max().unsqueeze(0)
        else:
            cv_new = input_tensor.abs().max().unsqueeze(0)
        cvn_new = input_tensor.min().unsqueeze(0) if self.minmax else -cv_new
        if self.Niter == 0 and self.training:
            with torch.no_grad():
                self.clip_val.copy_(cv_new)
                self.clip_valn.copy_(cvn_new)
        if self.training:
            out = self._quantize(input_tensor, cv_new, cvn_new)
            with torch.no_grad():
                self.clip_val.copy_(self.clip_val * (1.0 - self.movAvgFac) + cv_new * self.movAvgFac)
                self.clip_valn.copy_(self.clip_valn * (1.0 - self.movAvgFac) + cvn_new * self.movAvgFac)
        else:
            out = self._quantize(input_tensor, self.clip_val, self.clip_valn)
        self.Niter += 1
        return out

    def __repr__(self):
        per = f"per channel of {self.perCh}" if self.perCh else ""
        return (f"{self.quantizer_name}(num_bits={self.num_bits}, clip_val={self.clip_val[0]:.2f}, "
                f"{per}class={self.__class__.__name__})")


SAWB_COEFF = {103: (2.6, -1.71), 403: (12.035, -12.03), 703: (28.24, -30.81), 803: (31.76, -35.04)}
SAWB_BITS2CODE = {2: 103, 4: 403, 7: 703, 8: 803}


def sawb_params_code(num_bits, code, out, perCh=False):
    """Statistics-aware clip value  c1 * mean|w| + c0 * sqrt(mean w^2)  (quantizers.py:633-672):
    per tensor -> (clip, 2^bits - 2); per output channel -> (clip vector, None)."""
    if code not in SAWB_COEFF:
        raise ValueError(f"SAWB not implemented for code={code}")
    c0, c1 = SAWB_COEFF[code]
    with torch.no_grad():
        if perCh:
            dims = list(range(1, out.dim()))
            mu = torch.mean(out.abs(), dim=dims)
            std = torch.mean(out**2, dim=dims).sqrt()
            return c1 * mu + c0 * std, None
        x = out.flatten()
        mu = x.abs().mean()
        std = x.mul(x).mean().sqrt()
        return c1 * mu + c0 * std, 2**num_bits - 2


class SAWB(nn.Module):
    """Statistics-aware weight binning, zero-aligned (symmetric, 2^bits - 1 levels), forward only
    (quantizers.py:377-452).  In training mode a call recomputes ``clip_val`` from the weight
    statistics, in eval mode it uses the stored one.  ``dequantize=False`` returns the integer codes
    in [-(2^(bits-1) - 1), 2^(bits-1) - 1], which is how QLinearINT8Deploy.from_fms_mo takes the
    weights from it.  clipSTE and perCh select the per-channel formula (quantizers.py:503-572:
    ``torch.quantize_per_channel`` with scale = 2 clip / (2^bits - 2)); every other combination is
    per tensor (:455-500, :575-630):  round((clamp(w / clip, -1, 1) / 2 + 1/2) * (2^bits - 2)) - (2^(bits-1) - 1).
    The variants without zero alignment are training-time only and are not built."""

    def __init__(self, num_bits, dequantize=True, inplace=False, align_zero=False, clipSTE=True, perCh=False,
                 interp=False):
        super().__init__()
        if num_bits not in [2, 4, 8]:
            raise ValueError("FMS: SAWB supports 2, 4, and 8-bit quantization only.")
        if not align_zero:
            raise NotImplementedError("SAWB without zero alignment is a training-time quantizer, not built here")
        self.num_bits = num_bits
        self.dequantize = dequantize
        self.inplace = inplace
        self.align_zero = align_zero
        self.clipSTE = clipSTE
        self.perCh = perCh
        self.interp = interp
        self.register_buffer("clip_val", torch.zeros(perCh) if perCh else torch.Tensor([0.0]))

    @property
    def per_channel_formula(self):
        return bool(self.clipSTE and self.perCh)

    def forward(self, input_tensor):
        nb = self.num_bits
        with torch.no_grad():
            if self.per_channel_formula:
                if self.training:
                    clip_val, _ = sawb_params_code(nb, SAWB_BITS2CODE[nb], input_tensor, perCh=True)
                else:
                    clip_val = self.clip_val
                self.clip_val.copy_(clip_val)
                int_u = 2 ** (nb - 1) - 1
                scale = clip_val * 2 / (2**nb - 2)
                zero_point = torch.zeros_like(scale)
                if self.dequantize:
                    return torch.fake_quantize_per_channel_affine(
                        input_tensor.float(), scale.float(), zero_point.float(), axis=0, quant_min=-int_u,
                        quant_max=int_u).to(clip_val.dtype)
                return torch.quantize_per_channel(input_tensor, scale, zero_point, 0, torch.qint8) \
                    .int_repr().clamp(-int_u, int_u)
            scale = 2**nb - 2
            if self.training:
                clip_val, _ = sawb_params_code(nb, SAWB_BITS2CODE[nb], input_tensor)
            else:
                clip_val = self.clip_val
            if self.clipSTE and clip_val <= 0:  # "sometimes sawb returns negative clipvals" (:481-483)
                clip_val = input_tensor.abs().max()
            if clip_val.dim() == 0:
                clip_val = clip_val.unsqueeze(dim=0)
            self.clip_val.copy_(clip_val)
            clip_val = clip_val.to(input_tensor.device)
            output = input_tensor.mul(1 / clip_val).clamp(-1, 1).mul(0.5).add(0.5)
            output = torch.round(scale * output - 0.0)
            if self.dequantize:
                output = (output + 0.0) / scale
                return (2 * output - 1) * clip_val
            return output - scale / 2

    def __repr__(self):
        return f"{self.__class__.__name__}(num_bits={self.num_bits}, perCh={self.perCh}, clipSTE={self.clipSTE})"


def max_to_scale(x_max, float8_dtype, orig_dtype):
    """Multiplicative FP8 scale 448 / clamp(max, 1e-12), stored in the original dtype."""
    if float8_dtype != torch.float8_e4m3fn:
        raise NotImplementedError("only e4m3 is supported")
    res = E4M3_MAX_POS / torch.clamp(x_max, min=EPS)
    if orig_dtype is torch.float16:
        res = torch.clamp(res, max=torch.finfo(torch.float16).max)
    scale = torch.empty_like(x_max, dtype=orig_dtype)
    scale.copy_(res)
    return scale


def to_fp8_saturated(x, float8_dtype=torch.float8_e4m3fn, orig_dtype=torch.bfloat16, emulate=True):
    x = x.clamp(min=-E4M3_MAX_POS, max=E4M3_MAX_POS)
    return x.to(float8_dtype).to(orig_dtype) if emulate else x.to(float8_dtype)


def _to_fp8_scaled(x, x_max, float8_dtype, orig_dtype, emulate):
    x_scale = max_to_scale(x_max, float8_dtype, orig_dtype)
    x_scaled = x * x_scale
    if emulate:
        return (to_fp8_saturated(x_scaled, float8_dtype, orig_dtype, True) / x_scale).to(orig_dtype), x_scale
    return to_fp8_saturated(x_scaled, float8_dtype, orig_dtype, False), x_scale


def to_fp8_scaled(x, float8_dtype=torch.float8_e4m3fn, orig_dtype=torch.float16, emulate=True):
    return _to_fp8_scaled(x, torch.max(torch.abs(x)), float8_dtype, orig_dtype, emulate)


def to_fp8_scaled_perCh(x, float8_dtype=torch.float8_e4m3fn, orig_dtype=torch.float16, emulate=True):
    return _to_fp8_scaled(x, torch.max(torch.abs(x), dim=1, keepdim=True)[0], float8_dtype, orig_dtype, emulate)


def to_fp8_scaled_perToken(x, float8_dtype=torch.float8_e4m3fn, orig_dtype=torch.float16, emulate=True):
    return _to_fp8_scaled(x, torch.max(torch.abs(x), dim=-1, keepdim=True)[0], float8_dtype, orig_dtype, emulate)


class to_fp8(nn.Module):
    """FP8 (e4m3) emulation quantizer: q_mode in fp8_e4m3_sat | fp8_e4m3_scale (+perCh/perToken)."""

    def __init__(self, n_bits=8, q_mode="fp8_e4m3_sat", perCh=None, perToken=False, emulate=True):
        super().__init__()
        assert n_bits == 8, "only for 8-bit floating point conversion"
        if "e4m3" not in q_mode:
            # the reference names a non-existent torch dtype for e5m2, i.e. that mode never worked
            raise ValueError("FP8 only supports e4m3 here")
        self.q_mode = q_mode
        self.float8_dtype = torch.float8_e4m3fn
        self.emulate = emulate
        self.perCh = perCh
        self.perToken = perToken
        self.register_buffer("scale", torch.zeros(perCh) if perCh else torch.Tensor([0.0]))

    def forward(self, x):
        od = x.dtype
        if self.perCh:
            return to_fp8_scaled_perCh(x, self.float8_dtype, od, self.emulate)[0]
        if self.perToken:
            return to_fp8_scaled_perToken(x, self.float8_dtype, od, self.emulate)[0]
        if "_sat" in self.q_mode:
            return to_fp8_saturated(x, self.float8_dtype, od, self.emulate)
        if "_scale" in self.q_mode:
            return to_fp8_scaled(x, self.float8_dtype, od, self.emulate)[0]
        return None

    def __repr__(self):
        return f"{self.__class__.__name__}(q_mode={self.q_mode}, emulate={self.emulate})"


_OUT_OF_SCOPE = ("pact", "lsq", "qsilu", "dorefa", "fix", "brecq", "adaround", "qil", "custom")


def get_activation_quantizer(qa_mode="PACT", nbits=32, clip_val=None, clip_valn=None, non_neg=False,
                             align_zero=True, extend_act_range=False, use_swcap=False,
                             use_PT_native_Qfunc=False, use_subnormal=False):
    """Activation quantizer factory for the modes on the inference path:
    pertokenmax / perTokenmax / max_perCh (dynamic), max, maxsym, fp8_e4m3_{sat,scale}[_perToken]."""
    mode = qa_mode or ""
    if use_swcap or any(k in mode.lower() for k in _OUT_OF_SCOPE):
        raise NotImplementedError(f"activation quantizer '{qa_mode}' is a training-time quantizer, not built here")
    if "max" in mode:
        if "min" in mode:
            return Qmax(nbits, align_zero=align_zero, minmax=True)
        if "pertoken" in mode or "perToken" in mode:
            return QMaxDynamic(nbits, dim=-1)
        if "per_channel" in mode or "perCh" in mode:
            return QMaxDynamic(nbits, dim=-2)
        if "sym" in mode:
            return Qmax(nbits, align_zero=True, minmax=False, extend_act_range=extend_act_range)
        return Qmax(nbits, align_zero=align_zero, minmax=False)
    if "fp8" in mode:
        return to_fp8(nbits, q_mode=mode, perToken="perToken" in mode, emulate=True)
    raise ValueError(f"unrecognized activation quantization mode {qa_mode}")


def get_weight_quantizer(qw_mode="SAWB+", nbits=32, clip_val=None, clip_valn=None, align_zero=True,
                         w_shape=None, use_swcap=False, recompute=False, perGp=None,
                         use_subnormal=False):
    """Weight quantizer factory: sawb[+][perCh], max / maxperCh, fp8_e4m3_{sat,scale}[_perCh]."""
    mode = qw_mode or ""
    if use_swcap or any(k in mode.lower() for k in _OUT_OF_SCOPE):
        raise NotImplementedError(f"weight quantizer '{qw_mode}' is a training-time quantizer, not built here")
    nch = w_shape[0] if w_shape is not None and "perCh" in mode else False
    if "sawb" in mode:  # quantizers.py:256-268
        return SAWB(nbits, dequantize=True, inplace=False, align_zero=True, clipSTE="+" in mode, perCh=nch,
                    interp="interp" in mode)
    if "max" in mode:
        if "min" in mode or "perGp" in mode:
            raise NotImplementedError("minmax / per-group weight quantizers are not on the W8A8 path")
        return Qmax(nbits, align_zero=align_zero, minmax=False, perCh=nch)
    if "fp8" in mode:
        return to_fp8(nbits, q_mode=mode, emulate=True, perCh=nch)
    raise ValueError(f"unrecognized weight quantized mode {qw_mode}")
