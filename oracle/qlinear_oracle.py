"""CPU restatement of the reference's quantized-linear arithmetic.  TEST INFRASTRUCTURE ONLY.

This module is the checker for the HIP kernels: only ``tests/``, ``__graft_entry__.smoke()`` and
the ``cpu_baseline`` leg of ``bench.py`` may import it.  Nothing in the product package imports
it, and it is never the thing that is measured or shipped.

Every function follows one piece of foundation-model-stack/fms-model-optimizer (paths relative to
that repository) and keeps its operation order, dtypes and rounding, using plain torch CPU ops
(torch is the library the reference itself computes with).  Integer products are exact
(``torch._int_mm`` / int64 accumulation), never ``torch.matmul`` on int8 (which wraps to int8).

How each function is pinned (see tests/test_oracle_*.py):
  * act quantizers      -- closed form re-evaluated with exact rational arithmetic (fractions)
                           and explicit IEEE roundings; special rows (all-zero, single +-amax,
                           exact .5 ties); the C restatement in oracle/qlinear_ref.c
  * weight quantizer    -- invariants (|w| <= 127, row arg-max hits +-127) and
                           torch.fake_quantize_per_channel_affine away from ties
  * int GEMM            -- brute-force int64 loops; the C restatement
  * epilogue            -- exact rational re-evaluation
  * chunked int / fp    -- brute force per chunk; bit-level closed form of the truncation
                           (C restatement, all exponent classes, NaN/Inf)
  * fp8 cast            -- all 256 codes and all midpoints against torch's own cast
  * i8i8_aiu            -- the six stored vectors of the reference's own test-suite
                           (tests/golden/ref_w-*_a-*_sq-N.pt); its SmoothQuant branch, which no
                           stored vector exercises, by exactness under power-of-two scales
  * attention matmuls   -- scaled_bmm reduces to scaled_mm per batch entry; qbmm_int8_deploy:
                           the exact form equals the product of the dequantized operands
                           ((q1 - zp) s1) . (q2 s2) (closed form), the literal form equals it to
                           fp16 rounding where the fp16 matmul does not overflow (2-D operands)
  * AIU checkpoint conversion, column abs-max
                        -- closed forms (sqrt(a)/sqrt(wmax) at alpha = 0.5, rint(127 W s / cv) away
                           from ties), invariants (|q| <= 127, zero shift = integer row sums)
  * static / asymmetric deploy branches, from_torch_iW, fake zero shift, per-column dynamic
    scales, the cuBLAS / CUTLASS style modules
                        -- the output equals the float64 product of the dequantized operands
                           ((q - z) s_x) . (w s_w)^T + b (pins sign and size of the correction
                           term, the zero point's offset of 128 and the dimension of the row
                           sums); zero point 128 => no correction; clamp-then-round ==
                           round-then-clamp == torch.quantize_per_tensor away from ties and the
                           same end codes outside the clip range; the per-column quantizer is the
                           per-token one of the transposed tensor; the chunk loop equals the
                           chunked-kernel restatement (tests/test_oracle_pins_deploy.py)
  * SAWB (zero-aligned, forward only) -- the codes equal the index of the nearest of the
                           2^bits - 1 levels k clip / (2^(bits-1) - 1) found by search, the dequantized
                           values are those levels, the clip rule against closed-form moments of a
                           uniform grid and the negative-clip fallback on two-valued weights
  * FP8 emulation quantizers (to_fp8*)
                        -- the scale re-derived with exact rationals and explicit roundings
                           (reciprocal-then-multiply, fp16 clamp), the cast against the enumerated
                           e4m3 grid with ties to even, every element of the scaled quantizers
                           re-derived the same way
  * FP8Linear dynamic scale (computed inside torchao 0.11, not in the reference tree)
                        -- what a symmetric e4m3 scale must satisfy whatever library forms it:
                           quantizing a finite non-zero row with it puts the row maximum on the
                           top code 448 and nothing beyond it, the top code dequantizes back to
                           the row maximum within an fp32 rounding, the scale is fp32 for every
                           input dtype, a zero row gives the floor and zero codes (each shown to
                           fail for /240, /127, a 16-bit-rounded scale, a scale left in x's
                           dtype).  The value of the floor and the dtype the division runs in are
                           torchao's own choice and not derivable: both are arguments (defaults =
                           the reference's test helper, tests/aiu_addons/test_fp8_addon.py:65-79).
"""
from __future__ import annotations

import torch

E4M3_MAX = 448.0
DL8_MIN = 0.0087890625
DL16_MAX = 8581545984.0
DL16_MIN = 4.665707820095122e-10


# ------------------------------------------------------------------------------------------
# SmoothQuant scale
# ------------------------------------------------------------------------------------------
def smoothq_scale_qlinear(weight: torch.Tensor, act_scale: torch.Tensor, alpha: float, x_dtype):
    """QLinear.get_smoothq_scale (fms_mo/modules/linear.py:345-368): ``[1.0]`` when the stored
    activation scale sums to zero, else clamp(a^alpha / wmax^(1-alpha), 1e-5) cast to x's dtype."""
    if act_scale.sum().item() == 0.0:
        return torch.tensor([1.0]).to(x_dtype)
    wmax = weight.abs().max(dim=0, keepdim=True)[0].clamp(min=1e-5)
    return (act_scale.pow(alpha) / wmax.pow(1.0 - alpha)).clamp(min=1e-5).to(x_dtype)


def smoothq_scale_deploy(weight: torch.Tensor, act_scale: torch.Tensor, alpha):
    """QLinearINT8Deploy.from_fms_mo (linear.py:800-817): computed only if every a_k != 0, kept in
    the dtype of the stored activation scale; otherwise ``[1.0]`` in the weight dtype."""
    if not torch.all(act_scale != 0).item():
        return torch.tensor([1.0], dtype=weight.dtype)
    wmax = weight.abs().max(dim=0, keepdim=True)[0].clamp(min=1e-5)
    return (act_scale**alpha / wmax ** (1.0 - alpha)).clamp(min=1e-5).to(act_scale.dtype)


# ------------------------------------------------------------------------------------------
# Activation quantizers
# ------------------------------------------------------------------------------------------
def quant_act_pertoken_i8(x: torch.Tensor, smooth: torch.Tensor | None = None, saturate=False):
    """qa_dynamic_max_qfunc with reduce dim -1 (linear.py:1085-1100) after the optional
    ``x / smoothq_scale`` of QLinearINT8Deploy.forward (:1331-1334).

    Returns (q int8 [M,K], scale [M,1] in the dtype torch promotion gives, x' the divided input).
    ``saturate`` is NOT reference behaviour: it clamps to +-127 before the int8 cast."""
    if smooth is not None:
        x = x / smooth  # fp16 / fp32 tensor -> fp32 (torch type promotion)
    amax = x.abs().max(dim=-1, keepdim=True)[0]
    scale = amax.clamp(min=1e-5).div(127)
    r = torch.round(x / scale)
    if saturate:
        r = r.clamp(-127, 127)
    else:
        # the reference's float -> int8 cast wraps 128 to -128 (only reachable in bfloat16);
        # make the wrap explicit instead of relying on an out-of-range cast
        r = torch.where(r > 127, r - 256, r)
    return r.to(torch.int8), scale, x


def fake_quant_act_pertoken(x: torch.Tensor):
    """QMaxDynamic.forward, dim=-1 (fms_mo/quant/quantizers.py:3531-3534): Q/dQ in x's dtype."""
    amax = x.abs().max(dim=-1, keepdim=True)[0]
    scales = amax.clamp(min=1e-5).div(127)
    return x.div(scales).round().mul(scales)


def quant_act_static_raw(x: torch.Tensor, scale: torch.Tensor, zp: int, sym: int):
    """qa_raw_qfunc (linear.py:1061-1071)."""
    return torch.clamp((x / scale + zp - 128 + sym).round(), -128, 127).to(torch.int8)


def quant_act_pt_native(x: torch.Tensor, scale: torch.Tensor, zp: int, sym: int):
    """qa_pt_quant_func / qa_pt_qfunc_wrapped (linear.py:1025-1059): the library routine itself."""
    return torch.quantize_per_tensor(x.float(), float(scale.reshape(-1)[0]), int(zp) - 128 + int(sym),
                                     torch.qint8).int_repr()


def quant_act_fmo_mo(x, cvn, cv, quant_stepsize, quant_zero_point, sym: int):
    """qa_fmo_mo_qfunc (linear.py:1073-1083): clamp first, then round.  The operands are the
    module's tensors (``cvs``, ``quant_stepsize``, ``quant_zero_point``), so torch's type
    promotion decides the compute dtype exactly as in the reference."""
    r = torch.round(x.clamp(cvn, cv) / quant_stepsize - quant_zero_point) - (128 - int(sym))
    return r.to(torch.int8)


def _wrap_int8(r: torch.Tensor) -> torch.Tensor:
    """float -> int8 the way the reference's ``.to(torch.int8)`` behaves on x86 for integer values
    a little outside the range: two's-complement wrap (128 -> -128), made explicit."""
    r = torch.where(r > 127, r - 256, r)
    r = torch.where(r < -128, r + 256, r)
    return r.to(torch.int8)


def quant_act_dyn_max(x: torch.Tensor, dim: int = -1, nbits: int = 8):
    """qa_dynamic_max_qfunc (linear.py:1085-1100) for either reduce dimension: -1 = per token
    (scale [M,1]), -2 = per input channel over the tokens (scale [1,K]).  Returns (q, scale)."""
    amax = x.abs().max(dim=dim, keepdim=True)[0]
    levels = 2 ** (nbits - 1) - 1
    scale = amax.clamp(min=1e-5).div(levels)
    return _wrap_int8(torch.round(x / scale)), scale


def quant_act_fake_zero_shift(x: torch.Tensor, input_zp: torch.Tensor, nbits: int = 8):
    """qa_dyn_max_fake_zero_shift (linear.py:1102-1113): one dynamic scale for the whole tensor,
    amax / (127 - zp), codes shifted by zp.  input_zp: the module's 0-dim int tensor.
    Returns (q, input_scale 0-dim in x's dtype)."""
    amax = x.abs().max()
    levels = 2 ** (nbits - 1) - 1 - input_zp
    scale = amax.clamp(min=1e-5) / levels
    xq = torch.round(x / scale) + input_zp
    return _wrap_int8(xq), scale


# ------------------------------------------------------------------------------------------
# Weight quantizers
# ------------------------------------------------------------------------------------------
def qmax_perch_clipval(weight: torch.Tensor):
    """Qmax.forward, perCh symmetric branch (quantizers.py:3058-3063): cv_n = max_k |W_nk|."""
    return torch.max(weight.abs().reshape([weight.shape[0], -1]), dim=1).values


def fake_quant_weight_perch(weight: torch.Tensor, cv: torch.Tensor):
    """QmaxPerChSTE.forward (quantizers.py:3190-3224), 8 bits: scale = cv*2/254."""
    scale = cv * 2 / 254
    return torch.fake_quantize_per_channel_affine(
        weight.float(), scale.float(), torch.zeros_like(scale).float(), axis=0,
        quant_min=-127, quant_max=127,
    ).to(weight.dtype)


def quant_weight_deploy(weight: torch.Tensor, w_cv: torch.Tensor, smoothq_scale: torch.Tensor):
    """from_fms_mo weight path (linear.py:821,863-871).  Returns (int8 [N,K], w_scale)."""
    w_scale = w_cv * 2 / 254
    w = torch.round((weight * smoothq_scale).t() / w_scale).clamp(-127, 127).t()
    return w.to(torch.int).to(torch.int8), w_scale


SAWB_COEFF = {103: (2.6, -1.71), 403: (12.035, -12.03), 803: (31.76, -35.04)}


def sawb_clip(weight: torch.Tensor, num_bits: int = 8, perCh: bool = False):
    """sawb_params_code (quantizers.py:633-672) for the zero-aligned codes 103 / 403 / 803:
    clip = c1 * mean|w| + c0 * sqrt(mean w^2), per tensor or per output channel."""
    c0, c1 = SAWB_COEFF[{2: 103, 4: 403, 8: 803}[num_bits]]
    if perCh:
        dims = list(range(1, weight.dim()))
        return c1 * torch.mean(weight.abs(), dim=dims) + c0 * torch.mean(weight**2, dim=dims).sqrt()
    x = weight.flatten()
    return c1 * x.abs().mean() + c0 * x.mul(x).mean().sqrt()


def sawb_zero_forward(x: torch.Tensor, clip_val: torch.Tensor, num_bits: int = 8, dequantize: bool = True):
    """SAWBPlusZeroSTE / SAWBZeroSTE forward in eval mode (quantizers.py:486-494, 610-617):
    x / clip clamped to +-1, mapped to [0, 1], rounded onto 2^bits - 2 steps; integer codes
    (dequantize False) are that minus (2^bits - 2) / 2."""
    scale = 2**num_bits - 2
    if clip_val.dim() == 0:
        clip_val = clip_val.unsqueeze(0)
    out = x.mul(1 / clip_val).clamp(-1, 1).mul(0.5).add(0.5)
    out = torch.round(scale * out - 0.0)
    if dequantize:
        out = (out + 0.0) / scale
        return (2 * out - 1) * clip_val
    return out - scale / 2


def sawb_zero_perch_forward(x: torch.Tensor, clip_val: torch.Tensor, num_bits: int = 8, dequantize: bool = True):
    """SAWBPlusZeroPerChSTE forward in eval mode (quantizers.py:541-565)."""
    int_u = 2 ** (num_bits - 1) - 1
    scale = clip_val * 2 / (2**num_bits - 2)
    zp = torch.zeros_like(scale)
    if dequantize:
        return torch.fake_quantize_per_channel_affine(x.float(), scale.float(), zp.float(), axis=0,
                                                      quant_min=-int_u, quant_max=int_u).to(clip_val.dtype)
    return torch.quantize_per_channel(x, scale, zp, 0, torch.qint8).int_repr().clamp(-int_u, int_u)


# ------------------------------------------------------------------------------------------
# Integer GEMM and epilogue
# ------------------------------------------------------------------------------------------
def int_gemm(a_i8: torch.Tensor, w_i8: torch.Tensor) -> torch.Tensor:
    """Exact int32 C = A[M,K] . W[N,K]^T (cutlass_i8i32gemm.cu:29-62; utils.py:690-714)."""
    M, K = a_i8.shape
    if M > 16 and K % 8 == 0 and w_i8.shape[0] % 8 == 0:
        return torch._int_mm(a_i8.contiguous(), w_i8.t())
    return (a_i8.to(torch.int64) @ w_i8.to(torch.int64).t()).to(torch.int32)


def epilogue_ref(acc: torch.Tensor, input_scale: torch.Tensor, w_scale: torch.Tensor,
                 bias: torch.Tensor | None, org_dtype=torch.float16, acc_dtype=torch.float16):
    """iaddmm_int plain branch (linear.py:1185-1188) then ``.to(org_dtype)`` (:1338).  acc_dtype is
    fp16 in from_fms_mo (:777) and fp32 by default in from_torch_iW (:955)."""
    y = acc.float() * (input_scale * w_scale).to(torch.float16)
    if bias is not None:
        y = y + bias
    return y.to(acc_dtype).to(org_dtype)


def epilogue_f32(acc, input_scale, w_scale, bias, out_dtype):
    """Not reference arithmetic: the fp32-scale epilogue of FMSMO_EPI_F32 (fused multiply-add in
    fp64 is exact enough to give the correctly rounded fp32 fma for these magnitudes)."""
    sc = input_scale.float() * w_scale.float()
    y = acc.double() * sc.double()
    if bias is not None:
        y = y + bias.double()
    return y.float().to(out_dtype)


# ------------------------------------------------------------------------------------------
# Whole modules
# ------------------------------------------------------------------------------------------
def qlinear_forward(x, weight, bias, act_scale=None, alpha=0.5, w_clip_val=None):
    """QLinear.forward, qa_mode='pertokenmax', qw_mode='maxperCh', 8/8 bits (linear.py:248-305).

    ``w_clip_val=None`` behaves like a training-mode first call (clip values = fresh abs-max)."""
    if act_scale is not None:
        s = smoothq_scale_qlinear(weight, act_scale, alpha, x.dtype)
    else:
        s = torch.tensor([1.0]).to(x.dtype)
    qinput = fake_quant_act_pertoken(x / s).to(x.dtype)
    ws = weight * s
    cv = qmax_perch_clipval(ws) if w_clip_val is None else w_clip_val
    qweight = fake_quant_weight_perch(ws, cv).to(weight.dtype)
    return torch.nn.functional.linear(qinput, qweight, bias)


def deploy_prepare(weight, bias, w_clip_val, act_scale=None, alpha=0.5):
    """from_fms_mo with use_dynamic_max_act_Qfunc=-1, symmetric activations (linear.py:717-920):
    returns the module buffers {weight int8, w_scale, smoothq_scale, bias}."""
    if act_scale is not None:
        sq = smoothq_scale_deploy(weight, act_scale, torch.tensor([alpha], dtype=torch.float32))
    else:
        sq = torch.tensor([1.0], dtype=weight.dtype)
    w_i8, w_scale = quant_weight_deploy(weight, w_clip_val, sq)
    # symmetric activations: corr_term = 0, bias <- bias.float() - 0, cast back to W dtype
    new_bias = None if bias is None else (bias.float() - 0.0).to(weight.dtype)
    return {"weight": w_i8, "w_scale": w_scale, "smoothq_scale": sq, "bias": new_bias}


def deploy_forward(x, bufs):
    """QLinearINT8Deploy.forward + iaddmm_int plain branch (linear.py:1309-1338,1115-1188).
    Returns every intermediate: q_x, input_scale, acc, y."""
    org_dtype = x.dtype
    x2 = x.reshape(-1, x.shape[-1])
    sq = bufs["smoothq_scale"]
    use_sq = torch.all(sq != 1).item()
    q_x, input_scale, _ = quant_act_pertoken_i8(x2, sq if use_sq else None)
    acc = int_gemm(q_x, bufs["weight"])
    bias = bufs["bias"]
    y = acc.float() * (input_scale * bufs["w_scale"]).to(torch.float16)
    y = (y + bias) if bias is not None else y
    y = y.to(torch.float16).reshape(tuple(x.shape[:-1]) + (bufs["weight"].shape[0],))
    return {"q_x": q_x, "input_scale": input_scale, "acc": acc, "y": y.to(org_dtype)}


def deploy_prepare_general(weight, bias, w_cv, a_cv=None, a_cvn=None, sym_act=True, act_scale=None,
                           alpha=0.5, use_PT_native_Qfunc=False, use_dynamic_max_act_Qfunc=False,
                           sawb=None):
    """QLinearINT8Deploy.from_fms_mo (linear.py:717-920) for every activation-quantizer branch:
    dynamic max (-1 / -2), fake zero shift (1..64), PT-native static, fms_mo-formula static.
    ``sym_act`` is the reference's useSymAct (:765-769: 'sym' in qa_mode or qa_mode in
    pertokenmax / max).  a_cv / a_cvn: the activation quantizer's clip_val / clip_valn tensors
    (shape [1], fp32 as the quantizers register them) -- default 8.0 / -8.0 as at :793-794.
    ``sawb``: the weight quantizer is a SAWB (None | "tensor" | "perCh") and supplies the codes.
    Returns the module state as a dict (buffers under the reference's names plus the flags)."""
    w_dtype = weight.dtype
    sym = int(bool(sym_act))
    w_levels, a_levels = 2**8 - 2, 2**8 - 1 - sym
    a_cv = torch.tensor(8.0) if a_cv is None else a_cv
    a_cvn = torch.tensor(-8.0) if a_cvn is None else a_cvn
    sq = torch.tensor([1.0], dtype=w_dtype)
    if act_scale is not None:
        sq = smoothq_scale_deploy(weight, act_scale, torch.tensor([alpha], dtype=torch.float32))
    input_scale = torch.tensor(1.0)
    w_scale = w_cv * 2 / w_levels
    st = {"useSymAct": sym, "useDynMaxQfunc": use_dynamic_max_act_Qfunc,
          "usePTnativeQfunc": use_PT_native_Qfunc, "use_fake_zero_shift": False,
          "cvs": [a_cv, a_cvn, w_cv], "acc_dtype": torch.float16}
    if use_dynamic_max_act_Qfunc in [-1, -2]:
        input_zp = torch.tensor(128 - sym)
    elif 0 < use_dynamic_max_act_Qfunc < 65:
        st["use_fake_zero_shift"] = True
        input_zp = torch.tensor(use_dynamic_max_act_Qfunc)
    elif use_PT_native_Qfunc:
        input_scale = torch.tensor([(a_cv - a_cvn) / a_levels])
        input_zp = torch.round(-a_cvn / input_scale)
    else:
        quant_scale = a_levels / torch.tensor([a_cv - a_cvn])
        quant_stepsize = 1.0 / quant_scale
        quant_zero_point = torch.round(a_cvn * quant_scale)
        input_scale = quant_stepsize
        input_zp = -quant_zero_point
        w_scale = 1.0 / (w_levels / (w_cv * 2))
        st.update(quant_scale=quant_scale, quant_stepsize=quant_stepsize,
                  quant_zero_point=quant_zero_point)
    input_zp = input_zp.to(torch.int)
    if sawb is None:
        w_int = torch.round((weight * sq).t() / w_scale).clamp(-w_levels / 2, w_levels / 2).t().to(torch.int)
    else:  # isinstance(Qw, SAWB) (linear.py:859-861): the quantizer's integer output; sawb = "tensor" | "perCh"
        fwd = sawb_zero_perch_forward if sawb == "perCh" else sawb_zero_forward
        w_int = fwd(weight.float() * sq, w_cv, 8, dequantize=False).to(torch.int)
    if sym:
        corr_term_int = 0
        if st["use_fake_zero_shift"]:
            corr_term_int = input_zp * (w_int.sum(dim=1))
    else:
        corr_term_int = (input_zp - 128) * (w_int.sum(dim=1))
    corr_term = corr_term_int * w_scale.float() * input_scale.float()
    new_bias = (bias.float() - corr_term) if bias is not None else -corr_term
    if st["use_fake_zero_shift"]:
        new_bias = new_bias + corr_term
    if not torch.is_tensor(new_bias):  # symmetric, no bias: -0 broadcast to the bias shape
        new_bias = torch.zeros(weight.shape[0]) + new_bias
    if new_bias.dim() == 0:
        new_bias = new_bias.expand(weight.shape[0]).clone()
    st.update(weight=w_int.to(torch.int8), w_scale=w_scale, smoothq_scale=sq, input_scale=input_scale,
              input_zp=input_zp, corr_term=corr_term, bias=new_bias.to(w_dtype))
    return st


def deploy_from_torch_iW(w_int, bias, a_cv: float, a_cvn: float, w_cv: float, zero_shift,
                         use_PT_native_Qfunc=True, acc_dtype=torch.float):
    """QLinearINT8Deploy.from_torch_iW (linear.py:923-1023): the module state built from integer
    weights (any dtype holding integers), Python-float clip values and the per-channel
    ``zero_shift`` (list / tensor of integer row sums, or one float)."""
    st = {"useSymAct": 0, "useDynMaxQfunc": False, "usePTnativeQfunc": use_PT_native_Qfunc,
          "use_fake_zero_shift": False, "cvs": [a_cv, a_cvn, w_cv], "acc_dtype": acc_dtype}
    if use_PT_native_Qfunc:
        input_scale = torch.Tensor([(a_cv - a_cvn) / (2**8 - 1)])
        input_zp = torch.round(-a_cvn / input_scale).to(torch.int)
        w_scale = torch.Tensor([w_cv * 2 / (2**8 - 2)])
    else:
        quant_scale = (2**8 - 1) / torch.Tensor([a_cv - a_cvn])
        quant_stepsize = 1.0 / quant_scale
        quant_zero_point = torch.round(a_cvn * quant_scale)
        input_scale = quant_stepsize
        input_zp = -quant_zero_point
        w_scale = 1.0 / ((2**8 - 2) / torch.Tensor([w_cv * 2]))
        st.update(quant_scale=quant_scale, quant_stepsize=quant_stepsize,
                  quant_zero_point=quant_zero_point)
    zero_s = torch.Tensor(list(zero_shift)) if not isinstance(zero_shift, (int, float)) else torch.Tensor([zero_shift])
    corr_term = (input_zp - 128) * zero_s * w_scale * input_scale
    new_bias = (bias - corr_term).to(acc_dtype) if bias is not None else -corr_term.to(acc_dtype)
    st.update(weight=w_int.to(torch.int8), w_scale=w_scale, smoothq_scale=torch.tensor([1.0]),
              input_scale=input_scale, input_zp=input_zp, corr_term=corr_term, zero_shift=zero_s,
              bias=new_bias)
    return st


def deploy_forward_general(x, st, chunk_size=100000, truncate_lsb=0, max_acc_bits=32):
    """QLinearINT8Deploy.forward + iaddmm_int (linear.py:1309-1338, 1115-1188) on a module state
    from deploy_prepare_general / deploy_from_torch_iW: every activation-quantizer branch, the
    serial chunk loop (:1142-1175) and the plain branch (:1177-1188).  Integer products are exact.
    Returns {q_x, input_scale, acc, y}."""
    org_dtype = x.dtype
    x2 = x.reshape(-1, x.shape[-1])
    sq = st["smoothq_scale"]
    if torch.all(sq != 1).item():
        x2 = x2 / sq
    input_scale = st["input_scale"]
    if st["useDynMaxQfunc"] in [-1, -2]:
        q_x, input_scale = quant_act_dyn_max(x2, st["useDynMaxQfunc"])
    elif st["use_fake_zero_shift"]:
        q_x, input_scale = quant_act_fake_zero_shift(x2, st["input_zp"])
    elif st["usePTnativeQfunc"]:
        q_x = quant_act_static_raw(x2, input_scale, st["input_zp"], st["useSymAct"])
    else:
        q_x = quant_act_fmo_mo(x2, st["cvs"][1], st["cvs"][0], st["quant_stepsize"],
                               st["quant_zero_point"], st["useSymAct"])
    w = st["weight"]
    bias, w_scale = st["bias"], st["w_scale"]
    K = x2.shape[1]
    if K > chunk_size:
        acc = torch.zeros((x2.shape[0], w.shape[0]), dtype=torch.int)
        trun_scale = 1
        lo, hi = -(1 << (max_acc_bits - 1)), (1 << (max_acc_bits - 1)) - 1
        for k0 in range(0, K, chunk_size):
            p = int_gemm(q_x[:, k0:k0 + chunk_size].contiguous(), w[:, k0:k0 + chunk_size].contiguous())
            if max_acc_bits < 32:
                p = p.clamp(lo, hi)
            if truncate_lsb > 0:
                trun_scale = 1 << truncate_lsb
                p = torch.bitwise_right_shift(p + (1 << (truncate_lsb - 1)), truncate_lsb)
            acc += p
        y = (acc * (trun_scale * input_scale * w_scale) + bias).to(st["acc_dtype"])
    else:
        acc = int_gemm(q_x, w)
        updated_bias = bias
        if st["use_fake_zero_shift"]:
            updated_bias = bias - input_scale * st["corr_term"]
        y = (acc.float() * (input_scale * w_scale).to(torch.float16) + updated_bias).to(st["acc_dtype"])
    y = y.reshape(tuple(x.shape[:-1]) + (w.shape[0],)).to(org_dtype)
    return {"q_x": q_x, "input_scale": input_scale, "acc": acc, "y": y}


def deploy_forward_triton(x, st, chunk_size=32, truncate_lsb=0):
    """QLinearINT8Deploy.forward with use_int_kernel="triton" (linear.py:1213-1251 binds imatmul
    to tl_matmul(chunk_trun_bits=truncate_lsb, chunk_size=chunk_size); iaddmm_int then skips its
    PyTorch chunk loop, :1142, and takes the fp16-scale epilogue, :1177-1188).  max_acc_bits is
    not forwarded to the kernel by the reference.  Dynamic per-token activations only."""
    org_dtype = x.dtype
    x2 = x.reshape(-1, x.shape[-1])
    sq = st["smoothq_scale"]
    if torch.all(sq != 1).item():
        x2 = x2 / sq
    q_x, input_scale = quant_act_dyn_max(x2, st["useDynMaxQfunc"])
    cs = max(chunk_size, 32) if (chunk_size & (chunk_size - 1)) == 0 else 32
    acc = chunk_matmul_i8(q_x, st["weight"], None, cs, truncate_lsb, 32)
    y = (acc.float() * (input_scale * st["w_scale"]).to(torch.float16) + st["bias"]).to(st["acc_dtype"])
    y = y.reshape(tuple(x.shape[:-1]) + (st["weight"].shape[0],)).to(org_dtype)
    return {"q_x": q_x, "input_scale": input_scale, "acc": acc, "y": y}


def i8i32nt_from_fms_mo(weight, bias, a_cv, a_cvn, w_cv):
    """QLinearCublasI8I32NT.from_fms_mo (linear.py:1429-1489): asymmetric (quint8) activations with
    the zero-point correction folded into the bias.  The weight integers are what the per-channel
    max quantizer returns with ``dequantize = False`` (:1466-1469; QmaxPerChSTE.forward,
    fms_mo/quant/quantizers.py:3190-3224): the fake-quantized fp32 weights divided by the scale
    again, cast to int8 -- a truncating cast of a quotient that is an integer up to one rounding."""
    input_scale = (a_cv - a_cvn) / (2**8 - 1)
    input_zp = torch.round(-a_cvn / input_scale).to(torch.int)
    scale = w_cv * 2 / (2**8 - 2)
    w_scale = scale.float()
    wf = weight.float()
    fq = torch.fake_quantize_per_channel_affine(wf, scale.float(), torch.zeros_like(scale).float(),
                                                axis=0, quant_min=-127, quant_max=127).to(wf.dtype)
    w_i8 = (fq.t() / scale).t().to(torch.int8)
    corr_term = (w_scale * input_scale * (input_zp - 128) * w_i8.sum(dim=1)).to(bias.dtype)
    return {"weight": w_i8, "w_scale": w_scale, "input_scale": input_scale, "input_zp": input_zp,
            "bias": bias - corr_term, "input_dtype": torch.quint8}


def i8i32nt_forward(x, st):
    """QLinearCublasI8I32NT.forward / QLinearCutlassI8I32NT.forward (linear.py:1491-1535,
    1549-1583): static quantizer (uint8 codes shifted by -128, or int8 clamped to +-127), exact
    integer GEMM, ``input_scale * w_scale * acc + bias``.  Returns {q_x, acc, y}."""
    in_dtype = x.dtype
    if st["input_dtype"] == torch.quint8:
        q = torch.clamp((x / st["input_scale"] + st["input_zp"]).round(), 0, 255)
        q = (q.to(torch.int16) - 128).to(torch.int8)
    else:
        q = torch.clamp((x / st["input_scale"] + st["input_zp"]).round(), -127, 127).to(torch.int8)
    tar_shape = x.shape[:-1] + (st["weight"].shape[0],)
    acc = int_gemm(q.reshape(-1, q.shape[-1]).contiguous(), st["weight"]).reshape(tar_shape)
    y = st["input_scale"] * st["w_scale"] * acc + st["bias"]
    return {"q_x": q, "acc": acc, "y": y.to(in_dtype)}


def deploy_forward_fp(x, bufs):
    """iaddmm_FP (linear.py:1190-1211): the reference's fallback without an int kernel; needs
    every buffer in x's dtype."""
    x2 = x.reshape(-1, x.shape[-1])
    sq = bufs["smoothq_scale"]
    q_x, input_scale, _ = quant_act_pertoken_i8(x2, sq if torch.all(sq != 1).item() else None)
    y = torch.matmul(q_x * input_scale, bufs["weight"].t() * bufs["w_scale"]) + bufs["bias"]
    return y.reshape(tuple(x.shape[:-1]) + (bufs["weight"].shape[0],)).to(x.dtype)


# ------------------------------------------------------------------------------------------
# Chunked accumulation
# ------------------------------------------------------------------------------------------
def chunk_matmul_i8(a_i8, w_i8, c=None, chunk_size=64, trun_bits=0, max_acc_bits=32,
                    truncate_then_accumulate=True):
    """imatmul_kernel (fms_mo/custom_ext_kernels/triton_kernels.py:262-302).  a [M,K], w [N,K]."""
    M, K = a_i8.shape
    N = w_i8.shape[0]
    acc = torch.zeros(M, N, dtype=torch.int64) if c is None else c.to(torch.int64).clone()
    rb = (1 << (trun_bits - 1)) if trun_bits > 0 else 0
    lo, hi = -(1 << (max_acc_bits - 1)), (1 << (max_acc_bits - 1)) - 1

    def wrap32(t):
        return ((t + (1 << 31)) % (1 << 32)) - (1 << 31)

    for k0 in range(0, K, chunk_size):
        p = a_i8[:, k0:k0 + chunk_size].to(torch.int64) @ w_i8[:, k0:k0 + chunk_size].to(torch.int64).t()
        if not truncate_then_accumulate:
            p = wrap32(p + acc)
        if max_acc_bits < 32:
            p = p.clamp(lo, hi)
        if trun_bits != 0:
            p = wrap32(wrap32(p + rb) >> trun_bits << trun_bits)
        acc = wrap32(acc + p) if truncate_then_accumulate else p
    return acc.to(torch.int32)


def round_and_trun(p: torch.Tensor, trun_bits: int, clamp_dl16: bool = False) -> torch.Tensor:
    """round_and_trun_mask + round_and_trun (triton_kernels.py:432-465) on an fp32 tensor."""
    if clamp_dl16:
        trun_bits = 14
    u = p.contiguous().view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    rb = (1 << (trun_bits - 1)) if trun_bits > 0 else 0
    mask = (~((1 << trun_bits) - 1)) & 0xFFFFFFFF
    u = ((u + rb) & 0xFFFFFFFF) & mask
    u = torch.where(u >= (1 << 31), u - (1 << 32), u).to(torch.int32)
    x = u.view(torch.float32)
    if clamp_dl16:
        x = torch.where(x >= DL16_MAX, torch.full_like(x, float("inf")), x)
        x = torch.where(x <= -DL16_MAX, torch.full_like(x, float("-inf")), x)
        x = torch.where(x.abs() < DL16_MIN, torch.zeros_like(x), x)
    return x


def chunk_matmul_fp(a, w, c=None, chunk_size=64, trun_bits=0, clamp_dl16=False,
                    truncate_then_accumulate=True):
    """matmul_kernel / matmul_kernel_DABC (triton_kernels.py:162-187,379-409).  a [M,K] and
    w [N,K] hold the operand values (any float dtype); the per-chunk dot is formed in fp64 and
    rounded once to fp32 -- the reference leaves the fp32 summation order to tl.dot."""
    M, K = a.shape
    acc = torch.zeros(M, w.shape[0], dtype=torch.float32) if c is None else c.float().clone()
    for k0 in range(0, K, chunk_size):
        p = a[:, k0:k0 + chunk_size].double() @ w[:, k0:k0 + chunk_size].double().t()
        if not truncate_then_accumulate:
            p = p + acc.double()
        p = p.float()
        if clamp_dl16 or trun_bits > 0:
            p = round_and_trun(p, trun_bits, clamp_dl16)
        acc = (acc + p) if truncate_then_accumulate else p
    return acc


# ------------------------------------------------------------------------------------------
# FP8
# ------------------------------------------------------------------------------------------
def fp8_quant_fpxacc(t: torch.Tensor, per_tensor=False, dl8=False):
    """Dynamic FP8 Q of LinearFuncFPxFwdBwd.forward (linear.py:1939-1953): returns
    (e4m3 tensor, scale in t's dtype).  Reduction over dim 1 (per token / per out-channel)."""
    reduce_dim = None if per_tensor else 1
    scale = (t.abs().amax(dim=reduce_dim, keepdim=True) / E4M3_MAX).clamp(min=1e-5)
    q = (t / scale).to(torch.float8_e4m3fn)
    if dl8:
        f = q.to(torch.float32)
        f.masked_fill_(f.abs() < DL8_MIN, 0)
        q = f.to(torch.float8_e4m3fn)
    return q, scale


def fpxacc_forward(x, weight, bias=None, trun_bits=0, chunk_size=16, fp8_dyn=False,
                   clamp_acc_to_dl16=False):
    """LinearFuncFPxFwdBwd.forward (linear.py:1902-1975)."""
    org_dtype = x.dtype
    out_shape = x.shape[:-1] + (weight.shape[0],)
    x = x.reshape(-1, x.shape[-1])
    x_scale = torch.tensor(1.0, dtype=org_dtype)
    w_scale = x_scale.clone()
    if fp8_dyn:
        xq, x_scale = fp8_quant_fpxacc(x, fp8_dyn == "per_tensor", clamp_acc_to_dl16)
        wq, w_scale = fp8_quant_fpxacc(weight, fp8_dyn == "per_tensor", clamp_acc_to_dl16)
        x, weight = xq.to(torch.float32), wq.to(torch.float32)
    min_chunk = 16  # fp32 / 16-bit operands; the fp8-valued operands are fp32 tensors here
    cs = max(chunk_size, min_chunk) if (chunk_size & (chunk_size - 1)) == 0 else min_chunk
    acc = chunk_matmul_fp(x, weight, None, cs, trun_bits, clamp_acc_to_dl16)
    out = (acc.to(x.dtype) * x_scale * w_scale.t()).to(org_dtype).reshape(out_shape)
    if bias is not None:
        out = out + bias.to(org_dtype)
    return out


def int8train_forward(x, weight, bias=None, lsb_trun_bits=0, chunk_size=64, max_acc_bits=32):
    """LinearFuncINT8FwdFP32Bwd.forward (linear.py:2141-2189)."""
    org_dtype = x.dtype
    out_shape = x.shape[:-1] + (weight.shape[0],)
    x = x.reshape(-1, x.shape[-1])
    x_scale = x.abs().amax(dim=-1, keepdim=True) / 127
    w_scale = weight.abs().amax(dim=-1, keepdim=True) / 127
    x_i8 = torch.round(x / x_scale).to(torch.int8)
    w_i8 = torch.round(weight / w_scale).to(torch.int8)
    cs = max(chunk_size, 32) if (chunk_size & (chunk_size - 1)) == 0 else 32
    acc = chunk_matmul_i8(x_i8, w_i8, None, cs, lsb_trun_bits, max_acc_bits)
    out = (acc.to(torch.float) * x_scale * w_scale.t()).reshape(out_shape).to(org_dtype)
    if bias is not None:
        out = out + bias.to(org_dtype)
    return out, x_i8, w_i8, acc


def to_fp8_saturated(x, orig_dtype):
    """to_fp8_saturated, e4m3, emulate=True (fms_mo/quant/quantizers.py:5316-5333)."""
    x = x.clamp(min=-1 * E4M3_MAX, max=E4M3_MAX)
    return x.to(torch.float8_e4m3fn).to(orig_dtype)


def fp8_max_to_scale(x_max, orig_dtype):
    """max_to_scale, e4m3 (quantizers.py:5335-5351): 448 / clamp(x_max, 1e-12) in x_max's dtype,
    clamped to the fp16 maximum for fp16."""
    scale = torch.empty_like(x_max, dtype=orig_dtype)
    res = E4M3_MAX / torch.clamp(x_max, min=1e-12)
    if orig_dtype is torch.float16:
        res = torch.clamp(res, max=torch.finfo(torch.float16).max)
    scale.copy_(res)
    return scale


def to_fp8_scaled(x, granularity="tensor"):
    """to_fp8_scaled / to_fp8_scaled_perCh / to_fp8_scaled_perToken, e4m3, emulate=True
    (quantizers.py:5353-5421).  granularity: 'tensor' | 'perCh' (max over dim 1, weights [N,K]) |
    'perToken' (max over dim -1).  Returns (fake-quantized x in x's dtype, scale)."""
    orig_dtype = x.dtype
    if granularity == "tensor":
        x_max = torch.max(torch.abs(x))
    elif granularity == "perCh":
        x_max = torch.max(torch.abs(x), dim=1, keepdim=True)[0]
    else:
        x_max = torch.max(torch.abs(x), dim=-1, keepdim=True)[0]
    x_scale = fp8_max_to_scale(x_max, orig_dtype)
    x_scaled = x * x_scale
    return (to_fp8_saturated(x_scaled, orig_dtype) / x_scale).to(orig_dtype), x_scale


def to_fp8_forward(x, q_mode="fp8_e4m3_sat", perCh=None, perToken=False):
    """class to_fp8, forward (quantizers.py:5423-5488), emulate=True."""
    if perCh:
        return to_fp8_scaled(x, "perCh")[0]
    if perToken:
        return to_fp8_scaled(x, "perToken")[0]
    if "_sat" in q_mode:
        return to_fp8_saturated(x, x.dtype)
    if "_scale" in q_mode:
        return to_fp8_scaled(x, "tensor")[0]
    return None


def qlinear_fp8_forward(x, weight, bias, qa_mode, qw_mode, smoothq_scale=None):
    """QLinear.forward (fms_mo/modules/linear.py:248-305) with the FP8 emulation quantizers
    (quantizers.py:5309-5488): F.linear on the fake-quantized tensors, each already rounded to its
    own dtype, the products summed by torch's matmul in that dtype."""
    s = torch.tensor([1.0], dtype=x.dtype) if smoothq_scale is None else smoothq_scale
    xq = to_fp8_forward(x / s, qa_mode, perToken="perToken" in qa_mode).to(x.dtype)
    wq = to_fp8_forward(weight * s, qw_mode, perCh=weight.shape[0] if "perCh" in qw_mode else None).to(weight.dtype)
    return torch.nn.functional.linear(xq, wq, bias)


def fp8_quant_static(x: torch.Tensor, scale: torch.Tensor):
    """_quantize_affine_float8_custom (fms_mo/aiu_addons/fp8/fp8_linear.py:54-72)."""
    t = x.to(torch.float32) / scale
    return t.clamp(min=-E4M3_MAX, max=E4M3_MAX).to(torch.float8_e4m3fn)


def fp8_dynamic_scale(x: torch.Tensor, floor: float = 1e-12, in_x_dtype: bool = False,
                      per_tensor: bool = False):
    """Dynamic activation scale of FP8Linear (fms_mo/aiu_addons/fp8/fp8_linear.py:163-194 hands
    the computation to torchao's to_affine_quantized_floatx with scale_dtype=torch.float32;
    torchao 0.11 is not in the reference tree and not importable).  Fixed by the mathematics and
    pinned by tests/test_oracle_pins.py: a symmetric e4m3 scale maps the abs-max onto the top
    code 448, and the result is fp32.  Left open by them, hence arguments: the lower clamp
    (default: the reference's own test helper, tests/aiu_addons/test_fp8_addon.py:65-79) and
    whether the division by 448 runs on the fp32-widened abs-max or in x's dtype."""
    amax = x.abs().amax().reshape(1, 1) if per_tensor else x.abs().amax(dim=-1, keepdim=True)
    if in_x_dtype:
        return (amax / E4M3_MAX).clamp(min=floor).to(torch.float32)
    return (amax.to(torch.float32) / E4M3_MAX).clamp(min=floor)


def scaled_mm_cpu(mat1, mat2, scale1, scale2, bias=None, out_dtype=torch.float32):
    """_scaled_mm_cpu_out (fms_mo/aiu_addons/fp8/fp8_spyre_op.py:35-60).  mat2 is [K,N]."""
    m1 = (mat1.to(dtype=out_dtype) * scale1).to(dtype=out_dtype)
    m2 = (mat2.to(dtype=out_dtype) * scale2).to(dtype=out_dtype)
    if bias is not None:
        return torch.addmm(bias.to(dtype=out_dtype), m1, m2)
    return torch.mm(m1, m2)


def fp8_linear_forward(x, w_e4m3, weight_scale, bias=None, input_scale=None):
    """FP8Linear.forward with quantized activations (fp8_linear.py:217-283) evaluated with the
    CPU _scaled_mm.  weight_scale: (1,) per tensor or (N,1) per row; input_scale None = dynamic
    per token."""
    x2 = x.reshape(-1, x.shape[-1])
    s_x = fp8_dynamic_scale(x2) if input_scale is None else input_scale.to(torch.float32)
    qx = fp8_quant_static(x2, s_x)
    s_w = weight_scale.to(torch.float32)
    s_w = s_w.reshape(1, -1) if s_w.numel() > 1 else s_w.reshape(())
    s_xx = s_x if s_x.numel() > 1 else s_x.reshape(())
    y = scaled_mm_cpu(qx, w_e4m3.t(), s_xx, s_w, bias, out_dtype=x.dtype)
    return y.reshape(tuple(x.shape[:-1]) + (w_e4m3.shape[0],)), qx, s_x


# ------------------------------------------------------------------------------------------
# Attention matmuls
# ------------------------------------------------------------------------------------------
def scaled_bmm(mat1, mat2, scale1, scale2, out_dtype=None):
    """spyre::scaled_bmm (fms_mo/aiu_addons/fp8/fp8_spyre_op.py:102-140): _scaled_mm per batch
    entry with per-tensor scales.  mat1 [..., M, K], mat2 [..., K, N]."""
    assert mat1.shape[:-2] == mat2.shape[:-2]
    assert scale1.numel() == 1 and scale2.numel() == 1
    od = torch.float32 if out_dtype is None else out_dtype
    m1 = mat1.reshape(-1, *mat1.shape[-2:])
    m2 = mat2.reshape(-1, *mat2.shape[-2:])
    out = torch.empty((m1.shape[0], m1.shape[1], m2.shape[2]), dtype=od)
    for b in range(m1.shape[0]):
        out[b] = scaled_mm_cpu(m1[b], m2[b], scale1, scale2, out_dtype=od)
    return out.reshape(*mat1.shape[:-2], m1.shape[1], m2.shape[2])


def qbmm_quant(x, scale, zp):
    """QBmmINT8Deploy.qfunc_raw (fms_mo/modules/bmm.py:699-711)."""
    return torch.clamp((x / scale + zp).round(), -128, 127).to(torch.int8)


def qbmm_int8_deploy(m1, m2, m1_scale, m1_zp, m2_scale, m2_zp, literal=False):
    """QBmmINT8Deploy.forward (fms_mo/modules/bmm.py:719-748).  Returns (y, m1_i8, m2_i8).

    literal=True follows the reference line by line: the integer operands are multiplied by an
    fp16 matmul (whose fp16 result overflows beyond 65504 and is rounded to 11 bits) and the
    correction sums m2_i8 over dim 0, which is the reduction dimension only for a 2-D m2.
    literal=False is the product that line stands for: exact integer accumulation and the
    correction summed over the reduction dimension (dim -2) of every batch entry."""
    m1_i8 = qbmm_quant(m1, m1_scale, m1_zp - 128)
    m2_i8 = qbmm_quant(m2, m2_scale, m2_zp)
    if literal:
        corr = m1_scale.float() * (m1_zp - 128) * m2_i8.sum(dim=0) * m2_scale.float()
        x = torch.matmul(m1_i8.half(), m2_i8.half()) * m1_scale * m2_scale - corr
        return x.to(m1.dtype), m1_i8, m2_i8
    acc = torch.matmul(m1_i8.to(torch.int64), m2_i8.to(torch.int64))
    colsum = m2_i8.to(torch.int64).sum(dim=-2, keepdim=True)
    s = m1_scale.double() * m2_scale.double()
    x = acc.double() * s - (m1_zp - 128).double() * colsum.double() * s
    return x.to(m1.dtype), m1_i8, m2_i8


# ------------------------------------------------------------------------------------------
# fms_mo::i8i8_aiu (the op the reference's stored vectors exercise)
# ------------------------------------------------------------------------------------------
def i8i8_aiu_quant_act(x, a_cv, a_cvn, sq, activ_quant_type):
    """Quantize step of quant_dequant_activ (fms_mo/aiu_addons/i8i8/i8i8_aiu_op.py:203-231):
    returns (x_int, scale_x, zp_x) in the promoted dtype; x_int holds integers in [-127,127]
    or, for per_tensor_asymm, [0,255]."""
    if activ_quant_type == "per_tensor_symm":
        scale_x = 127 / a_cv
        return torch.round(x / sq * scale_x).clamp(-127, 127), scale_x, None
    if activ_quant_type == "per_tensor_asymm":
        scale_x = 255 / (a_cv - a_cvn)
        zp_x = a_cvn * scale_x
        return torch.round(x / sq * scale_x - zp_x).clamp(0, 255), scale_x, zp_x
    if activ_quant_type == "per_token":
        x_sq = x / sq
        a_cv_tok = x_sq.abs().max(dim=-1, keepdim=True)[0]
        scale_x = 127 / a_cv_tok
        return torch.round(x_sq * scale_x).clamp(-127, 127), scale_x, None
    raise NotImplementedError(activ_quant_type)


def i8i8_aiu(x, weight, bias, qdata, weight_quant_type, activ_quant_type, smoothquant):
    """fms_mo/aiu_addons/i8i8/i8i8_aiu_op.py:86-231."""
    dtype = x.dtype
    out_feat, in_feat = weight.size()
    if weight_quant_type == "per_tensor":
        i1 = 1
    elif weight_quant_type == "per_channel":
        i1 = out_feat
    else:
        raise NotImplementedError(weight_quant_type)
    i2 = i1 + i1
    i3, i4 = i2 + 1, i2 + 2
    i5 = i4 + (out_feat if activ_quant_type == "per_tensor_asymm" else 1)
    i6 = i5 + (in_feat if smoothquant else 1)
    if len(qdata) != i6:
        raise ValueError(f"qdata length ({len(qdata)}) does not match {i6}")
    w_cv, _, a_cv, a_cvn, _, sq = torch.tensor_split(qdata, (i1, i2, i3, i4, i5))

    x_int, scale_x, zp_x = i8i8_aiu_quant_act(x, a_cv, a_cvn, sq, activ_quant_type)
    if activ_quant_type == "per_tensor_asymm":
        x_dq = x_int.add(zp_x).div(scale_x).mul(sq)
    else:
        x_dq = x_int.div(scale_x).mul(sq)

    if weight_quant_type == "per_tensor":
        w_dq = (weight * w_cv / 127) / sq
    else:
        w_dq = (weight * w_cv.unsqueeze(dim=1) / 127) / sq
    return torch.nn.functional.linear(x_dq.to(dtype), w_dq.to(dtype), bias.to(dtype))


# ------------------------------------------------------------------------------------------
# AIU checkpoint conversion (offline weight path)
# ------------------------------------------------------------------------------------------
def aiu_convert_layer(weight, w_cv, sq_a_scale=None, sq_alpha=None, a_cv=None, a_cvn=None):
    """One layer of convert_sd_for_aiu: process_smoothquant (fms_mo/utils/aiu_utils.py:87-122),
    process_weight without SAWB recomputation (:237-279), process_zero_shift (:282-333).
    Returns a dict with ``weight`` (int8) and, when they apply, ``smoothq_scale`` (fp16) and
    ``zero_shift`` (fp32)."""
    out = {}
    pre = weight
    if sq_a_scale is not None and sum(sq_a_scale) != 0:
        sq_w_scale = weight.abs().max(dim=0, keepdim=True).values.clamp(min=1e-5)
        sq_scale = sq_a_scale.pow(sq_alpha) / sq_w_scale.pow(1 - sq_alpha)
        pre = weight * sq_scale
        out["smoothq_scale"] = sq_scale.squeeze().to(torch.float16)
    cv = w_cv.unsqueeze(dim=1) if w_cv.numel() > 1 else w_cv
    w_int = torch.clamp(127 / cv * pre, -127, 127).round()
    out["weight"] = w_int.to(torch.int8)
    if a_cv is not None and a_cvn is not None and not torch.equal(a_cv, -a_cvn):
        out["zero_shift"] = torch.sum(w_int, dim=1).to(torch.float32)
    return out


def aiu_recompute_narrow(weight_pre_quant, weight_int_as_fp, per_channel: bool):
    """recompute_weight_with_sawb (fms_mo/utils/aiu_utils.py:125-235) without SmoothQuant: when the
    integer weights are narrow (std below 20 levels, any row in per-channel mode) they are
    re-quantized with a SAWB quantizer in training mode (clip from the statistics, :633-672) and,
    per channel, kept where that clip value is below the row maximum.  Returns (integers or None,
    guarded clip value(s) in fp16 or None)."""
    if per_channel:
        recompute = any(w < 20 for w in weight_int_as_fp.std(dim=-1))
    else:
        recompute = weight_int_as_fp.std().item() < 20
    if not recompute:
        return None, None
    w32 = weight_pre_quant.to(torch.float32)
    clip = sawb_clip(w32, 8, perCh=per_channel)
    if per_channel:
        w_sawb = sawb_zero_perch_forward(w32, clip, 8, dequantize=False)
        cv_sawb = clip.to(torch.float16)
        cv_max = weight_pre_quant.abs().max(dim=-1)[0]
        w_int = torch.where((cv_sawb < cv_max)[:, None], w_sawb, weight_int_as_fp)
        return w_int, torch.where(cv_sawb < cv_max, cv_sawb, cv_max)
    if clip <= 0:  # SAWBPlusZeroSTE's safety check (:481-483)
        clip = w32.abs().max()
    w_sawb = sawb_zero_forward(w32, clip, 8, dequantize=False)
    cv_sawb = clip.reshape(1).to(torch.float16)
    cv_max = weight_pre_quant.abs().max()
    # per tensor the reference forms the guarded integers (:196-199) but returns the SAWB integers
    # themselves (:235) beside the guarded clip value: kept as it is
    return w_sawb, torch.min(cv_sawb, cv_max)


def absmax_cols(x):
    """comming_max of the SmoothQuant statistics hook (fms_mo/quant/ptq.py:2586-2595)."""
    return x.reshape(-1, x.shape[-1]).abs().max(dim=0).values.float()
