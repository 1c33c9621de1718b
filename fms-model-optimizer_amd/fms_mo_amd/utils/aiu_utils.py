"""AIU-style integer checkpoints: writer and reader, mirroring fms_mo/utils/aiu_utils.py.

Per quantized linear layer the converted state dict holds ``<layer>.weight`` (int8),
``<layer>.quantize_weight.clip_val`` / ``clip_valn`` and the activation clip values (fp16),
``<layer>.smoothq_scale`` (fp16, only with SmoothQuant) and ``<layer>.zero_shift`` (fp32, only with
asymmetric activations).  The two passes over a weight matrix (column abs-max for the SmoothQuant
scale, quantization + row sums) run as HIP kernels; the vectors of K or N elements between them
are torch arithmetic on the host, in the order the reference uses.

``recompute_narrow_weights`` (aiu_utils.py:125-235): layers whose integer weights are narrow (standard
deviation below 20 levels) are re-quantized with a SAWB quantizer's statistics-aware clip value,
kept only where that clip value lies below the row (tensor) maximum; a one-time host computation
with torch ops, as in the reference.
"""
from __future__ import annotations

import logging
from pathlib import Path

import torch

from .. import kernels
from ..quant.quantizers import SAWB

logger = logging.getLogger(__name__)

STD_THRESHOLD = 20

EXCLUDED_KEYS = ["calib_counter", "num_module_called", "smoothq_act_scale", "smoothq_alpha",
                 "obsrv_w_clipval", "obsrv_clipval", "obsrv_clipvaln"]


def get_quantized_linear_names(model_type: str) -> list[str]:
    """Unique identifiers of the quantized linear layers of a model family (aiu_utils.py:36-69)."""
    if model_type in ["granite", "llama"]:
        return ["self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj", "self_attn.o_proj",
                "mlp.gate_proj", "mlp.up_proj", "mlp.down_proj"]
    if model_type == "gpt_bigcode":
        return ["attn.c_attn", "attn.c_proj", "mlp.c_fc", "mlp.c_proj"]
    if model_type in ["bert", "roberta"]:
        return ["attention.self.query", "attention.self.key", "attention.self.value",
                "attention.output.dense", "intermediate.dense", "output.dense"]
    raise NotImplementedError(f"Model type {model_type} is not supported for quantized checkpoint saving")


def _gpu(t: torch.Tensor, device) -> torch.Tensor:
    if device is None:
        if not t.is_cuda and not torch.cuda.is_available():
            raise RuntimeError("checkpoint conversion runs its weight passes on an AMD GPU; none is visible")
        device = t.device if t.is_cuda else torch.device("cuda")
    return t.to(device)


def process_smoothquant(sd: dict, layer_name: str, new_sd: dict, device=None):
    """aiu_utils.py:87-122.  Returns (sq_scale [1,K] or None, smoothq_act_scale or None); the scaled
    weights themselves are not materialised -- the quantization kernel folds the scale in."""
    sq_scale = None
    sq_a_scale = None
    w = sd[layer_name + ".weight"]
    if layer_name + ".smoothq_alpha" in sd:
        sq_a_scale = sd[layer_name + ".smoothq_act_scale"]
        if sum(sq_a_scale) != 0:
            sq_alpha = sd[layer_name + ".smoothq_alpha"]
            # w.abs().max(dim=0, keepdim=True).values.clamp(min=1e-5): the pass over W on the GPU
            # (exact), the clamp in W's dtype
            col_max = kernels.absmax_cols(_gpu(w, device)).to(w.dtype).to(w.device)
            sq_w_scale = col_max.reshape(1, -1).clamp(min=1e-5)
            sq_scale = sq_a_scale.pow(sq_alpha) / sq_w_scale.pow(1 - sq_alpha)
            if sq_scale.abs().max() > torch.finfo(torch.float16).max:
                raise ValueError("Quantization parameters (qscale) exceeds float16 range. "
                                 "Aborted state dict saving.")
            new_sd[layer_name + ".smoothq_scale"] = sq_scale.squeeze().to(torch.float16).to("cpu")
    return sq_scale, sq_a_scale


def recompute_weight_with_sawb(weight_pre_quant, weight_int_as_fp, weight_per_channel: bool, sq_a_scale,
                               layer_name: str, new_sd: dict):
    """aiu_utils.py:125-235.  Returns (integer weights or None, recomputed?); overwrites the layer's
    weight clip values in ``new_sd`` when it recomputes."""
    weight_pre_quant = weight_pre_quant.to("cpu")
    weight_int_as_fp = weight_int_as_fp.to("cpu")
    if weight_per_channel:
        recompute = any(w < STD_THRESHOLD for w in weight_int_as_fp.std(dim=-1))
    else:
        recompute = weight_int_as_fp.std().item() < STD_THRESHOLD
    if not recompute:
        return None, False
    if sq_a_scale is not None and sum(sq_a_scale) != 0:
        raise ValueError("Weight recomputation while smoothquant is in use is not yet supported.")
    quantizer = SAWB(num_bits=8, dequantize=False, align_zero=True,
                     perCh=weight_int_as_fp.size(0) if weight_per_channel else False)
    quantizer.training = True  # the quantizer recomputes its clip value(s) from the weights
    weight_int_sawb = quantizer(weight_pre_quant.to(torch.float32))
    cv_sawb = quantizer.clip_val.to("cpu").to(torch.float16)
    if weight_per_channel:
        # SAWB rows only where the clip value does not exceed the row maximum
        cv_max = weight_pre_quant.abs().max(dim=-1)[0]
        weight_int_sawb = torch.where((cv_sawb < cv_max)[:, None], weight_int_sawb, weight_int_as_fp)
        cv_guarded = torch.where(cv_sawb < cv_max, cv_sawb, cv_max)
    else:
        # per tensor the reference guards the clip value only: it builds the guarded integers
        # (aiu_utils.py:196-199) and returns the SAWB integers regardless (:235)
        cv_max = weight_pre_quant.abs().max()
        cv_guarded = torch.min(cv_sawb, cv_max)
    new_sd[layer_name + ".quantize_weight.clip_val"] = cv_guarded
    new_sd[layer_name + ".quantize_weight.clip_valn"] = -cv_guarded
    return weight_int_sawb, True


def process_weight(sd: dict, layer_name: str, sq_scale, recompute_narrow_weights: bool, new_sd: dict,
                   device=None, weight_per_channel: bool = False, sq_a_scale=None):
    """aiu_utils.py:237-279: ``clamp(127 / w_cv * (W * sq_scale), -127, 127).round()`` -> int8, in
    one kernel pass that also returns the integer row sums.  With ``recompute_narrow_weights`` a
    layer whose integers are narrow is re-quantized by recompute_weight_with_sawb."""
    if layer_name + ".quantize_weight.clip_val" not in sd:
        return None, None
    w = sd[layer_name + ".weight"]
    w_cv = sd[layer_name + ".quantize_weight.clip_val"]
    if torch.any(w_cv.isclose(torch.tensor(0.0, dtype=w_cv.dtype, device=w_cv.device))):
        raise ValueError(f"Quantization clip values for {layer_name=} have near-zero values and "
                         "are likely uninitialized.")
    coef = 127 / w_cv                                   # [N] or [1], in the clip value's dtype
    wd = _gpu(w, device)
    smooth = None if sq_scale is None else sq_scale.reshape(-1).to(wd.device)
    q, row_sum = kernels.quant_weight_i8(wd, coef.to(wd.device), smooth, mode="mul", want_row_sum=True)
    t_sum = w.dtype if sq_scale is None else torch.promote_types(w.dtype, sq_scale.dtype)
    t_sum = torch.promote_types(t_sum, coef.dtype)
    if recompute_narrow_weights:
        w_pre = w if sq_scale is None else w * sq_scale.to(w.device)
        w_sawb, recomputed = recompute_weight_with_sawb(w_pre, q.to(w_pre.dtype), weight_per_channel, sq_a_scale,
                                                        layer_name, new_sd)
        if recomputed:
            q8 = w_sawb.to(torch.int8)
            new_sd[layer_name + ".weight"] = q8.to("cpu")
            return q8, q8.to(torch.int64).sum(dim=-1).to(t_sum)
    new_sd[layer_name + ".weight"] = q.to("cpu")
    # the reference sums the integer-valued weights in the dtype they were computed in (fp32
    # accumulation, one final rounding): round the exact integer sum to that dtype
    t = w.dtype if sq_scale is None else torch.promote_types(w.dtype, sq_scale.dtype)
    t = torch.promote_types(t, coef.dtype)
    return q, row_sum.to(t)


def process_zero_shift(sd: dict, layer_name: str, weight_int, row_sum, new_sd: dict) -> None:
    """aiu_utils.py:282-333: sum of the integer weights along in_features, only for asymmetric
    activations; stored in fp32."""
    a_cv_name = layer_name + ".quantize_feature.clip_val"
    a_cvn_name = a_cv_name + "n"
    if a_cv_name not in sd:
        return
    a_cv = sd[a_cv_name]
    a_cvn = sd.get(a_cvn_name)
    if not (a_cv is None or a_cvn is None or torch.equal(a_cv, -a_cvn)):
        if weight_int is None:
            logger.info("weights of %s are not quantized: no zero shift generated", layer_name)
        else:
            new_sd[layer_name + ".zero_shift"] = row_sum.to(torch.float32).to("cpu")


def convert_sd_for_aiu(model, recompute_narrow_weights: bool = False, weight_per_channel: bool = False,
                       quantized_layers: list[str] | None = None, device=None) -> dict:
    """aiu_utils.py:336-449.  ``model`` is any module whose state dict follows the fms_mo naming
    (``<layer>.weight``, ``<layer>.quantize_weight.clip_val``, ...); the layer identifiers come
    from ``model.config.model_type`` unless given."""
    if quantized_layers is None:
        model_type = getattr(getattr(model, "config", None), "model_type", None)
        if not model_type:
            raise ValueError("Could not determine model type to save quantized state dictionary.")
        quantized_layers = get_quantized_linear_names(model_type)
    sd = model.state_dict()
    new_sd: dict = {}
    for k, v in sd.items():
        if k.endswith(".weight") and any(q in k for q in quantized_layers):
            layer_name = k[:-7]
            sq_scale, sq_a_scale = process_smoothquant(sd, layer_name, new_sd, device)
            weight_int, row_sum = process_weight(sd, layer_name, sq_scale, recompute_narrow_weights,
                                                 new_sd, device, weight_per_channel, sq_a_scale)
            process_zero_shift(sd, layer_name, weight_int, row_sum, new_sd)
        elif all(ex not in k for ex in EXCLUDED_KEYS):
            if k not in new_sd:
                if v.abs().max() > torch.finfo(torch.float16).max:
                    raise ValueError(f"Quantization parameters ({k}) exceeds float16 range. "
                                     "Aborted state dict saving.")
                new_sd[k] = v.to("cpu").to(torch.float16)
    return new_sd


def save_sd_for_aiu(model, qcfg: dict | None = None, output_dir="./", file_name="qmodel_for_aiu.pt",
                    quantized_layers: list[str] | None = None, device=None) -> None:
    """aiu_utils.py:452-497."""
    if qcfg is not None:
        nbits_w = qcfg.get("nbits_w", None)
        if nbits_w is not None and nbits_w != 8:
            raise ValueError("Saving checkpoint in AIU-compliant format only supports INT8 "
                             f"quantization for now, but found {nbits_w=} in qcfg.")
    converted = convert_sd_for_aiu(
        model,
        recompute_narrow_weights=qcfg.get("recompute_narrow_weights", False) if qcfg else False,
        weight_per_channel="perch" in str(qcfg.get("qw_mode", "")).lower() if qcfg else False,
        quantized_layers=quantized_layers, device=device)
    torch.save(converted, Path(output_dir) / file_name)


def deploy_linear_from_aiu_sd(sd: dict, layer_name: str, device="cuda", **kwargs):
    """Reader: build a QLinearINT8Deploy from one layer of a converted state dict through
    ``from_torch_iW`` (fms_mo/modules/linear.py:923-1023).  Static per-tensor activation clip values
    are required (what from_torch_iW supports); the SmoothQuant scale, when present, is attached so
    the forward divides by it."""
    from ..modules.linear import QLinearINT8Deploy

    w_int = sd[layer_name + ".weight"]
    n, k = w_int.shape
    lin = torch.nn.Linear(k, n, bias=(layer_name + ".bias") in sd)
    with torch.no_grad():
        lin.weight.copy_(w_int.float())
        if lin.bias is not None:
            lin.bias.copy_(sd[layer_name + ".bias"].float())
    lin = lin.to(device)
    w_cv = sd[layer_name + ".quantize_weight.clip_val"].float().reshape(-1)
    if w_cv.numel() != 1:
        raise NotImplementedError("from_torch_iW takes a per-tensor weight clip value")
    a_cv = float(sd[layer_name + ".quantize_feature.clip_val"].float())
    a_cvn = float(sd[layer_name + ".quantize_feature.clip_valn"].float())
    zs = sd.get(layer_name + ".zero_shift")
    zero_shift = "[" + ",".join(repr(float(z)) for z in zs.reshape(-1)) + "]" if zs is not None else 0.0
    m = QLinearINT8Deploy.from_torch_iW(lin, "int8", a_cv, a_cvn, float(w_cv), zero_shift,
                                        target_device=device, **kwargs)
    if layer_name + ".smoothq_scale" in sd:
        m.smoothq_scale = sd[layer_name + ".smoothq_scale"].to(device)
    return m
