"""AIU-style integer checkpoints: writer and reader, mirroring fms_mo/utils/aiu_utils.py.

Per quantized linear layer the converted state dict holds ``<layer>.weight`` (int8),
``<layer>.quantize_weight.clip_val`` / ``clip_valn`` and the activation clip values (fp16),
``<layer>.smoothq_scale`` (fp16, only with SmoothQuant) and ``<layer>.zero_shift`` (fp32, only with
asymmetric activations).  The two passes over a weight matrix (column abs-max for the SmoothQuant
scale, quantization + row sums) run as HIP kernels; the vectors of K or N elements between them
are torch arithmetic on the host, in the order the reference uses.

Not carried over: the SAWB recomputation of narrow weight distributions
(``recompute_narrow_weights``, aiu_utils.py:125-235) needs the SAWB quantizer, which is a
training-time quantizer outside this package.
"""
from __future__ import annotations

import logging
from pathlib import Path

import torch

from .. import kernels

logger = logging.getLogger(__name__)

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


def process_weight(sd: dict, layer_name: str, sq_scale, recompute_narrow_weights: bool, new_sd: dict,
                   device=None):
    """aiu_utils.py:237-279: ``clamp(127 / w_cv * (W * sq_scale), -127, 127).round()`` -> int8, in
    one kernel pass that also returns the integer row sums."""
    if recompute_narrow_weights:
        raise NotImplementedError("SAWB recomputation of narrow weights is not part of this package")
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
    del weight_per_channel  # only steers the SAWB recomputation in the reference
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
            sq_scale, _ = process_smoothquant(sd, layer_name, new_sd, device)
            weight_int, row_sum = process_weight(sd, layer_name, sq_scale, recompute_narrow_weights,
                                                 new_sd, device)
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
