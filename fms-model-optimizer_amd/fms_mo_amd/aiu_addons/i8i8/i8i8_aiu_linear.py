"""W8A8 linear module around ``torch.ops.fms_mo.i8i8_aiu`` -- the single-GPU part of the
reference's fms_mo/aiu_addons/i8i8/i8i8_aiu_linear.py (:50-231, :241-272): same buffers, same
``qdata`` layout, same factory signature.  The tensor-parallel sharding map of the reference
(:312-410) belongs to ibm-fms' TP machinery and has no counterpart here."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Optional, Union
import copy

import torch

from .i8i8_aiu_op import register_aiu_i8i8_op

register_aiu_i8i8_op()


@dataclass
class W8A8LinearConfig:
    """Configuration for W8A8 Linear module (i8i8_aiu_linear.py:50-60)."""

    linear_type: str = "int8"
    bits: int = 8
    weight_per_channel: bool = False
    activ_quant_type: Optional[str] = "per_token"
    smoothquant: bool = False
    smoothquant_layers: Optional[list] = None


class W8A8LinearAIU(torch.nn.Module):
    """Holds int8 weights and the quantization metadata; forward is one call of the op."""

    def __init__(self, in_features: int, out_features: int, bias: bool, config: W8A8LinearConfig,
                 use_smoothquant: bool = False):
        super().__init__()
        if config.bits != 8:
            raise ValueError("Only INT8 quantization is supported by W8A8LinearAIU module")
        if config.activ_quant_type not in ["per_token", "per_tensor_symm", "per_tensor_asymm"]:
            raise ValueError(
                f"Unrecognized activation quantization type {config.activ_quant_type}. "
                "Choose between per_token, per_tensor_symm, per_tensor_asymm"
            )
        self.in_features = in_features
        self.out_features = out_features
        self.register_buffer("weight", torch.zeros(out_features, in_features, dtype=torch.int8))
        self.has_bias = bias
        self.register_buffer("bias", torch.zeros(out_features if bias else 1, dtype=torch.float16))
        if config.weight_per_channel:
            w_clip_size, self.weight_quant_type = out_features, "per_channel"
        else:
            w_clip_size, self.weight_quant_type = 1, "per_tensor"
        self.register_buffer("w_clip_val", torch.zeros(w_clip_size, dtype=torch.float16))
        self.register_buffer("w_clip_valn", torch.zeros(w_clip_size, dtype=torch.float16))
        # dummies for "per_token" (computed on the fly)
        self.register_buffer("a_clip_val", torch.zeros(1, dtype=torch.float16))
        self.register_buffer("a_clip_valn", torch.zeros(1, dtype=torch.float16))
        zero_shift_size = out_features if config.activ_quant_type == "per_tensor_asymm" else 1
        self.register_buffer("zero_shift", torch.zeros(zero_shift_size, dtype=torch.float32))
        self.activ_quant_type = config.activ_quant_type
        self.smoothquant = config.smoothquant and use_smoothquant
        self.register_buffer(
            "smoothquant_scale",
            torch.ones(in_features if self.smoothquant else 1, dtype=torch.float16),
        )
        if not hasattr(torch.ops, "fms_mo") or not hasattr(torch.ops.fms_mo, "i8i8_aiu"):
            raise ValueError("Custom AIU op `fms_mo.i8i8_aiu` has not been registered.")
        self.aiu_op = torch.ops.fms_mo.i8i8_aiu
        self.register_buffer("qdata", self._cat_qdata())

    def _cat_qdata(self):
        return torch.cat((self.w_clip_val, self.w_clip_valn, self.a_clip_val, self.a_clip_valn,
                          self.zero_shift, self.smoothquant_scale))

    def forward(self, x):
        return self.aiu_op(x, self.weight, self.bias, self.qdata, self.weight_quant_type,
                           self.activ_quant_type, self.smoothquant)

    def re_register_qdata(self) -> None:
        """Rebuild ``qdata`` after the individual metadata buffers were updated."""
        del self.qdata
        self.register_buffer("qdata", self._cat_qdata())

    def __repr__(self) -> str:
        return (f"{self.__class__.__name__}(in={self.in_features}, out={self.out_features}, "
                f"bias={self.has_bias}, wq={self.weight_quant_type}, "
                f"aq={self.activ_quant_type}, smoothq={self.smoothquant}, op={self.aiu_op})")


def update_from_partial(linear_config: dict[Union[str, Callable], Any]):
    """Fold the keywords of a ``functools.partial`` linear_type into a copy of the config."""
    updated = copy.deepcopy(linear_config)
    for k, v in linear_config["linear_type"].keywords.items():
        updated[k] = v
    return updated


def get_int8_aiu_linear(in_features: int, out_features: int, bias: bool,
                        linear_config: dict[Union[str, Callable], Any],
                        linear_type: Optional[str] = None,
                        use_smoothquant: bool = False) -> torch.nn.Module:
    """Factory with the reference's signature (i8i8_aiu_linear.py:241-272)."""
    cfg = None
    if callable(linear_config["linear_type"]):
        cfg = update_from_partial(linear_config)
        cfg["linear_type"] = linear_type
    if not cfg:
        cfg = linear_config
    return W8A8LinearAIU(in_features=in_features, out_features=out_features, bias=bias,
                         config=W8A8LinearConfig(**cfg), use_smoothquant=use_smoothquant)
