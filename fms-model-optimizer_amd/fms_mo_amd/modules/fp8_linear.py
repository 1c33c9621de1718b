"""FP8 (OCP e4m3) W8A8 linear.

Mirrors FP8Linear of fms_mo/aiu_addons/fp8/fp8_linear.py:105-311 without its torchao / ibm-fms
plumbing: same constructor ``(in_features, out_features, bias, linear_config)``, same parameters
(``weight`` e4m3 [N,K], ``weight_scale`` (1,) per tensor or (N,1) per row, optional static
``input_scale``), same ``linear_config`` keys:

    {"weights":           {"strategy": "tensor" | "channel", "symmetric": True, "dynamic": False},
     "input_activations": None | {"strategy": "tensor" | "token", "symmetric": True, "dynamic": bool}}

Forward: activations are quantized with  q = e4m3(clamp(f32(x) / scale, +-448))  (scale static
per tensor, or dynamic = amax / 448 per token or per tensor), then one FP8 MFMA GEMM with fp32
accumulation and the epilogue  y = out(acc * s_x[m] * s_w[n] + bias)  -- what the reference
obtains from torch._scaled_mm through torchao's addmm_float8_unwrapped_inference (:275-283).
The dynamic-scale rule inside torchao 0.11 is outside the reference tree.  What the mathematics
fixes is built in (the row maximum lands on the top code 448, the scale is fp32); the two
properties only torchao's source fixes are module attributes: ``dynamic_scale_floor`` (lower
clamp of the scale, default 1e-12 as in the reference's own test helper,
tests/aiu_addons/test_fp8_addon.py:65-79) and ``dynamic_scale_in_input_dtype`` (False: the
abs-max is widened to fp32 before the division by 448; True: the division runs in x's dtype and
its result is widened).
"""
from __future__ import annotations

import torch
from torch import nn

from .. import _lib as L
from .. import kernels


class FP8Linear(nn.Module):
    dynamic_scale_floor = 1e-12
    dynamic_scale_in_input_dtype = False

    def __init__(self, in_features: int, out_features: int, bias: bool, linear_config: dict):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.has_bias = bias
        self.linear_config = linear_config
        assert linear_config["weights"] is not None, "Weights must always be quantized for FP8Linear"
        assert linear_config["weights"]["symmetric"], "We only support symmetric weights for now"
        assert not linear_config["weights"]["dynamic"], "We only support pre-quantized weights for now"
        self.weight = nn.Parameter(torch.zeros(out_features, in_features, dtype=torch.float8_e4m3fn),
                                   requires_grad=False)
        w_shape = (1,) if linear_config["weights"]["strategy"] == "tensor" else (out_features, 1)
        self.weight_scale = nn.Parameter(torch.ones(w_shape), requires_grad=False)
        if self.has_bias:
            self.bias = nn.Parameter(torch.zeros(out_features))
        act = linear_config["input_activations"]
        if act is not None:
            assert act["symmetric"], "We only support symmetric input activations for now"
            if not act["dynamic"]:
                in_shape = (1,) if act["strategy"] == "tensor" else (in_features,)
                self.input_scale = nn.Parameter(torch.ones(in_shape), requires_grad=False)

    @classmethod
    def from_float(cls, weight, bias=None, per_channel=False, act="token"):
        """Quantize fp weights offline: scale = absmax / 448 (per tensor or per row), clamp 1e-12."""
        N, K = weight.shape
        cfg = {"weights": {"strategy": "channel" if per_channel else "tensor", "symmetric": True, "dynamic": False},
               "input_activations": None if act is None else
               {"strategy": act, "symmetric": True, "dynamic": True}}
        m = cls(K, N, bias is not None, cfg).to(weight.device)
        with torch.no_grad():
            w = weight.float()
            amax = w.abs().amax(dim=1, keepdim=True) if per_channel else w.abs().amax().reshape(1)
            scale = (amax / 448.0).clamp(min=1e-12)
            m.weight.data = (w / scale).clamp(-448, 448).to(torch.float8_e4m3fn)
            m.weight_scale.data = scale
            if bias is not None:
                m.bias.data = bias.detach().clone()
        return m

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if not x.is_cuda:
            raise RuntimeError("fms_mo_amd.FP8Linear runs on an AMD GPU only; there is no CPU path")
        act = self.linear_config["input_activations"]
        out_shape = tuple(x.shape[:-1]) + (self.out_features,)
        x2 = x.reshape(-1, x.shape[-1])
        with torch.no_grad():
            bias = self.bias if self.has_bias else None
            w_scale = self.weight_scale.float().reshape(-1)
            if act is None:
                # activations not quantized: dequantize the weight and do a regular matmul
                w = self.weight.to(x.dtype) * self.weight_scale.to(x.dtype)
                return torch.nn.functional.linear(x, w, bias.to(x.dtype) if bias is not None else None)
            if not act["dynamic"]:
                if self.input_scale.numel() != 1:
                    raise NotImplementedError("static activation scales are per tensor")
                q, s = kernels.quant_act_fp8_pertoken(x2, L.FP8_LINEAR, static_scale=self.input_scale.float())
            elif act["strategy"] == "tensor":
                # column abs-max and quantizer: two passes over x, the scale never leaves the device
                q, s = kernels.quant_act_fp8_dynamic(x2, L.FP8_LINEAR, True, self.dynamic_scale_floor,
                                                     self.dynamic_scale_in_input_dtype)
            elif self.dynamic_scale_floor != 1e-12 or self.dynamic_scale_in_input_dtype:
                q, s = kernels.quant_act_fp8_dynamic(x2, L.FP8_LINEAR, False, self.dynamic_scale_floor,
                                                     self.dynamic_scale_in_input_dtype)
            elif kernels.decode_linear_ok(x2, None, x2.shape[1]):
                # decode step of a few tokens: quantizer and weight-streaming matmul in one launch
                y, _ = kernels.decode_linear_fp8(x2, self.weight, w_scale, bias, out_dtype=x.dtype)
                return y.reshape(out_shape)
            else:
                q, s = kernels.quant_act_fp8_pertoken(x2, L.FP8_LINEAR)
            y = kernels.gemm_fp8_dq(q, self.weight, s, w_scale, bias, out_dtype=x.dtype)
        return y.reshape(out_shape)

    def __repr__(self) -> str:
        c = self.linear_config
        a = c["input_activations"]
        acts = "None" if a is None else f"(dynamic: {a['dynamic']}, strategy: {a['strategy']})"
        return (f"{self.__class__.__name__}(in={self.in_features}, out={self.out_features}, "
                f"bias={self.has_bias}, fp8_config=(acts: {acts}, weights: (dynamic: "
                f"{c['weights']['dynamic']}, strategy: {c['weights']['strategy']})))")


def get_fp8_linear(in_features: int, out_features: int, bias: bool, linear_config: dict) -> FP8Linear:
    """Factory with the signature ibm-fms expects from a registered linear type
    (fms_mo/aiu_addons/fp8/fp8_linear.py:313-320)."""
    return FP8Linear(in_features, out_features, bias, linear_config)
