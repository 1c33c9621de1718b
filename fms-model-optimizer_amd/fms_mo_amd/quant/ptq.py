"""SmoothQuant activation statistics (the part of fms_mo/quant/ptq.py the quantized-linear path
depends on): per-channel running abs-max of every linear layer's input, collected by forward
hooks.  The reduction over tokens runs in the HIP column abs-max kernel on the layer's device;
the running maxima stay on that device until ``get_act_scales`` returns them on the CPU (the
reference moves every batch's maximum to the CPU, ptq.py:2589)."""
from __future__ import annotations

from functools import partial

import torch
from torch import nn

from .. import kernels


@torch.no_grad()
def activation_stats(name, tensor, act_scales):
    """ptq.py:2584-2595: act_scales[name] = max(act_scales[name], max over tokens of |tensor|)."""
    hidden_dim = tensor.shape[-1]
    x = tensor.detach().reshape(-1, hidden_dim)
    if name in act_scales:
        kernels.absmax_cols(x, act_scales[name])
    else:
        act_scales[name] = kernels.absmax_cols(x)
    return act_scales


@torch.no_grad()
def input_stats_hook(m, x, _y, name, act_scales):
    """ptq.py:2598-2605 (linear layers: the first positional input)."""
    if isinstance(x, tuple):
        x = x[0].detach()
    activation_stats(name, x, act_scales)


@torch.no_grad()
def get_act_scales(model, dloader, qcfg: dict | None = None, device=None, n_samples: int = 100):
    """ptq.py:2608-2659: hook every nn.Linear (QLinear is one), run up to ``n_samples`` batches,
    return {module name: fp32 [in_features] on the CPU}."""
    model.eval()
    if device is not None:
        model.to(device)
    else:
        device = next(model.parameters()).device
    act_scales: dict = {}
    hooks = []
    for name, m in model.named_modules():
        if isinstance(m, nn.Linear):
            hooks.append(m.register_forward_hook(partial(input_stats_hook, name=name, act_scales=act_scales)))
    for data_mb, _ in zip(dloader, range(n_samples)):
        if qcfg is not None:
            qcfg["sample_id"] = qcfg.get("sample_id", 0) + 1
        if isinstance(data_mb, dict):
            model(**{k: (v.to(device) if torch.is_tensor(v) else v) for k, v in data_mb.items()})
        else:
            model(data_mb.to(device) if torch.is_tensor(data_mb) else data_mb)
    for h in hooks:
        h.remove()
    return {k: v.cpu() for k, v in act_scales.items()}
