"""Lowering of a prepared (fake-quant) model onto the deploy modules through a user-given class
mapping.  Mirrors lower_qmodel_to_ext_kernels and check_qclass_fallback_based_on_min_feat of
fms_mo/fx/utils.py:60-225; the graph plotting and tracing helpers of that file are not part of
the inference path and are not built."""
from __future__ import annotations

import logging

import torch

from ..custom_ext_kernels.utils import _parent_name, _run_once
from ..modules.linear import QLinear

logger = logging.getLogger(__name__)


def check_qclass_fallback_based_on_min_feat(ref_module, qclass_frontup, feat_thresh=16, qclass_fallback=None):
    """The class to lower ``ref_module`` to: ``qclass_frontup`` unless the layer's smaller feature
    dimension is below ``feat_thresh`` (the integer kernels read rows in 16-byte pieces), in which
    case ``qclass_fallback`` -- None here means "leave the module as it is", where the reference
    falls back to its torch-only debug classes (fx/utils.py:60-112)."""
    if isinstance(ref_module, torch.nn.Linear):
        min_feat_or_ch = min(ref_module.in_features, ref_module.out_features)
    elif isinstance(ref_module, torch.nn.Conv2d):
        min_feat_or_ch = min(ref_module.in_channels, ref_module.out_channels)
        qclass_fallback = None
    else:
        raise RuntimeError(f"Reference module {ref_module} is neither Linear nor Conv2d.")
    if min_feat_or_ch < feat_thresh:
        logger.info("%s has min feature size (%d) < %d. It is not lowered.", ref_module, min_feat_or_ch,
                    feat_thresh)
        return qclass_fallback
    return qclass_frontup


def lower_qmodel_to_ext_kernels(mod, exam_inp_eval, qcfg, useInductor=True, model_dtype=torch.float16,
                                **from_fms_mo_kwargs):
    """In-place swap of every module whose type is a key of ``qcfg["ext_kernel_mapping_mod"]`` for
    ``mapping[type].from_fms_mo(module, target_device=..., useInductor=...)``, then optionally
    torch.compile and one run on ``exam_inp_eval`` (fms_mo/fx/utils.py:120-225).  The model is moved
    to the host and cast to ``model_dtype`` first (buffers of the quantizers included), each module
    is converted on the target device, and the model is moved back at the end.  Extra keyword
    arguments (an extension) are handed to every ``from_fms_mo``."""
    mapping = qcfg["ext_kernel_mapping_mod"]
    curr_dev = getattr(mod, "device", next(mod.parameters()).device)
    mod.cpu().to(model_dtype)
    mod2swap = {n: m for n, m in mod.named_modules() if type(m) in mapping}
    for name, module in mod2swap.items():
        parent_name, module_name = _parent_name(name)
        parent_mod = mod.get_submodule(parent_name)
        qclass = mapping[type(module)]
        if isinstance(module, QLinear):
            qclass = check_qclass_fallback_based_on_min_feat(module, qclass_frontup=qclass)
            if qclass is None:
                continue
        module.to(curr_dev)
        new_module = qclass.from_fms_mo(module, target_device=curr_dev, useInductor=useInductor,
                                        **from_fms_mo_kwargs)
        setattr(parent_mod, module_name, new_module)
        module.to("cpu")
    mod.to(curr_dev)
    if useInductor:
        _run_once(mod, exam_inp_eval)  # the deploy modules cache host-side decisions on an eager call
        with torch.no_grad():
            mod = torch.compile(mod, mode="default" if useInductor is True else useInductor)
            _run_once(mod, exam_inp_eval)
    return mod
