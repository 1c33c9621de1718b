"""Custom-op registration and lowering helpers on top of the HIP kernels.

Mirrors the part of fms_mo/custom_ext_kernels/utils.py that belongs to the quantized-linear path:
``imatmul_ops_reg`` (torch.ops.fms_mo.{imatmul,iaddmm,q_iaddmm_dq,q_per_t_sym}, :642-802), the
native GEMM ops ``torch.ops.cutlass_gemm.i8i32nt`` (:336-364) and
``torch.ops.mygemm.gemm_nt_i8i32`` (:186-206), and the module-swap helpers
``lower_qmodel_cutlass`` / ``lower_qmodel_triton`` (:805-959).  Every op has a fake (meta)
implementation so that torch.compile traces through it; device kernels are registered for the
GPU dispatch key only, so a CPU tensor raises instead of silently taking another path.
"""
from __future__ import annotations

import logging

import torch

from .. import kernels

logger = logging.getLogger(__name__)

_LIBS = {}
_registered = set()


def _lib(ns):
    if ns not in _LIBS:
        _LIBS[ns] = torch.library.Library(ns, "FRAGMENT")
    return _LIBS[ns]


def _define(ns, name, schema, impl, fake):
    qual = f"{ns}::{name}"
    if qual in _registered or (hasattr(torch.ops, ns) and hasattr(getattr(torch.ops, ns), name)):
        return  # first registration wins, like the reference (utils.py:667-669)
    lib = _lib(ns)
    lib.define(f"{name}{schema}")
    lib.impl(name, impl, "CUDA")
    torch.library.register_fake(qual)(fake)
    _registered.add(qual)


def _w_rows(m2: torch.Tensor) -> torch.Tensor:
    """[K,N] operand -> the [N,K] row-major weight matrix the kernels read.  For the usual
    ``W.t()`` view this is the original storage; a row-major [K,N] tensor is transposed once."""
    w = m2.t()
    return w if w.stride(-1) == 1 else w.contiguous()


def _imatmul(m1, m2):
    assert m1.dtype == torch.int8 and m2.dtype == torch.int8, \
        "When using int matmul, inputs must be 2D and INT8."
    tar_shape = tuple(m1.shape[:-1]) + (m2.shape[1],)
    return kernels.gemm_i8_i32(m1.reshape(-1, m1.shape[-1]), _w_rows(m2)).reshape(tar_shape)


def _imatmul_fake(m1, m2):
    return torch.empty(tuple(m1.shape[:-1]) + (m2.shape[1],), dtype=torch.int32, device=m1.device)


def _iaddmm(bias, m1, m2, scale_i, scale_w):
    M = m1.shape[0]
    return kernels.gemm_i8_dq(m1, _w_rows(m2), scale_i.reshape(-1), scale_w.reshape(-1), bias,
                              out_dtype=torch.float32, exact_ref=False).reshape(M, m2.shape[1])


def _iaddmm_fake(bias, m1, m2, scale_i, scale_w):
    return torch.empty((m1.shape[0], m2.shape[1]), dtype=torch.float, device=m1.device)


def _q_iaddmm_dq(bias, m1, m2, scale_i, zp_i, scale_w):
    assert m2.dtype == torch.int8, f"weight tensor is of incorrect dtype {m2.dtype}"
    q = kernels.quant_act_i8_static(m1, float(scale_i.reshape(-1)[0]), int(zp_i.reshape(-1)[0]), 0)
    y = kernels.gemm_i8_dq(q, _w_rows(m2), scale_i.reshape(-1)[:1], scale_w.reshape(-1), bias,
                           out_dtype=torch.float32, exact_ref=False)
    return y.to(m1.dtype)


def _q_iaddmm_dq_fake(bias, m1, m2, scale_i, zp_i, scale_w):
    return torch.empty((m1.shape[0], m2.shape[1]), dtype=m1.dtype, device=m1.device)


def _q_per_t(x, s, zp):
    shp = x.shape
    q = kernels.quant_act_i8_static(x.reshape(-1, shp[-1]), float(s.reshape(-1)[0]),
                                    int(zp.reshape(-1)[0]) + 128, 2)  # 2: quantize_per_tensor arithmetic
    return q.reshape(shp)


def _q_per_t_fake(x, s, zp):
    return torch.empty(x.shape, dtype=torch.int8, device=x.device)


def imatmul_ops_reg(useINTkernel="hip", mm_func=None, AB_dtype=torch.float, D_dtype=torch.float):
    """Register torch.ops.fms_mo.{imatmul, iaddmm, q_iaddmm_dq, q_per_t_sym} on the HIP kernels.
    The arguments are accepted for call compatibility; there is one backend here."""
    if hasattr(torch.ops, "fms_mo") and hasattr(torch.ops.fms_mo, "imatmul"):
        logger.info("imatmul op has already been registered.")
        return
    _define("fms_mo", "imatmul", "(Tensor m1, Tensor m2) -> Tensor", _imatmul, _imatmul_fake)
    _define("fms_mo", "iaddmm",
            "(Tensor bias, Tensor m1, Tensor m2, Tensor scale_i, Tensor scale_w) -> Tensor",
            _iaddmm, _iaddmm_fake)
    _define("fms_mo", "q_iaddmm_dq",
            "(Tensor bias, Tensor m1, Tensor m2, Tensor scale_i, Tensor zp_i, Tensor scale_w) -> Tensor",
            _q_iaddmm_dq, _q_iaddmm_dq_fake)
    _define("fms_mo", "q_per_t_sym", "(Tensor x, Tensor s, Tensor zp) -> Tensor", _q_per_t, _q_per_t_fake)


def _i8i32nt(m1, m2):
    """A [M,K] int8 row-major, B passed as the [K,N] transposed view of a [N,K] weight."""
    return kernels.gemm_i8_i32(m1.contiguous(), _w_rows(m2))


def _gemm_nt_i8i32(x, w):
    """x [M,K] int8, w [N,K] int8 (weight layout)."""
    return kernels.gemm_i8_i32(x, w)


def native_gemm_ops_reg():
    """torch.ops.cutlass_gemm.i8i32nt(m1, m2) and torch.ops.mygemm.gemm_nt_i8i32(x, w)."""
    _define("cutlass_gemm", "i8i32nt", "(Tensor m1, Tensor m2) -> Tensor", _i8i32nt,
            lambda m1, m2: torch.empty((m1.shape[0], m2.shape[1]), dtype=torch.int32, device=m1.device))
    _define("mygemm", "gemm_nt_i8i32", "(Tensor x, Tensor w) -> Tensor", _gemm_nt_i8i32,
            lambda x, w: torch.empty((x.shape[0], w.shape[0]), dtype=torch.int32, device=x.device))


# the loader names of the reference; both end in the same registration here
def cutlass_ops_load_and_reg(qcfg=None, run_unit_test=False):
    native_gemm_ops_reg()


def cublas_ops_load_and_reg(qcfg=None, run_unit_test=False):
    native_gemm_ops_reg()


def _parent_name(target: str):
    """'a.b.c' -> ('a.b', 'c') (torch.ao.quantization.utils._parent_name)."""
    *parent, name = target.rsplit(".", 1)
    return (parent[0] if parent else ""), name


def _run_once(mod, exam_inp_eval):
    if exam_inp_eval is None:
        return
    with torch.no_grad():
        if isinstance(exam_inp_eval, dict):
            mod(**exam_inp_eval)
        elif isinstance(exam_inp_eval, (tuple, list)):
            mod(*exam_inp_eval)
        else:
            mod(exam_inp_eval)


def lower_qmodel_cutlass(mod, exam_inp_eval=None, qcfg=None, use_inductor=False, model_dtype=torch.float16,
                         **from_fms_mo_kwargs):
    """In-place swap of every 8-bit QLinear for QLinearINT8Deploy, then optionally torch.compile
    (fms_mo/custom_ext_kernels/utils.py:805-866).  Like the reference it passes no quantizer choice
    to from_fms_mo, i.e. the static fms_mo-formula activation quantizer is what the modules get;
    extra keyword arguments (an extension: e.g. use_dynamic_max_act_Qfunc=-1) are handed through.  As in the reference the model is first moved to
    the host and cast to ``model_dtype`` together with all quantizer buffers, which puts the
    offline scale arithmetic in that dtype with the host's roundings; each module is converted on
    the target device and the model is moved back at the end."""
    from ..modules.linear import QLinear, QLinearINT8Deploy

    curr_dev = getattr(mod, "device", next(mod.parameters()).device)
    mod.cpu().to(model_dtype)
    cutlass_ops_load_and_reg(qcfg)
    for name, m in list(mod.named_modules()):
        if isinstance(m, QLinear):
            if m.num_bits_weight != 8 or m.num_bits_feature != 8:
                logger.warning("Only support INT8 lowering for now, cannot lower %s", name)
                continue
            parent_name, module_name = _parent_name(name)
            parent_mod = mod.get_submodule(parent_name)
            m.to(curr_dev)
            new_module = QLinearINT8Deploy.from_fms_mo(m, target_device=curr_dev, use_inductor=use_inductor,
                                                       **from_fms_mo_kwargs)
            setattr(parent_mod, module_name, new_module)
            m.to("cpu")
    mod.to(curr_dev)
    if use_inductor is True:
        use_inductor = "default"
    if use_inductor:
        _run_once(mod, exam_inp_eval)  # the deploy modules cache host-side decisions on an eager call
        with torch.no_grad():
            mod = torch.compile(mod, mode=use_inductor)
            _run_once(mod, exam_inp_eval)
    logger.info("Model lowered %s.", "and compiled" if use_inductor else "")
    return mod


def lower_qmodel_triton(model, use_dyn_max_act=False, max_acc_bits=32, clamp_acc_to_dl16=False,
                        num_lsb_to_truncate=0, chunk_size=32, layer_to_exclude=None):
    """In-place swap QLinear -> QLinearINT8Deploy(use_int_kernel='triton') and nn.Linear ->
    LinearFPxAcc, both running the chunked-accumulation HIP kernels
    (fms_mo/custom_ext_kernels/utils.py:869-959): simulation of accumulators with fewer bits
    (max_acc_bits), LSB truncation per K chunk and the DL16 accumulator range."""
    from ..modules.linear import LinearFPxAcc, QLinear, QLinearINT8Deploy

    lin_fp_dyn_code = ("per_token" if use_dyn_max_act in [-1, -2]
                       else "per_tensor" if use_dyn_max_act else False)
    if layer_to_exclude is None:
        layer_to_exclude = []
    elif isinstance(layer_to_exclude, str):
        layer_to_exclude = [layer_to_exclude]
    elif not isinstance(layer_to_exclude, (list, tuple)):
        raise RuntimeError("layer_to_exclude has to be either str, list, or tuple.")
    for name, m in list(model.named_modules()):
        if not isinstance(m, (QLinear, torch.nn.Linear)) or name in layer_to_exclude:
            continue
        parent_name, module_name = _parent_name(name)
        parent_mod = model.get_submodule(parent_name)
        if isinstance(m, QLinear):
            new_lin = QLinearINT8Deploy.from_fms_mo(
                m, use_int_kernel="triton", use_dynamic_max_act_Qfunc=use_dyn_max_act,
                max_acc_bits=max_acc_bits, truncate_lsb=num_lsb_to_truncate, chunk_size=chunk_size)
        else:
            new_lin = LinearFPxAcc.from_nn(
                m, trun_bits=num_lsb_to_truncate, chunk_size=chunk_size, dynamic_fp8=lin_fp_dyn_code,
                clamp_acc_to_dl16=clamp_acc_to_dl16)
        setattr(parent_mod, module_name, new_lin)
    logger.info("Model lowering with the chunked-accumulation kernels is done.")
    return model
