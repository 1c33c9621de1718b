"""Host-side logic that needs no GPU: quantizer state machines, module construction and
conversion (offline weight preparation) against the oracle, op registration, chunk-size rules."""
import pickle

import pytest
import torch

from oracle import qlinear_oracle as O


def gen(seed):
    return torch.Generator().manual_seed(seed)


def make_qlinear(K=128, N=96, smoothq=False, bias=True, qw_mode="maxperCh", dtype=torch.float16):
    from fms_mo_amd.modules.linear import QLinear

    qcfg = {"smoothq": smoothq, "smoothq_alpha": 0.5}
    m = QLinear(K, N, bias=bias, num_bits_feature=8, qa_mode="pertokenmax", num_bits_weight=8,
                qw_mode=qw_mode, qcfg=qcfg, device="cpu")
    g = gen(0)
    with torch.no_grad():
        m.weight.copy_(0.02 * torch.randn(N, K, generator=g))
        if bias:
            m.bias.copy_(0.01 * torch.randn(N, generator=g))
    m.to(dtype)
    m.quantize_weight.float()       # quantizer buffers stay fp32, as when they are created after .half()
    if smoothq:
        m.smoothq_act_scale = m.smoothq_act_scale.float()
        m.smoothq_alpha = m.smoothq_alpha.float()
    return m


def test_quantizer_factories_and_scope():
    from fms_mo_amd.quant import quantizers as Q

    assert isinstance(Q.get_activation_quantizer("pertokenmax", 8), Q.QMaxDynamic)
    assert Q.get_activation_quantizer("max_perCh", 8).reduce_dim == -2
    assert isinstance(Q.get_activation_quantizer("maxsym", 8), Q.Qmax)
    assert Q.get_weight_quantizer("maxperCh", 8, w_shape=(16, 32)).perCh == 16
    assert not Q.get_weight_quantizer("max", 8, w_shape=(16, 32)).perCh
    assert isinstance(Q.get_weight_quantizer("fp8_e4m3_scale_perCh", 8, w_shape=(16, 32)), Q.to_fp8)
    sawb = Q.get_weight_quantizer("sawb+perCh", 8, w_shape=(16, 32))
    assert isinstance(sawb, Q.SAWB) and sawb.per_channel_formula and sawb.clip_val.shape == (16,)
    assert not Q.get_weight_quantizer("sawb", 8, w_shape=(16, 32)).per_channel_formula
    for mode in ["pact+", "lsq+", "brecq"]:
        with pytest.raises(NotImplementedError):
            Q.get_activation_quantizer(mode, 8)
    with pytest.raises(ValueError):  # SAWB is a weight quantizer only, as in the reference's factory
        Q.get_activation_quantizer("sawb+", 8)
    with pytest.raises(ValueError):
        Q.get_weight_quantizer("nonsense", 8)


def test_qmaxdynamic_matches_oracle():
    from fms_mo_amd.quant.quantizers import QMaxDynamic

    x = (torch.randn(8, 64, generator=gen(1)) * 2).half()
    assert torch.equal(QMaxDynamic(8, dim=-1)(x), O.fake_quant_act_pertoken(x))
    with pytest.raises(ValueError):
        QMaxDynamic(8, dim=0)


def test_qmax_state_machine_and_per_channel_levels():
    from fms_mo_amd.quant.quantizers import Qmax

    W = (0.02 * torch.randn(16, 64, generator=gen(2)))
    q = Qmax(8, align_zero=True, perCh=16)
    assert torch.all(q.clip_val == 0)
    q.train()
    out = q(W)
    cv = W.abs().amax(dim=1)
    assert torch.allclose(q.clip_val, cv)                              # first call copies, EMA of equal values
    assert torch.equal(out, O.fake_quant_weight_perch(W, cv))
    q.eval()
    out2 = q(W * 0.5)                                                  # eval: stored clip values define the grid
    assert torch.equal(out2, O.fake_quant_weight_perch(W * 0.5, q.clip_val))
    q.train()
    q(W * 2)
    assert torch.allclose(q.clip_val, 0.9 * cv + 0.1 * 2 * cv, rtol=1e-6)   # moving average, factor 0.1
    # per-tensor variant: 254 levels, symmetric
    qt = Qmax(8, align_zero=True)
    qt.train()
    o = qt(W)
    step = W.abs().max() * 2 / 254
    assert torch.allclose(o / step, torch.round(o / step), atol=1e-3)
    assert torch.allclose(o, W, atol=step.item() / 2 + 1e-7)


def test_fp8_emulation_quantizer_closed_form():
    from fms_mo_amd.quant.quantizers import to_fp8

    x = (torch.randn(4, 64, generator=gen(3)) * 5).bfloat16()
    q = to_fp8(8, "fp8_e4m3_scale", perToken=True)
    s = 448 / x.abs().amax(dim=-1, keepdim=True).clamp(min=1e-12)     # multiplicative scale, in bf16
    expect = ((x * s).clamp(-448, 448).to(torch.float8_e4m3fn).to(torch.bfloat16) / s).to(torch.bfloat16)
    assert torch.equal(q(x), expect)
    sat = to_fp8(8, "fp8_e4m3_sat")
    assert sat(torch.tensor([1000.0, -1000.0, 0.3])).tolist() == [448.0, -448.0, 0.3125]
    with pytest.raises(ValueError):
        to_fp8(8, "fp8_e5m2_sat")


def test_qlinear_constructor_surface():
    m = make_qlinear(smoothq=True)
    for attr in ["quantize_feature", "quantize_weight", "num_bits_feature", "num_bits_weight", "qa_mode",
                 "qw_mode", "smoothq", "smoothq_act_scale", "smoothq_alpha", "qcfg", "calib_counter",
                 "num_module_called"]:
        assert hasattr(m, attr)
    assert m.smoothq_act_scale.shape == (128,) and m.smoothq_alpha.item() == 0.5
    assert "QLinear(128,96" in repr(m)
    with pytest.raises(KeyError):
        from fms_mo_amd.modules.linear import QLinear

        QLinear(8, 8, device="cpu")      # qcfg is required, like the reference
    m.set_act_scale(torch.ones(128))
    s = m.get_smoothq_scale(torch.zeros(1, 128, dtype=torch.float16))
    assert s.dtype == torch.float16 and s.shape == (1, 128)
    assert torch.equal(s, O.smoothq_scale_qlinear(m.weight, m.smoothq_act_scale, 0.5, torch.float16))


@pytest.mark.parametrize("smoothq", [False, True])
def test_from_fms_mo_offline_preparation_matches_oracle(smoothq):
    from fms_mo_amd.modules.linear import QLinearINT8Deploy, prepare_deploy_weights

    m = make_qlinear(smoothq=smoothq)
    act_scale = None
    if smoothq:
        act_scale = torch.rand(128, generator=gen(4)) * 8 + 0.5
        m.set_act_scale(act_scale)
    with torch.no_grad():
        m.quantize_weight.train()
        m.quantize_weight(m.weight)            # one training-mode pass initialises clip_val
    m.eval()
    dep = QLinearINT8Deploy.from_fms_mo(m, use_int_kernel="cutlass", use_dynamic_max_act_Qfunc=-1,
                                        recalc_clipvals=False, target_device="cpu")
    bufs = O.deploy_prepare(m.weight.detach(), m.bias.detach(), m.quantize_weight.clip_val, act_scale, 0.5)
    assert dep.weight.dtype == torch.int8 and torch.equal(dep.weight, bufs["weight"])
    assert torch.equal(dep.w_scale, bufs["w_scale"])
    assert torch.equal(dep.smoothq_scale, bufs["smoothq_scale"])
    assert torch.equal(dep.bias, bufs["bias"])
    assert dep.input_zp.item() == 127 and torch.all(dep.corr_term == 0) and torch.all(dep.w_zp == 0)
    assert dep._get_name() == "QLinear_INT8" and "int_kernel=cutlass" in dep.extra_repr()
    for name in ["input_scale", "input_zp", "w_scale", "w_zp", "smoothq_scale", "corr_term", "bias"]:
        assert name in dict(dep.named_buffers())
    # the standalone helper used by the benchmark performs the same recipe
    if not smoothq:
        w8, ws, sq = prepare_deploy_weights(m.weight.detach(), None, 0.5, m.quantize_weight.clip_val)
        assert torch.equal(w8, bufs["weight"]) and torch.equal(ws, bufs["w_scale"])
    # forward on CPU raises instead of taking some other path
    with pytest.raises(RuntimeError, match="no CPU path"):
        dep(torch.zeros(2, 128, dtype=torch.float16))
    # pickling drops and rebinds the op handles
    dep2 = pickle.loads(pickle.dumps(dep))
    assert torch.equal(dep2.weight, dep.weight) and callable(dep2.iaddmm)


def test_static_activation_variants_of_from_fms_mo():
    from fms_mo_amd.modules.linear import QLinearINT8Deploy

    m = make_qlinear()
    m.qa_mode = "maxsym"
    m.quantize_feature.clip_val = torch.tensor([4.0])
    m.quantize_feature.clip_valn = torch.tensor([-4.0])
    dep = QLinearINT8Deploy.from_fms_mo(m, use_PT_native_Qfunc=True, target_device="cpu")
    assert dep.useSymAct and dep.input_scale.item() == pytest.approx(8.0 / 254)
    assert dep.input_zp.item() == 127
    dep2 = QLinearINT8Deploy.from_fms_mo(m, target_device="cpu")          # fms_mo formula
    assert "quant_stepsize" in dict(dep2.named_buffers())
    assert dep2.input_scale.item() == pytest.approx(8.0 / 254)
    dep3 = QLinearINT8Deploy.from_fms_mo(m, use_dynamic_max_act_Qfunc=5, target_device="cpu")
    assert dep3.use_fake_zero_shift and dep3.input_zp.item() == 5
    w_sum = dep3.weight.to(torch.int).sum(dim=1)
    assert torch.allclose(dep3.corr_term, 5 * w_sum * dep3.w_scale.float() * 1.0)


def test_from_torch_iw():
    from fms_mo_amd.modules.linear import QLinearINT8Deploy

    lin = torch.nn.Linear(64, 32)
    with torch.no_grad():
        lin.weight.copy_(torch.randint(-127, 128, (32, 64), generator=gen(5)).float())
    dep = QLinearINT8Deploy.from_torch_iW(lin, "int8", 6.0, -2.0, 0.3, 0.0, target_device="cpu")
    assert dep.weight.dtype == torch.int8 and torch.equal(dep.weight.float(), lin.weight)
    assert dep.input_scale.item() == pytest.approx(8.0 / 255) and dep.input_zp.item() == round(2.0 / (8.0 / 255))
    assert dep.w_scale.item() == pytest.approx(0.6 / 254)


def test_custom_ops_are_registered_with_fake_impls():
    from fms_mo_amd.custom_ext_kernels.utils import imatmul_ops_reg, native_gemm_ops_reg

    imatmul_ops_reg()
    native_gemm_ops_reg()
    for ns, op in [("fms_mo", "imatmul"), ("fms_mo", "iaddmm"), ("fms_mo", "q_iaddmm_dq"),
                   ("fms_mo", "q_per_t_sym"), ("cutlass_gemm", "i8i32nt"), ("mygemm", "gemm_nt_i8i32")]:
        assert hasattr(getattr(torch.ops, ns), op)
    m1 = torch.empty(2, 3, 64, dtype=torch.int8, device="meta")
    m2 = torch.empty(64, 48, dtype=torch.int8, device="meta")
    out = torch.ops.fms_mo.imatmul(m1, m2)
    assert out.shape == (2, 3, 48) and out.dtype == torch.int32
    with pytest.raises((NotImplementedError, RuntimeError)):
        torch.ops.fms_mo.imatmul(torch.zeros(2, 64, dtype=torch.int8), torch.zeros(64, 8, dtype=torch.int8))


def test_chunk_wrapper_argument_rules():
    from fms_mo_amd.custom_ext_kernels.hip_kernels import matmul_chunk_truncate

    a = torch.zeros(4, 64)
    with pytest.raises(AssertionError, match="Incompatible dimensions"):
        matmul_chunk_truncate(a, torch.zeros(32, 8))
    with pytest.raises(AssertionError, match="dtypes inconsistent"):
        matmul_chunk_truncate(a, torch.zeros(64, 8, dtype=torch.float16))
    with pytest.raises(AssertionError, match="23 mantissa bits"):
        matmul_chunk_truncate(a, torch.zeros(64, 8), chunk_trun_bits=23)
    with pytest.raises(RuntimeError, match="no CPU path"):
        matmul_chunk_truncate(a, torch.zeros(64, 8))


def test_fp8_linear_construction_and_offline_quantization():
    from fms_mo_amd.modules.fp8_linear import FP8Linear, get_fp8_linear

    cfg = {"weights": {"strategy": "channel", "symmetric": True, "dynamic": False},
           "input_activations": {"strategy": "token", "symmetric": True, "dynamic": True}}
    m = get_fp8_linear(64, 32, True, cfg)
    assert m.weight.dtype == torch.float8_e4m3fn and m.weight_scale.shape == (32, 1) and m.bias.shape == (32,)
    W = 0.02 * torch.randn(32, 64, generator=gen(6))
    f = FP8Linear.from_float(W, None, per_channel=True)
    scale = (W.abs().amax(dim=1, keepdim=True) / 448).clamp(min=1e-12)
    assert torch.equal(f.weight_scale.data, scale)
    assert torch.equal(f.weight.data.view(torch.uint8), (W / scale).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8))
    assert "FP8Linear(in=64, out=32" in repr(f)
    with pytest.raises(RuntimeError, match="no CPU path"):
        f(torch.zeros(2, 64, dtype=torch.bfloat16))


def test_fp16_quotient_from_reciprocal_rounds_like_ieee_division():
    """The act-quant kernel forms fp16 quotients as q1 = fma(fma(-q0, s, e), r, q0), q0 = e r, with
    r a 1-ulp reciprocal, and rounds q1 to fp16.  Check against correctly rounded division over
    every pair of fp16 significands (normal results) and over subnormal results, with the
    reciprocal perturbed by -1, 0, +1 ulp."""
    import numpy as np

    def f32(a):
        return a.astype(np.float32)

    def fma32(a, b, c):  # products of a 24-bit and an 11/24-bit number are exact in float64
        return f32(a.astype(np.float64) * b.astype(np.float64) + c.astype(np.float64))

    sig = (1024 + np.arange(1024)).astype(np.float32)
    e, s = np.meshgrid(sig, sig, indexing="ij")
    e, s = e.ravel(), s.ravel()
    cases = [(e, s), (e * np.float32(2.0 ** -24), s * np.float32(2.0 ** -9)),   # quotients ~2^-15: subnormal
             (e * np.float32(2.0 ** -20), s * np.float32(2.0 ** -6)),           # ~2^-14 boundary
             (e * np.float32(2.0 ** -10), s)]                                   # ~2^-10..2^-9
    for e, s in cases:
        exact = (e.astype(np.float64) / s.astype(np.float64)).astype(np.float16)
        r0 = f32(np.float64(1.0) / s.astype(np.float64))
        for ulps in (-1, 0, 1):
            r = (r0.view(np.int32) + ulps).view(np.float32)
            q0 = f32(e.astype(np.float64) * r.astype(np.float64))
            q1 = fma32(fma32(-q0, s, e), r, q0)
            got = q1.astype(np.float16)
            assert np.array_equal(got.view(np.uint16), exact.view(np.uint16)), ulps


def test_fp32_quotient_by_two_residual_corrections_is_correctly_rounded():
    """The fp32-compute act-quant kernel divides as q0 = x r1, q <- fma(fma(-s, q, x), r1, q) twice,
    r1 = one Newton step on a 1-ulp reciprocal.  Emulated with exact rational arithmetic (every
    fma rounded once) and compared with the correctly rounded quotient, for fp16-valued x and
    random fp32 divisors, the hardware reciprocal modelled as the exact one moved by -1/0/+1 ulp."""
    import random
    from fractions import Fraction

    import numpy as np

    def rn32(fr):  # round a Fraction to the nearest fp32, ties to even (normal range only)
        if fr == 0:
            return Fraction(0)
        sign = -1 if fr < 0 else 1
        a = abs(fr)
        e = a.numerator.bit_length() - a.denominator.bit_length()
        if Fraction(2) ** e > a:
            e -= 1
        ulp = Fraction(2) ** (e - 23)
        n = a / ulp
        f = n.numerator // n.denominator
        rem = n - f
        if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and f % 2 == 1):
            f += 1
        return sign * f * ulp

    def fma(a, b, c):
        return rn32(a * b + c)

    rnd = random.Random(7)
    for trial in range(4000):
        xv = Fraction(float(np.float16(rnd.choice([-1, 1]) * rnd.uniform(0.001, 60000.0))))
        sv = Fraction(float(np.float32(rnd.uniform(0.3, 3.0) * 2.0 ** rnd.randint(-20, 20))))
        for ulps in (-1, 0, 1):
            r0 = rn32(1 / sv)
            r0 = r0 + ulps * Fraction(2) ** (int(np.floor(np.log2(float(r0)))) - 23)
            r1 = fma(fma(-sv, r0, Fraction(1)), r0, r0)
            q = rn32(xv * r1)
            q = fma(fma(-sv, q, xv), r1, q)
            q = fma(fma(-sv, q, xv), r1, q)
            assert q == rn32(xv / sv), (float(xv), float(sv), ulps)


def test_bf16_quotient_from_reciprocal_rounds_like_ieee_division():
    """Same construction for bf16 operands (8-bit significands): all 128 x 128 pairs, reciprocal
    off by -1/0/+1 ulp, result rounded to bf16 (RNE on the upper 16 bits of the fp32 pattern)."""
    import numpy as np

    def to_bf16_bits(a32):
        u = a32.view(np.uint32).astype(np.uint64)
        return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)

    sig = (128 + np.arange(128)).astype(np.float32)
    e, s = np.meshgrid(sig, sig, indexing="ij")
    e, s = e.ravel(), s.ravel()
    for e_, s_ in [(e, s), (e * np.float32(2.0 ** -7), s), (e, s * np.float32(2.0 ** 5))]:
        exact = to_bf16_bits((e_.astype(np.float64) / s_.astype(np.float64)).astype(np.float32))
        r0 = (np.float64(1.0) / s_.astype(np.float64)).astype(np.float32)
        for ulps in (-1, 0, 1):
            r = (r0.view(np.int32) + ulps).view(np.float32)
            q0 = (e_.astype(np.float64) * r.astype(np.float64)).astype(np.float32)
            t = (-q0.astype(np.float64) * s_.astype(np.float64) + e_.astype(np.float64)).astype(np.float32)
            q1 = (t.astype(np.float64) * r.astype(np.float64) + q0.astype(np.float64)).astype(np.float32)
            assert np.array_equal(to_bf16_bits(q1), exact), ulps


def test_sawb_recompute_per_tensor_returns_the_sawb_integers_unguarded():
    """recompute_weight_with_sawb, per tensor, when the statistics-aware clip is not below the
    tensor maximum: the reference builds the guarded integers (fms_mo/utils/aiu_utils.py:196-199)
    but returns the SAWB integers themselves (:235) beside the guarded clip value.  The writer and
    the oracle reproduce that; per channel the guarded rows are what is returned."""
    from fms_mo_amd.utils import aiu_utils as A

    g = torch.Generator().manual_seed(5)
    w = (0.01 * torch.randn(8, 8, generator=g)).half()
    w[2, 3] = 1.0                          # one outlier among 64 weights: SAWB's clip exceeds it
    w_int = torch.round(w.float() * 127).clamp(-127, 127)
    assert w_int.std() < A.STD_THRESHOLD
    new_sd = {}
    got, recomputed = A.recompute_weight_with_sawb(w, w_int.to(w.dtype), False, None, "lin", new_sd)
    ref_int, ref_cv = O.aiu_recompute_narrow(w, w_int.to(w.dtype), False)
    clip = O.sawb_clip(w.float(), 8, perCh=False)
    assert recomputed and clip > w.abs().max()                      # the case in question
    assert torch.equal(new_sd["lin.quantize_weight.clip_val"], ref_cv)
    assert ref_cv.item() == w.abs().max().item()                    # the clip value is guarded ...
    assert torch.equal(got, ref_int)
    assert torch.equal(got, O.sawb_zero_forward(w.float(), clip, 8, dequantize=False))   # ... the integers are not
    assert not torch.equal(got, w_int)
    assert got.abs().max() < 127                                    # quantized against the larger clip
