"""GPU parity of the deploy branches beside the per-token one: static PT-native and fms_mo-formula
quantizers with asymmetric zero points (correction term folded into the bias), from_torch_iW,
dynamic per-channel (dim -2) and fake-zero-shift quantizers, the cuBLAS / CUTLASS style modules,
the lowering helpers, and the FP8 emulation quantizers.  Conversion runs on the CPU (the host
roundings of the reference's lowering helpers), the forward on the GPU; int8 codes and fp16 / fp32
outputs are compared bit for bit with the oracle."""
import pytest
import torch

from oracle import qlinear_oracle as O

pytestmark = pytest.mark.gpu


def gen(seed):
    return torch.Generator().manual_seed(seed)


def Kn():
    from fms_mo_amd import kernels

    return kernels


def bits(t):
    return t.contiguous().view(torch.int16 if t.element_size() == 2 else torch.int32)


def static_x(M, K, seed, dtype=torch.float16):
    """Off-centre activations with values beyond both clip values and exact ties of x / scale."""
    x = torch.randn(M, K, generator=gen(seed)) * 1.7 + 0.6
    x[0, :8] = torch.tensor([100.0, -100.0, 0.0, -0.0, 5.5, -3.25, 1e-4, -1e-4])
    return x.to(dtype)


def make_static_qlinear(K, N, qa_mode, a_cv, a_cvn, seed=0, dtype=torch.float16, bias=True, buffers_fp32=True):
    """A QLinear whose activation quantizer holds calibrated clip values (what PTQ / QAT leaves)."""
    from fms_mo_amd.modules.linear import QLinear

    m = QLinear(K, N, bias=bias, num_bits_feature=8, qa_mode=qa_mode, num_bits_weight=8,
                qw_mode="maxperCh", qcfg={"smoothq": False}, device="cpu")
    g = gen(seed)
    with torch.no_grad():
        m.weight.copy_(0.03 * torch.randn(N, K, generator=g))
        if bias:
            m.bias.copy_(0.05 * torch.randn(N, generator=g))
        m.quantize_feature.clip_val.fill_(a_cv)
        m.quantize_feature.clip_valn.fill_(a_cvn)
    m.to(dtype)
    if buffers_fp32:
        m.quantize_weight.float()
        m.quantize_feature.float()
        with torch.no_grad():   # the values the fp32 buffers would hold had they never been cast
            m.quantize_feature.clip_val.fill_(a_cv)
            m.quantize_feature.clip_valn.fill_(a_cvn)
    with torch.no_grad():
        m.quantize_weight.train()
        m.quantize_weight(m.weight)
    return m.eval()


# ----------------------------------------------------------------------- quantizer kernels
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("own_dtype", [True, False])
def test_static_quantizer_kernels_in_every_compute_dtype(dev, dtype, own_dtype):
    """The four static formulas with the scale tensor in x's dtype (T = that dtype) or fp32."""
    from fms_mo_amd import _lib as L

    x = static_x(33, 256, 1, dtype)
    sdt = dtype if own_dtype else torch.float32
    T = torch.promote_types(dtype, sdt)
    scale = torch.tensor([0.0343]).to(sdt)
    zp = torch.tensor([95], dtype=torch.int)
    xd = x.to(dev)
    for sym in (0, 1):
        ref = O.quant_act_static_raw(x, scale, zp, sym)
        q = Kn().quant_act_i8_static_t(xd, L.SQ_RAW, T, float(scale), 95, sym)
        assert torch.equal(q.cpu(), ref), ("raw", sym)
    # fms_mo formula: bounds, step and zero point as the module would hold them
    cvn, cv = torch.tensor([-3.25]).to(sdt), torch.tensor([5.5]).to(sdt)
    qs = 255 / torch.tensor([cv - cvn])
    step, qzp = 1.0 / qs, torch.round(cvn * qs)
    ref = O.quant_act_fmo_mo(x, cvn, cv, step, qzp, 0)
    q = Kn().quant_act_i8_static_t(xd, L.SQ_FMO, (x.clamp(cvn, cv) / step).dtype, float(step), float(qzp), 0,
                                   float(cvn), float(cv))
    assert torch.equal(q.cpu(), ref)
    assert ref.min() == -128 and ref.max() >= 126          # both clip values are hit
    # the uint8-shift and narrow-int8 quantizers of the cuBLAS / CUTLASS style modules
    r = (x / scale + zp).round()
    ref_u8 = (torch.clamp(r, 0, 255).to(torch.int16) - 128).to(torch.int8)
    ref_s8 = torch.clamp((x / scale + torch.tensor([3], dtype=torch.int)).round(), -127, 127).to(torch.int8)
    assert torch.equal(Kn().quant_act_i8_static_t(xd, L.SQ_U8_SHIFT, T, float(scale), 95).cpu(), ref_u8)
    assert torch.equal(Kn().quant_act_i8_static_t(xd, L.SQ_S8_NARROW, T, float(scale), 3).cpu(), ref_s8)


def test_static_quantizer_fp16_exact_ties(dev):
    """x / scale + zp lands exactly on .5 for a power-of-two scale: half to even in fp16."""
    from fms_mo_amd import _lib as L

    scale = torch.tensor([0.25], dtype=torch.float16)
    x = (torch.arange(-300, 300).float() * 0.125).half().reshape(1, -1)     # quotients k / 2
    x = torch.nn.functional.pad(x, (0, (-x.shape[1]) % 8))
    zp = torch.tensor([7], dtype=torch.int)
    ref = O.quant_act_static_raw(x, scale, zp, 0)
    q = Kn().quant_act_i8_static_t(x.to(dev), L.SQ_RAW, torch.float16, 0.25, 7, 0)
    assert torch.equal(q.cpu(), ref)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_static_quantizer_16bit_kernel_on_every_pattern(dev, dtype):
    """Contiguous rows in a 16-bit compute dtype take a kernel with a three-operation quotient instead
    of the IEEE division.  Every 16-bit pattern of x: bit-identical to the generic kernel (which a
    padded output selects) for all four formulas, NaN and infinities included, and to the oracle on
    the finite patterns.  Parameters outside the fast kernel's domain (a scale that is not a value
    of the dtype, fp16 quotients that overflow) must give the generic kernel's codes as well."""
    from fms_mo_amd import _lib as L

    code = L.F16 if dtype == torch.float16 else L.BF16
    pats = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype).reshape(8, 8192).contiguous()
    xd = pats.to(dev)
    M, K = pats.shape
    lib, st = L.load(), torch.cuda.current_stream().cuda_stream
    finite = torch.isfinite(pats.float())

    def both(mode, scale, zp, sym, lo, hi):
        qf = torch.empty(M, K, dtype=torch.int8, device=dev)
        qg = torch.empty(M, K + 8, dtype=torch.int8, device=dev)
        for q, ld in ((qf, K), (qg, K + 8)):
            assert lib.fmsmo_quant_act_i8_static_t(xd.data_ptr(), code, K, mode, code, scale, zp, sym, lo, hi,
                                                   q.data_ptr(), ld, M, K, st) == 0
        torch.cuda.synchronize()
        assert torch.equal(qf, qg[:, :K]), (mode, scale, zp, sym, lo, hi)
        return qf.cpu()

    t = lambda v: float(torch.tensor(v, dtype=dtype))
    for scale, zp, sym in ((t(0.0343), 95.0, 0), (t(0.0343), 95.0, 1), (t(1.0), 0.0, 0), (t(250.0), -5.0, 1),
                           (t(6.1e-5), 128.0, 0), (0.0343, 3.0, 0)):          # the last: not a value of the dtype
        q = both(L.SQ_RAW, scale, zp, sym, 0.0, 0.0)
        if t(scale) == scale:
            ref = O.quant_act_static_raw(pats, torch.tensor([scale], dtype=dtype), torch.tensor([int(zp)], dtype=torch.int), sym)
            assert torch.equal(q[finite], ref[finite]), ("raw", scale, zp, sym)
        both(L.SQ_U8_SHIFT, scale, zp, 0, 0.0, 0.0)
        both(L.SQ_S8_NARROW, scale, zp, 0, 0.0, 0.0)
    for (cvn, cv), sym in (((-3.25, 5.5), 0), ((-3.25, 5.5), 1), ((-0.01, 0.0), 0), ((-1e4, 1e4), 0)):
        cvn_t, cv_t = torch.tensor([cvn], dtype=dtype), torch.tensor([cv], dtype=dtype)
        qs = 255 / (cv_t - cvn_t)
        step, qzp = 1.0 / qs, torch.round(cvn_t * qs)
        q = both(L.SQ_FMO, float(step), float(qzp), sym, float(cvn_t), float(cv_t))
        ref = O.quant_act_fmo_mo(pats, cvn_t, cv_t, step, qzp, sym)
        assert torch.equal(q[finite], ref[finite]), ("fmo", cvn, cv, sym)
    # fp16 quotients that overflow to inf: the generic kernel's conversion, whichever kernel runs
    both(L.SQ_FMO, t(3.0e-5), 3.0, 1, -2.5, 3.0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_dynamic_per_tensor_quantizer_16bit_kernel_on_every_pattern(dev, dtype):
    """The per-tensor dynamic quantizer on contiguous 16-bit rows (fast quotient) against the generic
    kernel (padded output) on every 16-bit pattern of x, for abs-max values from under the 1e-5
    floor to infinity and NaN; and against the oracle's formula where the abs-max is the data's."""
    from fms_mo_amd import _lib as L

    code = L.F16 if dtype == torch.float16 else L.BF16
    pats = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype).reshape(8, 8192).contiguous()
    xd = pats.to(dev)
    M, K = pats.shape
    lib, st = L.load(), torch.cuda.current_stream().cuda_stream
    for amax in (1.0, 6.0, 65504.0, 1e-7, 3.0e-3, 1.0e21, 3.0e38, float("inf"), float("nan")):
        for levels, zp in ((127, 0), (126, 1), (110, 17), (63, 64)):
            col = torch.zeros(K, device=dev)
            col[K // 3] = amax
            out = []
            for ld in (K, K + 8):
                q = torch.empty(M, ld, dtype=torch.int8, device=dev)
                sc = torch.empty(1, dtype=torch.float32, device=dev)
                assert lib.fmsmo_quant_act_i8_dynamic(xd.data_ptr(), code, K, col.data_ptr(), 0, levels, zp,
                                                      q.data_ptr(), ld, sc.data_ptr(), M, K, st) == 0
                out.append((q[:, :K].clone(), sc.clone()))
            torch.cuda.synchronize()
            assert torch.equal(out[0][0], out[1][0]) and torch.equal(out[0][1], out[1][1]), (amax, levels, zp)
    # the data's own abs-max, finite values only: the oracle
    x = pats.clone()
    x[~torch.isfinite(x.float())] = 0
    for zp in (1, 64):
        ref_q, ref_s = O.quant_act_fake_zero_shift(x, torch.tensor(zp, dtype=torch.int))
        q, sc = Kn().quant_act_i8_dynamic(x.to(dev), False, 127 - zp, zp)
        assert torch.equal(sc.cpu().reshape(()), ref_s.float()) and torch.equal(q.cpu(), ref_q), zp


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_dynamic_per_tensor_and_per_column_quantizers(dev, dtype):
    x = (torch.randn(70, 384, generator=gen(2)) * torch.linspace(0.01, 4, 384)).to(dtype)
    x[:, 5] = 0                                              # an all-zero column: the 1e-5 floor
    for zp in (1, 17, 64):
        ref_q, ref_s = O.quant_act_fake_zero_shift(x, torch.tensor(zp, dtype=torch.int))
        q, s = Kn().quant_act_i8_dynamic(x.to(dev), False, 127 - zp, zp)
        assert torch.equal(s.cpu().reshape(()), ref_s.float()) and torch.equal(q.cpu(), ref_q), zp
    ref_q, ref_s = O.quant_act_dyn_max(x, -2)
    q, s = Kn().quant_act_i8_dynamic(x.to(dev), True, 127)
    assert torch.equal(s.cpu(), ref_s.float().reshape(-1)) and torch.equal(q.cpu(), ref_q)


# ------------------------------------------------------------------- deploy module, static
@pytest.mark.parametrize("pt_native", [True, False])
@pytest.mark.parametrize("regime", ["fp32_buffers", "all_fp16"])
@pytest.mark.parametrize("qa", [("minmax", 5.5, -3.25), ("max", 6.0, -6.0)])
def test_deploy_module_static_branches_bit_exact(dev, pt_native, regime, qa):
    """Asymmetric ('minmax': zero point != 128, non-zero correction term) and symmetric ('max')
    static activation quantizers, with the quantizer buffers left in fp32 (the quantizers are
    created after model.half() in the reference's flow) or cast to fp16 with the model (what its
    lowering helpers do first)."""
    from fms_mo_amd.modules.linear import QLinearINT8Deploy

    qa_mode, a_cv, a_cvn = qa
    K, N, M = 256, 192, 75
    m = make_static_qlinear(K, N, qa_mode, a_cv, a_cvn, seed=3, buffers_fp32=(regime == "fp32_buffers"))
    x = static_x(M, K, 4)
    dep = QLinearINT8Deploy.from_fms_mo(m, use_int_kernel="cutlass", use_PT_native_Qfunc=pt_native,
                                        recalc_clipvals=False, target_device=dev)
    Qa, Qw = m.quantize_feature, m.quantize_weight
    st = O.deploy_prepare_general(m.weight.detach(), m.bias.detach(), Qw.clip_val, Qa.clip_val, Qa.clip_valn,
                                  sym_act=(qa_mode == "max"), use_PT_native_Qfunc=pt_native)
    assert torch.equal(dep.weight.cpu(), st["weight"])
    assert int(dep.input_zp) == int(st["input_zp"]) and (qa_mode == "max" or int(dep.input_zp) != 128)
    assert torch.equal(dep.corr_term.cpu(), st["corr_term"]) and torch.equal(dep.bias.cpu(), st["bias"])
    assert torch.equal(dep.input_scale.cpu(), st["input_scale"]) and dep.w_scale.dtype == st["w_scale"].dtype
    if qa_mode == "minmax":
        assert dep.corr_term.abs().max() > 1e-2
    ref = O.deploy_forward_general(x, st)
    q = dep._quantize(x.to(dev))
    assert torch.equal(q.cpu(), ref["q_x"])
    y = dep(x.to(dev))
    assert y.dtype == torch.float16 and torch.equal(bits(y.cpu()), bits(ref["y"]))
    # a 3-D input and the PT-native library form of the same quantizer
    y3 = dep(x.to(dev).reshape(3, 25, K))
    assert torch.equal(bits(y3.cpu().reshape(M, N)), bits(ref["y"]))
    if pt_native and regime == "fp32_buffers":
        qt = dep.qa_pt_quant_func(x.to(dev))
        assert torch.equal(qt.cpu(), O.quant_act_pt_native(x, st["input_scale"], st["input_zp"], st["useSymAct"]))


def test_deploy_module_static_branches_random_layers(dev):
    """Sixteen seeded layers through the static branches: random clip values (asymmetric and
    symmetric), both formulas, both buffer regimes, with and without bias, any M, K a multiple of
    64, N a multiple of 8: buffers, integer codes and outputs are the oracle's bit for bit."""
    import random

    from fms_mo_amd.modules.linear import QLinearINT8Deploy

    rng = random.Random(13579)
    for case in range(16):
        sym = rng.random() < 0.4
        a_cv = round(rng.uniform(2.0, 8.0), 3)
        a_cvn = -a_cv if sym else -round(rng.uniform(0.5, 6.0), 3)
        pt_native, fp32_buffers, bias = rng.random() < 0.5, rng.random() < 0.5, rng.random() < 0.7
        K, N = 64 * rng.randint(1, 40), 8 * rng.randint(1, 120)
        M = rng.choice([1, rng.randint(2, 16), rng.randint(17, 300)])
        tag = (f"case {case}: sym={sym} cv={a_cv}/{a_cvn} pt_native={pt_native} fp32_buffers={fp32_buffers} "
               f"bias={bias} M={M} K={K} N={N}")
        m = make_static_qlinear(K, N, "max" if sym else "minmax", a_cv, a_cvn, seed=100 + case, bias=bias,
                                buffers_fp32=fp32_buffers)
        x = static_x(M, K, 200 + case)
        dep = QLinearINT8Deploy.from_fms_mo(m, use_int_kernel="cutlass", use_PT_native_Qfunc=pt_native,
                                            recalc_clipvals=False, target_device=dev)
        Qa, Qw = m.quantize_feature, m.quantize_weight
        st = O.deploy_prepare_general(m.weight.detach(), m.bias.detach() if bias else None, Qw.clip_val,
                                      Qa.clip_val, Qa.clip_valn, sym_act=sym, use_PT_native_Qfunc=pt_native)
        assert torch.equal(dep.weight.cpu(), st["weight"]) and int(dep.input_zp) == int(st["input_zp"]), tag
        assert torch.equal(bits(dep.corr_term.cpu()), bits(st["corr_term"])), tag
        assert torch.equal(bits(dep.bias.cpu()), bits(st["bias"])), tag
        ref = O.deploy_forward_general(x, st)
        assert torch.equal(dep._quantize(x.to(dev)).cpu(), ref["q_x"]), tag
        y = dep(x.to(dev))
        assert torch.equal(bits(y.cpu()), bits(ref["y"])), tag


@pytest.mark.parametrize("pt_native", [True, False])
@pytest.mark.parametrize("acc_dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("with_bias", [True, False])
def test_from_torch_iW_bit_exact(dev, pt_native, acc_dtype, with_bias):
    """A layer that already holds integer weights (AIU-style checkpoint) with per-channel zero
    shift: buffers, int8 codes and the output in the module's accumulator dtype (fp32 default)."""
    import json

    from fms_mo_amd.modules.linear import QLinearINT8Deploy

    K, N, M = 320, 128, 50
    g = gen(5)
    w_int = torch.randint(-127, 128, (N, K), generator=g).float()
    lin = torch.nn.Linear(K, N, bias=with_bias)
    with torch.no_grad():
        lin.weight.copy_(w_int)
        if with_bias:
            lin.bias.copy_(0.1 * torch.randn(N, generator=g))
    a_cv, a_cvn, w_cv = 4.75, -2.5, 0.21
    zero_shift = w_int.sum(dim=1).tolist()
    dep = QLinearINT8Deploy.from_torch_iW(lin, "int8", a_cv, a_cvn, w_cv, json.dumps(zero_shift),
                                          use_PT_native_Qfunc=pt_native, acc_dtype=acc_dtype,
                                          use_int_kernel="cutlass", target_device=dev)
    st = O.deploy_from_torch_iW(w_int, lin.bias.detach() if with_bias else None, a_cv, a_cvn, w_cv, zero_shift,
                                use_PT_native_Qfunc=pt_native, acc_dtype=acc_dtype)
    assert torch.equal(dep.weight.cpu(), st["weight"]) and torch.equal(dep.corr_term.cpu(), st["corr_term"])
    assert dep.bias.dtype == acc_dtype and torch.equal(dep.bias.detach().cpu(), st["bias"])
    assert int(dep.input_zp) == int(st["input_zp"]) != 128
    for dtype in (torch.float16, torch.float32):
        x = static_x(M, K, 6, dtype)
        ref = O.deploy_forward_general(x, st)
        assert torch.equal(dep._quantize(x.to(dev)).cpu(), ref["q_x"])
        y = dep(x.to(dev))
        assert y.dtype == dtype and torch.equal(bits(y.cpu()), bits(ref["y"])), dtype


# ----------------------------------------------------------------- deploy module, dynamic
@pytest.mark.parametrize("zp", [1, 17, 64])
def test_deploy_module_fake_zero_shift_bit_exact(dev, zp):
    from fms_mo_amd.modules.linear import QLinearINT8Deploy
    from tests.test_gpu_modules import make_qlinear

    K, N, M = 512, 256, 40
    m = make_qlinear(None, K, N, seed=7)
    x = static_x(M, K, 8)
    dep = QLinearINT8Deploy.from_fms_mo(m, use_int_kernel="cutlass", use_dynamic_max_act_Qfunc=zp,
                                        recalc_clipvals=False, target_device=dev)
    st = O.deploy_prepare_general(m.weight.detach(), m.bias.detach(), m.quantize_weight.clip_val,
                                  use_dynamic_max_act_Qfunc=zp)
    assert dep.use_fake_zero_shift and torch.equal(dep.corr_term.cpu(), st["corr_term"])
    assert torch.equal(dep.bias.cpu(), st["bias"])
    ref = O.deploy_forward_general(x, st)
    y = dep(x.to(dev))
    assert dep.input_scale.dim() == 0 and dep.input_scale.dtype == torch.float16
    assert torch.equal(dep.input_scale.cpu(), ref["input_scale"])
    assert torch.equal(dep._quantize(x.to(dev)).cpu(), ref["q_x"])
    assert torch.equal(bits(y.cpu()), bits(ref["y"]))


@pytest.mark.parametrize("qw_mode", ["sawb+", "sawb", "sawb+perCh"])
@pytest.mark.parametrize("smoothq", [False, True])
def test_deploy_module_from_a_sawb_weight_quantizer(dev, qw_mode, smoothq):
    """from_fms_mo takes the integer weights from a SAWB quantizer's own output (linear.py:859-861).
    The clip value comes from one training-mode pass over the weights (quantizers.py:633-672), the
    conversion runs on the CPU, the forward on the GPU; weights, scales, bias and output against
    the oracle, bit for bit."""
    from fms_mo_amd.modules.linear import QLinear, QLinearINT8Deploy
    from fms_mo_amd.quant.quantizers import SAWB

    K, N, M = 512, 192, 33
    m = QLinear(K, N, bias=True, num_bits_feature=8, qa_mode="pertokenmax", num_bits_weight=8,
                qw_mode=qw_mode, qcfg={"smoothq": smoothq, "smoothq_alpha": 0.5}, device="cpu")
    g = gen(21)
    with torch.no_grad():
        m.weight.copy_(0.02 * torch.randn(N, K, generator=g))
        m.bias.copy_(0.01 * torch.randn(N, generator=g))
    m.to(torch.float16)
    Qw = m.quantize_weight
    assert isinstance(Qw, SAWB) and Qw.per_channel_formula == (qw_mode == "sawb+perCh")
    Qw.float()
    act_scale = None
    if smoothq:
        act_scale = (torch.rand(K, generator=g) * 4 + 0.1)
        m.smoothq_act_scale = act_scale.clone()
        m.smoothq_alpha = m.smoothq_alpha.float()
    with torch.no_grad():
        Qw.train()
        Qw(m.weight.float())
    m.eval()
    ref_clip = O.sawb_clip(m.weight.detach().float(), 8, perCh=Qw.per_channel_formula)
    assert torch.equal(Qw.clip_val.reshape(-1), ref_clip.reshape(-1)) and (ref_clip > 0).all()
    dep = QLinearINT8Deploy.from_fms_mo(m, use_int_kernel="cutlass", use_dynamic_max_act_Qfunc=-1,
                                        recalc_clipvals=False, target_device=dev)
    st = O.deploy_prepare_general(m.weight.detach(), m.bias.detach(), Qw.clip_val, act_scale=act_scale,
                                  use_dynamic_max_act_Qfunc=-1,
                                  sawb="perCh" if Qw.per_channel_formula else "tensor")
    assert torch.equal(dep.weight.cpu(), st["weight"]) and st["weight"].abs().max() == 127
    assert torch.equal(dep.w_scale.cpu(), st["w_scale"]) and torch.equal(bits(dep.bias.cpu()), bits(st["bias"]))
    x = static_x(M, K, 22)
    ref = O.deploy_forward_general(x, st)
    y = dep(x.to(dev))
    if not smoothq:  # (with SmoothQuant the division is fused into the forward's quantizer launch)
        assert torch.equal(dep._quantize(x.to(dev)).cpu(), ref["q_x"])
    assert torch.equal(bits(y.cpu()), bits(ref["y"]))


def test_deploy_module_per_channel_dynamic_bit_exact(dev):
    """use_dynamic_max_act_Qfunc = -2: one scale per input channel over the tokens; the reference's
    [1,K] scale broadcasts against the [M,N] accumulator, so the layer is square."""
    from fms_mo_amd.modules.linear import QLinearINT8Deploy
    from tests.test_gpu_modules import make_qlinear

    K = N = 256
    m = make_qlinear(None, K, N, seed=9)
    x = (torch.randn(48, K, generator=gen(10)) * torch.linspace(0.1, 5, K)).half()
    dep = QLinearINT8Deploy.from_fms_mo(m, use_int_kernel="cutlass", use_dynamic_max_act_Qfunc=-2,
                                        recalc_clipvals=False, target_device=dev)
    st = O.deploy_prepare_general(m.weight.detach(), m.bias.detach(), m.quantize_weight.clip_val,
                                  use_dynamic_max_act_Qfunc=-2)
    ref = O.deploy_forward_general(x, st)
    y = dep(x.to(dev))
    assert dep.input_scale.shape == (1, K) and torch.equal(dep.input_scale.cpu(), ref["input_scale"])
    assert torch.equal(dep._quantize(x.to(dev)).cpu(), ref["q_x"])
    assert torch.equal(bits(y.cpu()), bits(ref["y"]))
    m2 = make_qlinear(None, 256, 128, seed=9)
    dep2 = QLinearINT8Deploy.from_fms_mo(m2, use_dynamic_max_act_Qfunc=-2, recalc_clipvals=False, target_device=dev)
    with pytest.raises(RuntimeError, match="in_features == out_features"):
        dep2(x.to(dev))


@pytest.mark.parametrize("cfg", [(48, 3, 20), (100, 0, 32), (96, 2, 32)])
def test_deploy_chunk_loop_with_any_chunk_size(dev, cfg):
    """Chunk sizes that are not powers of two (ragged last chunk included) run the reference's
    serial loop, one exact int32 GEMM per chunk."""
    from fms_mo_amd.modules.linear import QLinearINT8Deploy
    from tests.test_gpu_modules import make_qlinear

    chunk, t, accbits = cfg
    K, N = 520, 128
    m = make_qlinear(None, K, N, seed=11)
    x = static_x(37, K, 12)
    dep = QLinearINT8Deploy.from_fms_mo(m, use_int_kernel="cutlass", use_dynamic_max_act_Qfunc=-1,
                                        recalc_clipvals=False, chunk_size=chunk, truncate_lsb=t,
                                        max_acc_bits=accbits, target_device=dev)
    st = O.deploy_prepare_general(m.weight.detach(), m.bias.detach(), m.quantize_weight.clip_val,
                                  use_dynamic_max_act_Qfunc=-1)
    ref = O.deploy_forward_general(x, st, chunk_size=chunk, truncate_lsb=t, max_acc_bits=accbits)
    y = dep(x.to(dev))
    assert torch.equal(bits(y.cpu()), bits(ref["y"]))


# ------------------------------------------------------------ cuBLAS / CUTLASS style modules
@pytest.mark.parametrize("cls_name", ["QLinearCublasI8I32NT", "QLinearCutlassI8I32NT"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_i8i32nt_modules_bit_exact(dev, cls_name, dtype):
    import fms_mo_amd.modules.linear as ML

    cls = getattr(ML, cls_name)
    assert cls in ML.QLinear_modules
    K, N = 384, 160
    m = make_static_qlinear(K, N, "minmax", 5.0, -3.0, seed=13, dtype=dtype)
    Qa, Qw = m.quantize_feature, m.quantize_weight
    st = O.i8i32nt_from_fms_mo(m.weight.detach(), m.bias.detach(), Qa.clip_val, Qa.clip_valn, Qw.clip_val)
    mod = cls.from_fms_mo(m, target_device=dev)
    assert mod._get_name() == ("QuantizedLinear_cublasi8i32" if "Cublas" in cls_name else "QuantizedLinear_cutlassi8i32")
    assert torch.equal(mod.weight.cpu(), st["weight"]) and torch.equal(mod.bias.detach().cpu(), st["bias"])
    assert torch.equal(mod.input_zp.cpu(), st["input_zp"]) and mod.input_dtype == torch.quint8
    x = static_x(2 * 31, K, 14, dtype).reshape(2, 31, K)
    ref = O.i8i32nt_forward(x, st)
    y = mod(x.to(dev))
    assert y.shape == (2, 31, N) and y.dtype == dtype
    assert torch.equal(bits(y.cpu()), bits(ref["y"]))
    # symmetric (qint8) activations: clamp to +-127, zero point inside the rounding
    mod.input_dtype = torch.qint8
    st_s = dict(st, input_dtype=torch.qint8)
    ref_s = O.i8i32nt_forward(x, st_s)
    assert torch.equal(bits(mod(x.to(dev)).cpu()), bits(ref_s["y"]))
    if "Cublas" in cls_name:
        with pytest.raises(RuntimeError):
            mod(x.to(dev).reshape(1, 2, 31, K))


# --------------------------------------------------------------------------- lowering helpers
class TwoLayer(torch.nn.Module):
    def __init__(self, K, H, qa_mode="pertokenmax"):
        super().__init__()
        from fms_mo_amd.modules.linear import QLinear

        mk = lambda i, o: QLinear(i, o, bias=True, num_bits_feature=8, qa_mode=qa_mode, num_bits_weight=8,  # noqa: E731
                                  qw_mode="maxperCh", qcfg={"smoothq": False}, device="cpu")
        self.up, self.down = mk(K, H), mk(H, K)
        self.plain = torch.nn.Linear(K, K, bias=False)

    def forward(self, x):
        return self.plain(self.down(torch.nn.functional.gelu(self.up(x))))


def _two_layer(K=256, H=512, qa_mode="pertokenmax", seed=20):
    torch.manual_seed(seed)
    net = TwoLayer(K, H, qa_mode)
    with torch.no_grad():
        for lin in (net.up, net.down):
            lin.weight.mul_(0.5)
    net.half()
    for lin in (net.up, net.down):
        lin.quantize_weight.float()
        with torch.no_grad():
            lin.quantize_weight.train()
            lin.quantize_weight(lin.weight)
    return net.eval()


def _oracle_two_layer(net_cpu, x, **prep):
    """The same two deploy layers through the oracle (conversion from the fp16-cast CPU model)."""
    h = x
    outs = []
    for lin in (net_cpu.up, net_cpu.down):
        cv = lin.quantize_weight.clip_val
        st = O.deploy_prepare_general(lin.weight.detach(), lin.bias.detach(), cv, **prep)
        h = O.deploy_forward_general(h, st)["y"]
        outs.append(h)
        if lin is net_cpu.up:
            h = torch.nn.functional.gelu(h.float()).half()
    return outs


def test_lower_qmodel_to_ext_kernels_and_cutlass_helper(dev):
    import copy

    from fms_mo_amd.custom_ext_kernels.utils import lower_qmodel_cutlass
    from fms_mo_amd.fx.utils import lower_qmodel_to_ext_kernels
    from fms_mo_amd.modules.linear import QLinear, QLinearINT8Deploy

    net = _two_layer()
    ref_net = copy.deepcopy(net)
    ref_net.half()                                           # the helpers cast buffers to model_dtype
    for lin in (ref_net.up, ref_net.down):
        lin.quantize_weight.half()
    x = torch.randn(24, 256, generator=gen(21)).half()
    net.to(dev)
    qcfg = {"ext_kernel_mapping_mod": {QLinear: QLinearINT8Deploy}}
    low = lower_qmodel_to_ext_kernels(copy.deepcopy(net), x.to(dev), qcfg, useInductor=False,
                                      use_dynamic_max_act_Qfunc=-1, recalc_clipvals=False)
    assert isinstance(low.up, QLinearINT8Deploy) and isinstance(low.down, QLinearINT8Deploy)
    assert type(low.plain) is torch.nn.Linear and low.up.weight.is_cuda and low.up.weight.dtype == torch.int8
    refs = _oracle_two_layer(ref_net, x, use_dynamic_max_act_Qfunc=-1)
    up_out = low.up(x.to(dev))
    assert torch.equal(bits(up_out.cpu()), bits(refs[0]))
    # the cutlass helper passes no quantizer choice, like the reference: static fms_mo formula
    # with the default +-8 activation clip values for a quantizer without stored ones
    low2 = lower_qmodel_cutlass(copy.deepcopy(net), None, {}, use_inductor=False, recalc_clipvals=False)
    assert isinstance(low2.up, QLinearINT8Deploy) and not low2.up.usePTnativeQfunc and low2.up.useDynMaxQfunc is False
    refs2 = _oracle_two_layer(ref_net, x, sym_act=True)
    assert torch.equal(bits(low2.up(x.to(dev)).cpu()), bits(refs2[0]))
    # layers too narrow for the 16-byte rows of the kernels stay as they are
    small = TwoLayer(8, 8).half().to(dev)
    low3 = lower_qmodel_to_ext_kernels(small, None, qcfg, useInductor=False)
    assert isinstance(low3.up, QLinear)


def test_lowered_model_compiles_fullgraph_and_replays_from_a_hip_graph(dev):
    """The lowering helper, then torch.compile(fullgraph=True) and a HIP graph over the lowered
    model: every replay equals the eager result."""
    import copy

    from fms_mo_amd.fx.utils import lower_qmodel_to_ext_kernels
    from fms_mo_amd.modules.linear import QLinear, QLinearINT8Deploy

    net = _two_layer().to(dev)
    qcfg = {"ext_kernel_mapping_mod": {QLinear: QLinearINT8Deploy}}
    x = torch.randn(32, 256, generator=gen(22)).half().to(dev)
    low = lower_qmodel_to_ext_kernels(copy.deepcopy(net), x, qcfg, useInductor=False,
                                      use_dynamic_max_act_Qfunc=-1, recalc_clipvals=False)
    with torch.no_grad():
        eager = low(x).clone()
        comp = torch.compile(low, fullgraph=True)
        out = comp(x)
    torch.testing.assert_close(out.float(), eager.float(), rtol=2e-3, atol=2e-3)
    static_x_ = x.clone()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s), torch.no_grad():
        for _ in range(2):
            low(static_x_)
    torch.cuda.current_stream().wait_stream(s)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph), torch.no_grad():
        static_y = low(static_x_)
    for i in range(3):
        xi = torch.randn(32, 256, generator=gen(30 + i)).half().to(dev)
        static_x_.copy_(xi)
        graph.replay()
        torch.cuda.synchronize()
        with torch.no_grad():
            expect = low(xi)
        assert torch.equal(bits(static_y.cpu()), bits(expect.cpu())), i


@pytest.mark.parametrize("trunc", [0, 6])
def test_lower_qmodel_triton_swaps_both_kinds(dev, trunc):
    """lower_qmodel_triton against the oracle, layer by layer on the oracle's own intermediate
    activations: the two int8 layers bit-exact against deploy_forward_triton (codes, scales and
    outputs), the plain layer's dynamic-FP8 chunked matmul within rtol / atol 1e-2 of
    fpxacc_forward (the fp32 summation order inside a chunk is the matrix unit's)."""
    import copy

    from fms_mo_amd.custom_ext_kernels.utils import lower_qmodel_triton
    from fms_mo_amd.modules.linear import LinearFPxAcc, QLinearINT8Deploy

    net = _two_layer()
    ref_net = copy.deepcopy(net)
    net.to(dev)
    x = torch.randn(16, 256, generator=gen(23)).half()
    low = lower_qmodel_triton(net, use_dyn_max_act=-1, max_acc_bits=32, num_lsb_to_truncate=trunc, chunk_size=64,
                              layer_to_exclude=None)
    assert isinstance(low.up, QLinearINT8Deploy) and low.up.use_int_kernel == "triton"
    assert isinstance(low.plain, LinearFPxAcc) and low.plain.fp8_dyn == "per_token"
    h = x
    for name in ("up", "down"):
        lin = getattr(ref_net, name)
        st = O.deploy_prepare_general(lin.weight.detach(), lin.bias.detach(), lin.quantize_weight.clip_val,
                                      use_dynamic_max_act_Qfunc=-1)
        ref = O.deploy_forward_triton(h, st, chunk_size=64, truncate_lsb=trunc)
        mod = getattr(low, name)
        with torch.no_grad():
            y = mod(h.to(dev))
        assert torch.equal(mod.weight.cpu(), st["weight"]), name
        assert torch.equal(mod.input_scale.cpu().reshape(-1).float(), ref["input_scale"].float().reshape(-1)), name
        assert torch.equal(bits(y.cpu()), bits(ref["y"])), name
        h = ref["y"]
        if name == "up":
            h = torch.nn.functional.gelu(h.float()).half()
    ref_plain = O.fpxacc_forward(h, ref_net.plain.weight.detach(), None, trunc, 64, "per_token", False)
    with torch.no_grad():
        y_plain = low.plain(h.to(dev))
    torch.testing.assert_close(y_plain.cpu().float(), ref_plain.float(), rtol=1e-2, atol=1e-2)
    with torch.no_grad():
        assert torch.isfinite(low(x.to(dev))).all()
    net2 = _two_layer().to(dev)
    low2 = lower_qmodel_triton(net2, layer_to_exclude="plain")
    assert type(low2.plain) is torch.nn.Linear


# ------------------------------------------------------------------------------ FP8 emulation
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_fake_quant_fp8_kernels_bit_exact(dev, dtype):
    from fms_mo_amd import _lib as L

    x = (torch.randn(40, 256, generator=gen(24)) * torch.logspace(-4, 3, 40).reshape(-1, 1)).to(dtype)
    x[3].zero_()                                             # all-zero row: the 1e-12 floor / fp16 clamp
    x[4, :4] = torch.tensor([448.0, 464.0, 465.0, -1e4]).to(dtype)
    grid = torch.tensor([c for c in range(256) if (c & 0x7f) != 0x7f], dtype=torch.uint8).view(torch.float8_e4m3fn).float()
    x[5, :254] = grid.to(dtype)                              # every e4m3 value
    pos = torch.unique(grid[grid >= 0])
    mids = (pos[:-1] + pos[1:]) / 2                          # every midpoint (ties)
    x[6, :mids.numel()] = mids.to(dtype)
    xd = x.to(dev)
    y, q, s, inv = Kn().fake_quant_fp8(xd, L.F8E_SAT, True, True)
    ref = O.to_fp8_saturated(x, dtype)
    assert s is None and torch.equal(bits(y.cpu()), bits(ref))
    assert torch.equal(q.cpu().view(torch.uint8), x.clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8))
    for mode, gran in ((L.F8E_PER_ROW, "perToken"), (L.F8E_PER_ROW, "perCh"), (L.F8E_PER_TENSOR, "tensor")):
        y, q, s, inv = Kn().fake_quant_fp8(xd, mode, True, True)
        ref, ref_s = O.to_fp8_scaled(x, gran)
        assert torch.equal(s.cpu().reshape(-1), ref_s.float().reshape(-1)), gran
        assert torch.equal(bits(y.cpu()), bits(ref)), gran
        codes = (x * ref_s).clamp(-448, 448).to(torch.float8_e4m3fn)
        assert torch.equal(q.cpu().view(torch.uint8), codes.view(torch.uint8)), gran
        assert torch.equal(inv.cpu().reshape(-1), (1.0 / ref_s.float()).reshape(-1))


@pytest.mark.parametrize("modes", [("fp8_e4m3_scale_perToken", "fp8_e4m3_scale_perCh"),
                                   ("fp8_e4m3_scale", "fp8_e4m3_scale"), ("fp8_e4m3_sat", "fp8_e4m3_sat")])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_qlinear_fp8_modes_run_on_the_fp8_gemm(dev, modes, dtype):
    """QLinear with FP8 emulation quantizers: the eval forward multiplies the e4m3 codes on the FP8
    MFMA GEMM; within rtol / atol 1e-2 of the reference's F.linear on the fake-quantized tensors."""
    from fms_mo_amd.modules.linear import QLinear

    K, N, M = 512, 384, 96
    qa, qw = modes
    m = QLinear(K, N, bias=True, num_bits_feature=8, qa_mode=qa, num_bits_weight=8, qw_mode=qw,
                qcfg={"smoothq": False}, device="cpu")
    g = gen(25)
    sat = "sat" in qa
    with torch.no_grad():
        m.weight.copy_((3.0 if sat else 0.03) * torch.randn(N, K, generator=g))
        m.bias.copy_(0.1 * torch.randn(N, generator=g))
    m.to(dtype).eval()
    x = (torch.randn(M, K, generator=g) * (40.0 if sat else 1.0)).to(dtype)
    xq = O.to_fp8_forward(x, qa, perToken="perToken" in qa)
    wq = O.to_fp8_forward(m.weight.detach(), qw, perCh=N if "perCh" in qw else None)
    ref = torch.nn.functional.linear(xq.float(), wq.float(), m.bias.detach().float())
    # the reference's own evaluation (F.linear in x's dtype on the same tensors) is that product
    # rounded once more: the band below is stated against the exact product and covers both
    ref_mod = O.qlinear_fp8_forward(x, m.weight.detach(), m.bias.detach(), qa, qw).float()
    assert ((ref_mod - ref).abs() <= 1e-2 * ref.abs() + 1e-2 * max(1.0, float(ref.abs().mean()))).all()
    md = m.to(dev)
    with torch.no_grad():
        y = md(x.to(dev))
        y_again = md(x.to(dev))                               # cached weight codes
    assert y.dtype == dtype and md._wcache is not None and md._wcache[1].dtype == torch.float8_e4m3fn
    assert torch.equal(bits(y.cpu()), bits(y_again.cpu()))
    tol = 1e-2 * ref.abs() + 1e-2 * max(1.0, float(ref.abs().mean()))
    assert ((y.cpu().float() - ref).abs() <= tol).all()
    assert ((y.cpu().float() - ref_mod).abs() <= 2 * tol).all()
    md.train()
    with torch.no_grad():
        y_train = md(x.to(dev))                              # torch-op emulation path
    assert ((y_train.cpu().float() - ref).abs() <= 2 * tol).all()
    # a q_mode the reference's quantizer answers with None is not sent to the kernels
    md.eval()
    md.quantize_feature.q_mode, md.quantize_feature.perToken = "fp8_e4m3", False
    assert not md._fp8_path_ok(x.to(dev))


# ----------------------------------------------------------------- QLinear SmoothQuant cache
def test_qlinear_set_act_scale_invalidates_the_cached_weights(dev):
    """forward, set_act_scale(new), forward: the second forward must use weights and activations
    smoothed with the NEW scale (a cache keyed on a temporary tensor's address would not)."""
    from tests.test_gpu_modules import make_qlinear, outlier_x

    K, N = 512, 256
    m = make_qlinear(dev, K, N, smoothq=True, seed=26)
    x = outlier_x(64, K, 27)
    w_cpu, b_cpu = m.weight.detach().cpu(), m.bias.detach().cpu()
    cv = m.quantize_weight.clip_val.cpu()
    a1 = x.float().abs().amax(dim=0)
    a2 = (a1 * torch.linspace(0.2, 5, K)).clamp(min=1e-3)
    outs = []
    for a in (a1, a2, a1):
        m.set_act_scale(a.to(dev))
        with torch.no_grad():
            y = m(x.to(dev))
            assert torch.equal(bits(m(x.to(dev)).cpu()), bits(y.cpu()))
        # the weight clip values stay those of the unsmoothed weights (eval-mode semantics)
        ref = O.qlinear_forward(x, w_cpu, b_cpu, a, 0.5, w_clip_val=cv)
        d = (y.cpu().float() - ref.float()).abs()
        assert (d > 1e-2 + 1e-2 * ref.float().abs()).float().mean() < 2e-3, "stale SmoothQuant cache"
        outs.append(y.cpu())
    assert torch.equal(bits(outs[0]), bits(outs[2])) and not torch.equal(bits(outs[0]), bits(outs[1]))
    # zeroed statistics switch SmoothQuant off again
    m.set_act_scale(torch.zeros(K, device=dev))
    with torch.no_grad():
        y0 = m(x.to(dev))
    ref0 = O.qlinear_forward(x, w_cpu, b_cpu, None, 0.5, w_clip_val=cv)
    d0 = (y0.cpu().float() - ref0.float()).abs()
    assert (d0 > 1e-2 + 1e-2 * ref0.float().abs()).float().mean() < 2e-3


def test_qlinear_smoothq_train_mode_backward_twice_without_optimizer_step(dev):
    """Gradient accumulation: two forward / backward passes of a SmoothQuant QLinear in training
    mode with no weight update in between.  The SmoothQuant scale depends on the weights, so it is
    rebuilt inside every call's autograd graph (the reference recomputes it in every forward,
    linear.py:345-368); the tensor cached for the kernel paths is detached and never enters one."""
    from tests.test_gpu_modules import make_qlinear, outlier_x

    K, N = 256, 128
    m = make_qlinear(dev, K, N, smoothq=True, seed=31, dtype=torch.float32)
    x = outlier_x(32, K, 32, dtype=torch.float32).to(dev)
    m.set_act_scale(x.abs().amax(dim=0))
    with torch.no_grad():
        m.eval()
        m(x)                                   # fills the cache on the no-grad kernel path first
    assert m._sqcache is not None and not m._sqcache[1].requires_grad
    m.train()
    grads = []
    for _ in range(2):
        m.zero_grad()
        y = m(x)
        y.float().pow(2).mean().backward()     # a second backward through a freed graph would raise
        assert m.weight.grad is not None and torch.isfinite(m.weight.grad).all()
        grads.append(m.weight.grad.clone())
    assert torch.equal(grads[0], grads[1])
    assert grads[0].abs().sum() > 0


def test_dynamic_quantizers_store_the_abs_max_as_clip_values(dev):
    """qa_dynamic_max_qfunc (dim -2) and qa_dyn_max_fake_zero_shift leave +-amax in cvs[0:2] like
    the reference (linear.py:1085-1113), not scale * levels; a changed input_zp buffer is seen by
    the next forward."""
    from fms_mo_amd.modules.linear import QLinearINT8Deploy
    from tests.test_gpu_modules import make_qlinear

    m = make_qlinear(None, 256, 256, seed=33)
    x = static_x(40, 256, 34, torch.float16)
    x[:, 7] *= 1e-7                              # a column whose scale is governed by the 1e-5 clamp

    dep = QLinearINT8Deploy.from_fms_mo(m, use_dynamic_max_act_Qfunc=-2, recalc_clipvals=False, target_device=dev)
    dep(x.to(dev))
    amax = x.abs().amax(dim=0, keepdim=True)
    assert torch.equal(dep.cvs[0].cpu(), amax) and torch.equal(dep.cvs[1].cpu(), -amax)
    fz = QLinearINT8Deploy.from_fms_mo(m, use_dynamic_max_act_Qfunc=5, recalc_clipvals=False, target_device=dev)
    assert fz.use_fake_zero_shift
    fz(x.to(dev))
    assert torch.equal(fz.cvs[0].cpu(), x.abs().max()) and torch.equal(fz.cvs[1].cpu(), -x.abs().max())
    s5 = fz.input_scale.clone()
    with torch.no_grad():
        fz.input_zp.fill_(9)
    fz(x.to(dev))
    ref_q, ref_s = O.quant_act_fake_zero_shift(x, torch.tensor(9, dtype=torch.int))
    assert torch.equal(fz.input_scale.cpu(), ref_s) and not torch.equal(fz.input_scale, s5)
