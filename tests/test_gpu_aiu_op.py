"""``torch.ops.fms_mo.i8i8_aiu`` on the GPU: activation codes bit-exact against the CPU oracle's
restatement of the reference op, outputs against the six vectors the reference's own test-suite
stores (tests/golden/ref_w-*.pt) and against the oracle at larger shapes, the zero-shift bias
kernel, and the module wrapped around the op."""
import glob
import os

import pytest
import torch

from oracle import qlinear_oracle as O

pytestmark = pytest.mark.gpu

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "ref_w-*.pt")))
MODES = ["per_token", "per_tensor_symm", "per_tensor_asymm"]


def gen(seed):
    return torch.Generator().manual_seed(seed)


def op():
    from fms_mo_amd.aiu_addons.i8i8.i8i8_aiu_op import register_aiu_i8i8_op

    if not (hasattr(torch.ops, "fms_mo") and hasattr(torch.ops.fms_mo, "i8i8_aiu")):
        register_aiu_i8i8_op()
    return torch.ops.fms_mo.i8i8_aiu


def make_case(seed, M, K, N, xdt, mdt, per_channel, act, smooth):
    """Synthetic operands in the layout of the reference's fixtures
    (tests/aiu_addons/conftest.py:105-147): integer weights, clip values, qdata."""
    g = gen(seed)
    x = torch.randn(M, K, generator=g)
    x[:, 3] *= 20.0  # an outlier channel, the case SmoothQuant exists for
    x = x.to(xdt)
    w_int = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int32).to(torch.int8)
    w_cv = (torch.rand(N if per_channel else 1, generator=g) * 0.5 + 0.05).to(mdt)
    sq = (torch.rand(K, generator=g) * 3 + 0.25).to(mdt) if smooth else torch.ones(1, dtype=mdt)
    xs = (x.float() / sq.float())
    if act == "per_token":
        a_cv, a_cvn = torch.zeros(1, dtype=mdt), torch.zeros(1, dtype=mdt)
    elif act == "per_tensor_symm":
        a_cv = (xs.abs().max() * 0.8).reshape(1).to(mdt)  # clips a few values
        a_cvn = -a_cv
    else:
        a_cv = (xs.max() * 0.8).reshape(1).to(mdt)
        a_cvn = (xs.min() * 0.6).reshape(1).to(mdt)
    zs = w_int.sum(dim=1).to(mdt) if act == "per_tensor_asymm" else torch.zeros(1, dtype=mdt)
    qdata = torch.cat((w_cv, -w_cv, a_cv, a_cvn, zs, sq))
    bias = (0.1 * torch.randn(N, generator=g)).to(xdt)
    return x, w_int, bias, qdata, w_cv, a_cv, a_cvn, sq


@pytest.mark.parametrize("act", MODES)
@pytest.mark.parametrize("xdt,mdt", [(torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16),
                                     (torch.float16, torch.float32), (torch.float32, torch.float32)])
@pytest.mark.parametrize("smooth", [False, True])
@pytest.mark.parametrize("shape", [(37, 256), (16, 4096), (5, 24576)])
def test_activation_codes_bit_exact(dev, act, xdt, mdt, smooth, shape):
    from fms_mo_amd import _lib as L
    from fms_mo_amd import kernels

    M, K = shape
    x, _, _, _, _, a_cv, a_cvn, sq = make_case(11, M, K, 8, xdt, mdt, False, act, smooth)
    x[2, 7] = 0.0
    ref_int, scale_x, zp_x = O.i8i8_aiu_quant_act(x, a_cv, a_cvn, sq, act)
    mode = {"per_token": L.MS_PER_TOKEN, "per_tensor_symm": L.MS_SYMM,
            "per_tensor_asymm": L.MS_ASYMM}[act]
    clip = None if act == "per_token" else torch.cat((a_cv, a_cvn)).to(dev)
    q, a_meta = kernels.quant_act_i8_mulscale(x.to(dev), mode, clip=clip,
                                              smooth=sq.to(dev) if smooth else None, meta_dtype=mdt)
    got = q.cpu().to(torch.int32) + (128 if act == "per_tensor_asymm" else 0)
    assert torch.equal(got, ref_int.to(torch.int32))
    inv = (1.0 / scale_x.float()).reshape(-1)
    if act == "per_token":
        assert torch.equal(a_meta.cpu(), inv)
    else:
        assert torch.equal(a_meta.cpu()[:1], inv)
        if act == "per_tensor_asymm":
            assert a_meta.cpu()[1].item() == zp_x.float().item()


@pytest.mark.parametrize("act", MODES)
@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("K", [256, 14336])
def test_activation_codes_rows_off_the_fast_path(dev, act, dt, K):
    """Rows the row-walking 16-bit kernel hands to its IEEE routine, between ordinary rows: a
    quotient x / smooth that overflows the dtype (per-tensor modes: the code saturates), a row whose
    maximum is so small that 127 / max overflows (per token: every code +-127, output scale 0), a
    divisor far outside the fast quotient's range (bf16).  All of them are finite in torch's own
    arithmetic, so the oracle defines them; the neighbours must stay bit-exact too."""
    from fms_mo_amd import _lib as L
    from fms_mo_amd import kernels

    g = gen(77)
    M = 9
    x = torch.randn(M, K, generator=g).to(dt)
    sq = (torch.rand(K, generator=g) * 3 + 0.25).to(dt)
    big = 6.0e4 if dt == torch.float16 else 3.0e38
    if act == "per_token":
        tiny = 2.0 ** -24 if dt == torch.float16 else 2.0 ** -130
        x[4] = torch.where(torch.rand(K, generator=g) < 0.5, -1.0, 1.0).to(dt) * tiny * 3
        sq[:] = 1.0
        sq[5] = 0.5
    else:
        if dt == torch.bfloat16 and act == "per_tensor_symm":
            sq[6] = 2.0 ** -70  # outside the fast quotient's divisor range: the whole block goes IEEE
            x[:, 6] = (torch.randn(M, generator=g) * 2.0 ** -72).to(dt)
        x[3, 17] = big
        sq[17] = 0.25  # x / smooth = inf in the compute dtype
        x[6, 200] = -big
        sq[200] = 0.5
    xs = x.float() / sq.float()
    fin = xs[torch.isfinite(xs) & (xs.abs() < 100)]
    a_cv = (fin.max() * 0.8).reshape(1).to(dt)
    a_cvn = -a_cv if act != "per_tensor_asymm" else (fin.min() * 0.6).reshape(1).to(dt)
    ref_int, scale_x, zp_x = O.i8i8_aiu_quant_act(x, a_cv, a_cvn, sq, act)
    mode = {"per_token": L.MS_PER_TOKEN, "per_tensor_symm": L.MS_SYMM, "per_tensor_asymm": L.MS_ASYMM}[act]
    clip = None if act == "per_token" else torch.cat((a_cv, a_cvn)).to(dev)
    q, a_meta = kernels.quant_act_i8_mulscale(x.to(dev), mode, clip=clip, smooth=sq.to(dev), meta_dtype=dt)
    got = q.cpu().to(torch.int32) + (128 if act == "per_tensor_asymm" else 0)
    assert torch.equal(got, ref_int.to(torch.int32))
    if act == "per_token":
        assert torch.equal(a_meta.cpu(), (1.0 / scale_x.float()).reshape(-1))
        assert a_meta[4].item() == 0.0 and torch.all(got[4].abs() == 127)


def test_all_zero_row_gives_zero_codes_and_zero_scale(dev):
    from fms_mo_amd import _lib as L
    from fms_mo_amd import kernels

    x = torch.randn(4, 64, generator=gen(5)).half()
    x[1] = 0.0
    q, a = kernels.quant_act_i8_mulscale(x.to(dev), L.MS_PER_TOKEN)
    assert torch.all(q[1] == 0) and a[1].item() == 0.0
    assert torch.all(q[0].abs().max() == 127)


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p) for p in GOLDEN])
def test_op_matches_the_reference_vectors(dev, path):
    d = torch.load(path, weights_only=True)
    x = d["x"].to(torch.float16)
    y = op()(x.to(dev), d["w_int"].to(dev), d["bias"].to(dev), d["qdata"].to(torch.float16).to(dev),
             d["weight_quant_type"], d["activ_quant_type"], d["smoothquant"])
    ref = d["reference_out"]
    assert y.shape == ref.shape and y.dtype == torch.float16
    # The stored outputs come from the floating-point simulation (fp16 operands, fp16 F.linear with
    # its own accumulation order), the op here multiplies the integer codes exactly and rounds
    # once.  Observed on these six vectors (K = 7, |y| up to 10.5): at most 4.3e-3 absolute where
    # |y| < 8 and one fp16 ulp (7.8e-3) above; the band asserted is that with a small margin, half
    # the W8A8 path's stated 1e-2 / 1e-2.
    torch.testing.assert_close(y.cpu().float(), ref.float(), rtol=1e-3, atol=5e-3)


def exact_from_oracle_codes(x, w_int, bias, w_cv, a_cv, a_cvn, sq, act):
    """float64 evaluation of the op from the oracle's integers: what exact integer hardware
    returns before the output cast."""
    x_int, scale_x, zp_x = O.i8i8_aiu_quant_act(x, a_cv, a_cvn, sq, act)
    xi = x_int.double()
    if act == "per_tensor_asymm":
        xi = xi + zp_x.double()
    acc = xi @ w_int.double().t()
    return acc / scale_x.double() * (w_cv.double() / 127) + bias.double()


@pytest.mark.parametrize("act", MODES)
@pytest.mark.parametrize("per_channel", [False, True])
@pytest.mark.parametrize("xdt,mdt", [(torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16),
                                     (torch.float16, torch.float32)])
@pytest.mark.parametrize("smooth", [False, True])
@pytest.mark.parametrize("shape", [(64, 1024, 512), (1, 4096, 1024), (300, 2048, 768)])
def test_op_against_oracle(dev, act, per_channel, xdt, mdt, smooth, shape):
    M, K, N = shape
    x, w_int, bias, qdata, w_cv, a_cv, a_cvn, sq = make_case(21, M, K, N, xdt, mdt, per_channel, act,
                                                             smooth)
    y = op()(x.to(dev), w_int.to(dev), bias.to(dev), qdata.to(dev),
             "per_channel" if per_channel else "per_tensor", act, smooth)
    assert y.dtype == xdt and y.shape == (M, N)
    exact = exact_from_oracle_codes(x, w_int, bias, w_cv, a_cv, a_cvn, sq, act)
    # integers are identical to the reference's, accumulation is exact: what remains is the fp32
    # epilogue and the cast to the output dtype (half an ulp: 2^-11 fp16, 2^-8 bf16)
    ulp = 2.0 ** -8 if xdt == torch.bfloat16 else 2.0 ** -11
    err = (y.cpu().double() - exact).abs()
    assert torch.all(err <= 1.1 * ulp * exact.abs() + 1e-3 * exact.abs().max() * ulp + 1e-6)
    # and the reference's floating-point simulation of the same node (oracle restatement)
    sim = O.i8i8_aiu(x, w_int, bias, qdata,
                     "per_channel" if per_channel else "per_tensor", act, smooth)
    scale = sim.float().abs().max()
    assert torch.all((y.cpu().float() - sim.float()).abs() <= 1e-2 * sim.float().abs() + 1e-2 * scale)


def test_random_nodes_codes_bit_exact_and_outputs_within_an_ulp(dev):
    """Forty seeded nodes over all three activation modes, both weight modes, the dtype pairs the
    op serves, any M, K a multiple of 64 and any N a multiple of 8: the integer activation codes
    are the oracle's and the output is the exact value of those integers within the output cast."""
    import random

    from fms_mo_amd import _lib as L
    from fms_mo_amd import kernels

    rng = random.Random(97531)
    for case in range(40):
        act = rng.choice(MODES)
        per_channel, smooth = rng.random() < 0.5, rng.random() < 0.5
        xdt, mdt = rng.choice([(torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16),
                               (torch.float16, torch.float32)])
        M = rng.choice([1, rng.randint(2, 16), rng.randint(17, 400)])
        K = 64 * rng.choice([rng.randint(1, 16), rng.randint(16, 230)])
        N = 8 * rng.randint(1, 150)
        tag = f"case {case}: {act} per_channel={per_channel} smooth={smooth} {xdt}/{mdt} M={M} K={K} N={N}"
        x, w_int, bias, qdata, w_cv, a_cv, a_cvn, sq = make_case(8000 + case, M, K, N, xdt, mdt, per_channel,
                                                                 act, smooth)
        ref_int, scale_x, zp_x = O.i8i8_aiu_quant_act(x, a_cv, a_cvn, sq, act)
        mode = {"per_token": L.MS_PER_TOKEN, "per_tensor_symm": L.MS_SYMM, "per_tensor_asymm": L.MS_ASYMM}[act]
        clip = None if act == "per_token" else torch.cat((a_cv, a_cvn)).to(dev)
        q, _ = kernels.quant_act_i8_mulscale(x.to(dev), mode, clip=clip, smooth=sq.to(dev) if smooth else None,
                                             meta_dtype=mdt)
        got = q.cpu().to(torch.int32) + (128 if act == "per_tensor_asymm" else 0)
        assert torch.equal(got, ref_int.to(torch.int32)), tag
        y = op()(x.to(dev), w_int.to(dev), bias.to(dev), qdata.to(dev),
                 "per_channel" if per_channel else "per_tensor", act, smooth)
        exact = exact_from_oracle_codes(x, w_int, bias, w_cv, a_cv, a_cvn, sq, act)
        ulp = 2.0 ** -8 if xdt == torch.bfloat16 else 2.0 ** -11
        err = (y.cpu().double() - exact).abs()
        # beside the output cast: the product term and (asymmetric mode) the zero-point correction
        # are each rounded to fp32 before they cancel
        dq = (w_cv.double() / 127) / scale_x.double()
        terms = (ref_int.double() @ w_int.double().t()).abs() * dq + bias.double().abs()
        if act == "per_tensor_asymm":
            terms = terms + (zp_x.double() * w_int.double().sum(dim=1)).abs() * dq
        assert torch.all(err <= 1.1 * ulp * exact.abs() + 4e-7 * terms + 1e-6), tag


def test_three_dimensional_input_and_dummy_bias(dev):
    x, w_int, _, qdata, *_ = make_case(31, 6 * 5, 128, 64, torch.float16, torch.float16, True,
                                       "per_token", False)
    x3 = x.reshape(6, 5, 128)
    zero = torch.zeros(1, dtype=torch.float16)
    y = op()(x3.to(dev), w_int.to(dev), zero.to(dev), qdata.to(dev), "per_channel", "per_token", False)
    assert y.shape == (6, 5, 64)
    sim = O.i8i8_aiu(x3, w_int, zero, qdata, "per_channel", "per_token", False)
    torch.testing.assert_close(y.cpu().float(), sim.float(), rtol=1e-2, atol=1e-2 * sim.float().abs().max().item())


def test_qdata_length_is_validated(dev):
    x, w_int, bias, qdata, *_ = make_case(32, 4, 64, 32, torch.float16, torch.float16, False,
                                          "per_token", False)
    with pytest.raises((ValueError, RuntimeError)):
        op()(x.to(dev), w_int.to(dev), bias.to(dev), qdata[:-1].to(dev), "per_tensor", "per_token", False)
    with pytest.raises((NotImplementedError, RuntimeError)):
        op()(x.to(dev), w_int.to(dev), bias.to(dev), qdata.to(dev), "per_group", "per_token", False)


@pytest.mark.parametrize("per_channel", [False, True])
def test_zero_shift_bias_kernel(dev, per_channel):
    from fms_mo_amd import kernels

    g = gen(41)
    N, K = 515, 4096
    w = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int32).to(torch.int8)
    ws = torch.rand(N if per_channel else 1, generator=g) * 0.01
    meta = torch.tensor([0.0123, -37.5])
    bias = torch.randn(N, generator=g).half()
    out = kernels.zero_shift_bias(w.to(dev), ws.to(dev), meta.to(dev), bias=bias.to(dev))
    ref = bias.double() + (128.0 + meta[1].double()) * w.sum(dim=1).double() * meta[0].double() * ws.double()
    torch.testing.assert_close(out.cpu().double(), ref, rtol=1e-6, atol=1e-6)
    out0 = kernels.zero_shift_bias(w.to(dev), ws.to(dev), meta.to(dev), bias=None)
    torch.testing.assert_close(out0.cpu().double(), ref - bias.double(), rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("act", MODES)
def test_module_forward_and_state_dict(dev, act):
    from fms_mo_amd.aiu_addons.i8i8.i8i8_aiu_linear import W8A8LinearAIU, get_int8_aiu_linear

    M, K, N = 48, 512, 256
    x, w_int, bias, qdata, w_cv, a_cv, a_cvn, sq = make_case(51, M, K, N, torch.float16, torch.float16,
                                                             True, act, True)
    lin = get_int8_aiu_linear(K, N, True, {"linear_type": "int8", "weight_per_channel": True,
                                           "activ_quant_type": act, "smoothquant": True},
                              use_smoothquant=True)
    assert isinstance(lin, W8A8LinearAIU) and lin.qdata.dtype == torch.float32
    sd = {"weight": w_int, "bias": bias.half(), "w_clip_val": w_cv, "w_clip_valn": -w_cv,
          "a_clip_val": a_cv, "a_clip_valn": a_cvn, "smoothquant_scale": sq,
          "zero_shift": (w_int.sum(dim=1).float() if act == "per_tensor_asymm" else torch.zeros(1))}
    lin.load_state_dict(sd, strict=False)
    lin.re_register_qdata()
    lin = lin.to(dev)
    y = lin(x.to(dev))
    sim = O.i8i8_aiu(x, w_int, bias, lin.qdata.cpu(), "per_channel", act, True)
    scale = sim.float().abs().max()
    assert torch.all((y.cpu().float() - sim.float()).abs() <= 1e-2 * sim.float().abs() + 1e-2 * scale)
    assert "W8A8LinearAIU(in=512, out=256" in repr(lin)


def test_op_schema_and_shape_only_twin(dev):
    x, w_int, bias, qdata, *_ = make_case(61, 8, 128, 64, torch.float16, torch.float16, False,
                                          "per_tensor_symm", False)
    args = (x.to(dev), w_int.to(dev), bias.to(dev), qdata.to(dev), "per_tensor", "per_tensor_symm", False)
    op()  # make sure it is registered
    torch.library.opcheck(torch.ops.fms_mo.i8i8_aiu.default, args,
                          test_utils=("test_schema", "test_faketensor"))


def _replay_equals_eager(fn, inputs, static_in):
    """Capture fn(static_in) once, replay it for every input with eager work and synchronisations
    in between; every replay must equal the eager result bit for bit."""
    eager = [fn(x).clone() for x in inputs]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn(static_in)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = fn(static_in)
    for _ in range(2):
        for x, ref in zip(inputs, eager):
            static_in.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(static_out.view(torch.int16), ref.view(torch.int16))
            fn(x)
            torch.cuda.synchronize()


@pytest.mark.parametrize("act", MODES)
def test_node_replays_from_a_hip_graph(dev, act):
    """Nothing in the node reads a value back to the host (clip values, zero point and scales stay
    on the device), so it can be captured; asymmetric activations add the zero-shift bias kernel."""
    M, K, N = 40, 1024, 768
    x, w_int, bias, qdata, *_ = make_case(71, M, K, N, torch.float16, torch.float16, True, act, True)
    w, b, qd = w_int.to(dev), bias.to(dev), qdata.to(dev)
    f = op()
    xs = [(x * (0.5 + 0.25 * i)).to(dev) for i in range(3)]
    _replay_equals_eager(lambda t: f(t, w, b, qd, "per_channel", act, True), xs, xs[0].clone())


@pytest.mark.parametrize("act", MODES)
def test_node_at_llama3_8b_down_projection(dev, act):
    """M = 4096 tokens through the 14336 -> 4096 projection: codes against the oracle on a sample of
    rows, outputs against the float64 evaluation of the oracle's integers on those rows."""
    M, K, N = 4096, 14336, 4096
    x, w_int, bias, qdata, w_cv, a_cv, a_cvn, sq = make_case(81, M, K, N, torch.float16, torch.float16,
                                                             True, act, True)
    y = op()(x.to(dev), w_int.to(dev), bias.to(dev), qdata.to(dev), "per_channel", act, True).cpu()
    rows = torch.tensor([0, 1, 777, 2048, 4095])
    exact = exact_from_oracle_codes(x[rows], w_int, bias, w_cv, a_cv, a_cvn, sq, act)
    err = (y[rows].double() - exact).abs()
    assert torch.all(err <= 1.1 * 2.0 ** -11 * exact.abs() + 4e-6 * exact.abs().max() + 1e-6)
