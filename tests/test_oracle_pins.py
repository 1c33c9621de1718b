"""Pins of the CPU oracle that do not need the reference: exact re-evaluation in another
arithmetic (numpy float64 + explicit roundings), an independent C restatement
(oracle/qlinear_ref.c), closed forms, invariants and brute force on small inputs.  Each check is
chosen so that a plausible slip (multiply by 127/amax instead of dividing by amax/127, a clamp
that is not there, truncation instead of half-to-even, a transposed operand, rounding the scale
after instead of before the multiply) fails it."""
import ctypes
import os
import subprocess

import numpy as np
import pytest
import torch

from oracle import qlinear_oracle as O

ORACLE_DIR = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle")


@pytest.fixture(scope="session")
def cref():
    so = os.path.join(ORACLE_DIR, "_build", "libqlinear_ref.so")
    if not os.path.exists(so):
        subprocess.run(["make", "-C", ORACLE_DIR], check=True)
    lib = ctypes.CDLL(so)
    lib.ref_round_f16.restype = ctypes.c_float
    lib.ref_round_f16.argtypes = [ctypes.c_float]
    lib.ref_round_bf16.restype = ctypes.c_float
    lib.ref_round_bf16.argtypes = [ctypes.c_float]
    lib.ref_epilogue.restype = ctypes.c_float
    lib.ref_epilogue.argtypes = [ctypes.c_int32, ctypes.c_float, ctypes.c_float, ctypes.c_float]
    lib.ref_round_and_trun.restype = ctypes.c_float
    lib.ref_round_and_trun.argtypes = [ctypes.c_float, ctypes.c_int, ctypes.c_int]
    lib.ref_e4m3.restype = ctypes.c_uint8
    lib.ref_e4m3.argtypes = [ctypes.c_float]
    return lib


def gen(seed):
    return torch.Generator().manual_seed(seed)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


# --------------------------------------------------------------------- activation quantizer
@pytest.mark.parametrize("dtype,T", [(torch.float16, 0), (torch.bfloat16, 1), (torch.float32, 2)])
def test_act_quant_vs_c_restatement(cref, dtype, T):
    x = (torch.randn(64, 512, generator=gen(1)) * 2.5).to(dtype)
    x[0].zero_()
    x[1].zero_(); x[1, 3] = 7.0
    q, s, _ = O.quant_act_pertoken_i8(x)
    xf = x.float().contiguous()
    qc = torch.empty(64, 512, dtype=torch.int8)
    sc = torch.empty(64, dtype=torch.float32)
    cref.ref_quant_act_pertoken(_ptr(xf), 64, 512, T, _ptr(qc), _ptr(sc))
    assert torch.equal(sc, s.float().reshape(-1))
    assert torch.equal(qc, q)


def test_act_quant_fp16_vs_float64_closed_form():
    """rnd_f16(a / b) == float16(float64(a) / float64(b)) (53 >= 2*11 + 2 makes the double
    rounding innocuous), so numpy in float64 re-derives every scale and quotient independently."""
    x = (torch.randn(32, 256, generator=gen(2)) * 3).half()
    q, s, _ = O.quant_act_pertoken_i8(x)
    xn = x.numpy().astype(np.float64)
    amax = np.abs(xn).max(axis=1, keepdims=True)
    eps16 = np.float64(np.float16(1e-5))
    sn = np.float16(np.maximum(amax, eps16) / 127.0).astype(np.float64)
    qn = np.rint(np.float16(xn / sn).astype(np.float64))
    assert np.array_equal(sn.reshape(-1), s.numpy().astype(np.float64).reshape(-1))
    assert np.array_equal(qn.astype(np.int8), q.numpy())
    # a plausible mistake -- multiplying by 127/amax -- is NOT the same function
    wrong = np.rint(np.float16(xn * np.float16(127.0 / amax).astype(np.float64)).astype(np.float64))
    assert not np.array_equal(wrong.astype(np.int8), q.numpy())


def test_act_quant_special_rows():
    x = torch.zeros(4, 64, dtype=torch.float16)
    x[1, 7] = -5.0                      # lone extreme -> -127
    x[2, :] = torch.linspace(-1, 1, 64).half()
    x[3, 0] = 127.0                     # scale exactly 1 -> identity on integers, ties to even
    x[3, 1] = 2.5
    x[3, 2] = 3.5
    x[3, 3] = -0.5
    q, s, _ = O.quant_act_pertoken_i8(x)
    assert torch.all(q[0] == 0)
    assert s[0, 0].item() == (torch.tensor(1e-5).half() / 127).item()
    assert q[1, 7].item() == -127 and q[1].abs().sum().item() == 127
    assert q[2, 0].item() == -127 and q[2, -1].item() == 127
    assert s[3, 0].item() == 1.0
    assert q[3, :4].tolist() == [127, 2, 4, 0]      # 2.5 -> 2, 3.5 -> 4, -0.5 -> -0 (half to even)


def test_bf16_wrap_census():
    """Every bf16 amax in (0.01, 1000): how often does the row maximum quantize to 128 (and wrap
    to -128)?  Never in fp16."""
    bits = torch.arange(0x3C00, 0x4500, dtype=torch.int32).to(torch.int16)  # bf16 0.0078 .. 2048
    v = bits.view(torch.bfloat16)
    v = v[(v > 0.01) & (v < 1000)]
    q, _, _ = O.quant_act_pertoken_i8(v.reshape(-1, 1))
    wraps = (q.reshape(-1) == -128).sum().item()
    assert 2130 <= v.numel() <= 2136 and wraps == 357
    h = torch.arange(0x2000, 0x6400, dtype=torch.int32).to(torch.int16).view(torch.float16)
    h = h[(h > 0.01) & (h < 1000)]
    qh, _, _ = O.quant_act_pertoken_i8(h.reshape(-1, 1))
    assert (qh.reshape(-1) == 127).all()


def test_fake_quant_equals_q_times_scale():
    x = (torch.randn(16, 128, generator=gen(3)) * 2).half()
    q, s, _ = O.quant_act_pertoken_i8(x)
    assert torch.equal(O.fake_quant_act_pertoken(x), (q.half() * s))


def test_static_quant_against_torch_quantize_per_tensor_away_from_ties():
    x = (torch.randn(8, 256, generator=gen(4)) * 3).float()
    scale, zp = 0.05, 131
    q = O.quant_act_static_raw(x, torch.tensor([scale]), zp, 0)
    ref = torch.quantize_per_tensor(x, scale, zp - 128, torch.qint8).int_repr()
    assert (q != ref).float().mean() < 1e-3   # only exact ties of x/scale may differ (mul vs div)


# --------------------------------------------------------------------------- weights / SmoothQuant
def test_weight_quant_invariants_and_fake_quant_agreement():
    W = (0.02 * torch.randn(64, 256, generator=gen(5))).half()
    cv = O.qmax_perch_clipval(W).float()
    w_i8, w_scale = O.quant_weight_deploy(W, cv, torch.tensor([1.0], dtype=torch.float16))
    assert w_i8.abs().max() <= 127
    arg = W.abs().argmax(dim=1)
    assert torch.all(w_i8[torch.arange(64), arg].abs() == 127)       # every row hits +-127 at its arg-max
    assert torch.allclose(w_scale, cv / 127)
    fq = O.fake_quant_weight_perch(W.float(), cv)
    assert ((w_i8.float() * w_scale[:, None]) - fq).abs().max() <= w_scale.max() * 1.001
    assert ((w_i8.float() * w_scale[:, None]) != fq).float().mean() < 1e-3   # differ at ties only


def test_smoothquant_scale_closed_form_and_invariance():
    W = (0.02 * torch.randn(32, 64, generator=gen(6))).float()
    a = torch.rand(64, generator=gen(7)) * 10 + 0.1
    s = O.smoothq_scale_deploy(W, a, torch.tensor([0.5]))
    expect = torch.sqrt(a) / torch.sqrt(W.abs().amax(dim=0))
    assert torch.allclose(s.reshape(-1), expect, rtol=1e-6)
    x = torch.randn(8, 64, generator=gen(8))
    assert torch.allclose((x / s) @ (W * s).t(), x @ W.t(), rtol=1e-4, atol=1e-5)
    assert O.smoothq_scale_qlinear(W, torch.zeros(64), 0.5, torch.float16).tolist() == [1.0]
    a0 = a.clone(); a0[3] = 0
    assert O.smoothq_scale_deploy(W.half(), a0, torch.tensor([0.5])).tolist() == [1.0]


# -------------------------------------------------------------------------------- GEMM / epilogue
def test_int_gemm_vs_c_brute_force(cref):
    a = torch.randint(-128, 128, (33, 96), generator=gen(9), dtype=torch.int8)
    w = torch.randint(-128, 128, (40, 96), generator=gen(10), dtype=torch.int8)
    c = torch.empty(33, 40, dtype=torch.int32)
    cref.ref_gemm_i8(_ptr(a), _ptr(w), 33, 40, 96, _ptr(c))
    assert torch.equal(O.int_gemm(a, w), c)
    # the fast path (torch._int_mm) as well
    a2 = torch.randint(-128, 128, (64, 128), generator=gen(11), dtype=torch.int8)
    w2 = torch.randint(-128, 128, (48, 128), generator=gen(12), dtype=torch.int8)
    c2 = torch.empty(64, 48, dtype=torch.int32)
    cref.ref_gemm_i8(_ptr(a2), _ptr(w2), 64, 48, 128, _ptr(c2))
    assert torch.equal(O.int_gemm(a2, w2), c2)
    # extreme values: -128 * -128 * K stays exact
    a3 = torch.full((17, 4096), -128, dtype=torch.int8)
    assert O.int_gemm(a3, a3[:8])[0, 0].item() == 128 * 128 * 4096


def test_epilogue_vs_c_and_fp16_scale_rounding(cref):
    acc = torch.randint(-400000, 400000, (24, 16), generator=gen(13), dtype=torch.int32)
    s_a = (torch.rand(24, 1, generator=gen(14)) * 0.05 + 1e-3).half()
    s_w = (torch.rand(16, generator=gen(15)) * 1e-3 + 1e-5).float()
    bias = (torch.randn(16, generator=gen(16)) * 0.01).half()
    y = O.epilogue_ref(acc, s_a, s_w, bias)
    for m in range(24):
        for n in range(16):
            r = cref.ref_epilogue(int(acc[m, n]), float(s_a[m, 0]), float(s_w[n]), float(bias[n]))
            assert r == y[m, n].item(), (m, n)
    # a tie of the fp16 subnormal scale: 369.5 * 2^-24 rounds to the even neighbour 370 * 2^-24
    tie = 369.5 * 2.0**-24
    assert cref.ref_round_f16(tie) == 370 * 2.0**-24
    assert torch.tensor(tie).half().item() == 370 * 2.0**-24


def test_round_f16_bf16_helpers_vs_torch(cref):
    v = torch.cat([torch.randn(2000, generator=gen(17)) * 100, torch.randn(2000, generator=gen(18)) * 1e-5,
                   torch.tensor([0.0, 65504.0, 65519.9, 65520.0, 6.0e-8, 2.98e-8, 2.99e-8, 1e-5])])
    for x in v.tolist():
        assert cref.ref_round_f16(x) == torch.tensor(x).half().float().item(), x
        assert cref.ref_round_bf16(x) == torch.tensor(x).bfloat16().float().item(), x


# --------------------------------------------------------------------------------- chunked paths
def test_round_and_trun_bit_level(cref):
    vals = torch.cat([torch.randn(300, generator=gen(19)) * 10.0 ** torch.randint(-12, 12, (300,), generator=gen(20)).float(),
                      torch.tensor([0.0, -0.0, 1.0, -1.0, 3.4e38, 1e-45, float("inf"), float("-inf"),
                                    8581545984.0, 8581545983.0, 4.665707820095122e-10, 4.6e-10])])
    for t in (0, 1, 7, 8, 14, 16, 22):
        for dl16 in (0, 1):
            out = O.round_and_trun(vals.clone(), t, bool(dl16))
            for i, x in enumerate(vals.tolist()):
                r = cref.ref_round_and_trun(x, t, dl16)
                o = out[i].item()
                assert (r == o) or (r != r and o != o), (x, t, dl16, r, o)
    # closed form: t bits cleared, round half away in magnitude, carry may bump the exponent
    x = torch.tensor([1.0 + 2.0**-16 + 2.0**-17, 2.0 - 2.0**-23])
    y = O.round_and_trun(x, 8)
    assert y[0].item() == 1.0 + 2.0**-15 and y[1].item() == 2.0
    assert torch.equal(O.round_and_trun(x, 0), x)
    nan = O.round_and_trun(torch.tensor([float("nan")]), 8)
    assert nan.isnan().all()


@pytest.mark.parametrize("cfg", [(64, 0, 32), (64, 8, 32), (32, 8, 18), (128, 4, 24), (64, 16, 32)])
def test_chunk_i8_vs_c(cref, cfg):
    chunk, t, bits = cfg
    a = torch.randint(-128, 128, (20, 300), generator=gen(21), dtype=torch.int8)
    w = torch.randint(-128, 128, (24, 300), generator=gen(22), dtype=torch.int8)
    d = torch.empty(20, 24, dtype=torch.int32)
    cref.ref_chunk_i8(_ptr(a), _ptr(w), 20, 24, 300, chunk, t, bits, _ptr(d))
    assert torch.equal(O.chunk_matmul_i8(a, w, None, chunk, t, bits), d)


def test_chunk_i8_properties():
    a = torch.randint(-128, 128, (16, 512), generator=gen(23), dtype=torch.int8)
    w = torch.randint(-128, 128, (16, 512), generator=gen(24), dtype=torch.int8)
    exact = O.int_gemm(a, w)
    assert torch.equal(O.chunk_matmul_i8(a, w, None, 64, 0, 32), exact)          # no truncation == GEMM
    assert torch.equal(O.chunk_matmul_i8(a, w, None, 512, 0, 32), exact)
    d8 = O.chunk_matmul_i8(a, w, None, 64, 8, 32)
    assert torch.all(d8 % 256 == 0)                                              # low t bits cleared
    assert (d8 - exact).abs().max() <= 8 * 128                                   # <= chunks * 2^(t-1)
    # the PyTorch chunk loop of iaddmm_int gives the same numbers after its 2^t scaling
    acc = torch.zeros(16, 16, dtype=torch.int32)
    for k0 in range(0, 512, 64):
        p = O.int_gemm(a[:, k0:k0 + 64].contiguous(), w[:, k0:k0 + 64].contiguous())
        acc += torch.bitwise_right_shift(p + 128, 8)
    assert torch.equal(acc * 256, d8)
    # MSB clamp: bigger chunks overflow an 18-bit accumulator more (reference test_triton_mm.py:120-123)
    e32 = (O.chunk_matmul_i8(a, w, None, 32, 8, 18) - exact).abs().float().norm()
    e128 = (O.chunk_matmul_i8(a, w, None, 128, 8, 18) - exact).abs().float().norm()
    assert e128 >= e32


def test_chunk_fp_exact_on_integers_and_tolerance():
    a = torch.randint(-6, 7, (12, 256), generator=gen(25)).float()
    w = torch.randint(-6, 7, (10, 256), generator=gen(26)).float()
    exact = a @ w.t()
    assert torch.equal(O.chunk_matmul_fp(a, w, None, 64, 0), exact)
    d = O.chunk_matmul_fp(a, w, None, 64, 16)
    per_chunk = torch.stack([O.round_and_trun(a[:, k:k + 64] @ w[:, k:k + 64].t(), 16) for k in range(0, 256, 64)]).sum(0)
    assert torch.equal(d, per_chunk)
    x = torch.randn(64, 512, generator=gen(27))
    y = torch.randn(48, 512, generator=gen(28))
    ref = x.double() @ y.double().t()
    rel = lambda t: ((O.chunk_matmul_fp(x, y, None, 64, t).double() - ref).norm() / ref.norm()).item()
    assert rel(0) < 1e-5 and rel(8) < 1e-3 and rel(16) < 1e-1 and rel(8) > rel(0)


# ---------------------------------------------------------------------------------------- fp8
def test_e4m3_cast_c_vs_torch(cref):
    codes = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float()
    vals = torch.unique(codes[~codes.isnan()])
    mids = (vals[:-1] + vals[1:]) / 2
    pts = torch.cat([vals, mids, torch.nextafter(mids, mids + 1), torch.nextafter(mids, mids - 1),
                     torch.tensor([464.0, 464.1, -464.0, 500.0, float("inf"), 2.0**-10, 2.0**-10 * 1.0001]),
                     torch.randn(3000, generator=gen(29)) * 50])
    t = pts.to(torch.float8_e4m3fn).view(torch.uint8)
    for x, code in zip(pts.tolist(), t.tolist()):
        assert cref.ref_e4m3(x) == code, x
    # all 256 codes survive a round trip through the oracle's quantizer at scale 1
    finite = vals.reshape(1, -1)
    assert torch.equal(O.fp8_quant_static(finite, torch.tensor(1.0)).float(), finite)


def test_fp8_quantizers_closed_forms():
    x = (torch.randn(6, 128, generator=gen(30)) * 3).bfloat16()
    q, s = O.fp8_quant_fpxacc(x)
    assert s.dtype == torch.bfloat16 and torch.equal(s, (x.abs().amax(dim=1, keepdim=True) / 448).clamp(min=1e-5))
    assert q.float().abs().max() <= 448
    assert torch.all(q.float().abs().amax(dim=1) >= 416)          # the row maximum lands on the top codes
    qd, _ = O.fp8_quant_fpxacc(x * 1e-3 + 0, dl8=True)
    f = qd.float()
    assert torch.all((f == 0) | (f.abs() >= O.DL8_MIN))


def _fp8_scale_properties(x, s, floor, exact):
    """The properties a symmetric per-row e4m3 scale has whatever library computes it; returns the
    list of those that fail.  ``exact``: the division ran on the fp32-widened abs-max."""
    bad = []
    xf = x.to(torch.float32)
    amax = xf.abs().amax(dim=-1, keepdim=True)
    live = (amax > 448 * floor * 1.01).reshape(-1)       # rows the floor does not govern
    if s.dtype != torch.float32:
        bad.append("dtype")
    s32 = s.to(torch.float32).reshape(-1, 1)
    q = O.fp8_quant_static(x, s32).to(torch.float32)
    if not torch.all(q[live].abs().amax(dim=-1) == 448):
        bad.append("row maximum on the top code")
    # nothing beyond the top code before the clamp: quotients stay within one e4m3 rounding of 448
    if not torch.all((xf / s32)[live].abs().amax(dim=-1) < 464):
        bad.append("no quotient beyond the top code")
    # the top code dequantizes to the row maximum: within an fp32 rounding when the division was
    # exact, within half a unit in the last place of x's dtype when it ran there
    err = (448 * s32.double() - amax.double()).abs()
    if exact:
        tol = amax.double() * 2.0 ** -23
    else:
        st = s32.to(x.dtype)                                  # spacing of x's dtype at the scale
        ulp = ((st.view(torch.int16) + 1).view(x.dtype).double() - st.double()).abs()
        tol = 448 * 0.5 * ulp * 1.001
    if not torch.all((err <= tol)[live]):
        bad.append("top code dequantizes to the row maximum")
    zero = (amax == 0).reshape(-1)
    if zero.any() and not (torch.all(s32[zero] == torch.tensor(floor, dtype=torch.float32))
                           and torch.all(q[zero] == 0)):
        bad.append("zero rows")
    return bad


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_fp8_dynamic_scale_pinned_by_invariants(dtype):
    """FP8Linear's dynamic scale is formed inside torchao (absent).  The checks below are not the
    oracle's formula retyped: they are what any correct symmetric e4m3 scale satisfies, and each
    plausible wrong rule is shown to fail at least one.  Two properties stay torchao's own and are
    arguments of the oracle and of the kernel (fmsmo_quant_act_fp8_dynamic): the floor's value and
    the dtype the division runs in."""
    g = gen(77)
    x = (torch.randn(64, 256, generator=g) * torch.logspace(-3, 3, 64).reshape(-1, 1)).to(dtype)
    x[5] = 0
    x[9, 3] = x[9].abs().max() * -2          # the maximum is a negative element
    for floor in (1e-12, 1e-5):
        assert _fp8_scale_properties(x, O.fp8_dynamic_scale(x, floor), floor, True) == []
    if dtype != torch.float32:
        s_t = O.fp8_dynamic_scale(x, 1e-5, in_x_dtype=True)
        assert _fp8_scale_properties(x, s_t, float(torch.tensor(1e-5).to(dtype)), False) == []
        assert torch.equal(s_t, s_t.to(dtype).float())            # a value of x's dtype, widened
    # wrong rules, each caught
    amax = x.float().abs().amax(dim=-1, keepdim=True)
    wrong = {
        "e4m3fnuz maximum": (amax / 240).clamp(min=1e-12),
        "int8 levels": (amax / 127).clamp(min=1e-12),
        "e5m2 maximum": (amax / 57344).clamp(min=1e-12),
        "reciprocal": (448 / amax.clamp(min=1e-12)),
        "no floor": amax / 448,
    }
    if dtype != torch.float32:
        wrong["left in x's dtype"] = (x.abs().amax(dim=-1, keepdim=True) / 448).clamp(min=1e-12)
        wrong["rounded to x's dtype"] = (amax / 448).clamp(min=1e-12).to(dtype).float()
    for name, s_bad in wrong.items():
        if name == "rounded to x's dtype" and dtype == torch.float16:
            # fp16 rounds the floor itself to zero; the live rows still show the rounding
            s_bad = s_bad.clamp(min=1e-12)
        assert _fp8_scale_properties(x, s_bad, 1e-12, True) != [], name
    # per tensor: the same properties for the flattened tensor
    s_pt = O.fp8_dynamic_scale(x, per_tensor=True)
    assert s_pt.numel() == 1
    assert _fp8_scale_properties(x.reshape(1, -1), s_pt.reshape(1, 1), 1e-12, True) == []


def test_fp8_dynamic_scale_defaults():
    x = (torch.randn(6, 128, generator=gen(30)) * 3).bfloat16()
    sd = O.fp8_dynamic_scale(x)
    assert sd.dtype == torch.float32 and sd.shape == (6, 1)
    z = torch.zeros(2, 16, dtype=torch.bfloat16)
    assert O.fp8_dynamic_scale(z).min().item() == pytest.approx(1e-12)
    assert O.fp8_dynamic_scale(z, floor=1e-5).min().item() == pytest.approx(1e-5)


def test_scaled_mm_cpu_is_plain_dequantized_matmul():
    a = torch.randint(-8, 9, (8, 32), generator=gen(31)).float().to(torch.float8_e4m3fn)
    w = torch.randint(-8, 9, (6, 32), generator=gen(32)).float().to(torch.float8_e4m3fn)
    y = O.scaled_mm_cpu(a, w.t(), torch.tensor(0.5), torch.tensor(0.25), None, torch.float32)
    assert torch.equal(y, (a.float() * 0.5) @ (w.float() * 0.25).t())


# -------------------------------------------------------------------------------- whole modules
def test_deploy_forward_consistency():
    g = gen(33)
    x = torch.randn(24, 128, generator=g).half()
    W = (0.02 * torch.randn(40, 128, generator=g)).half()
    b = (0.01 * torch.randn(40, generator=g)).half()
    bufs = O.deploy_prepare(W, b, O.qmax_perch_clipval(W).float())
    out = O.deploy_forward(x, bufs)
    # dequantized integer result == fake-quant operands multiplied in high precision
    xhat = out["q_x"].double() * out["input_scale"].double()
    what = bufs["weight"].double() * bufs["w_scale"].double()[:, None]
    ref = xhat @ what.t() + b.double()
    assert torch.allclose(out["y"].double(), ref, rtol=5e-3, atol=5e-3)
    # 3-D input is flattened and restored
    out3 = O.deploy_forward(x.reshape(2, 12, 128), bufs)
    assert out3["y"].shape == (2, 12, 40) and torch.equal(out3["y"].reshape(24, 40), out["y"])
    # all-fp16 regime: the reference's own CPU fallback (iaddmm_FP) agrees at tolerance level
    bufs16 = {k: (v.half() if v.is_floating_point() else v) for k, v in bufs.items()}
    yfp = O.deploy_forward_fp(x, bufs16)
    assert torch.allclose(yfp.float(), out["y"].float(), rtol=2e-2, atol=2e-2)


def test_qlinear_forward_with_smoothquant_close_to_fp():
    g = gen(34)
    x = torch.randn(32, 256, generator=g)
    x[:, :3] *= 50
    W = 0.02 * torch.randn(48, 256, generator=g)
    a = x.abs().amax(dim=0)
    y = O.qlinear_forward(x, W, None, a, 0.5)
    y0 = O.qlinear_forward(x, W, None)
    ref = x @ W.t()
    e = lambda t: ((t - ref).norm() / ref.norm()).item()
    assert e(y) < 0.02 and e(y) < e(y0)          # SmoothQuant helps with outlier channels


# ------------------------------------------------------------------------------------------
# AIU checkpoint conversion
# ------------------------------------------------------------------------------------------
def test_aiu_convert_layer_closed_forms_and_invariants():
    g = torch.Generator().manual_seed(5)
    w = 0.03 * torch.randn(64, 128, generator=g)
    w_cv = w.abs().amax(dim=1)
    a = torch.rand(128, generator=g) * 4 + 0.1
    out = O.aiu_convert_layer(w, w_cv, a, torch.tensor([0.5]), torch.tensor(2.0), torch.tensor(-1.0))
    q = out["weight"]
    assert q.dtype == torch.int8 and q.abs().max() <= 127
    # alpha = 0.5: s_k = sqrt(a_k) / sqrt(max_n |W_nk|)
    s = (a.double().sqrt() / w.abs().amax(dim=0).double().sqrt())
    assert torch.allclose(out["smoothq_scale"].double(), s, rtol=1e-3)
    # q = rint(127 W s / cv) away from ties, clamped
    t = (127.0 * w.double() * s / w_cv.double()[:, None]).clamp(-127, 127)
    away = (t - t.round()).abs() < 0.49
    assert torch.equal(q.double()[away], t.round()[away])
    # zero shift = integer row sums, fp32, only for asymmetric activations
    assert torch.equal(out["zero_shift"], q.sum(dim=1).float())
    sym = O.aiu_convert_layer(w, w_cv, None, None, torch.tensor(2.0), torch.tensor(-2.0))
    assert "zero_shift" not in sym and "smoothq_scale" not in sym
    # every row reaches +-127 at its arg-max when the clip value is the row maximum
    assert torch.equal(sym["weight"].abs().amax(dim=1), torch.full((64,), 127, dtype=torch.int8))
    # all-zero activation scale switches SmoothQuant off
    off = O.aiu_convert_layer(w, w_cv, torch.zeros(128), torch.tensor([0.5]))
    assert "smoothq_scale" not in off and torch.equal(off["weight"], sym["weight"])


def test_absmax_cols_is_a_running_maximum():
    x = torch.tensor([[1.0, -5.0], [-3.0, 2.0]])
    assert torch.equal(O.absmax_cols(x), torch.tensor([3.0, 5.0]))
    assert torch.equal(O.absmax_cols(x.reshape(1, 2, 2).half()), torch.tensor([3.0, 5.0]))


# ------------------------------------------------------------------ attention matmuls
def test_qbmm_exact_form_is_the_product_of_the_dequantized_operands():
    """(q1 - zp) s1 and q2 s2 are the dequantized operands; their float64 product is what the
    quantize -> integer matmul -> dequantize-with-correction chain must return.  A wrong sign, a
    correction summed over the wrong dimension or applied to the wrong operand fails this."""
    g = torch.Generator().manual_seed(3)
    m1 = torch.randn(2, 3, 17, 29, generator=g, dtype=torch.float64)
    m2 = torch.randn(2, 3, 29, 11, generator=g, dtype=torch.float64)
    s1, z1 = torch.tensor([0.031], dtype=torch.float64), torch.tensor([113], dtype=torch.int)
    s2, z2 = torch.tensor([0.027], dtype=torch.float64), torch.tensor([0], dtype=torch.int)
    y, q1, q2 = O.qbmm_int8_deploy(m1, m2, s1, z1, s2, z2)
    dq1 = (q1.double() - (z1 - 128).double()) * s1
    dq2 = q2.double() * s2
    torch.testing.assert_close(y, dq1 @ dq2, rtol=1e-12, atol=1e-12)
    # the codes are a faithful quantization: dequantized operands within half a step (unclipped)
    inside = (m1 / s1 + (z1 - 128)).abs() < 127
    assert torch.all(((dq1 - m1).abs() <= 0.5 * s1 + 1e-12)[inside])


def test_qbmm_literal_form_agrees_where_the_reference_forward_is_well_defined():
    g = torch.Generator().manual_seed(4)
    m1 = (0.2 * torch.randn(12, 8, generator=g)).half()
    m2 = (0.2 * torch.randn(8, 9, generator=g)).half()
    s1, z1 = torch.tensor([0.02]), torch.tensor([128], dtype=torch.int)
    s2, z2 = torch.tensor([0.02]), torch.tensor([0], dtype=torch.int)
    lit, q1, q2 = O.qbmm_int8_deploy(m1, m2, s1, z1, s2, z2, literal=True)
    ex, q1e, q2e = O.qbmm_int8_deploy(m1, m2, s1, z1, s2, z2)
    assert torch.equal(q1, q1e) and torch.equal(q2, q2e)
    assert (q1.int() @ q2.int()).abs().max() < 2048  # exactly representable in the fp16 matmul
    torch.testing.assert_close(lit.float(), ex.float(), rtol=2e-3, atol=1e-4)


def test_scaled_bmm_is_scaled_mm_per_batch_entry():
    g = torch.Generator().manual_seed(5)
    a = torch.randn(2, 3, 5, 16, generator=g).to(torch.float8_e4m3fn)
    b = torch.randn(2, 3, 16, 7, generator=g).to(torch.float8_e4m3fn)
    s1, s2 = torch.tensor([0.5]), torch.tensor([0.25])
    y = O.scaled_bmm(a, b, s1, s2, torch.float32)
    ref = torch.matmul(a.float() * 0.5, b.float() * 0.25)
    torch.testing.assert_close(y, ref, rtol=1e-6, atol=1e-6)
    assert O.scaled_bmm(a, b, s1, s2).dtype == torch.float32
