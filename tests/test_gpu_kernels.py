"""Parity of every HIP kernel against the CPU oracle, called through the C ABI (ctypes)."""
import pytest
import torch

from oracle import qlinear_oracle as O

pytestmark = pytest.mark.gpu


def K():
    from fms_mo_amd import kernels

    return kernels


def gen(seed):
    return torch.Generator().manual_seed(seed)


# ----------------------------------------------------------------------------- act quant int8
def _special_rows(x):
    x = x.clone()
    x[0].zero_()                       # all-zero row -> scale = T(1e-5)/127, q = 0
    x[1].zero_(); x[1, 5] = -3.0       # single +-amax -> q = -127
    x[2] = x[2].abs()                  # non-negative row
    return x


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(67, 4096), (5, 14336), (33, 64), (3, 20000)])
def test_quant_act_i8_pertoken(dev, dtype, shape):
    M, Kd = shape
    Kd = Kd // 8 * 8
    x = _special_rows((torch.randn(M, Kd, generator=gen(1)) * 3).to(dtype))
    q_ref, s_ref, _ = O.quant_act_pertoken_i8(x)
    q, s = K().quant_act_i8_pertoken(x.to(dev))
    assert torch.equal(s.cpu(), s_ref.float().reshape(-1))
    assert torch.equal(q.cpu(), q_ref)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("Kd", [64, 4096, 14336])
def test_quant_act_row_maximum_found_in_every_lane_and_wave(dev, dtype, Kd):
    """The row maximum is reduced across lanes with DPP row operations and across waves through
    LDS: one row per 16-byte chunk position, its only large element inside that chunk, so a lane,
    row of lanes or wave that the reduction skipped shows up as a wrong scale in its rows."""
    nchunk = Kd // 8
    rows = torch.arange(nchunk)
    x = torch.full((nchunk, Kd), 0.001)
    x[rows, rows * 8 + rows % 8] = (rows % 7 + 1).float() * torch.where(rows % 2 == 0, 1.0, -1.0)
    x = x.to(dtype)
    sm = (torch.rand(Kd, generator=gen(5)) + 0.5).to(dtype)
    for smooth in (None, sm):
        q_ref, s_ref, _ = O.quant_act_pertoken_i8(x, smooth)
        q, s = K().quant_act_i8_pertoken(x.to(dev), None if smooth is None else smooth.to(dev))
        assert torch.equal(s.cpu(), s_ref.float().reshape(-1))
        assert torch.equal(q.cpu(), q_ref)
    q8, s8 = K().quant_act_fp8_pertoken(x.to(dev))
    assert torch.equal(s8.cpu(), O.fp8_dynamic_scale(x).reshape(-1))


def test_quant_act_i8_bf16_wraps_like_reference(dev):
    # amax = 0.0103759765625 in bfloat16 quantises to 127.5 -> rint 128 -> int8 -128
    x = torch.zeros(2, 64, dtype=torch.bfloat16)
    x[0, 3] = 0.0103759765625
    x[0, 4] = -0.005
    x[1, 7] = -0.0103759765625
    q_ref, s_ref, _ = O.quant_act_pertoken_i8(x)
    assert q_ref[0, 3].item() == -128 and q_ref[1, 7].item() == -128  # the hazard exists
    q, s = K().quant_act_i8_pertoken(x.to(dev))
    assert torch.equal(q.cpu(), q_ref) and torch.equal(s.cpu(), s_ref.float().reshape(-1))
    q_sat, _ = K().quant_act_i8_pertoken(x.to(dev), saturate=True)
    q_ref_sat, _, _ = O.quant_act_pertoken_i8(x, saturate=True)
    assert torch.equal(q_sat.cpu(), q_ref_sat) and q_sat[0, 3].item() == 127


@pytest.mark.parametrize("sdtype", [torch.float32, torch.float16])
def test_quant_act_i8_smoothquant(dev, sdtype):
    M, Kd = 48, 4096
    x = torch.randn(M, Kd, generator=gen(2))
    idx = torch.randperm(Kd, generator=gen(3))[:41]
    x[:, idx] *= 50
    x = x.half()
    smooth = (torch.rand(Kd, generator=gen(4)) * 4 + 0.05).to(sdtype)
    q_ref, s_ref, _ = O.quant_act_pertoken_i8(x, smooth.reshape(1, -1))
    q, s = K().quant_act_i8_pertoken(x.to(dev), smooth.to(dev))
    assert torch.equal(s.cpu(), s_ref.float().reshape(-1))
    assert torch.equal(q.cpu(), q_ref)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(4133, 64), (2500, 4096), (530, 14336), (300, 28672), (70, 32768)])
def test_quant_act_i8_rows_walked_by_one_block(dev, dtype, shape):
    """More rows than resident blocks (each block quantizes several rows, prefetching the next),
    16-bit SmoothQuant divisors with a narrow range so that every x / smooth rounding shows in q."""
    M, Kd = shape
    g = gen(11)
    x = ((torch.rand(M, Kd, generator=g) + 0.5) * torch.sign(torch.randn(M, Kd, generator=g))).to(dtype)
    x = _special_rows(x)
    smooth = (torch.rand(Kd, generator=g) * 1.5 + 0.5).to(dtype)
    for sm in (None, smooth):
        q_ref, s_ref, _ = O.quant_act_pertoken_i8(x, None if sm is None else sm.reshape(1, -1))
        q, s = K().quant_act_i8_pertoken(x.to(dev), None if sm is None else sm.to(dev))
        assert torch.equal(s.cpu(), s_ref.float().reshape(-1))
        assert torch.equal(q.cpu(), q_ref)


def test_quant_act_i8_bf16_division_all_patterns(dev):
    """Every finite bf16 bit pattern of moderate magnitude as x against bf16 divisors that make
    exact ties and inexact neighbours; plus divisors outside the fast path's range."""
    bits = torch.arange(0, 1 << 16, dtype=torch.int32)
    vals = bits.to(torch.int16).view(torch.bfloat16)
    keep = torch.isfinite(vals) & (vals.float().abs() < 1e30) & ((vals.float().abs() > 1e-30) | (vals == 0))
    vals = vals[keep]
    Kd = 64
    vals = vals[: vals.numel() // Kd * Kd].reshape(-1, Kd)
    for sval in (2.0, 0.5, 3.0, 0.33203125, 1.0078125, 1.9921875, 1e-25, 1e25):
        smooth = torch.full((Kd,), sval, dtype=torch.bfloat16)
        q_ref, s_ref, _ = O.quant_act_pertoken_i8(vals, smooth.reshape(1, -1))
        q, s = K().quant_act_i8_pertoken(vals.to(dev), smooth.to(dev))
        ok = torch.isfinite(s_ref.float().reshape(-1))
        assert torch.equal(s.cpu()[ok], s_ref.float().reshape(-1)[ok]), sval
        assert torch.equal(q.cpu()[ok], q_ref[ok]), sval


@pytest.mark.parametrize("shape", [(4133, 64), (2500, 4096), (300, 6144), (530, 14336)])
def test_quant_act_i8_fp16_x_fp32_smooth_rows(dev, shape):
    """fp16 x with an fp32 SmoothQuant scale: torch promotes to fp32, the quantizer runs in fp32
    (the reference's example flow keeps quantizer buffers fp32).  Includes divisors outside the
    fast path's range (block-wide IEEE fallback) and rows that overflow to inf."""
    M, Kd = shape
    g = gen(12)
    x = ((torch.rand(M, Kd, generator=g) * 3 + 0.01) * torch.sign(torch.randn(M, Kd, generator=g))).half()
    x = _special_rows(x)
    x[5, 3] = 65504.0
    base = torch.rand(Kd, generator=g) * 1.5 + 0.5
    for variant in ("plain", "tiny_divisor", "huge_divisor"):
        smooth = base.clone()
        if variant == "tiny_divisor":
            smooth[7] = 1e-30      # x / 1e-30 stays finite in fp32 only for small x; outside 2^-60
        if variant == "huge_divisor":
            smooth[9] = 3e30
        q_ref, s_ref, _ = O.quant_act_pertoken_i8(x, smooth.reshape(1, -1))
        q, s = K().quant_act_i8_pertoken(x.to(dev), smooth.to(dev))
        ok = torch.isfinite(s_ref.float().reshape(-1))
        assert torch.equal(s.cpu()[ok], s_ref.float().reshape(-1)[ok]), variant
        assert torch.equal(q.cpu()[ok], q_ref[ok]), variant


@pytest.mark.parametrize("shape", [(2500, 4096), (300, 6144), (530, 14336)])
def test_quant_act_i8_bf16_x_fp32_smooth_rows(dev, shape):
    """bf16 x with an fp32 SmoothQuant scale (a bf16 model with fp32 quantizer buffers): fp32
    arithmetic as above, plus what bf16's range adds -- rows of tiny values (maximum below 2^-80:
    IEEE path), tiny and huge elements inside ordinary rows, rows that overflow."""
    M, Kd = shape
    g = gen(13)
    x = ((torch.rand(M, Kd, generator=g) * 3 + 0.01) * torch.sign(torch.randn(M, Kd, generator=g))).bfloat16()
    x = _special_rows(x)
    x[5, 3] = 3.0e38                                   # overflows after the divide: scale inf
    x[6] = (x[6].float() * 1e-30).bfloat16()           # whole row tiny: maximum ~3e-30 < 2^-80
    x[7] = (x[7].float() * 2.0 ** -110).bfloat16()     # and deeper still
    x[8, ::5] = (x[8, ::5].float() * 1e-36).bfloat16() # tiny elements in an ordinary row
    x[9, 11] = 1.0e30                                  # one huge, finite element
    base = torch.rand(Kd, generator=g) * 1.5 + 0.5
    for variant in ("plain", "tiny_divisor", "huge_divisor"):
        smooth = base.clone()
        if variant == "tiny_divisor":
            smooth[7] = 1e-30
        if variant == "huge_divisor":
            smooth[9] = 3e30
        q_ref, s_ref, _ = O.quant_act_pertoken_i8(x, smooth.reshape(1, -1))
        q, s = K().quant_act_i8_pertoken(x.to(dev), smooth.to(dev))
        ok = torch.isfinite(s_ref.float().reshape(-1))
        assert torch.equal(s.cpu()[ok], s_ref.float().reshape(-1)[ok]), variant
        assert torch.equal(q.cpu()[ok], q_ref[ok]), variant


def test_quant_act_i8_fp16_division_ties_and_subnormals(dev):
    """Every finite fp16 bit pattern as x against divisors that make exact ties (powers of two on
    subnormal quotients), tiny and huge quotients: x / smooth must round like torch's fp16
    division.  One column per row group keeps the per-row scale from hiding the quotient."""
    bits = torch.arange(0, 1 << 16, dtype=torch.int32)
    vals = bits.to(torch.int16).view(torch.float16)
    vals = vals[torch.isfinite(vals)]                       # 63488 values
    Kd = 64
    vals = vals[: vals.numel() // Kd * Kd].reshape(-1, Kd)  # [992, 64], similar magnitudes per row
    for sval in (2.0, 4.0, 0.5, 3.0, 0.3330078125, 1.0009765625, 1.9990234375, 6.103515625e-05, 1024.0):
        smooth = torch.full((Kd,), sval, dtype=torch.float16)
        q_ref, s_ref, _ = O.quant_act_pertoken_i8(vals, smooth.reshape(1, -1))
        q, s = K().quant_act_i8_pertoken(vals.to(dev), smooth.to(dev))
        assert torch.equal(s.cpu(), s_ref.float().reshape(-1)), sval
        ok = torch.isfinite(s_ref.float().reshape(-1))   # rows that overflowed hold inf / inf = nan
        assert torch.equal(q.cpu()[ok], q_ref[ok]), sval
        assert torch.equal(q.cpu()[~ok] == 0, q_ref[~ok] == 0), sval   # finite / inf = 0 there


def test_quant_act_i8_static(dev):
    x = (torch.randn(37, 1024, generator=gen(5)) * 4).half()
    for scale, zp, sym in [(0.0627, 128, 1), (0.031, 117, 0), (0.05, 128, 0)]:
        q_ref = O.quant_act_static_raw(x, torch.tensor([scale]), zp, sym)
        q = K().quant_act_i8_static(x.to(dev), scale, zp, sym)
        assert torch.equal(q.cpu(), q_ref)


@pytest.mark.parametrize("xdt", [torch.float16, torch.bfloat16, torch.float32])
def test_quant_act_i8_static_every_pattern_and_range(dev, xdt):
    """x / scale runs without the range scaling and fix-up of the IEEE sequence where the plain
    operations give the same quotient; outside that range, and for non-finite x, it falls back.
    Every 16-bit pattern except NaN (fp32: random values over the whole exponent range, zeros and
    infinities), scales inside and outside the fast range."""
    if xdt == torch.float32:
        g = gen(77)
        mant = torch.rand(65536, generator=g) + 1.0
        expo = torch.randint(-140, 128, (65536,), generator=g).float()
        x = mant * torch.exp2(expo) * torch.where(torch.rand(65536, generator=g) < 0.5, -1.0, 1.0)
        x[:4] = torch.tensor([0.0, -0.0, float("inf"), float("-inf")])
    else:
        x = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(xdt)
        x = x[~torch.isnan(x)]
    x = x[: x.numel() // 64 * 64].reshape(-1, 64)
    for scale in (0.0371, 1.0, 2.0 ** -19, 2.0 ** -30, 3.0e5, 7.0e7, 1.1e-3):
        for zp, sym in ((128, 1), (117, 0)):
            q_ref = O.quant_act_static_raw(x, torch.tensor([scale]), zp, sym)
            q = K().quant_act_i8_static(x.to(dev), scale, zp, sym)
            assert torch.equal(q.cpu(), q_ref), f"scale {scale} zp {zp} sym {sym}"


# ------------------------------------------------------------------------------ act quant fp8
def test_fp8_cast_all_codes_and_midpoints(dev):
    codes = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float()
    vals = codes[~codes.isnan()]
    vals = torch.unique(vals)
    mids = (vals[:-1] + vals[1:]) / 2
    eps = torch.cat([torch.nextafter(mids, mids + 1), torch.nextafter(mids, mids - 1)])
    extra = torch.tensor([448.0, 449.0, 463.9, 464.0, -464.0, 1e-10, -1e-10, 0.0, 2.0**-10, 2.0**-9])
    t = torch.cat([vals, mids, eps, extra])
    t = t[t.abs() <= 464.0]
    n = t.numel() // 8 * 8
    t = t[:n].reshape(1, n)
    # static scale 1.0, FP8_LINEAR clamps to +-448 first, exactly like the oracle
    ref = O.fp8_quant_static(t, torch.tensor(1.0))
    from fms_mo_amd import _lib as L

    q, _ = K().quant_act_fp8_pertoken(t.to(dev), L.FP8_LINEAR, static_scale=1.0)
    assert torch.equal(q.cpu().view(torch.uint8), ref.view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_quant_act_fp8_dynamic_all_codes_midpoints_and_many_rows(dev, dtype):
    """Dynamic per-token path on 16-bit inputs: a row whose maximum is 448 (scale exactly 1) holding
    every e4m3 value, every midpoint and the 16-bit neighbours of the midpoints; more rows than
    resident blocks; rows with inf."""
    from fms_mo_amd import _lib as L

    codes = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float()
    vals = torch.unique(codes[~codes.isnan()])
    mids = ((vals[:-1] + vals[1:]) / 2).to(dtype)
    up = torch.nextafter(mids, torch.full_like(mids, 1e4)).float()
    dn = torch.nextafter(mids, torch.full_like(mids, -1e4)).float()
    t = torch.cat([vals, mids.float(), up, dn, torch.tensor([0.0, -0.0, 2.0**-10, 2.0**-9, 1e-7])])
    t = t[t.abs() <= 448.0]
    n = (t.numel() + 7) // 8 * 8
    row = torch.zeros(n)
    row[: t.numel()] = t
    g = gen(31)
    x = (torch.randn(2600, n, generator=g) * 3)
    x[0] = row
    x[1] = row * 0.5
    x[2] = row * 3.0
    x[7, 5] = float("inf")
    x = x.to(dtype)
    s_ref = O.fp8_dynamic_scale(x)
    q_ref = O.fp8_quant_static(x, s_ref)
    q, s = K().quant_act_fp8_pertoken(x.to(dev), L.FP8_LINEAR)
    ok = torch.isfinite(s_ref.reshape(-1))
    assert torch.equal(s.cpu()[ok], s_ref.reshape(-1)[ok])
    assert torch.equal(q.cpu().view(torch.uint8)[ok], q_ref.view(torch.uint8)[ok])
    for dl8 in (False, True):
        q_ref, s_ref = O.fp8_quant_fpxacc(x, per_tensor=False, dl8=dl8)
        q, s = K().quant_act_fp8_pertoken(x.to(dev), L.FP8_FPXACC_DL8 if dl8 else L.FP8_FPXACC)
        ok = torch.isfinite(s_ref.float().reshape(-1))
        assert torch.equal(s.cpu()[ok], s_ref.float().reshape(-1)[ok])
        assert torch.equal(q.cpu().view(torch.uint8)[ok], q_ref.view(torch.uint8)[ok])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_quant_act_fp8_linear(dev, dtype):
    from fms_mo_amd import _lib as L

    x = _special_rows((torch.randn(40, 4096, generator=gen(6)) * 2).to(dtype))
    s_ref = O.fp8_dynamic_scale(x)
    q_ref = O.fp8_quant_static(x, s_ref)
    q, s = K().quant_act_fp8_pertoken(x.to(dev), L.FP8_LINEAR)
    assert torch.equal(s.cpu(), s_ref.reshape(-1))
    assert torch.equal(q.cpu().view(torch.uint8), q_ref.view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("per_tensor", [False, True])
def test_quant_act_fp8_dynamic_scale_rules(dev, dtype, per_tensor):
    """fmsmo_quant_act_fp8_dynamic: floor and division dtype of the dynamic scale as the caller
    states them, per token and per tensor (column abs-max on the device, nothing read back);
    scales and codes bit-exact against the oracle."""
    from fms_mo_amd import _lib as L

    for Kd, scale in ((4096, 2.0), (14336, 0.01), (64, 300.0), (20000, 1.0)):
        x = _special_rows((torch.randn(37, Kd, generator=gen(61)) * scale).to(dtype))
        x[5] = x[5] * 1e-4                                  # a row far below the tensor's maximum
        for floor, in_xt in ((1e-12, False), (1e-5, False), (1e-5, True), (2e-3, True), (2e-3, False)):
            if in_xt and dtype == torch.float16 and floor < 1e-7:
                continue
            s_ref = O.fp8_dynamic_scale(x, floor, in_xt, per_tensor)
            q_ref = O.fp8_quant_static(x, s_ref)
            q, s = K().quant_act_fp8_dynamic(x.to(dev), L.FP8_LINEAR, per_tensor, floor, in_xt)
            assert s.dtype == torch.float32
            assert torch.equal(s.cpu(), s_ref.reshape(-1)), (Kd, floor, in_xt)
            assert torch.equal(q.cpu().view(torch.uint8), q_ref.view(torch.uint8)), (Kd, floor, in_xt)
    # the defaults of the per-token entry point are (1e-12, fp32)
    q0, s0 = K().quant_act_fp8_pertoken(x.to(dev), L.FP8_LINEAR)
    q1, s1 = K().quant_act_fp8_dynamic(x.to(dev), L.FP8_LINEAR, False, 1e-12, False)
    assert torch.equal(s0, s1) and torch.equal(q0.view(torch.uint8), q1.view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("dl8", [False, True])
def test_quant_act_fp8_fpxacc_per_tensor(dev, dtype, dl8):
    """The per-tensor scales of LinearFuncFPxFwdBwd.forward (amax / 448 in x's dtype, floor 1e-5)
    from the device-side column abs-max."""
    from fms_mo_amd import _lib as L

    for Kd, scale in ((4096, 2.0), (12800, 0.05), (72, 100.0)):
        x = _special_rows((torch.randn(29, Kd, generator=gen(62)) * scale).to(dtype))
        q_ref, s_ref = O.fp8_quant_fpxacc(x, per_tensor=True, dl8=dl8)
        q, s = K().quant_act_fp8_dynamic(x.to(dev), L.FP8_FPXACC_DL8 if dl8 else L.FP8_FPXACC,
                                         True, 1e-5, True)
        assert torch.equal(s.cpu(), s_ref.float().reshape(-1))
        assert torch.equal(q.cpu().view(torch.uint8), q_ref.view(torch.uint8))
    z = torch.zeros(8, 64, dtype=dtype)
    q, s = K().quant_act_fp8_dynamic(z.to(dev), L.FP8_FPXACC, True, 1e-5, True)
    assert s.item() == torch.tensor(1e-5).to(dtype).float().item() and not q.cpu().view(torch.uint8).any()


def test_quant_act_fp8_dynamic_rejects_bad_options(dev):
    from fms_mo_amd import _lib as L

    x = torch.randn(4, 64, device=dev).half()
    for floor in (0.0, -1.0, float("nan"), 2.0 ** 61):
        with pytest.raises(L.FmsMoHipError):
            K().quant_act_fp8_dynamic(x, L.FP8_LINEAR, False, floor, False)
    with pytest.raises(L.FmsMoHipError):      # an fp16 floor that rounds to zero would divide by it
        K().quant_act_fp8_dynamic(x, L.FP8_LINEAR, False, 1e-12, True)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("dl8", [False, True])
def test_quant_act_fp8_fpxacc(dev, dtype, dl8):
    from fms_mo_amd import _lib as L

    x = _special_rows((torch.randn(40, 2048, generator=gen(7)) * 2).to(dtype))
    x[3] *= 1e-4
    q_ref, s_ref = O.fp8_quant_fpxacc(x, per_tensor=False, dl8=dl8)
    q, s = K().quant_act_fp8_pertoken(x.to(dev), L.FP8_FPXACC_DL8 if dl8 else L.FP8_FPXACC)
    assert torch.equal(s.cpu(), s_ref.float().reshape(-1))
    assert torch.equal(q.cpu().view(torch.uint8), q_ref.view(torch.uint8))


def test_quantizers_random_shapes_dtypes_and_magnitudes(dev):
    """Eighty seeded cases over row counts, row lengths (any multiple of 8), dtypes, divisor
    dtypes and magnitudes from 1e-3 to 1e3: whichever quantizer kernel serves a case (packed
    16-bit row walker in any chunk count, fp32-divisor walker, generic one-row-per-block), codes
    and scales are the oracle's, for the int8, the e4m3 and the static int8 quantizers."""
    import random

    from fms_mo_amd import _lib as L

    rng = random.Random(2468)
    kn = K()
    for case in range(80):
        M = rng.choice([rng.randint(1, 8), rng.randint(9, 300), rng.randint(300, 3000)])
        Kd = 8 * rng.choice([rng.randint(1, 64), rng.randint(64, 1024), rng.randint(1024, 4200)])
        if M > 300:
            Kd = min(Kd, 8 * 640)
        dt = rng.choice([torch.float16, torch.bfloat16, torch.float32])
        mag = 10.0 ** rng.uniform(-3, 3 if dt != torch.float16 else 2)
        tag = f"case {case}: M={M} K={Kd} {dt} mag={mag:.3g}"
        g = gen(3000 + case)
        x = (torch.randn(M, Kd, generator=g) * mag).to(dt)
        if M >= 3:
            x = _special_rows(x)
        kind = rng.choice(["none", "same", "f32"])
        sm = None
        if kind != "none":
            sm = (torch.rand(Kd, generator=g) * 3 + 0.1).to(dt if kind == "same" else torch.float32)
        q_ref, s_ref, _ = O.quant_act_pertoken_i8(x, None if sm is None else sm.reshape(1, -1))
        q, s = kn.quant_act_i8_pertoken(x.to(dev), None if sm is None else sm.to(dev))
        assert torch.equal(s.cpu(), s_ref.float().reshape(-1)), tag + f" smooth={kind}"
        assert torch.equal(q.cpu(), q_ref), tag + f" smooth={kind}"
        s8_ref = O.fp8_dynamic_scale(x)
        q8_ref = O.fp8_quant_static(x, s8_ref)
        q8, s8 = kn.quant_act_fp8_pertoken(x.to(dev), L.FP8_LINEAR)
        assert torch.equal(s8.cpu(), s8_ref.reshape(-1)), tag
        assert torch.equal(q8.cpu().view(torch.uint8), q8_ref.view(torch.uint8)), tag
        scale = mag * rng.uniform(0.01, 0.05)
        zp, sym = rng.choice([(128, 1), (rng.randint(100, 156), 0)])
        qs_ref = O.quant_act_static_raw(x, torch.tensor([scale]), zp, sym)
        qs = kn.quant_act_i8_static(x.to(dev), scale, zp, sym)
        assert torch.equal(qs.cpu(), qs_ref), tag + f" static scale={scale:.4g} zp={zp} sym={sym}"


# ---------------------------------------------------------------------------------- int8 GEMM
def _rand_i8(shape, seed):
    return torch.randint(-128, 128, shape, generator=gen(seed), dtype=torch.int8)


@pytest.mark.parametrize("shape", [(512, 4096, 4096), (300, 520, 1024), (256, 256, 64),
                                   (17, 4096, 4096), (1000, 1200, 256), (129, 130, 80),
                                   (64, 72, 4112), (2048, 2304, 512),
                                   # large ragged shapes, K in whole 128-byte slabs: the first three
                                   # run 256x192 tiles (fuller last round), the last one 256x256
                                   (4000, 4100, 384), (4097, 4095, 128), (3900, 4352, 256), (4000, 4000, 384)])
def test_gemm_i8_i32_exact(dev, shape):
    M, N, Kd = shape
    a, w = _rand_i8((M, Kd), 11), _rand_i8((N, Kd), 12)
    ref = O.int_gemm(a, w)
    c = K().gemm_i8_i32(a.to(dev), w.to(dev))
    assert torch.equal(c.cpu(), ref)


@pytest.mark.parametrize("shape", [
    # a few rows: the weight-streaming decode kernels store their int32 sums (row kernel, MFMA
    # streaming kernel with whole and half row groups, streamed activations, generic decode kernel,
    # batches of up to 64 rows)
    (1, 4096, 4096), (2, 1000, 4096), (1, 520, 14336), (3, 4096, 14336), (4, 6144, 4096), (9, 264, 12800),
    (16, 4096, 4096), (16, 1000, 2048), (5, 300, 384), (16, 4104, 14336), (24, 4096, 4096), (33, 520, 2048),
    (64, 6144, 4096), (32, 1000, 8192),
    # few output tiles, long reduction: K slices through the workspace
    (17, 4096, 14336), (128, 4096, 4096), (100, 1000, 8192), (512, 4096, 4096), (300, 520, 14336),
    (1024, 2048, 4096)])
def test_gemm_i8_i32_small_batches(dev, shape):
    M, N, Kd = shape
    g = torch.Generator(device=dev).manual_seed(M + N + Kd)
    a = torch.randint(-128, 128, (M, Kd), generator=g, dtype=torch.int8, device=dev)
    w = torch.randint(-128, 128, (N, Kd), generator=g, dtype=torch.int8, device=dev)
    ref = (a.double() @ w.double().t()).to(torch.int32)
    c = K().gemm_i8_i32(a, w)
    assert c.dtype == torch.int32 and torch.equal(c, ref)
    if M * N * Kd <= 2 ** 28:  # the oracle itself on the smaller ones
        assert torch.equal(c.cpu(), O.int_gemm(a.cpu(), w.cpu()))


def test_gemm_i8_i32_with_and_without_workspace(dev):
    """The C entry points: with a workspace the K slices, without one the single pass; the same
    bits, and a workspace that is too small or NULL is simply not used."""
    from fms_mo_amd import _lib as L

    lib = L.load()
    M, N, Kd = 100, 1024, 8192
    a, w = _rand_i8((M, Kd), 15).to(dev), _rand_i8((N, Kd), 16).to(dev)
    ref = O.int_gemm(a.cpu(), w.cpu())
    need = lib.fmsmo_gemm_workspace_bytes(M, N, Kd)
    assert need > 0
    st = torch.cuda.current_stream().cuda_stream
    for nbytes in (need, need - 16, 0):
        ws = torch.empty((max(nbytes, 16),), dtype=torch.uint8, device=dev)
        c = torch.full((M, N), -7, dtype=torch.int32, device=dev)
        L.call("fmsmo_gemm_i8_i32_ws", a.data_ptr(), Kd, w.data_ptr(), Kd, c.data_ptr(), N, M, N, Kd,
               ws.data_ptr() if nbytes else None, nbytes, st)
        torch.cuda.synchronize()
        assert torch.equal(c.cpu(), ref)


def test_gemm_i8_i32_random_shapes_cover_every_kernel_choice(dev):
    """Forty seeded shapes between 17 and ~4500 rows / columns: whatever kernel and tile shape the
    library picks for a shape (fmsmo_gemm_plan names it), the int32 result must equal the exact
    product, here taken in float64 on the GPU (|acc| < 2^53) so that large shapes stay cheap."""
    import random

    rng = random.Random(1234)
    seen = set()
    for case in range(40):
        M = rng.choice([rng.randint(17, 300), rng.randint(300, 2100), rng.randint(2100, 4500)])
        N = rng.choice([rng.randint(8, 300), rng.randint(300, 2100), rng.randint(2100, 6200)])
        Kd = rng.choice([16 * rng.randint(1, 40), 64 * rng.randint(1, 24), 128 * rng.randint(1, 16)])
        g = torch.Generator(device=dev).manual_seed(100 + case)
        a = torch.randint(-128, 128, (M, Kd), generator=g, dtype=torch.int8, device=dev)
        w = torch.randint(-128, 128, (N, Kd), generator=g, dtype=torch.int8, device=dev)
        plan = K().gemm_plan(M, N, Kd)
        seen.add(plan[:3])
        c = K().gemm_i8_i32(a, w)
        ref = (a.double() @ w.double().t()).to(torch.int32)
        assert torch.equal(c, ref), f"M={M} N={N} K={Kd} plan={plan}"
    # the sample reaches the generic kernel, both MFMA pipelines and all five tile shapes
    assert {p[0] for p in seen} >= {1, 2, 3}
    assert {p[1:] for p in seen if p[0] in (1, 2)} >= {(256, 256), (256, 192), (256, 128), (128, 256), (128, 128)}


def test_gemm_i8_dq_random_shapes_scales_and_epilogues(dev):
    """Thirty seeded shapes from 17 rows up: per-row or single activation scale, per-column or
    single weight scale, bias of any dtype or none, 16-bit and fp32 outputs, the reference epilogue
    (bit-exact against the oracle) and both fp32-scale forms."""
    import random

    from fms_mo_amd import _lib as L

    rng = random.Random(9753)
    kn = K()
    for case in range(30):
        M = rng.choice([rng.randint(17, 300), rng.randint(300, 2100), rng.randint(2100, 4500)])
        N = rng.choice([rng.randint(8, 300), rng.randint(300, 2100), rng.randint(2100, 6200)])
        Kd = rng.choice([16 * rng.randint(1, 40), 64 * rng.randint(1, 24), 128 * rng.randint(1, 40)])
        g = torch.Generator(device=dev).manual_seed(4000 + case)
        # every third case: operands that are column slices of wider buffers (row stride > K)
        pa, pw = (16 * rng.randint(1, 8), 16 * rng.randint(1, 8)) if case % 3 == 2 else (0, 0)
        a = torch.randint(-128, 128, (M, Kd + pa), generator=g, dtype=torch.int8, device=dev)[:, :Kd]
        w = torch.randint(-128, 128, (N, Kd + pw), generator=g, dtype=torch.int8, device=dev)[:, :Kd]
        acc = (a.double() @ w.double().t()).to(torch.int32).cpu()
        an, wn = rng.choice([1, M]), rng.choice([1, N])
        s_a = (torch.rand(an, 1, generator=gen(4100 + case)) * 0.05 + 1e-3).half()
        s_w = (torch.rand(wn, generator=gen(4200 + case)) * 1e-2 + 1e-4).float()
        bdt = rng.choice([None, torch.float16, torch.bfloat16, torch.float32])
        bias = None if bdt is None else (torch.randn(N, generator=gen(4300 + case)) * 0.1).to(bdt)
        bd = None if bias is None else bias.to(dev)
        odt = rng.choice([torch.float16, torch.bfloat16, torch.float32])
        tag = f"case {case}: M={M} N={N} K={Kd} a_scales={an} w_scales={wn} bias={bdt} out={odt} plan={kn.gemm_plan(M, N, Kd)}"
        sad, swd = s_a.float().reshape(-1).to(dev), s_w.to(dev)
        acc_dt = torch.float32 if odt == torch.float32 else torch.float16
        ref = O.epilogue_ref(acc, s_a, s_w, bias, odt, acc_dtype=acc_dt)
        y = kn.gemm_i8_dq(a, w, sad, swd, bd, out_dtype=odt, exact_ref=True).cpu()
        bits = torch.int32 if odt == torch.float32 else torch.int16
        assert torch.equal(y.view(bits), ref.view(bits)), tag
        ref2 = O.epilogue_f32(acc, s_a, s_w, bias, odt)
        y2 = kn.gemm_i8_dq(a, w, sad, swd, bd, out_dtype=odt, exact_ref=False).cpu()
        # (the oracle's fma is emulated in float64: a rare double rounding may differ by one ulp)
        torch.testing.assert_close(y2.float(), ref2.float(), rtol=1e-2, atol=1e-2, msg=tag + " fp32-scale fma")
        assert (y2.view(bits) != ref2.view(bits)).float().mean().item() < 1e-5, tag + " fp32-scale fma"
        ref3 = (acc.float() * (s_a.float() * s_w.float()))
        if bias is not None:
            ref3 = ref3 + bias.float()
        y3 = kn.gemm_i8_dq(a, w, sad, swd, bd, out_dtype=odt, epilogue=L.EPI_F32_MULADD).cpu()
        assert torch.equal(y3.view(bits), ref3.to(odt).view(bits)), tag + " fp32-scale mul+add"


def test_gemm_i8_i32_strided_rows(dev):
    big_a, big_w = _rand_i8((200, 2048 + 64), 13), _rand_i8((300, 2048 + 128), 14)
    a, w = big_a[:, :2048], big_w[:, :2048]
    c = K().gemm_i8_i32(a.to(dev)[:, :], w.to(dev)[:, :])
    ad, wd = big_a.to(dev)[:, :2048], big_w.to(dev)[:, :2048]
    assert ad.stride(0) == 2048 + 64
    c2 = K().gemm_i8_i32(ad, wd)
    ref = O.int_gemm(a.contiguous(), w.contiguous())
    assert torch.equal(c.cpu(), ref) and torch.equal(c2.cpu(), ref)


@pytest.mark.parametrize("out_dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(512, 4096, 4096), (300, 520, 1024), (16, 512, 1024), (1, 256, 128),
                                   (2048, 6100, 256),   # 256x192 tiles, ragged last column tile
                                   (2000, 4090, 384)])  # 256x128 tiles, ragged last row and column tiles
def test_gemm_i8_dq_reference_epilogue_bit_exact(dev, shape, out_dtype):
    M, N, Kd = shape
    a, w = _rand_i8((M, Kd), 21), _rand_i8((N, Kd), 22)
    s_a = (torch.rand(M, 1, generator=gen(23)) * 0.05 + 1e-3).half()
    s_w = (torch.rand(N, generator=gen(24)) * 1e-3 + 1e-5).float()
    bias = (torch.randn(N, generator=gen(25)) * 0.01).half()
    acc = O.int_gemm(a, w)
    ref = O.epilogue_ref(acc, s_a, s_w, bias, out_dtype)
    y = K().gemm_i8_dq(a.to(dev), w.to(dev), s_a.float().to(dev), s_w.to(dev), bias.to(dev),
                       out_dtype=out_dtype, exact_ref=True)
    assert torch.equal(y.cpu().view(torch.int16), ref.view(torch.int16))
    # fp32-scale epilogue: within the tolerance the task states for 16-bit outputs
    y2 = K().gemm_i8_dq(a.to(dev), w.to(dev), s_a.float().to(dev), s_w.to(dev), bias.to(dev),
                        out_dtype=out_dtype, exact_ref=False)
    ref2 = O.epilogue_f32(acc, s_a, s_w, bias, out_dtype)
    torch.testing.assert_close(y2.cpu().float(), ref2.float(), rtol=1e-2, atol=1e-2)


def test_c1_config_deploy_forward(dev):
    """The reference's CPU-runnable configuration: x fp16 [512,4096] ~N(0,1), W fp16 [4096,4096] ~N(0,0.02), bias
    ~N(0,0.01), per-token act / per-channel weight int8, seed 0."""
    g = gen(0)
    x = torch.randn(512, 4096, generator=g).half()
    W = (0.02 * torch.randn(4096, 4096, generator=g)).half()
    b = (0.01 * torch.randn(4096, generator=g)).half()
    bufs = O.deploy_prepare(W, b, O.qmax_perch_clipval(W).float())
    ref = O.deploy_forward(x, bufs)
    q, s = K().quant_act_i8_pertoken(x.to(dev))
    assert torch.equal(q.cpu(), ref["q_x"])
    assert torch.equal(s.cpu(), ref["input_scale"].float().reshape(-1))
    wq = bufs["weight"].to(dev)
    acc = K().gemm_i8_i32(q, wq)
    assert torch.equal(acc.cpu(), ref["acc"])
    y = K().gemm_i8_dq(q, wq, s, bufs["w_scale"].to(dev), bufs["bias"].to(dev),
                       out_dtype=torch.float16, exact_ref=True)
    assert torch.equal(y.cpu().view(torch.int16), ref["y"].view(torch.int16))
    # fp32-scale epilogue (no fp16 rounding of s_x*s_w): within the stated tolerance of the
    # reference's dequantized result
    y32 = K().gemm_i8_dq(q, wq, s, bufs["w_scale"].to(dev), bufs["bias"].to(dev),
                         out_dtype=torch.float16, exact_ref=False)
    torch.testing.assert_close(y32.cpu().float(), ref["y"].float(), rtol=1e-2, atol=1e-2)
    # The reference's fake-quant QLinear.forward (fp16 Q/dQ operands, fp16 F.linear) is a
    # different rounding path: its own deploy path already leaves the 1e-2 band on ~0.015 % of
    # the outputs (CPU oracle vs CPU oracle), so only the bulk is compared.
    y_fake = O.qlinear_forward(x, W, b)
    for out in (y, y32):
        d = (out.cpu().float() - y_fake.float()).abs()
        assert (d > 1e-2 + 1e-2 * y_fake.float().abs()).float().mean() < 1e-3
        assert d.max() < 5e-2


# ------------------------------------------------------------------------------ skinny (decode)
@pytest.mark.parametrize("M", [1, 2, 4, 16, 7])
@pytest.mark.parametrize("NK", [(4096, 4096), (6144, 4096), (4096, 14336), (1000, 384),
                                (1000, 5120), (520, 11008), (300, 13824)])  # Llama-2 reduction lengths
def test_gemv_i8_matches_gemm_semantics(dev, M, NK):
    N, Kd = NK
    a, w = _rand_i8((M, Kd), 31), _rand_i8((N, Kd), 32)
    s_a = (torch.rand(M, 1, generator=gen(33)) * 0.05 + 1e-3).bfloat16()
    s_w = (torch.rand(N, generator=gen(34)) * 1e-3 + 1e-5).float()
    bias = (torch.randn(N, generator=gen(35)) * 0.01).bfloat16()
    acc = O.int_gemm(a, w)
    ref = O.epilogue_ref(acc, s_a, s_w, bias, torch.bfloat16)
    y = K().gemm_i8_dq(a.to(dev), w.to(dev), s_a.float().to(dev), s_w.to(dev), bias.to(dev),
                       out_dtype=torch.bfloat16, exact_ref=True, force_gemv=True)
    assert torch.equal(y.cpu().view(torch.int16), ref.view(torch.int16))
    y_auto = K().gemm_i8_dq(a.to(dev), w.to(dev), s_a.float().to(dev), s_w.to(dev), bias.to(dev),
                            out_dtype=torch.bfloat16, exact_ref=True)
    assert torch.equal(y_auto.cpu().view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("M", [1, 2, 3, 5, 8, 9, 16])
@pytest.mark.parametrize("NKd", [(1000, 14336), (8200, 14336), (1000, 12800), (520, 8192), (520, 16384)])
def test_decode_long_rows(dev, M, NKd):
    """Long reductions (14336 and 12800: the shallow two-step pipeline of the streaming kernel;
    one or two tokens go to the row kernel or to the streaming kernel depending on K and operand
    type).  N = 1000: ragged last group of 16 weight rows; N = 8200: several groups per block.
    int8 bit-exact, e4m3 exact on small integers."""
    N, Kd = NKd
    a, w = _rand_i8((M, Kd), 36), _rand_i8((N, Kd), 37)
    s_a = (torch.rand(M, 1, generator=gen(38)) * 0.05 + 1e-3).half()
    s_w = (torch.rand(N, generator=gen(39)) * 1e-3 + 1e-5).float()
    bias = (torch.randn(N, generator=gen(40)) * 0.01).half()
    ref = O.epilogue_ref(O.int_gemm(a, w), s_a, s_w, bias, torch.float16)
    y = K().gemm_i8_dq(a.to(dev), w.to(dev), s_a.float().to(dev), s_w.to(dev), bias.to(dev),
                       out_dtype=torch.float16, exact_ref=True)
    assert torch.equal(y.cpu().view(torch.int16), ref.view(torch.int16))
    a8 = torch.randint(-3, 4, (M, Kd), generator=gen(41)).float()
    w8 = torch.randint(-3, 4, (N, Kd), generator=gen(42)).float()
    one = torch.ones(1, device=dev)
    y8 = K().gemm_fp8_dq(a8.to(torch.float8_e4m3fn).to(dev), w8.to(torch.float8_e4m3fn).to(dev), one, one,
                         None, out_dtype=torch.float32)
    assert torch.equal(y8.cpu(), a8 @ w8.t())


def test_decode_range_random_shapes(dev):
    """Sixty seeded shapes with 1..64 tokens: whichever decode kernel serves a shape (row kernel,
    streaming kernel in any of its instantiations, generic kernel, K slices), the int32 sums are
    the exact product, the reference epilogue gives the oracle's bits, e4m3 is exact on small
    integers, and the fused linear (where it serves the shape) equals quantizer + matmul."""
    import random

    rng = random.Random(4321)
    kn = K()
    for case in range(60):
        M = rng.choice([1, 2, 3, 4, rng.randint(5, 16), rng.randint(17, 32), rng.randint(33, 64)])
        N = rng.choice([rng.randint(1, 64), rng.randint(65, 3000), 8 * rng.randint(1, 800), 16 * rng.randint(1, 400)])
        Kd = rng.choice([16 * rng.randint(1, 64), 128 * rng.randint(1, 128),
                         1024 * rng.choice([1, 2, 4, 5, 8, 11, 13, 14, 16]), 12800, 14336])
        tag = f"case {case}: M={M} N={N} K={Kd}"
        g = torch.Generator(device=dev).manual_seed(500 + case)
        # every third case: operands that are column slices of wider buffers (row stride > K)
        pa, pw = (16 * rng.randint(1, 8), 16 * rng.randint(1, 8)) if case % 3 == 2 else (0, 0)
        a = torch.randint(-128, 128, (M, Kd + pa), generator=g, dtype=torch.int8, device=dev)[:, :Kd]
        w = torch.randint(-128, 128, (N, Kd + pw), generator=g, dtype=torch.int8, device=dev)[:, :Kd]
        acc = (a.double() @ w.double().t()).to(torch.int32)
        assert torch.equal(kn.gemm_i8_i32(a, w), acc), tag
        s_a = (torch.rand(M, 1, generator=gen(600 + case)) * 0.05 + 1e-3).half()
        s_w = (torch.rand(N, generator=gen(700 + case)) * 1e-3 + 1e-5).float()
        bias = (torch.randn(N, generator=gen(800 + case)) * 0.01).half() if case % 3 else None
        ref = O.epilogue_ref(acc.cpu(), s_a, s_w, bias, torch.float16)
        y = kn.gemm_i8_dq(a, w, s_a.float().to(dev), s_w.to(dev), None if bias is None else bias.to(dev),
                          out_dtype=torch.float16, exact_ref=True)
        assert torch.equal(y.cpu().view(torch.int16), ref.view(torch.int16)), tag
        a8 = torch.randint(-3, 4, (M, Kd), generator=g, device=dev).float()
        w8 = torch.randint(-3, 4, (N, Kd), generator=g, device=dev).float()
        one = torch.ones(1, device=dev)
        y8 = kn.gemm_fp8_dq(a8.to(torch.float8_e4m3fn), w8.to(torch.float8_e4m3fn), one, one, None,
                            out_dtype=torch.float32)
        assert torch.equal(y8, a8 @ w8.t()), tag
        if M <= 4:
            dt = torch.float16 if case % 2 else torch.bfloat16
            x = (torch.randn(M, Kd, generator=gen(900 + case)) * 2).to(dt).to(dev)
            sm = (torch.rand(Kd, generator=gen(1000 + case)) * 3 + 0.2).to(dt).to(dev) if case % 4 < 2 else None
            if kn.decode_linear_ok(x, sm, Kd):
                b16 = None if bias is None else bias.to(dt).to(dev)
                q, s = kn.quant_act_i8_pertoken(x, sm)
                r2 = kn.gemm_i8_dq(q, w, s, s_w.to(dev), b16, out_dtype=dt, exact_ref=False)
                y2, s2 = kn.decode_linear_i8(x, w, s_w.to(dev), b16, sm, out_dtype=dt, exact_ref=False)
                assert torch.equal(s2.view(torch.int32), s.view(torch.int32)), tag
                assert torch.equal(y2.view(torch.int16), r2.view(torch.int16)), tag


def _rand_fp8(shape, seed, scale=1.0):
    return (torch.randn(shape, generator=gen(seed)) * scale).clamp(-448, 448).to(torch.float8_e4m3fn)


@pytest.mark.parametrize("M", [1, 4, 16, 128, 2048])
def test_gemm_fp8_dq(dev, M):
    N, Kd = 1024, 4096
    a, w = _rand_fp8((M, Kd), 41, 2.0), _rand_fp8((N, Kd), 42, 0.5)
    s_a = torch.rand(M, generator=gen(43)) * 0.05 + 1e-3
    s_w = torch.rand(N, generator=gen(44)) * 0.01 + 1e-4
    bias = (torch.randn(N, generator=gen(45)) * 0.1).bfloat16()
    exact = (a.double() @ w.double().t()) * s_a.double()[:, None] * s_w.double()[None, :] + bias.double()
    y = K().gemm_fp8_dq(a.to(dev), w.to(dev), s_a.to(dev), s_w.to(dev), bias.to(dev),
                        out_dtype=torch.bfloat16)
    torch.testing.assert_close(y.cpu().double(), exact, rtol=1e-2, atol=1e-2)
    # the reference's CPU _scaled_mm (bf16 operands) agrees at the same tolerance
    ref = O.scaled_mm_cpu(a, w.t(), s_a[:, None], s_w[None, :], bias, out_dtype=torch.bfloat16)
    torch.testing.assert_close(y.cpu().float(), ref.float(), rtol=2e-2, atol=2e-2)


def test_gemm_fp8_random_shapes_and_fused_decode(dev):
    """Forty seeded e4m3 products from one row to a few thousand: every route (decode kernels, K
    slices, tiles) against the float64 product of the same codes within the stated tolerance,
    single or per-row / per-column scales, any bias dtype; where the fused decode linear serves a
    shape it returns the quantizer's scales and the GEMM's outputs bit for bit."""
    import random

    from fms_mo_amd import _lib as L

    rng = random.Random(11235)
    kn = K()
    for case in range(40):
        M = rng.choice([1, 2, 3, 4, rng.randint(5, 64), rng.randint(65, 600), rng.randint(600, 3000)])
        N = rng.choice([rng.randint(8, 300), 16 * rng.randint(1, 300), rng.randint(300, 5000)])
        Kd = rng.choice([64 * rng.randint(1, 32), 128 * rng.randint(1, 112), 1024 * rng.choice([1, 2, 4, 8, 14]), 12800])
        if M > 600:
            Kd = min(Kd, 4096)
        an, wn = rng.choice([1, M]), rng.choice([1, N])
        bdt = rng.choice([None, torch.float16, torch.bfloat16, torch.float32])
        odt = rng.choice([torch.float16, torch.bfloat16, torch.float32])
        tag = f"case {case}: M={M} N={N} K={Kd} a_scales={an} w_scales={wn} bias={bdt} out={odt}"
        a = _rand_fp8((M, Kd), 7000 + case, 2.0).to(dev)
        w = _rand_fp8((N, Kd), 7100 + case, 0.5).to(dev)
        s_a = (torch.rand(an, generator=gen(7200 + case)) * 0.05 + 1e-3).to(dev)
        s_w = (torch.rand(wn, generator=gen(7300 + case)) * 0.01 + 1e-4).to(dev)
        bias = None if bdt is None else (torch.randn(N, generator=gen(7400 + case)) * 0.1).to(bdt).to(dev)
        exact = (a.double() @ w.double().t()) * s_a.double()[:, None] * s_w.double()[None, :]
        if bias is not None:
            exact = exact + bias.double()
        y = kn.gemm_fp8_dq(a, w, s_a, s_w, bias, out_dtype=odt)
        torch.testing.assert_close(y.double(), exact, rtol=1e-2, atol=1e-2, msg=tag)
        # fp32 accumulation: far inside the tolerance when the output is fp32
        if odt == torch.float32:
            torch.testing.assert_close(y.double(), exact, rtol=1e-4, atol=1e-4 * exact.abs().max().item(), msg=tag)
        if M <= 4:
            dt = torch.float16 if case % 2 else torch.bfloat16
            x = (2.0 * torch.randn(M, Kd, generator=gen(7500 + case))).to(dt).to(dev)
            if kn.decode_linear_ok(x, None, Kd):
                b16 = None if bias is None else bias.to(dt)
                sw_n = s_w if wn == N else s_w.expand(N).contiguous()
                q, s = kn.quant_act_fp8_pertoken(x, L.FP8_LINEAR)
                ref = kn.gemm_fp8_dq(q, w, s, sw_n, b16, out_dtype=dt)
                y2, s2 = kn.decode_linear_fp8(x, w, sw_n, b16, out_dtype=dt)
                assert torch.equal(s2.view(torch.int32), s.view(torch.int32)), tag
                assert torch.equal(y2.view(torch.int16), ref.view(torch.int16)), tag


@pytest.mark.parametrize("shape", [(256, 512, 1024), (4000, 4100, 384), (4097, 4095, 128), (4000, 4000, 384)])
def test_gemm_fp8_integer_valued_is_exact(dev, shape):
    # small-integer operands: every product and partial sum is exact in fp32, so any MFMA
    # summation order must give the exact integer result (the large ragged shapes run 256x192
    # tiles, the last one 256x256, with K in whole 128-byte slabs)
    M, N, Kd = shape
    a = torch.randint(-4, 5, (M, Kd), generator=gen(46)).float().to(torch.float8_e4m3fn)
    w = torch.randint(-4, 5, (N, Kd), generator=gen(47)).float().to(torch.float8_e4m3fn)
    exact = a.float() @ w.float().t()
    one = torch.ones(1)
    y = K().gemm_fp8_dq(a.to(dev), w.to(dev), one.to(dev), one.to(dev), None, out_dtype=torch.float32)
    assert torch.equal(y.cpu(), exact)
    y16 = K().gemm_fp8_dq(a[:16].contiguous().to(dev), w.to(dev), one.to(dev), one.to(dev), None,
                          out_dtype=torch.float32, force_gemv=True)
    assert torch.equal(y16.cpu(), exact[:16])


@pytest.mark.parametrize("bias_dt", [None, torch.float16, torch.bfloat16, torch.float32])
def test_gemm_dq_with_columns_cut_off_the_last_round(dev, bias_dt):
    """2048 x 25600 outputs are 800 tiles of 256 x 256: three full rounds over 256 compute units
    and 32 tiles more, so the library runs the last 1024 columns as a second, small GEMM.
    Per-column scales, bias (every dtype) and output of both parts must line up: int8 bit-exact
    against the reference epilogue (fp16 and fp32 accumulator dtype) and the fp32 forms, e4m3 exact
    on small integers with per-column scales that are powers of two.  Without a bias nothing is
    added: a product of -0.0 (a scale product that underflows in fp16, a negative sum) stays -0.0,
    as in the reference, whose deploy module then holds -corr_term = -0.0 as its bias buffer
    (linear.py:897-911)."""
    from fms_mo_amd import _lib as L

    M, N, Kd = 2048, 25600, 128
    if L.load().fmsmo_gemm_tail_columns(M, N, Kd) != 1024:
        pytest.skip("tuning overrides switch the cut off")
    assert L.load().fmsmo_gemm_tail_columns(1100, 14080, Kd) == 0   # 128 x 256 tiles: nothing to cut
    a, w = _rand_i8((M, Kd), 51), _rand_i8((N, Kd), 52)
    s_a = (torch.rand(M, 1, generator=gen(53)) * 0.05 + 1e-3).half()
    s_w = (torch.rand(N, generator=gen(54)) * 1e-3 + 1e-5).float()
    bias = None if bias_dt is None else (torch.randn(N, generator=gen(55)) * 0.01).to(bias_dt)
    bz = torch.full((N,), -0.0) if bias is None else bias
    acc = O.int_gemm(a, w)
    ad, wd, sad, swd = a.to(dev), w.to(dev), s_a.float().to(dev), s_w.to(dev)
    bd = None if bias is None else bias.to(dev)
    ref = O.epilogue_ref(acc, s_a, s_w, bz, torch.float16)
    y = K().gemm_i8_dq(ad, wd, sad, swd, bd, out_dtype=torch.float16, exact_ref=True)
    assert torch.equal(y.cpu().view(torch.int16), ref.view(torch.int16))
    ref32 = O.epilogue_ref(acc, s_a, s_w, bz, torch.float32, acc_dtype=torch.float32)
    y32 = K().gemm_i8_dq(ad, wd, sad, swd, bd, out_dtype=torch.float32, exact_ref=True)
    assert torch.equal(y32.cpu().view(torch.int32), ref32.view(torch.int32))
    ref_ma = ((s_a.float() * s_w) * acc + bz.float()).to(torch.bfloat16)
    y_ma = K().gemm_i8_dq(ad, wd, sad, swd, bd, out_dtype=torch.bfloat16, epilogue=L.EPI_F32_MULADD)
    assert torch.equal(y_ma.cpu().view(torch.int16), ref_ma.view(torch.int16))
    a8 = torch.randint(-4, 5, (M, Kd), generator=gen(56)).float()
    w8 = torch.randint(-4, 5, (N, Kd), generator=gen(57)).float()
    s8 = torch.tensor([0.5, 1.0, 2.0, 4.0])[torch.randint(0, 4, (N,), generator=gen(58))]
    one = torch.ones(M)
    b8 = None if bias is None else bias.float().to(bias_dt)
    y8 = K().gemm_fp8_dq(a8.to(torch.float8_e4m3fn).to(dev), w8.to(torch.float8_e4m3fn).to(dev), one.to(dev),
                         s8.to(dev), None if b8 is None else b8.to(dev), out_dtype=torch.float32)
    exact8 = (a8 @ w8.t()).double() * s8[None, :].double() + (0 if b8 is None else b8.double())
    assert torch.equal(y8.cpu(), exact8.float())


# ------------------------------------------------------------------------- chunked accumulation
@pytest.mark.parametrize("cfg", [dict(chunk_size=64, chunk_trun_bits=0, max_acc_bits=32),
                                 dict(chunk_size=64, chunk_trun_bits=8, max_acc_bits=32),
                                 dict(chunk_size=32, chunk_trun_bits=8, max_acc_bits=18),
                                 dict(chunk_size=128, chunk_trun_bits=4, max_acc_bits=24),
                                 dict(chunk_size=256, chunk_trun_bits=7, max_acc_bits=32),
                                 dict(chunk_size=64, chunk_trun_bits=8, max_acc_bits=32,
                                      truncate_then_accumulate=False)])
@pytest.mark.parametrize("shape", [(64, 64, 64), (256, 256, 256), (300, 200, 1040), (130, 257, 4096)])
def test_chunk_i8_bit_exact(dev, cfg, shape):
    M, N, Kd = shape
    a, w = _rand_i8((M, Kd), 51), _rand_i8((N, Kd), 52)
    ocfg = dict(cfg)
    ocfg["trun_bits"] = ocfg.pop("chunk_trun_bits")
    ref = O.chunk_matmul_i8(a, w, None, **ocfg)
    d = K().matmul_chunk(a.to(dev), w.to(dev), None, **cfg)
    assert torch.equal(d.cpu(), ref)


def test_chunk_i8_random_shapes_and_settings(dev):
    """Twenty-five seeded cases: any M and N, K a multiple of 16 (ragged last chunk included),
    every chunk size, truncation from 0 to 12 bits, accumulator widths from 14 to 32 bits, both
    orders of truncation and accumulation, with and without an initial accumulator."""
    import random

    rng = random.Random(1357)
    for case in range(25):
        M, N = rng.randint(1, 300), rng.randint(1, 300)
        Kd = 16 * rng.randint(2, 200)
        cfg = dict(chunk_size=rng.choice([32, 64, 128, 256]), chunk_trun_bits=rng.randint(0, 12),
                   max_acc_bits=rng.choice([14, 16, 18, 20, 24, 32]),
                   truncate_then_accumulate=rng.random() < 0.7)
        g = gen(5000 + case)
        a = torch.randint(-128, 128, (M, Kd), generator=g, dtype=torch.int8)
        w = torch.randint(-128, 128, (N, Kd), generator=g, dtype=torch.int8)
        c = torch.randint(-10**6, 10**6, (M, N), generator=g, dtype=torch.int32) if case % 3 == 0 else None
        ocfg = dict(cfg)
        ocfg["trun_bits"] = ocfg.pop("chunk_trun_bits")
        ref = O.chunk_matmul_i8(a, w, c, **ocfg)
        d = K().matmul_chunk(a.to(dev), w.to(dev), None if c is None else c.to(dev), **cfg)
        assert torch.equal(d.cpu(), ref), f"case {case}: M={M} N={N} K={Kd} {cfg} c={'yes' if c is not None else 'no'}"


def test_chunk_i8_initial_accumulator(dev):
    a, w = _rand_i8((100, 512), 53), _rand_i8((90, 512), 54)
    c = torch.randint(-10**6, 10**6, (100, 90), generator=gen(55), dtype=torch.int32)
    ref = O.chunk_matmul_i8(a, w, c, 64, 8, 32)
    d = K().matmul_chunk(a.to(dev), w.to(dev), c.to(dev), chunk_size=64, chunk_trun_bits=8)
    assert torch.equal(d.cpu(), ref)


@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("t", [0, 7, 8, 16])
def test_chunk_fp_integer_valued_bit_exact(dev, dtype, t):
    # integer-valued operands make every chunk dot exact in fp32 -> the truncation is bit-pinned
    M, N, Kd = 130, 200, 1024
    a = torch.randint(-6, 7, (M, Kd), generator=gen(56)).float().to(dtype)
    w = torch.randint(-6, 7, (N, Kd), generator=gen(57)).float().to(dtype)
    ref = O.chunk_matmul_fp(a.float(), w.float(), None, 64, t)
    d = K().matmul_chunk(a.to(dev), w.to(dev), None, chunk_size=64, chunk_trun_bits=t)
    assert torch.equal(d.cpu(), ref)


@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float16, torch.bfloat16, torch.float32])
def test_chunk_fp_random_within_reference_tolerance(dev, dtype):
    # the reference's own bounds (tests/triton_kernels/test_triton_mm.py:81-82): relative
    # Frobenius error vs a plain matmul < 1e-5 without truncation, < 1e-3 with 8 bits.
    # e4m3: the gfx950 fp8 MFMA keeps fewer guard bits when aligning addends than a chain of
    # fp32 FMAs (measured 1.3e-5), so the no-truncation bound is 5e-5 for that operand type.
    M, N, Kd = 256, 256, 2048
    a = torch.randn(M, Kd, generator=gen(58)).to(dtype)
    w = torch.randn(N, Kd, generator=gen(59)).to(dtype)
    exact = a.double() @ w.double().t()
    b0 = 5e-5 if dtype == torch.float8_e4m3fn else 1e-5
    for t, bound in [(0, b0), (8, 1e-3)]:
        d = K().matmul_chunk(a.to(dev), w.to(dev), None, chunk_size=64, chunk_trun_bits=t).cpu().double()
        rel = torch.linalg.norm(d - exact) / torch.linalg.norm(exact)
        assert rel < bound, (t, rel)
        ref = O.chunk_matmul_fp(a.float(), w.float(), None, 64, t).double()
        rel2 = torch.linalg.norm(d - ref) / torch.linalg.norm(ref)
        assert rel2 < bound


def test_chunk_fp_dl16_and_dabc(dev):
    M, N, Kd = 64, 64, 512
    a = torch.randint(-3, 4, (M, Kd), generator=gen(60)).float().to(torch.float8_e4m3fn)
    w = torch.randint(-3, 4, (N, Kd), generator=gen(61)).float().to(torch.float8_e4m3fn)
    c = torch.randint(-100, 100, (M, N), generator=gen(62)).float()
    ref = O.chunk_matmul_fp(a.float(), w.float(), c, 64, 0, clamp_dl16=True)
    d = K().matmul_chunk(a.to(dev), w.to(dev), c.to(dev), chunk_size=64, clamp_acc_to_dl16=True)
    assert torch.equal(d.cpu(), ref)
    ref2 = O.chunk_matmul_fp(a.float(), w.float(), c, 32, 12, truncate_then_accumulate=False)
    d2 = K().matmul_chunk(a.to(dev), w.to(dev), c.to(dev), chunk_size=32, chunk_trun_bits=12,
                          truncate_then_accumulate=False)
    assert torch.equal(d2.cpu(), ref2)


# ---------------------------------------------------------------------------------- grouped MoE
def test_grouped_gemm_equals_per_expert_linear(dev):
    E, N, Kd, T = 8, 512, 1024, 1500
    g = gen(70)
    logits = torch.rand(T // 2, E, generator=g)
    top2 = logits.topk(2, dim=-1).indices.reshape(-1)           # uneven rows per expert
    order = torch.argsort(top2, stable=True)
    counts = torch.bincount(top2, minlength=E)
    offsets = torch.zeros(E + 1, dtype=torch.int32)
    offsets[1:] = counts.cumsum(0)
    a = _rand_i8((T, Kd), 71)[order]
    w = _rand_i8((E, N, Kd), 72)
    s_a = (torch.rand(T, generator=gen(73)) * 0.05 + 1e-3).half()
    s_w = (torch.rand(E, N, generator=gen(74)) * 1e-3 + 1e-5).float()
    bias = (torch.randn(E, N, generator=gen(75)) * 0.01).half()
    y = K().grouped_gemm_i8_dq(a.to(dev), w.to(dev), offsets.to(dev), s_a.float().to(dev),
                               s_w.to(dev), bias.to(dev), out_dtype=torch.float16, exact_ref=True).cpu()
    for e in range(E):
        lo, hi = offsets[e].item(), offsets[e + 1].item()
        if hi == lo:
            continue
        acc = O.int_gemm(a[lo:hi], w[e])
        ref = O.epilogue_ref(acc, s_a[lo:hi, None], s_w[e], bias[e], torch.float16)
        assert torch.equal(y[lo:hi].view(torch.int16), ref.view(torch.int16)), e


@pytest.mark.parametrize("counts", [
    # rows beyond an expert's last whole 256-row tile: none, 1, 64, 65, 128, 129, 255; empty and
    # tiny experts; an expert of exactly one tile
    [256, 257, 320, 321, 384, 385, 511, 0],
    [0, 0, 5, 0, 130, 64, 1, 0],
    [1069, 1029, 997, 985],
    [128, 128, 128, 128, 128, 128],
    [700]])
@pytest.mark.parametrize("NK", [(520, 256), (256, 1088)])
@pytest.mark.parametrize("exact_ref,out_dtype", [(True, torch.float16), (False, torch.float32)])
def test_grouped_gemm_row_remainders(dev, counts, NK, exact_ref, out_dtype):
    """Every row of every expert must come out exactly once and equal the per-expert product,
    whatever the split of the rows (K in whole 128-byte slabs and not: both grouped kernels)."""
    N, Kd = NK
    E = len(counts)
    offsets = torch.zeros(E + 1, dtype=torch.int32)
    offsets[1:] = torch.tensor(counts).cumsum(0)
    T = int(offsets[-1])
    a = _rand_i8((T, Kd), 76)
    w = _rand_i8((E, N, Kd), 77)
    s_a = (torch.rand(T, generator=gen(78)) * 0.05 + 1e-3).float()
    s_w = (torch.rand(E, N, generator=gen(79)) * 1e-3 + 1e-5).float()
    bias = (torch.randn(E, N, generator=gen(80)) * 0.01).half()
    y = K().grouped_gemm_i8_dq(a.to(dev), w.to(dev), offsets.to(dev), s_a.to(dev), s_w.to(dev), bias.to(dev),
                               out_dtype=out_dtype, exact_ref=exact_ref).cpu()
    bits = torch.int32 if out_dtype == torch.float32 else torch.int16
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi == lo:
            continue
        ref = K().gemm_i8_dq(a[lo:hi].to(dev), w[e].to(dev), s_a[lo:hi].to(dev), s_w[e].to(dev), bias[e].to(dev),
                             out_dtype=out_dtype, exact_ref=exact_ref).cpu()
        assert torch.equal(y[lo:hi].view(bits), ref.view(bits)), e
        if exact_ref and hi - lo <= 400:
            acc = O.int_gemm(a[lo:hi], w[e])
            want = O.epilogue_ref(acc, s_a[lo:hi, None].half(), s_w[e], bias[e], torch.float16)
            # (the oracle takes the token scales in fp16, the kernel in fp32: compare where equal)
            same = s_a[lo:hi].half().float() == s_a[lo:hi]
            assert torch.equal(y[lo:hi][same].view(bits), want[same].view(bits))


@pytest.mark.parametrize("counts", [
    [700, 0, 13, 1300, 256, 511],        # 13 row tiles x 24 column tiles = 312 tiles
    [300, 300, 300, 300, 300, 300, 300, 300, 300, 300, 300, 300]])   # 24 x 24 = 576: every block walks tiles of several experts
def test_grouped_gemm_more_tiles_than_compute_units(dev, counts):
    """The blocks of the grouped kernel are persistent (one per compute unit) and walk the tile
    sequence themselves: with more tiles than compute units a block computes tiles of different
    experts one after the other (accumulators, weight descriptor, scales re-made per tile).  Every
    row must equal the per-expert product, bit for bit."""
    N, Kd = 6144, 256
    E = len(counts)
    offsets = torch.zeros(E + 1, dtype=torch.int32)
    offsets[1:] = torch.tensor(counts).cumsum(0)
    T = int(offsets[-1])
    a = _rand_i8((T, Kd), 176).to(dev)
    w = _rand_i8((E, N, Kd), 177).to(dev)
    s_a = (torch.rand(T, generator=gen(178)) * 0.05 + 1e-3).float().to(dev)
    s_w = (torch.rand(E, N, generator=gen(179)) * 1e-3 + 1e-5).float().to(dev)
    bias = (torch.randn(E, N, generator=gen(180)) * 0.01).half().to(dev)
    y = K().grouped_gemm_i8_dq(a, w, offsets.to(dev), s_a, s_w, bias, out_dtype=torch.float16, exact_ref=True)
    y2 = K().grouped_gemm_i8_dq(a, w, offsets.to(dev), s_a, s_w, bias, out_dtype=torch.float16, exact_ref=True)
    assert torch.equal(y.view(torch.int16), y2.view(torch.int16))
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi == lo:
            continue
        ref = K().gemm_i8_dq(a[lo:hi], w[e], s_a[lo:hi], s_w[e], bias[e], out_dtype=torch.float16, exact_ref=True)
        assert torch.equal(y[lo:hi].view(torch.int16), ref.view(torch.int16)), e
    # one expert against the oracle's integers
    e = 2
    lo, hi = int(offsets[e]), int(offsets[e + 1])
    acc = O.int_gemm(a[lo:hi].cpu(), w[e].cpu())
    sa16 = s_a[lo:hi].cpu()
    same = sa16.half().float() == sa16
    want = O.epilogue_ref(acc, sa16[:, None].half(), s_w[e].cpu(), bias[e].cpu(), torch.float16)
    assert torch.equal(y[lo:hi].cpu()[same].view(torch.int16), want[same].view(torch.int16))


def test_grouped_gemm_random_expert_splits(dev):
    """Twelve seeded cases: 1 to 12 experts, a random split of the rows (empty experts included),
    any N, K in whole 128-byte slabs and not, per-expert bias or none: every expert's rows equal
    the plain GEMM on that expert's rows and weights, bit for bit."""
    import random

    rng = random.Random(8642)
    for case in range(12):
        E = rng.randint(1, 12)
        counts = [rng.choice([0, rng.randint(1, 40), rng.randint(40, 700)]) for _ in range(E)]
        if sum(counts) == 0:
            counts[0] = 33
        N = rng.choice([rng.randint(8, 200), rng.randint(200, 1500)])
        Kd = rng.choice([64 * rng.randint(1, 30), 128 * rng.randint(1, 24)])
        exact_ref = case % 2 == 0
        out_dtype = torch.float16 if exact_ref else rng.choice([torch.float32, torch.bfloat16])
        offsets = torch.zeros(E + 1, dtype=torch.int32)
        offsets[1:] = torch.tensor(counts).cumsum(0)
        T = int(offsets[-1])
        a = _rand_i8((T, Kd), 6000 + case).to(dev)
        w = _rand_i8((E, N, Kd), 6100 + case).to(dev)
        s_a = (torch.rand(T, generator=gen(6200 + case)) * 0.05 + 1e-3).float().to(dev)
        s_w = (torch.rand(E, N, generator=gen(6300 + case)) * 1e-3 + 1e-5).float().to(dev)
        bias = (torch.randn(E, N, generator=gen(6400 + case)) * 0.01).half().to(dev) if case % 3 else None
        y = K().grouped_gemm_i8_dq(a, w, offsets.to(dev), s_a, s_w, bias, out_dtype=out_dtype, exact_ref=exact_ref)
        bits = torch.int32 if out_dtype == torch.float32 else torch.int16
        for e in range(E):
            lo, hi = int(offsets[e]), int(offsets[e + 1])
            if hi == lo:
                continue
            ref = K().gemm_i8_dq(a[lo:hi], w[e], s_a[lo:hi], s_w[e], None if bias is None else bias[e],
                                 out_dtype=out_dtype, exact_ref=exact_ref)
            assert torch.equal(y[lo:hi].view(bits), ref.view(bits)), f"case {case}: counts={counts} N={N} K={Kd} expert {e}"


# ------------------------------------------------------------------------------ error behaviour
def test_clock_probe_reports_a_plausible_core_clock(dev):
    # diagnostic entry point: block 0 of a 256-row-tile GEMM stores {core, 100 MHz} counter pairs
    a, w = _rand_i8((4096, 256), 71).to(dev), _rand_i8((4096, 256), 72).to(dev)
    buf = torch.zeros(6, dtype=torch.int64, device=dev)
    K().clock_probe(buf)
    try:
        c = K().gemm_i8_i32(a, w)
    finally:
        K().clock_probe(None)
    torch.cuda.synchronize()
    t = buf.cpu().tolist()
    assert t[0] < t[2] < t[4] and t[1] <= t[3] <= t[5] and t[5] > t[1]
    assert 300.0 < K().core_clock_mhz(buf) < 2700.0
    # switched off: the buffer stays as it is, the result is the same
    buf.zero_()
    c2 = K().gemm_i8_i32(a, w)
    torch.cuda.synchronize()
    assert int(buf.abs().sum()) == 0 and torch.equal(c, c2)
    with pytest.raises(ValueError):
        K().clock_probe(torch.zeros(6, dtype=torch.int32, device=dev))


def test_errors_are_raised_not_swallowed(dev):
    from fms_mo_amd._lib import FmsMoHipError

    a = _rand_i8((8, 24), 80).to(dev)      # K not a multiple of 16
    w = _rand_i8((8, 24), 81).to(dev)
    with pytest.raises(FmsMoHipError):
        K().gemm_i8_i32(a, w)
    with pytest.raises(TypeError):
        K().gemm_i8_i32(a.float(), w)
    with pytest.raises(RuntimeError):
        K().gemm_i8_i32(a.cpu(), w.cpu())


# ------------------------------------------------------------------ split-K (workspace) GEMMs
def _plain_i8_dq(a, w, a_s, w_s, bias, out_dtype, exact_ref):
    """fmsmo_gemm_i8_dq without a workspace: the single-pass kernels."""
    from fms_mo_amd import _lib as L
    from fms_mo_amd import kernels as Kn

    M, K = a.shape
    N = w.shape[0]
    y = torch.empty((M, N), dtype=out_dtype, device=a.device)
    L.call("fmsmo_gemm_i8_dq", a.data_ptr(), K, w.data_ptr(), K, a_s.data_ptr(), a_s.numel(),
           w_s.data_ptr(), w_s.numel(), None if bias is None else bias.data_ptr(),
           Kn._DT[bias.dtype] if bias is not None else 0, L.EPI_REF_F16 if exact_ref else L.EPI_F32,
           y.data_ptr(), Kn._DT[out_dtype], N, M, N, K, torch.cuda.current_stream().cuda_stream)
    return y


@pytest.mark.parametrize("shape", [(17, 4096, 14336), (64, 4096, 4096), (200, 1024, 1536), (128, 4096, 4096),
                                   (100, 520, 2048), (128, 6144, 4096), (1000, 1024, 14336),
                                   # long reductions from 384 rows: register-staged 256 x 128 tiles
                                   (384, 4096, 14336), (700, 1000, 8192), (768, 4096, 14336), (513, 264, 12800)])
@pytest.mark.parametrize("exact_ref,out_dtype", [(True, torch.float16), (False, torch.bfloat16), (False, torch.float32)])
def test_split_k_int8_is_bit_identical_to_single_pass(dev, shape, exact_ref, out_dtype):
    from fms_mo_amd import _lib as L
    from fms_mo_amd import kernels as Kn

    M, N, Kd = shape
    assert L.load().fmsmo_gemm_workspace_bytes(M, N, Kd) > 0
    g = torch.Generator().manual_seed(91)
    a = torch.randint(-128, 128, (M, Kd), generator=g, dtype=torch.int32).to(torch.int8).to(dev)
    w = torch.randint(-128, 128, (N, Kd), generator=g, dtype=torch.int32).to(torch.int8).to(dev)
    a_s = (torch.rand(M, generator=g) * 1e-2).to(dev)
    w_s = (torch.rand(N, generator=g) * 1e-2).to(dev)
    bias = torch.randn(N, generator=g).half().to(dev)
    for b in (None, bias):
        y = Kn.gemm_i8_dq(a, w, a_s, w_s, b, out_dtype=out_dtype, exact_ref=exact_ref)
        ref = _plain_i8_dq(a, w, a_s, w_s, b, out_dtype, exact_ref)
        assert torch.equal(y.view(torch.int16 if out_dtype != torch.float32 else torch.int32),
                           ref.view(torch.int16 if out_dtype != torch.float32 else torch.int32))
    # and against exact integer arithmetic on a sample of rows
    acc = O.int_gemm(a[:5].cpu(), w.cpu())
    exact = acc.double() * a_s[:5].cpu().double()[:, None] * w_s.cpu().double()[None, :]
    y = Kn.gemm_i8_dq(a, w, a_s, w_s, None, out_dtype=torch.float32, exact_ref=False)
    torch.testing.assert_close(y[:5].cpu().double(), exact, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("shape", [(512, 4096, 4096), (129, 4096, 4096), (256, 6144, 4096), (1024, 2000, 4096),
                                   (500, 4090, 8192), (300, 4096, 2048),     # 128 x 64 tiles, 128-byte stages
                                   (1024, 4096, 8192), (512, 6144, 4096), (1000, 4000, 1152),  # 128 x 128
                                   (200, 13824, 5120),
                                   (100, 14336, 4096), (48, 13824, 5120), (33, 14330, 8192)])  # one row of 128 x 64 tiles
def test_one_pass_tiles_with_128_byte_stages(dev, shape):
    """A few hundred rows through a projection that fills half a round of 128 x 64 tiles or more
    (and a round of 128 x 128 tiles) run in one pass even when a workspace is offered: int8
    bit-exact against the oracle's epilogue on the exact product, e4m3 exact on small integers,
    ragged last tiles included."""
    M, N, Kd = shape
    kn = K()
    plan = kn.gemm_plan(M, N, Kd, with_workspace=True)
    assert plan[3] == 1 and plan[1] == 128, plan
    g = torch.Generator(device=dev).manual_seed(M + N)
    a = torch.randint(-128, 128, (M, Kd), generator=g, dtype=torch.int8, device=dev)
    w = torch.randint(-128, 128, (N, Kd), generator=g, dtype=torch.int8, device=dev)
    acc = (a.double() @ w.double().t()).to(torch.int32)
    assert torch.equal(kn.gemm_i8_i32(a, w), acc)
    s_a = (torch.rand(M, 1, generator=gen(61)) * 0.05 + 1e-3).half()
    s_w = (torch.rand(N, generator=gen(62)) * 1e-3 + 1e-5).float()
    bias = (torch.randn(N, generator=gen(63)) * 0.01).half()
    ref = O.epilogue_ref(acc.cpu(), s_a, s_w, bias, torch.float16)
    y = kn.gemm_i8_dq(a, w, s_a.float().reshape(-1).to(dev), s_w.to(dev), bias.to(dev), out_dtype=torch.float16,
                      exact_ref=True)
    assert torch.equal(y.cpu().view(torch.int16), ref.view(torch.int16))
    a8 = torch.randint(-4, 5, (M, Kd), generator=g, device=dev).float()
    w8 = torch.randint(-4, 5, (N, Kd), generator=g, device=dev).float()
    one = torch.ones(1, device=dev)
    y8 = kn.gemm_fp8_dq(a8.to(torch.float8_e4m3fn), w8.to(torch.float8_e4m3fn), one, one, None,
                        out_dtype=torch.float32)
    assert torch.equal(y8, a8 @ w8.t())


@pytest.mark.parametrize("shape", [(17, 4096, 14336), (64, 4096, 4096), (200, 1024, 1536), (100, 520, 2048),
                                   (512, 4096, 14336), (700, 1000, 8192)])
def test_split_k_fp8(dev, shape):
    from fms_mo_amd import kernels as Kn

    M, N, Kd = shape
    g = torch.Generator().manual_seed(92)
    # integer-valued operands: every partial sum is exact, so the split result is the exact product
    a = torch.randint(-8, 9, (M, Kd), generator=g).float().to(torch.float8_e4m3fn).to(dev)
    w = torch.randint(-8, 9, (N, Kd), generator=g).float().to(torch.float8_e4m3fn).to(dev)
    one = torch.ones(1, device=dev)
    y = Kn.gemm_fp8_dq(a, w, one, one, None, out_dtype=torch.float32)
    ref = a.cpu().double() @ w.cpu().double().t()
    assert torch.equal(y.cpu().double(), ref)
    # general operands: within the tolerance of the fp8 path
    a = torch.randn(M, Kd, generator=g).to(torch.float8_e4m3fn).to(dev)
    w = torch.randn(N, Kd, generator=g).to(torch.float8_e4m3fn).to(dev)
    a_s = (torch.rand(M, generator=g) + 0.5).to(dev)
    w_s = (torch.rand(N, generator=g) + 0.5).to(dev)
    y = Kn.gemm_fp8_dq(a, w, a_s, w_s, None, out_dtype=torch.bfloat16)
    ref = (a.cpu().double() @ w.cpu().double().t()) * a_s.cpu().double()[:, None] * w_s.cpu().double()[None, :]
    torch.testing.assert_close(y.cpu().double(), ref, rtol=1e-2, atol=1e-2 * ref.abs().max().item())


# ------------------------------------------------------------------ 17 .. 64 tokens, one weight pass
@pytest.mark.parametrize("M", [17, 24, 32, 33, 48, 64])
@pytest.mark.parametrize("NK", [(4096, 4096), (520, 1024), (1000, 2048), (256, 8192), (6144, 4096), (1000, 5120)])
def test_batched_decode_i8_bit_exact(dev, M, NK):
    """Batches of up to 64 tokens run through the weight-streaming kernel where their activation
    fragments fit in registers (K = 1024, 2048, 4096; 8192 up to 32 tokens) and through the tiled /
    split-K kernels otherwise; every route returns the reference epilogue bit for bit."""
    N, Kd = NK
    a, w = _rand_i8((M, Kd), 131), _rand_i8((N, Kd), 132)
    s_a = (torch.rand(M, 1, generator=gen(133)) * 0.05 + 1e-3).half()
    s_w = (torch.rand(N, generator=gen(134)) * 1e-3 + 1e-5).float()
    bias = (torch.randn(N, generator=gen(135)) * 0.01).half()
    acc = O.int_gemm(a, w)
    ref = O.epilogue_ref(acc, s_a, s_w, bias, torch.float16)
    y = K().gemm_i8_dq(a.to(dev), w.to(dev), s_a.float().to(dev), s_w.to(dev), bias.to(dev),
                       out_dtype=torch.float16, exact_ref=True)
    assert torch.equal(y.cpu().view(torch.int16), ref.view(torch.int16))
    # without a bias nothing is added: the same bits, the sign of a zero product included
    y = K().gemm_i8_dq(a.to(dev), w.to(dev), s_a.float().to(dev), s_w.to(dev), None,
                       out_dtype=torch.float16, exact_ref=True)
    assert torch.equal(y.cpu().view(torch.int16), O.epilogue_ref(acc, s_a, s_w, None, torch.float16).view(torch.int16))
    y32 = K().gemm_i8_dq(a.to(dev), w.to(dev), torch.ones(1, device=dev), torch.ones(1, device=dev), None,
                         out_dtype=torch.float32, exact_ref=False)
    assert torch.equal(y32.cpu().double(), acc.double())


@pytest.mark.parametrize("M", [17, 32, 40, 64])
@pytest.mark.parametrize("NK", [(4096, 4096), (520, 1024), (256, 8192), (1000, 5120)])
def test_batched_decode_fp8(dev, M, NK):
    N, Kd = NK
    a = torch.randint(-8, 9, (M, Kd), generator=gen(141)).float().to(torch.float8_e4m3fn)
    w = torch.randint(-8, 9, (N, Kd), generator=gen(142)).float().to(torch.float8_e4m3fn)
    one = torch.ones(1, device=dev)
    y = K().gemm_fp8_dq(a.to(dev), w.to(dev), one, one, None, out_dtype=torch.float32)
    assert torch.equal(y.cpu().double(), a.double() @ w.double().t())  # integer-valued operands: exact
    a, w = _rand_fp8((M, Kd), 143, 2.0), _rand_fp8((N, Kd), 144, 0.5)
    s_a = torch.rand(M, generator=gen(145)) * 0.05 + 1e-3
    s_w = torch.rand(N, generator=gen(146)) * 0.01 + 1e-4
    bias = (torch.randn(N, generator=gen(147)) * 0.1).bfloat16()
    exact = (a.double() @ w.double().t()) * s_a.double()[:, None] * s_w.double()[None, :] + bias.double()
    y = K().gemm_fp8_dq(a.to(dev), w.to(dev), s_a.to(dev), s_w.to(dev), bias.to(dev), out_dtype=torch.bfloat16)
    torch.testing.assert_close(y.cpu().double(), exact, rtol=1e-2, atol=1e-2 * exact.abs().max().item())


def test_split_k_gemm_replays_from_a_hip_graph(dev):
    """The workspace of the split form comes from torch's allocator inside the capture (the
    library allocates nothing): the captured GEMM must replay bit-identically on new inputs."""
    from fms_mo_amd import _lib as L

    M, N, Kd = 128, 1024, 4096
    assert L.load().fmsmo_gemm_workspace_bytes(M, N, Kd) > 0
    w = _rand_i8((N, Kd), 152).to(dev)
    s_a = (torch.rand(M, generator=gen(153)) * 0.05 + 1e-3).to(dev)
    s_w = (torch.rand(N, generator=gen(154)) * 1e-3 + 1e-5).to(dev)
    bias = (torch.randn(N, generator=gen(155)) * 0.01).half().to(dev)
    xs = [_rand_i8((M, Kd), 160 + i).to(dev) for i in range(3)]
    fn = lambda a: K().gemm_i8_dq(a, w, s_a, s_w, bias, out_dtype=torch.float16, exact_ref=True)
    eager = [fn(a).clone() for a in xs]
    static_a = xs[0].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn(static_a)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = fn(static_a)
    for _ in range(2):
        for a, ref in zip(xs, eager):
            static_a.copy_(a)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out.view(torch.int16), ref.view(torch.int16))
            fn(a)
            torch.cuda.synchronize()


# ------------------------------------------------------------------ fused decode linear
@pytest.mark.parametrize("NK", [(4096, 4096), (6144, 4096), (520, 1024), (1000, 2048), (256, 8192), (28672, 4096),
                                (96, 1536), (64, 3584),
                                # long rows: the streaming kernel's fused form (whole and half row
                                # groups, fewer and more than one group per compute unit)
                                (4096, 14336), (1000, 14336), (4104, 14336), (8200, 14336), (24, 14336),
                                (4096, 12800), (1016, 12800), (1024, 4096), (1000, 4096), (4104, 4096)])
@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("smooth", [False, True])
def test_fused_decode_linear_is_bit_identical_to_the_two_kernels(dev, NK, dt, smooth):
    N, Kd = NK
    kn = K()
    x = torch.randn(1, Kd, generator=gen(171)).to(dt)
    x[:, 5] *= 30.0
    sm = (torch.rand(Kd, generator=gen(172)) * 3 + 0.2).to(dt) if smooth else None
    w = _rand_i8((N, Kd), 173).to(dev)
    s_w = (torch.rand(N, generator=gen(174)) * 1e-3 + 1e-5).to(dev)
    bias = (torch.randn(N, generator=gen(175)) * 0.01).to(dt).to(dev)
    xd, smd = x.to(dev), None if sm is None else sm.to(dev)
    assert kn.decode_linear_ok(xd, smd, Kd)
    for exact_ref, od in ((True, torch.float16), (False, dt)):
        q, s = kn.quant_act_i8_pertoken(xd, smd)
        ref = kn.gemm_i8_dq(q, w, s, s_w, bias, out_dtype=od, exact_ref=exact_ref)
        y, s_f = kn.decode_linear_i8(xd, w, s_w, bias, smd, out_dtype=od, exact_ref=exact_ref)
        assert torch.equal(s_f, s)
        assert torch.equal(y.view(torch.int16), ref.view(torch.int16))
    # the scale against the oracle as well (the codes are checked through the matmul above)
    _, s_ref, _ = O.quant_act_pertoken_i8(x if sm is None else x / sm)
    assert torch.equal(s_f.cpu(), s_ref.reshape(-1).float())


@pytest.mark.parametrize("NK", [(4096, 4096), (6144, 4096), (28672, 4096), (1000, 4096), (24, 4096),
                                (4096, 14336), (1000, 14336), (8200, 14336), (4104, 12800)])
@pytest.mark.parametrize("M", [2, 3, 4])
@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("smooth", [False, True])
def test_fused_decode_linear_several_tokens(dev, NK, M, dt, smooth):
    """A decode step of a few sequences: the streaming kernel quantizes all token rows itself.
    Rows off the quantizer's fast path (zeros, an infinity, an overflow after the SmoothQuant
    divide) sit between ordinary ones.  Scales and outputs are the two kernels' bit for bit."""
    N, Kd = NK
    kn = K()
    x = torch.randn(M, Kd, generator=gen(176)).to(dt)
    x[:, 5] *= 30.0
    x[M - 1] *= 0.01
    sm = (torch.rand(Kd, generator=gen(177)) * 3 + 0.2).to(dt) if smooth else None
    if M >= 3:
        x[1] = 0.0
    if M == 4 or Kd == 12800:
        x[2 if M > 2 else 0, 100] = float("inf")
    overflow = M == 3 and dt == torch.float16 and smooth
    if overflow:
        x[2, 7] = 60000.0
        sm[7] = 0.25  # 60000 / 0.25 overflows fp16
    xd, smd = x.to(dev), None if sm is None else sm.to(dev)
    if not kn.decode_linear_ok(xd, smd, Kd):
        assert M > 3 and Kd > 4096  # long rows are served up to three tokens
        return
    w = _rand_i8((N, Kd), 178).to(dev)
    s_w = (torch.rand(N, generator=gen(179)) * 1e-3 + 1e-5).to(dev)
    bias = (torch.randn(N, generator=gen(180)) * 0.01).to(dt).to(dev)
    for exact_ref, od in ((True, torch.float16), (False, torch.float32)):
        q, s = kn.quant_act_i8_pertoken(xd, smd)
        ref = kn.gemm_i8_dq(q, w, s, s_w, bias, out_dtype=od, exact_ref=exact_ref)
        y, s_f = kn.decode_linear_i8(xd, w, s_w, bias, smd, out_dtype=od, exact_ref=exact_ref)
        assert torch.equal(s_f.view(torch.int32), s.view(torch.int32))
        bits = torch.int32 if od == torch.float32 else torch.int16
        assert torch.equal(y.view(bits), ref.view(bits))
    if not (M == 4 or Kd == 12800 or overflow):
        _, s_ref, _ = O.quant_act_pertoken_i8(x if sm is None else x / sm)
        assert torch.equal(s_f.cpu(), s_ref.reshape(-1).float())


@pytest.mark.parametrize("NK", [(1000, 4096), (4096, 14336), (256, 2048)])
@pytest.mark.parametrize("M", [1, 3])
@pytest.mark.parametrize("smooth", [None, "same", "fp32"])
def test_fused_decode_linear_strided_operands(dev, NK, M, smooth):
    """Token rows and weight rows that are slices of wider buffers (row stride larger than K)."""
    N, Kd = NK
    kn = K()
    xb = torch.randn(M, Kd + 64, generator=gen(221)).half().to(dev)
    wb = _rand_i8((N, Kd + 128), 222).to(dev)
    x, w = xb[:, :Kd], wb[:, :Kd]
    assert x.stride(0) == Kd + 64 and w.stride(0) == Kd + 128
    sm = None
    if smooth is not None:
        sm = (torch.rand(Kd, generator=gen(223)) * 3 + 0.2).to(torch.float16 if smooth == "same" else torch.float32).to(dev)
    if not kn.decode_linear_ok(x, sm, Kd):
        return
    s_w = (torch.rand(N, generator=gen(224)) * 1e-3 + 1e-5).to(dev)
    q, s = kn.quant_act_i8_pertoken(x.contiguous(), sm)
    ref = kn.gemm_i8_dq(q, w.contiguous(), s, s_w, None, out_dtype=torch.float16, exact_ref=True)
    y, s_f = kn.decode_linear_i8(x, w, s_w, None, sm, out_dtype=torch.float16, exact_ref=True)
    assert torch.equal(s_f.view(torch.int32), s.view(torch.int32))
    assert torch.equal(y.view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("NK", [(4096, 4096), (520, 4096), (4096, 14336), (264, 12800)])
@pytest.mark.parametrize("M", [1, 2, 3, 4])
def test_fused_decode_linear_bf16_divisor_outside_the_fast_range(dev, NK, M):
    """A bf16 SmoothQuant divisor outside 2^-60 .. 2^60 sends every row through the IEEE division
    routine (the fast quotient's residual could leave the normal range); scales and outputs must
    still be the stand-alone quantizer's."""
    N, Kd = NK
    kn = K()
    x = torch.randn(M, Kd, generator=gen(211)).bfloat16()
    sm = (torch.rand(Kd, generator=gen(212)) * 3 + 0.2).bfloat16()
    sm[11] = 1e-20
    sm[Kd - 3] = 3e19
    xd, smd = x.to(dev), sm.to(dev)
    if not kn.decode_linear_ok(xd, smd, Kd):
        assert M > 3 and Kd > 4096
        return
    w = _rand_i8((N, Kd), 213).to(dev)
    s_w = (torch.rand(N, generator=gen(214)) * 1e-3 + 1e-5).to(dev)
    q, s = kn.quant_act_i8_pertoken(xd, smd)
    ref = kn.gemm_i8_dq(q, w, s, s_w, None, out_dtype=torch.float32, exact_ref=False)
    y, s_f = kn.decode_linear_i8(xd, w, s_w, None, smd, out_dtype=torch.float32, exact_ref=False)
    assert torch.equal(s_f.view(torch.int32), s.view(torch.int32))
    assert torch.equal(y.view(torch.int32), ref.view(torch.int32))
    _, s_ref, _ = O.quant_act_pertoken_i8(x, sm)
    assert torch.equal(s_f.cpu(), s_ref.reshape(-1).float())


@pytest.mark.parametrize("NK", [(4096, 4096), (6144, 4096), (1000, 4096), (4096, 14336), (1016, 12800)])
@pytest.mark.parametrize("M", [2, 3, 4])
@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
def test_fused_decode_linear_fp8_several_tokens(dev, NK, M, dt):
    """The same for e4m3 weights: scales and codes are the stand-alone quantizer's bit for bit
    (codes through an exact product with weight rows that hold a single one); with random weights
    the fp32 sums may be added in another order than by the two kernels (rtol 1e-5)."""
    from fms_mo_amd import _lib as L

    N, Kd = NK
    kn = K()
    x = (2.0 * torch.randn(M, Kd, generator=gen(186))).to(dt)
    x[0, 3] = -0.0
    x[M - 1] = 0.0
    if M >= 3:
        x[1, 9] = float("inf")
    xd = x.to(dev)
    if not kn.decode_linear_ok(xd, None, Kd):
        assert M > 3 and Kd > 4096  # long rows are served up to three tokens
        return
    q, s = kn.quant_act_fp8_pertoken(xd, L.FP8_LINEAR)
    n_id = min(N, Kd)
    w_id = torch.zeros(N, Kd)
    w_id[torch.arange(n_id), torch.arange(n_id)] = 1.0
    w_id = w_id.to(torch.float8_e4m3fn).to(dev)
    y_id, s_f = kn.decode_linear_fp8(xd, w_id, torch.ones(N, device=dev), None, out_dtype=torch.float32)
    assert torch.equal(s_f.view(torch.int32), s.view(torch.int32))
    want = q.float()[:, :n_id] * s.reshape(-1, 1)
    fin = torch.ones(M, dtype=torch.bool)
    if M >= 3:
        fin[1] = False
    flat = lambda t: torch.nan_to_num(t, nan=7.0, posinf=1e30, neginf=-1e30)
    # (the row with the infinity has the scale inf: its outputs are NaN = 0 * inf but for column 9)
    assert torch.equal(flat(y_id[:, :n_id]), flat(want))
    w = _rand_fp8((N, Kd), 187, 0.5).to(dev)
    s_w = (torch.rand(N, generator=gen(188)) * 0.01 + 1e-4).to(dev)
    bias = (torch.randn(N, generator=gen(189)) * 0.1).to(dt).to(dev)
    ref = kn.gemm_fp8_dq(q, w, s, s_w, bias, out_dtype=torch.float32)
    y, _ = kn.decode_linear_fp8(xd, w, s_w, bias, out_dtype=torch.float32)
    torch.testing.assert_close(y[fin.to(dev)], ref[fin.to(dev)], rtol=1e-5, atol=1e-5)
    assert torch.equal(flat(y[~fin.to(dev)]), flat(ref[~fin.to(dev)]))


@pytest.mark.parametrize("NK", [(4096, 4096), (6144, 4096), (28672, 4096), (1000, 4096), (24, 4096),
                                (4096, 14336), (1000, 14336), (8200, 14336), (4104, 12800)])
@pytest.mark.parametrize("M", [1, 2, 3])
@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("special", [None, "rows", "divisor"])
def test_fused_decode_linear_fp32_divisors(dev, NK, M, dt, special):
    """fp16 / bf16 activations with fp32 SmoothQuant divisors (quantizer buffers left in fp32 under
    a 16-bit model): torch promotes the quantizer to fp32.  Scales, codes (through the exact int32
    product) and outputs equal the two kernels' bit for bit; the scales equal the oracle's.  Rows
    and divisors off the fast division path (zeros, an infinity, a tiny bf16 row; a divisor
    outside 2^-60 .. 2^60) take IEEE divisions in both."""
    N, Kd = NK
    kn = K()
    x = torch.randn(M, Kd, generator=gen(201)).to(dt)
    x[:, 5] *= 30.0
    sm = (torch.rand(Kd, generator=gen(202)) * 3 + 0.2).float()
    if special == "rows":
        if M == 1:
            x[0, 100] = float("inf")
        elif dt == torch.bfloat16:
            x[0] = x[0] * 1e-30  # a row whose largest quotient lies under 2^-80
            x[1] = 0.0
        else:
            x[0, 100] = float("inf")
            x[1] = 0.0
    elif special == "divisor":
        sm[11] = 1e-20
    xd, smd = x.to(dev), sm.to(dev)
    if not kn.decode_linear_ok(xd, smd, Kd):
        assert M > 2 or (M > 1 and Kd > 4096)  # fp32 divisors: two tokens at K = 4096, one at long rows
        return
    w = _rand_i8((N, Kd), 203).to(dev)
    s_w = (torch.rand(N, generator=gen(204)) * 1e-3 + 1e-5).to(dev)
    bias = (torch.randn(N, generator=gen(205)) * 0.01).to(dt).to(dev)
    q, s = kn.quant_act_i8_pertoken(xd, smd, compute_dtype=torch.float32)
    for exact_ref, od in ((True, torch.float16), (False, torch.float32)):
        ref = kn.gemm_i8_dq(q, w, s, s_w, bias, out_dtype=od, exact_ref=exact_ref)
        y, s_f = kn.decode_linear_i8(xd, w, s_w, bias, smd, out_dtype=od, exact_ref=exact_ref)
        assert torch.equal(s_f.view(torch.int32), s.view(torch.int32))
        bits = torch.int32 if od == torch.float32 else torch.int16
        assert torch.equal(y.view(bits), ref.view(bits))
    # the codes themselves, through the exact integer product with rows that hold a single one
    n_id = min(N, Kd)
    w_id = torch.zeros(N, Kd, dtype=torch.int8)
    w_id[torch.arange(n_id), torch.arange(n_id)] = 1
    y_id, _ = kn.decode_linear_i8(xd, w_id.to(dev), torch.ones(N, device=dev), None, smd, out_dtype=torch.float32,
                                  exact_ref=False)
    fin = torch.isfinite(s)
    want = q.float()[:, :n_id] * s.reshape(-1, 1)
    assert torch.equal(y_id[:, :n_id][fin], want[fin])
    if special is None:
        _, s_ref, _ = O.quant_act_pertoken_i8(x, sm)
        assert s_ref.dtype == torch.float32 and torch.equal(s_f.cpu(), s_ref.reshape(-1))


@pytest.mark.parametrize("row", ["zeros", "inf", "overflow"])
@pytest.mark.parametrize("Kd", [4096, 14336])
def test_fused_decode_linear_special_rows(dev, row, Kd):
    """Rows that leave the fast division path (all zeros, an infinity, an fp16 overflow after the
    SmoothQuant divide) must come out like the stand-alone quantizer's."""
    kn = K()
    N = 512
    x = torch.randn(1, Kd, generator=gen(181)).half()
    sm = (torch.rand(Kd, generator=gen(182)) * 3 + 0.2).half()
    if row == "zeros":
        x[0] = 0.0
    elif row == "inf":
        x[0, 100] = float("inf")
    else:
        x[0, 7] = 60000.0
        sm[7] = 0.25  # 60000 / 0.25 overflows fp16
    w = _rand_i8((N, Kd), 183).to(dev)
    s_w = (torch.rand(N, generator=gen(184)) * 1e-3 + 1e-5).to(dev)
    for smd in (None, sm.to(dev)):
        q, s = kn.quant_act_i8_pertoken(x.to(dev), smd)
        ref = kn.gemm_i8_dq(q, w, s, s_w, None, out_dtype=torch.float32, exact_ref=False)
        y, s_f = kn.decode_linear_i8(x.to(dev), w, s_w, None, smd, out_dtype=torch.float32, exact_ref=False)
        assert torch.equal(s_f.view(torch.int32), s.view(torch.int32))
        assert torch.equal(y.view(torch.int32), ref.view(torch.int32))


def test_fused_decode_linear_rejects_what_it_does_not_serve(dev):
    kn = K()
    x = torch.randn(2, 4096, device=dev).half()
    assert kn.decode_linear_ok(x, None, 4096)                              # a few tokens at K = 4096
    assert not kn.decode_linear_ok(torch.randn(5, 4096, device=dev).half(), None, 4096)
    assert not kn.decode_linear_ok(torch.randn(2, 2048, device=dev).half(), None, 2048)
    assert not kn.decode_linear_ok(x[:1].float(), None, 4096)              # fp32 activations
    assert not kn.decode_linear_ok(torch.randn(1, 16384, device=dev).half(), None, 16384)  # long rows
    assert kn.decode_linear_ok(torch.randn(3, 14336, device=dev).half(), None, 14336)
    assert not kn.decode_linear_ok(torch.randn(4, 14336, device=dev).half(), None, 14336)
    assert kn.decode_linear_ok(torch.randn(1, 14336, device=dev).half(), None, 14336)
    assert kn.decode_linear_ok(x[:1], torch.ones(4096, device=dev), 4096)      # fp32 divisors: K = 4096 ...
    assert not kn.decode_linear_ok(torch.randn(1, 2048, device=dev).half(), torch.ones(2048, device=dev), 2048)
    assert not kn.decode_linear_ok(torch.randn(2, 14336, device=dev).half(), torch.ones(14336, device=dev), 14336)
    assert kn.decode_linear_ok(x[:1], None, 4096)
    w = torch.zeros(64, 2048, dtype=torch.int8, device=dev)
    with pytest.raises(RuntimeError):
        kn.decode_linear_i8(x[:, :2048].contiguous(), w, torch.ones(1, device=dev))


@pytest.mark.parametrize("NK", [(4096, 4096), (6144, 4096), (520, 1024), (1000, 2048), (256, 8192), (96, 1536)])
@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("special", [None, "zeros", "inf"])
def test_fused_decode_linear_fp8_is_bit_identical_to_the_two_kernels(dev, NK, dt, special):
    from fms_mo_amd import _lib as L

    N, Kd = NK
    kn = K()
    x = (2.0 * torch.randn(1, Kd, generator=gen(191))).to(dt)
    x[0, 3] = -0.0
    if special == "zeros":
        x[0] = 0.0
    elif special == "inf":
        x[0, 9] = float("inf")
    w = _rand_fp8((N, Kd), 192, 0.5).to(dev)
    s_w = (torch.rand(N, generator=gen(193)) * 0.01 + 1e-4).to(dev)
    bias = (torch.randn(N, generator=gen(194)) * 0.1).to(dt).to(dev)
    xd = x.to(dev)
    assert kn.decode_linear_ok(xd, None, Kd)
    for od in (dt, torch.float32):
        q, s = kn.quant_act_fp8_pertoken(xd, L.FP8_LINEAR)
        ref = kn.gemm_fp8_dq(q, w, s, s_w, bias, out_dtype=od)
        y, s_f = kn.decode_linear_fp8(xd, w, s_w, bias, out_dtype=od)
        assert torch.equal(s_f.view(torch.int32), s.view(torch.int32))
        bits = torch.int32 if od == torch.float32 else torch.int16
        assert torch.equal(y.view(bits), ref.view(bits))


@pytest.mark.parametrize("NK", [(4096, 14336), (1000, 14336), (8200, 14336), (4096, 12800), (1016, 12800)])
@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("special", [None, "zeros", "inf"])
def test_fused_decode_linear_fp8_long_rows(dev, NK, dt, special):
    """Long rows take the streaming kernel's fused form.  The quantized token is the stand-alone
    quantizer's bit for bit (scale; codes through an exact product with power-of-two weights);
    the product with random weights equals the two kernels' up to the order of the fp32 sums,
    which differs where they stream the weights in another shape (rtol 1e-5 on fp32 outputs)."""
    from fms_mo_amd import _lib as L

    N, Kd = NK
    kn = K()
    x = (2.0 * torch.randn(1, Kd, generator=gen(195))).to(dt)
    x[0, 3] = -0.0
    if special == "zeros":
        x[0] = 0.0
    elif special == "inf":
        x[0, 9] = float("inf")
    xd = x.to(dev)
    assert kn.decode_linear_ok(xd, None, Kd)
    q, s = kn.quant_act_fp8_pertoken(xd, L.FP8_LINEAR)
    # (a) codes: weight row n = one power of two at column n (mod Kd) -> y[n] is code n exactly
    n_id = min(N, Kd)
    w_id = torch.zeros(N, Kd)
    w_id[torch.arange(n_id), torch.arange(n_id)] = 1.0
    w_id = w_id.to(torch.float8_e4m3fn).to(dev)
    ones = torch.ones(N, device=dev)
    y_id, s_f = kn.decode_linear_fp8(xd, w_id, ones, None, out_dtype=torch.float32)
    assert torch.equal(s_f.view(torch.int32), s.view(torch.int32))
    want = q.float()[0, :n_id] * s
    got = y_id[0, :n_id]
    assert torch.equal(torch.nan_to_num(got, nan=7.0), torch.nan_to_num(want, nan=7.0))
    # (b) random weights against the two kernels
    w = _rand_fp8((N, Kd), 196, 0.5).to(dev)
    s_w = (torch.rand(N, generator=gen(197)) * 0.01 + 1e-4).to(dev)
    bias = (torch.randn(N, generator=gen(198)) * 0.1).to(dt).to(dev)
    ref = kn.gemm_fp8_dq(q, w, s, s_w, bias, out_dtype=torch.float32)
    y, _ = kn.decode_linear_fp8(xd, w, s_w, bias, out_dtype=torch.float32)
    if special == "inf":
        assert torch.equal(torch.isnan(y), torch.isnan(ref))
    else:
        torch.testing.assert_close(y, ref, rtol=1e-5, atol=1e-5)


# ------------------------------------------------------------------ chunked matmuls, fused epilogue
def _chunk_epilogue_ref(acc, a_s, w_s, bias, epi, out):
    """The four epilogues restated with torch CPU ops in the reference's operation order."""
    from fms_mo_amd import _lib as L

    a_s, w_s = a_s.reshape(-1, 1), w_s.reshape(1, -1)
    if epi == L.EPI_REF_F16:      # iaddmm_int's plain branch (linear.py:1185-1188)
        return O.epilogue_ref(acc, a_s, w_s, bias, org_dtype=out,
                              acc_dtype=torch.float32 if out == torch.float32 else torch.float16)
    if epi == L.EPI_F32_MULADD:   # the last line of its chunk loop (linear.py:1166-1175)
        y = acc.float() * (a_s * w_s)
        return (y if bias is None else y + bias).to(out)
    if epi == L.EPI_SEQ_OUT:      # LinearFuncFPxFwdBwd / LinearFuncINT8FwdFP32Bwd (linear.py:1955-1975, 2180-2189)
        y = (acc.float() * a_s * w_s).to(out)
        return y if bias is None else y + bias.to(out)
    return O.epilogue_f32(acc, a_s, w_s, bias, out)


@pytest.mark.parametrize("shape", [(70, 200, 4096), (33, 96, 80), (300, 130, 1024), (129, 257, 320)])
def test_matmul_chunk_i8_fused_epilogues_bit_exact(dev, shape):
    """fmsmo_matmul_chunk_i8_dq: the chunked accumulator is the oracle's, and every epilogue applied
    to it inside the kernel gives the bits of the reference's torch expression."""
    from fms_mo_amd import _lib as L

    M, N, Kd = shape
    g = gen(91)
    a = torch.randint(-127, 128, (M, Kd), generator=g, dtype=torch.int8)
    w = torch.randint(-127, 128, (N, Kd), generator=g, dtype=torch.int8)
    a_s = (torch.rand(M, generator=g) * 1e-2 + 1e-3).half().float()
    w_s = (torch.rand(N, generator=g) * 1e-3 + 1e-4)
    bias16 = (torch.randn(N, generator=g) * 0.1).half()
    cases = [(64, 5, 32, L.EPI_F32_MULADD, torch.float16, bias16, True),
             (64, 7, 20, L.EPI_F32_MULADD, torch.float32, bias16.float(), True),
             (32, 6, 32, L.EPI_REF_F16, torch.float16, bias16, True),
             (128, 3, 32, L.EPI_REF_F16, torch.float32, None, True),
             (64, 8, 24, L.EPI_SEQ_OUT, torch.bfloat16, bias16.bfloat16(), True),
             (64, 8, 32, L.EPI_SEQ_OUT, torch.float16, bias16.float(), True),     # bias rounded to the output dtype
             (32, 4, 32, L.EPI_SEQ_OUT, torch.float32, None, False),
             (64, 0, 32, L.EPI_F32, torch.bfloat16, bias16, True),                # nothing to round: the plain GEMM
             (64, 0, 32, L.EPI_SEQ_OUT, torch.float16, bias16, True),
             (256, 9, 32, L.EPI_F32, torch.float16, bias16.float(), True)]
    for cs, t, mab, epi, out, bias, per_row in cases:
        tag = (shape, cs, t, mab, epi, out)
        acc = O.chunk_matmul_i8(a, w, None, cs, t, mab)
        sa = a_s if per_row else a_s[:1]
        ref = _chunk_epilogue_ref(acc, sa if per_row else sa.expand(M), w_s, bias, epi, out)
        y = K().matmul_chunk_dq(a.to(dev), w.to(dev), sa.to(dev), w_s.to(dev), None if bias is None else bias.to(dev),
                                epi, out, chunk_size=cs, chunk_trun_bits=t, max_acc_bits=mab)
        assert y.dtype == out and y.shape == (M, N), tag
        assert torch.equal(y.cpu().view(torch.int32 if out == torch.float32 else torch.int16),
                           ref.view(torch.int32 if out == torch.float32 else torch.int16)), tag
    # one scale per tensor on the weight side too
    acc = O.chunk_matmul_i8(a, w, None, 64, 5, 32)
    ref = _chunk_epilogue_ref(acc, a_s, w_s[:1].expand(N), bias16, L.EPI_F32_MULADD, torch.float16)
    y = K().matmul_chunk_dq(a.to(dev), w.to(dev), a_s.to(dev), w_s[:1].to(dev), bias16.to(dev), L.EPI_F32_MULADD,
                            torch.float16, chunk_size=64, chunk_trun_bits=5)
    assert torch.equal(y.cpu().view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float16, torch.bfloat16, torch.float32])
def test_matmul_chunk_fp_fused_epilogues_match_the_two_step_form(dev, dtype):
    """fmsmo_matmul_chunk_fp_dq against fmsmo_matmul_chunk_fp followed by the reference's torch
    expression on its fp32 accumulator: the same kernel accumulates, so the outputs are equal bit
    for bit; on integer-valued operands (exact in any summation order) also against the oracle."""
    from fms_mo_amd import _lib as L

    g = gen(92)
    for (M, N, Kd), cs, t, dl16 in (((70, 200, 1024), 64, 8, False), ((33, 96, 144), 32, 10, False),
                                    ((150, 130, 512), 16 if dtype != torch.float8_e4m3fn else 32, 12, True)):
        a = torch.randint(-6, 7, (M, Kd), generator=g).float().to(dtype)
        w = torch.randint(-6, 7, (N, Kd), generator=g).float().to(dtype)
        a_s = (torch.rand(M, generator=g) * 1e-1 + 1e-2).bfloat16().float()
        w_s = (torch.rand(N, generator=g) * 1e-2 + 1e-3).bfloat16().float()
        bias = (torch.randn(N, generator=g)).bfloat16()
        acc_gpu = K().matmul_chunk(a.to(dev), w.to(dev), None, chunk_size=cs, chunk_trun_bits=t,
                                   clamp_acc_to_dl16=dl16).cpu()
        acc_ref = O.chunk_matmul_fp(a.float(), w.float(), None, cs, t, dl16)
        assert torch.equal(acc_gpu, acc_ref)
        for epi, out, b in ((L.EPI_SEQ_OUT, torch.bfloat16, bias), (L.EPI_SEQ_OUT, torch.float16, None),
                            (L.EPI_SEQ_OUT, torch.float32, bias.float()), (L.EPI_F32_MULADD, torch.float16, bias),
                            (L.EPI_F32, torch.float32, bias)):
            ref = _chunk_epilogue_ref(acc_ref, a_s, w_s, b, epi, out)
            y = K().matmul_chunk_dq(a.to(dev), w.to(dev), a_s.to(dev), w_s.to(dev), None if b is None else b.to(dev),
                                    epi, out, chunk_size=cs, chunk_trun_bits=t, clamp_acc_to_dl16=dl16)
            v = torch.int32 if out == torch.float32 else torch.int16
            assert torch.equal(y.cpu().view(v), ref.view(v)), (dtype, M, N, Kd, epi, out)
    # real-valued operands: equal to the unfused kernel's accumulator put through the same expression
    a = torch.randn(96, 768, generator=g).to(dtype)
    w = (torch.randn(160, 768, generator=g) * 0.5).to(dtype)
    acc = K().matmul_chunk(a.to(dev), w.to(dev), None, chunk_size=64, chunk_trun_bits=9).cpu()
    ref = _chunk_epilogue_ref(acc, a_s[:96], w_s[:1].expand(160), None, L.EPI_SEQ_OUT, torch.bfloat16)
    y = K().matmul_chunk_dq(a.to(dev), w.to(dev), a_s[:96].to(dev), w_s[:1].to(dev), None, L.EPI_SEQ_OUT,
                            torch.bfloat16, chunk_size=64, chunk_trun_bits=9)
    assert torch.equal(y.cpu().view(torch.int16), ref.view(torch.int16))
