"""Attention matmuls on the GPU: the affine int8 quantizer (plain and transposing) bit-exact
against the CPU oracle, the batched int8 / e4m3 MFMA matmuls against exact integer / float64
products, ``QBmmINT8Deploy`` and ``spyre::scaled_bmm`` against the oracle's restatements."""
import types

import pytest
import torch

from oracle import qlinear_oracle as O

pytestmark = pytest.mark.gpu


def gen(seed):
    return torch.Generator().manual_seed(seed)


def K():
    from fms_mo_amd import kernels

    return kernels


@pytest.mark.parametrize("xdt,sdt", [(torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16),
                                     (torch.float16, torch.float32), (torch.float32, torch.float32)])
@pytest.mark.parametrize("shape", [(3, 64, 128), (2, 77, 100), (1, 300, 24), (5, 1, 72)])
@pytest.mark.parametrize("transpose", [False, True])
def test_affine_quantizer_bit_exact(dev, xdt, sdt, shape, transpose):
    B, R, C = shape
    x = (3 * torch.randn(B, R, C, generator=gen(7))).to(xdt)
    scale = torch.tensor([0.0371], dtype=sdt)
    for zp in (torch.tensor([0], dtype=torch.int), torch.tensor([37 - 128], dtype=torch.int)):
        ref = O.qbmm_quant(x, scale, zp)
        T = torch.promote_types(xdt, sdt)
        q = K().quant_i8_affine(x.to(dev), float(scale), float(zp), T, transpose=transpose).cpu()
        inner = R if transpose else C
        pad = (inner + 63) // 64 * 64
        want = ref.transpose(1, 2) if transpose else ref
        assert q.shape == (B, C if transpose else R, pad)
        assert torch.equal(q[..., :inner], want)
        assert torch.all(q[..., inner:] == 0)


@pytest.mark.parametrize("xdt", [torch.float16, torch.bfloat16])
def test_affine_quantizer_every_16_bit_pattern(dev, xdt):
    """The scalar division runs without the IEEE sequence where that is exact (scale a value of
    the compute dtype, or fp16 x with an fp32 scale): every 16-bit pattern of x except NaN, whose
    int8 cast is undefined in the reference -- zeros of both signs, subnormals, the largest finite
    values, both infinities -- against scales from 2^-20 to 600 and two zero points."""
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    x = bits.view(xdt)
    x = x[~torch.isnan(x)]
    x = x[: x.numel() // 64 * 64].reshape(1, -1, 64)
    scales = [0.0371, 1.0, 2.0 ** -20, 600.0, 3.0517578125e-05, 0.3333]
    for sdt in (xdt, torch.float32):
        if sdt == torch.float32 and xdt == torch.bfloat16:
            continue  # promoted to fp32 with bf16 x: plain IEEE path, covered above
        for sv in scales:
            scale = torch.tensor([sv], dtype=sdt)
            for zp in (0, -91):
                ref = O.qbmm_quant(x, scale, torch.tensor([zp], dtype=torch.int))
                q = K().quant_i8_affine(x.to(dev), float(scale), float(zp), torch.promote_types(xdt, sdt)).cpu()
                assert torch.equal(q[..., :64], ref), f"scale {sv} ({sdt}) zp {zp}"


def test_affine_quantizer_strided_input(dev):
    """A [b, h, s, d] tensor viewed as K^T ([.., d, s], unit stride along d): the module quantizes
    the untransposed view, a slice along the last dimension takes the scalar path."""
    x = torch.randn(2, 4, 50, 64, generator=gen(8)).half()
    scale, zp = torch.tensor([0.05]).half(), torch.tensor([0], dtype=torch.int)
    q = K().quant_i8_affine(x.to(dev)[..., 3:43], float(scale), 0.0, torch.float16).cpu()
    assert torch.equal(q[..., :40], O.qbmm_quant(x[..., 3:43], scale, zp).reshape(8, 50, 40))


@pytest.mark.parametrize("shape", [(4, 256, 256, 128), (3, 300, 333, 128), (3, 100, 77, 64), (2, 300, 128, 320),
                                   (3, 300, 100, 640), (2, 700, 128, 1024),  # tall tiles, staggered reduction
                                   (5, 64, 40, 192), (1, 513, 700, 256),
                                   (40, 520, 700, 128)])  # 600 ragged tiles of the K = 128 kernel: its blocks walk several
@pytest.mark.parametrize("with_bias", [False, True])
def test_bmm_i8_exact(dev, shape, with_bias):
    B, M, N, Kd = shape
    g = gen(9)
    a = torch.randint(-128, 128, (B, M, Kd), generator=g, dtype=torch.int32).to(torch.int8)
    b = torch.randint(-128, 128, (B, N, Kd), generator=g, dtype=torch.int32).to(torch.int8)
    bias = torch.randn(B, N, generator=g) if with_bias else None
    sa, sb = torch.tensor([2.0 ** -7]), torch.tensor([2.0 ** -9])
    y = K().bmm_i8_dq(a.to(dev), b.to(dev), sa.to(dev), sb.to(dev),
                      bias=bias.to(dev) if with_bias else None, out_dtype=torch.float32).cpu()
    acc = torch.matmul(a.to(torch.int64), b.to(torch.int64).transpose(1, 2))
    ref = acc.double() * 2.0 ** -16 + (bias.double().unsqueeze(1) if with_bias else 0.0)
    # power-of-two scales: the only rounding is int32 -> fp32 and the final add
    torch.testing.assert_close(y.double(), ref, rtol=2e-7, atol=1e-6)


@pytest.mark.parametrize("shape", [(4, 256, 256, 128), (3, 300, 333, 128), (3, 100, 77, 64), (2, 130, 128, 384),
                                   (3, 300, 100, 640), (40, 520, 700, 128)])
def test_bmm_fp8_exact_on_integer_operands(dev, shape):
    B, M, N, Kd = shape
    g = gen(10)
    a = torch.randint(-8, 9, (B, M, Kd), generator=g).float().to(torch.float8_e4m3fn)
    b = torch.randint(-8, 9, (B, N, Kd), generator=g).float().to(torch.float8_e4m3fn)
    s = torch.tensor([0.5])
    y = K().bmm_fp8_dq(a.to(dev), b.to(dev), s.to(dev), s.to(dev), out_dtype=torch.float32).cpu()
    ref = torch.matmul(a.double(), b.double().transpose(1, 2)) * 0.25
    assert torch.equal(y.double(), ref)


def test_bmm_random_shapes_exact(dev):
    """Thirty seeded batched products: any batch count, M and N, K a multiple of 64 up to 1024,
    with and without the per-column bias: int8 exact up to the fp32 conversion (power-of-two
    scales), e4m3 exact on small integers; whichever batched kernel serves the shape."""
    import random

    rng = random.Random(86420)
    for case in range(30):
        B = rng.choice([1, rng.randint(2, 8), rng.randint(8, 48)])
        M, N = rng.choice([1, rng.randint(2, 130), rng.randint(130, 700)]), rng.randint(1, 700)
        Kd = 64 * rng.randint(1, 16)
        if B * M * N > 12e6:
            B = max(1, int(12e6 // (M * N)))
        tag = f"case {case}: B={B} M={M} N={N} K={Kd}"
        g = gen(9000 + case)
        a = torch.randint(-128, 128, (B, M, Kd), generator=g, dtype=torch.int32).to(torch.int8)
        b = torch.randint(-128, 128, (B, N, Kd), generator=g, dtype=torch.int32).to(torch.int8)
        bias = torch.randn(B, N, generator=g) if case % 2 else None
        sa, sb = torch.tensor([2.0 ** -7]), torch.tensor([2.0 ** -9])
        y = K().bmm_i8_dq(a.to(dev), b.to(dev), sa.to(dev), sb.to(dev),
                          bias=None if bias is None else bias.to(dev), out_dtype=torch.float32).cpu()
        acc = torch.matmul(a.to(dev).double(), b.to(dev).double().transpose(1, 2)).cpu()
        ref = acc * 2.0 ** -16 + (bias.double().unsqueeze(1) if bias is not None else 0.0)
        torch.testing.assert_close(y.double(), ref, rtol=2e-7, atol=1e-6, msg=tag)
        a8 = torch.randint(-8, 9, (B, M, Kd), generator=g).float().to(torch.float8_e4m3fn)
        b8 = torch.randint(-8, 9, (B, N, Kd), generator=g).float().to(torch.float8_e4m3fn)
        s = torch.tensor([0.5])
        y8 = K().bmm_fp8_dq(a8.to(dev), b8.to(dev), s.to(dev), s.to(dev), out_dtype=torch.float32).cpu()
        ref8 = torch.matmul(a8.to(dev).double(), b8.to(dev).double().transpose(1, 2)).cpu() * 0.25
        assert torch.equal(y8.double(), ref8), tag


def stub_qbmm(clip1, clipn1, clip2, mode="asym", nbits1=8, dtype=torch.float32):
    m = torch.nn.Module()
    m.num_bits_m1, m.num_bits_m2, m.qm1_mode = nbits1, 8, mode
    m.quantize_m1 = types.SimpleNamespace(clip_val=torch.tensor([clip1], dtype=dtype),
                                          clip_valn=torch.tensor([clipn1], dtype=dtype), num_bits=nbits1)
    m.quantize_m2 = types.SimpleNamespace(clip_val=torch.tensor([clip2], dtype=dtype), num_bits=8)
    m.register_parameter("dummy", torch.nn.Parameter(torch.zeros(1)))
    return m


@pytest.mark.parametrize("xdt,sdt", [(torch.float16, torch.float32), (torch.float16, torch.float16),
                                     (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("case", ["qk", "pv", "2d", "ragged"])
def test_qbmm_int8_deploy_against_oracle(dev, xdt, sdt, case):
    from fms_mo_amd.modules.bmm import QBmmINT8Deploy

    g = gen(11)
    if case == "qk":  # Q [b,h,s,d] @ K^T (a transposed view)
        m1 = torch.randn(2, 4, 96, 128, generator=g).to(xdt)
        m2 = torch.randn(2, 4, 80, 128, generator=g).to(xdt).transpose(-1, -2)
        src = stub_qbmm(3.0, -3.5, 3.2, dtype=sdt)
    elif case == "pv":  # softmax output (unidirectional, 7 bit) @ V [b,h,s,d]
        m1 = torch.softmax(torch.randn(2, 4, 96, 160, generator=g), dim=-1).to(xdt)
        m2 = torch.randn(2, 4, 160, 128, generator=g).to(xdt)
        src = stub_qbmm(1.0, 0.0, 3.0, mode="sym", nbits1=7, dtype=sdt)
    elif case == "2d":
        m1 = torch.randn(70, 200, generator=g).to(xdt)
        m2 = torch.randn(200, 50, generator=g).to(xdt)
        src = stub_qbmm(2.5, -2.0, 2.8, dtype=sdt)
    else:
        m1 = torch.randn(3, 77, 45, generator=g).to(xdt)
        m2 = torch.randn(3, 45, 19, generator=g).to(xdt)
        src = stub_qbmm(2.5, -2.5, 2.8, mode="sym", dtype=sdt)
    mod_cpu = QBmmINT8Deploy.from_fms_mo(src, target_device="cpu")
    ref, r1, r2 = O.qbmm_int8_deploy(m1.double(), m2.double(), mod_cpu.m1_scale.double(), mod_cpu.m1_zp,
                                     mod_cpu.m2_scale.double(), mod_cpu.m2_zp)
    _, q1_ref, q2_ref = O.qbmm_int8_deploy(m1, m2, mod_cpu.m1_scale, mod_cpu.m1_zp, mod_cpu.m2_scale,
                                           mod_cpu.m2_zp)
    mod = QBmmINT8Deploy.from_fms_mo(src, target_device=dev)
    assert mod.m1_scale.device.type == "cuda" and mod._get_name() == "QBmmINT8Deploy"
    q1, q2 = mod.quantize_operands(m1.to(dev), m2.to(dev))
    k, n = m2.shape[-2:]
    assert torch.equal(q1.cpu()[..., :k].reshape(q1_ref.shape), q1_ref)
    assert torch.equal(q2.cpu()[..., :k].transpose(1, 2).reshape(q2_ref.shape), q2_ref)
    y = mod(m1.to(dev), m2.to(dev))
    assert y.dtype == xdt and y.shape == ref.shape
    # exact integers; what is left is the fp32 epilogue and the output cast
    acc = torch.matmul(q1_ref.double(), q2_ref.double())
    s = mod_cpu.m1_scale.double() * mod_cpu.m2_scale.double()
    exact = acc * s - (mod_cpu.m1_zp - 128).double() * q2_ref.double().sum(dim=-2, keepdim=True) * s
    ulp = 2.0 ** -8 if xdt == torch.bfloat16 else 2.0 ** -11
    err = (y.cpu().double() - exact).abs()
    # the product term and the zero-point correction are each rounded to fp32 before they cancel
    terms = (acc * s).abs() + ((mod_cpu.m1_zp - 128).double() * q2_ref.double().sum(dim=-2, keepdim=True) * s).abs()
    assert torch.all(err <= 1.1 * ulp * exact.abs() + 4e-7 * terms + 1e-7)


def test_qbmm_literal_reference_on_two_dimensional_operands(dev):
    """Where the reference's own forward is well defined (2-D m2, products small enough for its
    fp16 matmul) the integer path agrees with it to fp16 rounding."""
    from fms_mo_amd.modules.bmm import QBmmINT8Deploy

    g = gen(12)
    m1 = (0.2 * torch.randn(40, 16, generator=g)).half()
    m2 = (0.2 * torch.randn(16, 24, generator=g)).half()
    src = stub_qbmm(3.0, -3.0, 3.0, mode="sym")
    mod_cpu = QBmmINT8Deploy.from_fms_mo(src, target_device="cpu")
    lit, _, _ = O.qbmm_int8_deploy(m1, m2, mod_cpu.m1_scale, mod_cpu.m1_zp, mod_cpu.m2_scale,
                                   mod_cpu.m2_zp, literal=True)
    y = QBmmINT8Deploy.from_fms_mo(src, target_device=dev)(m1.to(dev), m2.to(dev))
    torch.testing.assert_close(y.cpu().float(), lit.float(), rtol=1e-2, atol=1e-2 * lit.float().abs().max().item())


@pytest.mark.parametrize("out_dtype", [None, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case", ["qk", "pv", "ragged"])
def test_scaled_bmm_against_oracle(dev, out_dtype, case):
    from fms_mo_amd.aiu_addons.fp8.fp8_spyre_op import register_spyre_scaled_bmm

    register_spyre_scaled_bmm()
    g = gen(13)
    if case == "qk":
        m1 = torch.randn(2, 4, 96, 128, generator=g)
        m2 = torch.randn(2, 4, 80, 128, generator=g).transpose(-1, -2)
    elif case == "pv":
        m1 = torch.rand(2, 4, 96, 160, generator=g)
        m2 = torch.randn(2, 4, 160, 128, generator=g)
    else:
        m1 = torch.randn(3, 50, 72, generator=g)
        m2 = torch.randn(3, 72, 33, generator=g)
    s1, s2 = torch.tensor([0.02]), torch.tensor([0.03])
    a = (m1 / s1).clamp(-448, 448).to(torch.float8_e4m3fn)
    b = (m2 / s2).clamp(-448, 448).to(torch.float8_e4m3fn)
    y = torch.ops.spyre.scaled_bmm(a.to(dev), b.to(dev), s1.to(dev), s2.to(dev), out_dtype)
    ref = O.scaled_bmm(a, b, s1, s2, torch.float32)
    assert y.dtype == (torch.float32 if out_dtype is None else out_dtype) and y.shape == ref.shape
    torch.testing.assert_close(y.cpu().float(), ref, rtol=1e-2, atol=1e-2 * ref.abs().max().item())


def test_scaled_bmm_schema_and_shape_only_twin(dev):
    from fms_mo_amd.aiu_addons.fp8.fp8_spyre_op import register_spyre_scaled_bmm

    register_spyre_scaled_bmm()
    a = torch.randn(2, 64, 128).to(torch.float8_e4m3fn).to(dev)
    b = torch.randn(2, 128, 64).to(torch.float8_e4m3fn).to(dev)
    s = torch.tensor([0.5], device=dev)
    # (the schema check of opcheck hashes its inputs with ops that float8 tensors do not have)
    torch.library.opcheck(torch.ops.spyre.scaled_bmm.default, (a, b, s, s, torch.bfloat16),
                          test_utils=("test_faketensor",))


def test_attention_shapes_of_llama3_8b(dev):
    """32 heads, head dimension 128, 2048 tokens: Q.K^T and P.V of one sequence against float64
    products of the same integer codes, computed on the GPU by torch."""
    g = torch.Generator(device=dev).manual_seed(14)
    h, s, d = 32, 2048, 128
    q1 = torch.randint(-128, 128, (h, s, d), generator=g, device=dev, dtype=torch.int32).to(torch.int8)
    k1 = torch.randint(-128, 128, (h, s, d), generator=g, device=dev, dtype=torch.int32).to(torch.int8)
    one = torch.ones(1, device=dev)
    y = K().bmm_i8_dq(q1, k1, one, one, out_dtype=torch.float32)
    ref = torch.matmul(q1.double(), k1.double().transpose(1, 2))
    assert torch.equal(y.double(), ref)  # |acc| <= 2^21: exact in fp32
    p = torch.randint(0, 128, (h, s, s), generator=g, device=dev, dtype=torch.int32).to(torch.int8)
    vt = torch.randint(-128, 128, (h, d, s), generator=g, device=dev, dtype=torch.int32).to(torch.int8)
    y = K().bmm_i8_dq(p, vt, one, one, out_dtype=torch.float32)
    ref = torch.matmul(p.double(), vt.double().transpose(1, 2))
    torch.testing.assert_close(y.double(), ref, rtol=1e-7, atol=0)


def test_qbmm_replays_from_a_hip_graph(dev):
    """Scales and zero points are cached on the host at conversion, the correction is computed on
    the device: forward holds only kernel launches and can be captured."""
    from fms_mo_amd.modules.bmm import QBmmINT8Deploy

    g = gen(15)
    mod = QBmmINT8Deploy.from_fms_mo(stub_qbmm(3.0, -3.5, 3.2), target_device=dev)
    k = torch.randn(2, 4, 80, 128, generator=g).half().to(dev)
    qs = [torch.randn(2, 4, 96, 128, generator=g).half().to(dev) for _ in range(3)]
    fn = lambda q: mod(q, k.transpose(-1, -2))
    eager = [fn(q).clone() for q in qs]
    static_q = qs[0].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn(static_q)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = fn(static_q)
    for _ in range(2):
        for q, ref in zip(qs, eager):
            static_q.copy_(q)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out.view(torch.int16), ref.view(torch.int16))
            fn(q)
            torch.cuda.synchronize()
