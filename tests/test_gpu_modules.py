"""The drop-in modules and custom ops on the GPU against the CPU oracle."""
import pytest
import torch

from oracle import qlinear_oracle as O

pytestmark = pytest.mark.gpu


def gen(seed):
    return torch.Generator().manual_seed(seed)


def make_qlinear(dev, K, N, smoothq=False, bias=True, seed=0, dtype=torch.float16):
    from fms_mo_amd.modules.linear import QLinear

    m = QLinear(K, N, bias=bias, num_bits_feature=8, qa_mode="pertokenmax", num_bits_weight=8,
                qw_mode="maxperCh", qcfg={"smoothq": smoothq, "smoothq_alpha": 0.5}, device="cpu")
    g = gen(seed)
    with torch.no_grad():
        m.weight.copy_(0.02 * torch.randn(N, K, generator=g))
        if bias:
            m.bias.copy_(0.01 * torch.randn(N, generator=g))
    m.to(dtype)
    m.quantize_weight.float()
    if smoothq:
        m.smoothq_act_scale = m.smoothq_act_scale.float()
        m.smoothq_alpha = m.smoothq_alpha.float()
    with torch.no_grad():
        m.quantize_weight.train()
        m.quantize_weight(m.weight)       # one training-mode pass initialises the weight clip values
    m.eval()
    return m if dev is None else m.to(dev)


def outlier_x(M, K, seed, dtype=torch.float16):
    g = gen(seed)
    x = torch.randn(M, K, generator=g)
    idx = torch.randperm(K, generator=g)[: max(1, round(0.01 * K))]
    x[:, idx] *= 50
    return x.to(dtype)


@pytest.mark.parametrize("smoothq", [False, True])
@pytest.mark.parametrize("shape", [(3, 40, 256, 384), (1, 512, 1024, 512), (1, 1, 4096, 512), (1, 3, 1024, 384),
                                   (2, 2, 2048, 256)])
def test_deploy_module_bit_exact_vs_oracle(dev, smoothq, shape):
    """Conversion (offline weight / scale preparation) runs on the CPU like the reference's
    lower_qmodel_cutlass (custom_ext_kernels/utils.py:830); the forward runs on the GPU."""
    from fms_mo_amd.modules.linear import QLinearINT8Deploy

    B, S, K, N = shape
    m = make_qlinear(None, K, N, smoothq=smoothq)
    x = outlier_x(B * S, K, 5).reshape(B, S, K)
    act_scale = None
    if smoothq:
        act_scale = x.reshape(-1, K).float().abs().amax(dim=0)
        m.set_act_scale(act_scale)
    dep = QLinearINT8Deploy.from_fms_mo(m, use_int_kernel="cutlass", use_dynamic_max_act_Qfunc=-1,
                                        recalc_clipvals=False, target_device=dev)
    y = dep(x.to(dev))
    bufs = O.deploy_prepare(m.weight.detach(), m.bias.detach(), m.quantize_weight.clip_val, act_scale, 0.5)
    ref = O.deploy_forward(x, bufs)
    assert torch.equal(dep.weight.cpu(), bufs["weight"]) and torch.equal(dep.w_scale.cpu(), bufs["w_scale"])
    assert y.shape == (B, S, N) and y.dtype == torch.float16
    assert torch.equal(dep.input_scale.cpu().reshape(-1), ref["input_scale"].float().reshape(-1))
    assert torch.equal(y.cpu().view(torch.int16), ref["y"].view(torch.int16))


def test_deploy_module_random_layers_bit_exact_vs_oracle(dev):
    """Fourteen seeded layers: any batch shape from one token to a few hundred, K and N off the
    tile sizes, with and without bias, with and without SmoothQuant: buffers, input scales and
    outputs are the oracle's, bit for bit (a layer without bias keeps the sign of a zero output)."""
    import random

    from fms_mo_amd.modules.linear import QLinearINT8Deploy

    rng = random.Random(7531)
    for case in range(14):
        B, S = rng.choice([(1, 1), (1, rng.randint(2, 16)), (rng.randint(2, 4), rng.randint(1, 90))])
        K = rng.choice([64 * rng.randint(1, 40), 128 * rng.randint(1, 40), 1024 * rng.choice([1, 2, 4])])
        N = rng.choice([8 * rng.randint(1, 100), rng.randint(10, 1200)])
        smoothq, bias = rng.random() < 0.5, rng.random() < 0.6
        tag = f"case {case}: B={B} S={S} K={K} N={N} smoothq={smoothq} bias={bias}"
        m = make_qlinear(None, K, N, smoothq=smoothq, bias=bias, seed=case)
        x = outlier_x(B * S, K, 7000 + case).reshape(B, S, K)
        act_scale = None
        if smoothq:
            act_scale = x.reshape(-1, K).float().abs().amax(dim=0)
            m.set_act_scale(act_scale)
        dep = QLinearINT8Deploy.from_fms_mo(m, use_int_kernel="cutlass", use_dynamic_max_act_Qfunc=-1,
                                            recalc_clipvals=False, target_device=dev)
        y = dep(x.to(dev))
        bufs = O.deploy_prepare(m.weight.detach(), m.bias.detach() if bias else None,
                                m.quantize_weight.clip_val, act_scale, 0.5)
        ref = O.deploy_forward(x, bufs)
        assert torch.equal(dep.weight.cpu(), bufs["weight"]) and torch.equal(dep.w_scale.cpu(), bufs["w_scale"]), tag
        assert torch.equal(dep.input_scale.cpu().reshape(-1), ref["input_scale"].float().reshape(-1)), tag
        assert torch.equal(y.cpu().view(torch.int16), ref["y"].view(torch.int16)), tag


@pytest.mark.parametrize("smoothq", [False, True])
def test_deploy_module_iaddmm_FP_vs_oracle(dev, smoothq):
    """use_int_kernel=False: the reference's emulation without an integer kernel
    (iaddmm_FP, linear.py:1190-1211): torch.matmul on the dequantized operands, every buffer in
    x's dtype.  The quantizer is still the device kernel: scales bit-exact, output within
    rtol / atol 1e-2 of the oracle (an fp16 matmul's summation order is the library's)."""
    from fms_mo_amd.modules.linear import QLinearINT8Deploy

    B, S, K, N = 2, 37, 512, 384
    m = make_qlinear(None, K, N, smoothq=smoothq)
    x = outlier_x(B * S, K, 9).reshape(B, S, K)
    act_scale = None
    if smoothq:
        act_scale = x.reshape(-1, K).float().abs().amax(dim=0)
        m.set_act_scale(act_scale)
    dep = QLinearINT8Deploy.from_fms_mo(m, use_int_kernel=False, use_dynamic_max_act_Qfunc=-1,
                                        recalc_clipvals=False, target_device=dev).half()
    assert dep.use_int_kernel is False and dep.iaddmm.__func__ is QLinearINT8Deploy.iaddmm_FP
    for name in ("w_scale", "bias", "smoothq_scale"):
        assert getattr(dep, name).dtype == torch.float16, name
    y = dep(x.to(dev))
    bufs = O.deploy_prepare(m.weight.detach(), m.bias.detach(), m.quantize_weight.clip_val, act_scale, 0.5)
    bufs16 = {k: (v.half() if torch.is_tensor(v) and v.is_floating_point() else v) for k, v in bufs.items()}
    ref = O.deploy_forward_fp(x, bufs16)
    assert y.shape == (B, S, N) and y.dtype == torch.float16
    x2 = x.reshape(-1, K)
    _, s_ref, _ = O.quant_act_pertoken_i8(x2, bufs16["smoothq_scale"] if smoothq else None)
    assert torch.equal(dep.input_scale.cpu().reshape(-1).float(), s_ref.float().reshape(-1))
    torch.testing.assert_close(y.cpu().float(), ref.float(), rtol=1e-2, atol=1e-2)
    # and it agrees with the integer-kernel module on the same layer at the same tolerance
    dep_i = QLinearINT8Deploy.from_fms_mo(m, use_int_kernel="cutlass", use_dynamic_max_act_Qfunc=-1,
                                          recalc_clipvals=False, target_device=dev)
    torch.testing.assert_close(y.float(), dep_i(x.to(dev)).float(), rtol=1e-2, atol=1e-2)


def test_deploy_module_converted_on_gpu_matches_within_tolerance(dev):
    """Converting on the GPU uses the GPU's pow / division roundings for the offline scales, so it
    is only tolerance-equal to the CPU-converted module."""
    from fms_mo_amd.modules.linear import QLinearINT8Deploy

    K, N = 512, 256
    m = make_qlinear(None, K, N, smoothq=True)
    x = outlier_x(64, K, 5)
    m.set_act_scale(x.float().abs().amax(dim=0))
    dep_cpu = QLinearINT8Deploy.from_fms_mo(m, use_dynamic_max_act_Qfunc=-1, recalc_clipvals=False, target_device=dev)
    dep_gpu = QLinearINT8Deploy.from_fms_mo(m.to(dev), use_dynamic_max_act_Qfunc=-1, recalc_clipvals=False)
    assert (dep_cpu.weight != dep_gpu.weight).float().mean() < 1e-3
    torch.testing.assert_close(dep_gpu(x.to(dev)).float(), dep_cpu(x.to(dev)).float(), rtol=1e-2, atol=1e-2)


def test_qlinear_eval_forward_within_tolerance_of_fake_quant(dev):
    K, N = 1024, 768
    m = make_qlinear(dev, K, N, smoothq=True)
    x = outlier_x(300, K, 6)
    a = x.float().abs().amax(dim=0)
    m.set_act_scale(a.to(dev))
    m.train()
    with torch.no_grad():
        y_train = m(x.to(dev))            # torch-op fake-quant path (also sets clip_val)
    m.eval()
    with torch.no_grad():
        y = m(x.to(dev))                  # integer path on the HIP kernels
    assert m.num_module_called.item() == 2 and y.dtype == torch.float16
    ref = O.qlinear_forward(x, m.weight.detach().cpu(), m.bias.detach().cpu(), a, 0.5,
                            w_clip_val=m.quantize_weight.clip_val.cpu())
    d = (y.cpu().float() - ref.float()).abs()
    assert (d > 1e-2 + 1e-2 * ref.float().abs()).float().mean() < 1e-3 and d.max() < 5e-2
    # the training-mode forward quantizes the weights on the grid of the CURRENT abs-max
    ref_train = O.qlinear_forward(x, m.weight.detach().cpu(), m.bias.detach().cpu(), a, 0.5)
    d2 = (y_train.cpu().float() - ref_train.float()).abs()
    assert (d2 > 1e-2 + 1e-2 * ref_train.float().abs()).float().mean() < 1e-2


def test_deploy_chunked_branches(dev):
    from fms_mo_amd.modules.linear import QLinearINT8Deploy

    K, N = 512, 256
    x = outlier_x(64, K, 7)
    m = make_qlinear(None, K, N)
    bufs = O.deploy_prepare(m.weight.detach(), m.bias.detach(), m.quantize_weight.clip_val)
    q_x, s_x, _ = O.quant_act_pertoken_i8(x)
    # cutlass + chunk loop: clamp to 24 bits, drop 4 LSBs per 64-chunk, fp32 scales
    dep = QLinearINT8Deploy.from_fms_mo(m, use_int_kernel="cutlass", use_dynamic_max_act_Qfunc=-1,
                                        recalc_clipvals=False, chunk_size=64, truncate_lsb=4, max_acc_bits=24,
                                        target_device=dev)
    y = dep(x.to(dev)).cpu()
    acc = O.chunk_matmul_i8(q_x, bufs["weight"], None, 64, 4, 24)
    ref = (acc * (s_x * bufs["w_scale"]) + bufs["bias"]).to(torch.float16)
    assert torch.equal(y.view(torch.int16), ref.view(torch.int16))
    # triton flavour: chunked kernel + fp16-scale epilogue
    dep2 = QLinearINT8Deploy.from_fms_mo(m, use_int_kernel="triton", use_dynamic_max_act_Qfunc=-1,
                                         recalc_clipvals=False, chunk_size=64, truncate_lsb=8, target_device=dev)
    y2 = dep2(x.to(dev)).cpu()
    acc2 = O.chunk_matmul_i8(q_x, bufs["weight"], None, 64, 8, 32)
    ref2 = O.epilogue_ref(acc2, s_x, bufs["w_scale"], bufs["bias"])
    assert torch.equal(y2.view(torch.int16), ref2.view(torch.int16))


def test_custom_ops(dev):
    from fms_mo_amd.custom_ext_kernels.utils import imatmul_ops_reg, native_gemm_ops_reg

    imatmul_ops_reg()
    native_gemm_ops_reg()
    a = torch.randint(-128, 128, (2, 9, 256), generator=gen(8), dtype=torch.int8)
    w = torch.randint(-128, 128, (96, 256), generator=gen(9), dtype=torch.int8)
    ref = O.int_gemm(a.reshape(-1, 256), w).reshape(2, 9, 96)
    ad, wd = a.to(dev), w.to(dev)
    assert torch.equal(torch.ops.fms_mo.imatmul(ad, wd.t()).cpu(), ref)                 # W.t() view
    assert torch.equal(torch.ops.fms_mo.imatmul(ad, wd.t().contiguous()).cpu(), ref)    # row-major [K,N]
    assert torch.equal(torch.ops.cutlass_gemm.i8i32nt(ad[0], wd.t()).cpu(), ref[0])
    assert torch.equal(torch.ops.mygemm.gemm_nt_i8i32(ad[0], wd).cpu(), ref[0])
    s_i, s_w = torch.tensor([0.02]), torch.rand(96, generator=gen(10)) * 1e-2
    bias = torch.randn(96, generator=gen(11))
    y = torch.ops.fms_mo.iaddmm(bias.to(dev), ad[0], wd.t(), s_i.to(dev), s_w.to(dev)).cpu()
    torch.testing.assert_close(y, s_i.float() * ref[0] * s_w + bias, rtol=1e-5, atol=1e-5)
    x = (torch.randn(9, 256, generator=gen(12)) * 2).half()
    zp = torch.tensor([131])
    y2 = torch.ops.fms_mo.q_iaddmm_dq(bias.to(dev), x.to(dev), wd.t(), s_i.to(dev), zp.to(dev), s_w.to(dev)).cpu()
    q = torch.clamp((x / s_i + zp - 128).round(), -128, 127).to(torch.int8)
    exp = (s_i.float() * O.int_gemm(q, w) * s_w + bias).to(torch.float16)
    torch.testing.assert_close(y2.float(), exp.float(), rtol=2e-3, atol=2e-3)
    q3 = torch.ops.fms_mo.q_per_t_sym(x.float().to(dev), s_i.to(dev), torch.tensor([3]).to(dev)).cpu()
    exp3 = torch.quantize_per_tensor(x.float(), 0.02, 3, torch.qint8).int_repr()
    assert torch.equal(q3, exp3)


def test_linear_fpx_acc_like_reference_test(dev):
    """fms-model-optimizer tests/triton_kernels/test_triton_mm.py:125-149 (fp32 Linear, 512 tokens)."""
    from fms_mo_amd.modules.linear import LinearFPxAcc

    torch.manual_seed(23)
    for fin, fout in [(64, 128), (256, 1024)]:
        lin = torch.nn.Linear(fin, fout).to(dev)
        inputs = torch.randn((512, fin)).to(dev)
        for t in [0, 8, 12, 16]:
            fpx = LinearFPxAcc.from_nn(lin, trun_bits=t)
            with torch.no_grad():
                base = lin(inputs)
                rel = (torch.norm(fpx(inputs) - base) / torch.norm(base)).item()
            assert rel < (1e-2 if t > 10 else 1e-4), (fin, t, rel)


@pytest.mark.parametrize("dl16", [False, True])
def test_linear_fpx_acc_dynamic_fp8_vs_oracle(dev, dl16):
    from fms_mo_amd.modules.linear import LinearFPxAcc

    lin = torch.nn.Linear(256, 192).to(torch.bfloat16)
    x = (torch.randn(40, 256, generator=gen(13)) * 2).bfloat16()
    fpx = LinearFPxAcc.from_nn(lin.to(dev), trun_bits=8, chunk_size=64, dynamic_fp8="per_token",
                               clamp_acc_to_dl16=dl16)
    y = fpx(x.to(dev)).cpu()
    ref = O.fpxacc_forward(x, lin.weight.detach().cpu(), lin.bias.detach().cpu(), 8, 64, "per_token", dl16)
    torch.testing.assert_close(y.float(), ref.float(), rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_linear_fpx_acc_per_tensor_fp8_vs_oracle(dev, dtype):
    """dynamic_fp8="per_tensor": both scales come from the device-side abs-max (no torch
    reductions, nothing read back); codes are the oracle's, so on a chunk of the whole reduction
    without truncation the output is the oracle's up to the fp32 summation order."""
    from fms_mo_amd import _lib as L
    from fms_mo_amd import kernels as kn
    from fms_mo_amd.modules.linear import LinearFPxAcc

    lin = torch.nn.Linear(256, 192).to(dtype)
    x = (torch.randn(40, 256, generator=gen(16)) * 2).to(dtype)
    fpx = LinearFPxAcc.from_nn(lin.to(dev), trun_bits=8, chunk_size=64, dynamic_fp8="per_tensor")
    y = fpx(x.to(dev)).cpu()
    w = lin.weight.detach().cpu()
    ref = O.fpxacc_forward(x, w, lin.bias.detach().cpu(), 8, 64, "per_tensor", False)
    torch.testing.assert_close(y.float(), ref.float(), rtol=2e-2, atol=2e-2)
    for t in (x, w):
        q_ref, s_ref = O.fp8_quant_fpxacc(t, per_tensor=True)
        q, s = kn.quant_act_fp8_dynamic(t.to(dev), L.FP8_FPXACC, True, 1e-5, True)
        assert torch.equal(q.cpu().view(torch.uint8), q_ref.view(torch.uint8))
        assert torch.equal(s.cpu().reshape(()), s_ref.float().reshape(()))


def test_qlinear_int8_train_forward_vs_oracle(dev):
    from fms_mo_amd.modules.linear import QLinearINT8Train

    lin = torch.nn.Linear(512, 128).half()
    x = (torch.randn(64, 512, generator=gen(14))).half()
    m = QLinearINT8Train.from_fms_mo(lin.to(dev), lsb_trun_bits=8, chunk_size=64, max_acc_bits=24)
    y = m(x.to(dev)).cpu()
    ref, _, _, _ = O.int8train_forward(x, lin.weight.detach().cpu(), lin.bias.detach().cpu(), 8, 64, 24)
    assert torch.equal(y.view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("cfg", [("tensor", "token", True), ("channel", "token", True),
                                 ("tensor", "tensor", True), ("tensor", "tensor", False)])
def test_fp8_linear_vs_oracle(dev, cfg):
    from fms_mo_amd.modules.fp8_linear import FP8Linear

    wstrat, astrat, dynamic = cfg
    g = gen(15)
    W = 0.02 * torch.randn(384, 512, generator=g)
    b = 0.1 * torch.randn(384, generator=g)
    x = torch.randn(2, 50, 512, generator=g).bfloat16()
    m = FP8Linear.from_float(W, b, per_channel=wstrat == "channel", act=astrat)
    if not dynamic:
        m.linear_config["input_activations"]["dynamic"] = False
        m.input_scale = torch.nn.Parameter(torch.tensor([0.0123]), requires_grad=False)
    y = m.to(dev)(x.to(dev)).cpu()
    assert y.shape == (2, 50, 384) and y.dtype == torch.bfloat16 and torch.isfinite(y).all()
    x2 = x.reshape(-1, 512)
    if not dynamic:
        in_scale = torch.tensor([0.0123])
    elif astrat == "tensor":
        in_scale = (x2.abs().amax().float() / 448).clamp(min=1e-12).reshape(1)
    else:
        in_scale = None
    ref, qx, s_x = O.fp8_linear_forward(x, m.weight.data.cpu(), m.weight_scale.data.cpu(), b.bfloat16(), in_scale)
    exact = (qx.double() * s_x.double()) @ (m.weight.data.cpu().double() * m.weight_scale.data.cpu().double()).t() + b.double()
    torch.testing.assert_close(y.reshape(-1, 384).double(), exact, rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(y.float(), ref.float(), rtol=3e-2, atol=3e-2)


def test_fp8_linear_dynamic_scale_rule_attributes(dev):
    """The floor and the division dtype of the dynamic activation scale are module attributes
    (the two properties only torchao's source fixes); each setting matches the oracle with the
    same arguments, per token and per tensor."""
    from fms_mo_amd import kernels as kn
    from fms_mo_amd.modules.fp8_linear import FP8Linear

    g = gen(17)
    W = 0.02 * torch.randn(256, 512, generator=g)
    x = torch.randn(48, 512, generator=g).bfloat16()
    x[3] = 0
    for astrat in ("token", "tensor"):
        m = FP8Linear.from_float(W, None, per_channel=False, act=astrat).to(dev)
        for floor, in_xt in ((1e-12, False), (1e-5, True), (1e-3, False)):
            m.dynamic_scale_floor, m.dynamic_scale_in_input_dtype = floor, in_xt
            y = m(x.to(dev)).cpu()
            s_x = O.fp8_dynamic_scale(x, floor, in_xt, astrat == "tensor")
            ref, qx, _ = O.fp8_linear_forward(x, m.weight.data.cpu(), m.weight_scale.data.cpu(), None,
                                              s_x if astrat == "token" else s_x.reshape(1))
            q, s = kn.quant_act_fp8_dynamic(x.to(dev), 0, astrat == "tensor", floor, in_xt)
            assert torch.equal(q.cpu().view(torch.uint8), qx.view(torch.uint8))
            assert torch.equal(s.cpu(), s_x.reshape(-1))
            torch.testing.assert_close(y.float(), ref.float(), rtol=3e-2, atol=3e-2)


def test_swapped_mlp_replays_from_a_hip_graph(dev):
    """The reference's route to a speed-up is capturing the lowered model (torch.compile /
    CUDA graphs, examples/QAT_INT8/README.md:116-122).  A gated MLP of three deploy modules is
    captured once and replayed with new inputs, with eager work and synchronisations between the
    replays; every replay must equal the eager result bit for bit.  No entry point allocates,
    synchronises or clears memory, so the capture holds only kernel launches."""
    from fms_mo_amd.modules.linear import QLinearINT8Deploy

    H, I, T = 512, 1536, 48
    mods = {}
    for name, k, n, seed in [("gate", H, I, 1), ("up", H, I, 2), ("down", I, H, 3)]:
        q = make_qlinear(None, k, n, smoothq=True, seed=seed)
        q.set_act_scale(torch.rand(k, generator=gen(10 + seed)) * 3 + 0.2)
        mods[name] = QLinearINT8Deploy.from_fms_mo(q, use_int_kernel="cutlass", use_dynamic_max_act_Qfunc=-1,
                                                   recalc_clipvals=False, target_device=dev)

    def mlp(x):
        return mods["down"](torch.nn.functional.silu(mods["gate"](x)) * mods["up"](x))

    xs = [outlier_x(T, H, 20 + i).to(dev) for i in range(4)]
    eager = [mlp(x).clone() for x in xs]            # also warms the cached host-side checks
    static_x = xs[0].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        mlp(static_x)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_y = mlp(static_x)
    for rnd in range(2):
        for x, ref in zip(xs, eager):
            static_x.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(static_y.view(torch.int16), ref.view(torch.int16))
            _ = mlp(x)                               # eager work between replays
            torch.cuda.synchronize()


def test_swapped_mlp_traces_without_graph_breaks(dev):
    """torch.compile must see the lowered modules as operator calls (the reference registers its
    integer matmuls as torch.ops.fms_mo.* for this, custom_ext_kernels/utils.py:642-802): the
    kernel wrappers are torch.ops.fms_mo_amd.* with shape-only twins.  ``fullgraph=True`` turns
    any graph break into an error; the backend replays the traced graph with the real kernels."""
    from fms_mo_amd.modules.linear import QLinearINT8Deploy

    H, I, T = 512, 1536, 48
    mods = {}
    for name, k, n, seed in [("gate", H, I, 1), ("up", H, I, 2), ("down", I, H, 3)]:
        q = make_qlinear(None, k, n, smoothq=True, seed=seed)
        q.set_act_scale(torch.rand(k, generator=gen(10 + seed)) * 3 + 0.2)
        mods[name] = QLinearINT8Deploy.from_fms_mo(q, use_int_kernel="cutlass", use_dynamic_max_act_Qfunc=-1,
                                                   recalc_clipvals=False, target_device=dev)

    class MLP(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.gate, self.up, self.down = mods["gate"], mods["up"], mods["down"]

        def forward(self, x):
            return self.down(torch.nn.functional.silu(self.gate(x)) * self.up(x))

    mlp = MLP()
    xs = [outlier_x(T, H, 30 + i).to(dev) for i in range(3)]
    eager = [mlp(x).clone() for x in xs]
    compiled = torch.compile(mlp, backend="aot_eager", fullgraph=True)
    for x, ref in zip(xs, eager):
        y = compiled(x)
        assert torch.equal(y.view(torch.int16), ref.view(torch.int16))
    ops = [n for n in dir(torch.ops.fms_mo_amd) if not n.startswith("_")]
    assert {"quant_act_i8_pertoken", "gemm_i8_dq"} <= set(ops)


def test_operator_twins_agree_with_the_kernels_on_shapes(dev):
    from fms_mo_amd import kernels

    x = torch.randn(24, 256, device=dev).half()
    sm = (torch.rand(256, device=dev) + 0.5).half()
    w = torch.randint(-127, 128, (96, 256), dtype=torch.int8, device=dev)
    ws = torch.rand(96, device=dev)
    q, s = kernels.quant_act_i8_pertoken(x, sm)
    torch.library.opcheck(torch.ops.fms_mo_amd.quant_act_i8_pertoken.default, (x, sm, torch.float16, False),
                          test_utils=("test_schema", "test_faketensor"))
    torch.library.opcheck(torch.ops.fms_mo_amd.gemm_i8_dq.default,
                          (q, w, s, ws, None, torch.float16, 0, False),
                          test_utils=("test_schema", "test_faketensor"))
    torch.library.opcheck(torch.ops.fms_mo_amd.quant_act_i8_static.default, (x, 0.05, 128, 0),
                          test_utils=("test_schema", "test_faketensor"))


@pytest.mark.parametrize("smoothq", [False, True])
@pytest.mark.parametrize("buffers", ["fp16", "fp32"])
@pytest.mark.parametrize("K,N", [(4096, 1024), (14336, 512), (1024, 768)])
def test_decode_step_equals_the_rows_of_a_larger_batch(dev, smoothq, buffers, K, N):
    """The deployed module takes the fused one-launch path for a decode step of a few tokens, with
    its buffers cast to fp16 (the lowering helper's flow) or left in fp32 under fp16 activations
    (the SmoothQuant divide then promotes the quantizer to fp32).  Per-token quantization makes
    every output row a function of its own input row only, so the decode step must reproduce, bit
    for bit, the corresponding rows of a 40-token batch (which runs the quantizer and the GEMM as
    two kernels)."""
    from fms_mo_amd.modules.linear import QLinearINT8Deploy

    m = make_qlinear(None, K, N, smoothq=smoothq, seed=7)
    x = outlier_x(40, K, 9)
    if smoothq:
        m.set_act_scale(x.float().abs().amax(dim=0))
    dep = QLinearINT8Deploy.from_fms_mo(m, use_int_kernel="cutlass", use_dynamic_max_act_Qfunc=-1,
                                        recalc_clipvals=False, target_device="cpu")
    dep = dep.half().to(dev) if buffers == "fp16" else dep.to(dev)
    if smoothq:
        assert dep.smoothq_scale.dtype == (torch.float16 if buffers == "fp16" else torch.float32)
    xd = x.to(dev)
    full = dep(xd).clone()
    full_scale = dep.input_scale.clone()
    for M in (1, 2, 4):  # fused launch where it is served; else quantizer and decode kernel
        y = dep(xd[:M])
        assert torch.equal(y.view(torch.int16), full[:M].view(torch.int16))
        assert torch.equal(dep.input_scale.reshape(-1), full_scale.reshape(-1)[:M])
