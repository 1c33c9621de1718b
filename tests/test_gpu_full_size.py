"""Parity at the full sizes of the benchmark configurations, through properties that do not need
a full-size CPU product: exact checksums (row / column sums of an integer GEMM equal the product
with the summed operand), sampled sub-blocks recomputed by the oracle, the invariants of the
truncation (low bits zero), and equality between kernels that must agree (grouped vs per-expert,
skinny-M vs tiled).  Element-wise kernels (activation quantizers) are compared in full."""
import pytest
import torch

from oracle import qlinear_oracle as O

pytestmark = pytest.mark.gpu

LLAMA = [("qkv", 4096, 6144), ("o", 4096, 4096), ("gate_up", 4096, 28672), ("down", 14336, 4096)]
M_TOK = 4096


def K():
    from fms_mo_amd import kernels

    return kernels


def gen(seed):
    return torch.Generator().manual_seed(seed)


def _rand_i8_dev(shape, seed, dev):
    g = torch.Generator(device=dev).manual_seed(seed)
    return torch.randint(-128, 128, shape, generator=g, dtype=torch.int8, device=dev)


def _sample(n, k, seed):
    return torch.randperm(n, generator=gen(seed))[:k].sort().values


@pytest.mark.parametrize("name,Kd,N", LLAMA)
def test_int8_gemm_checksums_and_sampled_blocks_full_size(dev, name, Kd, N):
    a, w = _rand_i8_dev((M_TOK, Kd), 101, dev), _rand_i8_dev((N, Kd), 102, dev)
    c = K().gemm_i8_i32(a, w)
    assert c.shape == (M_TOK, N) and c.dtype == torch.int32
    # |sums| < 4096 * 14336 * 128 * 128 < 2^53: float64 arithmetic on them is exact
    col_sum = c.to(torch.float64).sum(dim=0)
    ref_col = a.to(torch.float64).sum(dim=0) @ w.to(torch.float64).t()
    assert torch.equal(col_sum, ref_col)
    row_sum = c.to(torch.float64).sum(dim=1)
    ref_row = a.to(torch.float64) @ w.to(torch.float64).sum(dim=0)
    assert torch.equal(row_sum, ref_row)
    # sampled rows x columns recomputed exactly on the CPU, including both edges of the matrix
    mi = torch.unique(torch.cat([_sample(M_TOK, 48, 1), torch.tensor([0, 255, 256, M_TOK - 1])]))
    ni = torch.unique(torch.cat([_sample(N, 48, 2), torch.tensor([0, 255, 256, N - 1])]))
    ref = O.int_gemm(a[mi.to(dev)].cpu(), w[ni.to(dev)].cpu())
    assert torch.equal(c[mi.to(dev)][:, ni.to(dev)].cpu(), ref)


@pytest.mark.parametrize("name,Kd,N", LLAMA)
def test_smoothquant_linear_full_size_sampled_bit_exact(dev, name, Kd, N):
    """Config 2 end to end (SmoothQuant divide + per-token quantizer + GEMM + reference epilogue):
    the quantizer output is compared in full, the fp16 result on sampled rows / columns."""
    g = gen(1)
    x = torch.randn(M_TOK, Kd, generator=g)
    idx = torch.randperm(Kd, generator=g)[: round(0.01 * Kd)]
    x[:, idx] *= 50
    x = x.half()
    w8 = torch.randint(-127, 128, (N, Kd), generator=g, dtype=torch.int8)
    w_scale = (torch.rand(N, generator=g) * 1e-3 + 1e-5).float()
    bias = (torch.randn(N, generator=g) * 0.01).half()
    smooth = (x.float().abs().amax(dim=0).sqrt().clamp(min=1e-5) * 3).half()
    for sm in (smooth, smooth.float()):     # fp16 module buffers, fp32 quantizer buffers
        q_ref, s_ref, _ = O.quant_act_pertoken_i8(x, sm.reshape(1, -1))
        q, s = K().quant_act_i8_pertoken(x.to(dev), sm.to(dev))
        assert torch.equal(q.cpu(), q_ref)
        assert torch.equal(s.cpu(), s_ref.float().reshape(-1))
    # the epilogue takes the per-token scale as the module stores it (x's dtype)
    y = K().gemm_i8_dq(q, w8.to(dev), s, w_scale.to(dev), bias.to(dev), out_dtype=torch.float16,
                       exact_ref=True)
    mi, ni = _sample(M_TOK, 64, 3), _sample(N, 64, 4)
    acc = O.int_gemm(q_ref[mi], w8[ni])
    ref = O.epilogue_ref(acc, s_ref.reshape(-1, 1)[mi], w_scale[ni], bias[ni], torch.float16)
    got = y[mi.to(dev)][:, ni.to(dev)].cpu()
    assert torch.equal(got.view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("name,Kd,N", LLAMA)
@pytest.mark.parametrize("M", [1, 2, 4, 16])
def test_decode_shapes_full_size_equal_exact_product(dev, name, Kd, N, M):
    """Config 3, int8: the skinny-M kernels against the exact integer product (the CPU computes
    it for all N at these small M) and the bf16 epilogue."""
    a = torch.randint(-128, 128, (M, Kd), generator=gen(5), dtype=torch.int8)
    w = _rand_i8_dev((N, Kd), 103, dev)
    s_a = (torch.rand(M, 1, generator=gen(6)) * 0.05 + 1e-3).bfloat16()
    s_w = (torch.rand(N, generator=gen(7)) * 1e-3 + 1e-5).float()
    a_pad = torch.cat([a, torch.zeros(32 - M, Kd, dtype=torch.int8)])   # the oracle's fast path needs M > 16
    acc = O.int_gemm(a_pad, w.cpu())[:M]
    ref = O.epilogue_ref(acc, s_a, s_w, None, torch.bfloat16)
    y = K().gemm_i8_dq(a.to(dev), w, s_a.float().to(dev), s_w.to(dev), None, out_dtype=torch.bfloat16,
                       exact_ref=True)
    assert torch.equal(y.cpu().view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("name,Kd,N", LLAMA)
@pytest.mark.parametrize("M", [1, 2, 4, 16])
def test_decode_shapes_full_size_fp8(dev, name, Kd, N, M):
    """Config 3, fp8: e4m3 operands with small-integer values make every product and partial sum
    exact in fp32, so any summation order must give the same result; random operands are held
    to the stated rtol / atol of 1e-2 against the float64 product."""
    g = gen(8)
    ai = torch.randint(-3, 4, (M, Kd), generator=g).float()
    wi = torch.randint(-3, 4, (N, Kd), generator=g).float()
    a8, w8 = ai.to(torch.float8_e4m3fn), wi.to(torch.float8_e4m3fn)
    one_a, one_w = torch.ones(M), torch.ones(N)
    y = K().gemm_fp8_dq(a8.to(dev), w8.to(dev), one_a.to(dev), one_w.to(dev), None, out_dtype=torch.float32)
    assert torch.equal(y.cpu(), ai @ wi.t())
    ar = (torch.randn(M, Kd, generator=g)).to(torch.float8_e4m3fn)
    wr = (torch.randn(N, Kd, generator=g) * 0.5).to(torch.float8_e4m3fn)
    s_a = torch.rand(M, generator=g) * 0.02 + 1e-3
    s_w = torch.rand(N, generator=g) * 0.02 + 1e-3
    y = K().gemm_fp8_dq(ar.to(dev), wr.to(dev), s_a.to(dev), s_w.to(dev), None, out_dtype=torch.bfloat16)
    ref = (ar.double() @ wr.double().t()) * s_a.double()[:, None] * s_w.double()[None, :]
    torch.testing.assert_close(y.cpu().double(), ref, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("name,Kd,N", [("qkv", 4096, 6144), ("o", 4096, 4096), ("gate_up", 4096, 25600),
                                       ("down", 12800, 4096)])
def test_fp8_linear_config_full_size(dev, name, Kd, N):
    """Config 4 (M = 2048, bf16, per-tensor weight scale, dynamic per-token activation scale):
    e4m3 bytes and scales of the quantizer in full; the GEMM on sampled rows / columns against
    the float64 product of the dequantized operands; integer-valued operands exactly."""
    from fms_mo_amd import _lib as L

    M = 2048
    g = gen(3)
    x = torch.randn(M, Kd, generator=g).bfloat16()
    w = 0.02 * torch.randn(N, Kd, generator=g)
    ws = (w.abs().amax() / 448).reshape(1).float()
    w8 = (w / ws).clamp(-448, 448).to(torch.float8_e4m3fn)
    s_ref = O.fp8_dynamic_scale(x)
    q_ref = O.fp8_quant_static(x, s_ref)
    q, s = K().quant_act_fp8_pertoken(x.to(dev), L.FP8_LINEAR)
    assert torch.equal(s.cpu(), s_ref.reshape(-1))
    assert torch.equal(q.cpu().view(torch.uint8), q_ref.view(torch.uint8))
    y = K().gemm_fp8_dq(q, w8.to(dev), s, ws.to(dev), None, out_dtype=torch.bfloat16)
    mi, ni = _sample(M, 64, 9), _sample(N, 64, 10)
    ref = (q_ref[mi].double() @ w8[ni].double().t()) * s_ref.reshape(-1, 1)[mi].double() * ws.double()
    torch.testing.assert_close(y[mi.to(dev)][:, ni.to(dev)].cpu().double(), ref, rtol=1e-2, atol=1e-2)
    # exactness on integer-valued operands, full size, via checksums
    gd = torch.Generator(device=dev).manual_seed(11)
    ai = torch.randint(-2, 3, (M, Kd), generator=gd, device=dev).float()
    wi = torch.randint(-2, 3, (N, Kd), generator=gd, device=dev).float()
    one = torch.ones(1, device=dev)
    yi = K().gemm_fp8_dq(ai.to(torch.float8_e4m3fn), wi.to(torch.float8_e4m3fn), one, one, None,
                         out_dtype=torch.float32)
    assert torch.equal(yi.double().sum(dim=0), ai.double().sum(dim=0) @ wi.double().t())
    assert torch.equal(yi.double().sum(dim=1), ai.double() @ wi.double().sum(dim=0))


def _mixtral_routing(T=4096, E=8, seed=4):
    logits = torch.rand(T, E, generator=gen(seed))
    flat = logits.topk(2, dim=-1).indices.reshape(-1)
    counts = torch.bincount(flat, minlength=E)
    offsets = torch.zeros(E + 1, dtype=torch.int32)
    offsets[1:] = counts.cumsum(0)
    return offsets


@pytest.mark.parametrize("name,Kd,N", [("w1", 4096, 14336), ("w2", 14336, 4096)])
def test_moe_grouped_full_size_equals_per_expert_linear(dev, name, Kd, N):
    """Config 5: 8 experts, 8192 routed rows, uneven split.  The grouped launch must equal the
    tiled GEMM run expert by expert (bit-exact, same epilogue), which in turn is checked against
    the oracle on sampled rows / columns of every expert."""
    E = 8
    offsets = _mixtral_routing()
    T = int(offsets[-1])
    assert T == 8192 and len(set((offsets[1:] - offsets[:-1]).tolist())) > 1
    a = _rand_i8_dev((T, Kd), 104, dev)
    w = _rand_i8_dev((E, N, Kd), 105, dev)
    s_a = (torch.rand(T, generator=gen(12)) * 0.05 + 1e-3).half()
    s_w = (torch.rand(E, N, generator=gen(13)) * 1e-3 + 1e-5).float()
    bias = (torch.randn(E, N, generator=gen(14)) * 0.01).half()
    y = K().grouped_gemm_i8_dq(a, w, offsets.to(dev), s_a.float().to(dev), s_w.to(dev), bias.to(dev),
                               out_dtype=torch.float16, exact_ref=True)
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        ye = K().gemm_i8_dq(a[lo:hi], w[e], s_a[lo:hi].float().to(dev), s_w[e].to(dev), bias[e].to(dev),
                            out_dtype=torch.float16, exact_ref=True)
        assert torch.equal(y[lo:hi].view(torch.int16), ye.view(torch.int16)), e
        mi = torch.unique(torch.cat([_sample(hi - lo, 24, 20 + e), torch.tensor([0, hi - lo - 1])]))
        ni = _sample(N, 32, 40 + e)
        acc = O.int_gemm(a[lo:hi][mi.to(dev)].cpu(), w[e][ni.to(dev)].cpu())
        ref = O.epilogue_ref(acc, s_a[lo:hi][mi].reshape(-1, 1), s_w[e][ni], bias[e][ni], torch.float16)
        got = y[lo:hi][mi.to(dev)][:, ni.to(dev)].cpu()
        assert torch.equal(got.view(torch.int16), ref.view(torch.int16)), e


@pytest.mark.parametrize("t", [7, 16])
def test_chunk_truncate_on_down_projection_full_size(dev, t):
    """Config 5, chunk-truncate emulation on one expert's w2 (K-chunk 64): every chunk partial has
    its low t bits cleared, so the int32 result has them cleared too; sampled rows / columns are
    recomputed by the oracle; t = 0 equals the plain product."""
    M, Kd, N = 1069, 14336, 4096
    a, w = _rand_i8_dev((M, Kd), 106, dev), _rand_i8_dev((N, Kd), 107, dev)
    d = K().matmul_chunk(a, w, None, chunk_size=64, chunk_trun_bits=t)
    assert int((d & ((1 << t) - 1)).abs().max()) == 0
    mi = torch.unique(torch.cat([_sample(M, 24, 60), torch.tensor([0, M - 1])]))
    ni = _sample(N, 32, 61)
    ref = O.chunk_matmul_i8(a[mi.to(dev)].cpu(), w[ni.to(dev)].cpu(), None, chunk_size=64, trun_bits=t)
    assert torch.equal(d[mi.to(dev)][:, ni.to(dev)].cpu(), ref)
    d0 = K().matmul_chunk(a, w, None, chunk_size=64, chunk_trun_bits=0)
    assert torch.equal(d0, K().gemm_i8_i32(a, w))


def test_chunk_truncate_fp_full_size(dev):
    """The fp32-accumulator variant on the same shape: integer-valued fp16 operands keep every
    chunk partial an exact small integer, so rounding away t = 8 mantissa bits is reproducible
    bit for bit by the oracle on sampled rows / columns; low mantissa bits of each chunk are zero."""
    M, Kd, N = 1069, 14336, 4096
    gd = torch.Generator(device=dev).manual_seed(108)
    a = torch.randint(-4, 5, (M, Kd), generator=gd, device=dev).half()
    w = torch.randint(-4, 5, (N, Kd), generator=gd, device=dev).half()
    d = K().matmul_chunk(a, w, None, chunk_size=64, chunk_trun_bits=8)
    mi, ni = _sample(M, 16, 62), _sample(N, 32, 63)
    ref = O.chunk_matmul_fp(a[mi.to(dev)].cpu(), w[ni.to(dev)].cpu(), None, chunk_size=64, trun_bits=8)
    assert torch.equal(d[mi.to(dev)][:, ni.to(dev)].cpu(), ref)
