"""The entry point that allocates nothing (fmsmo_gemm_i8_dq_noalloc: split-K partial sums in the
library's own static device array) against fmsmo_gemm_i8_dq_ws with a caller's workspace, through
the C ABI, bit for bit, on calls in a row that share the array -- the second smaller than the first,
so whatever the first left behind in the array must not leak into it."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _operands(M, N, K, seed, dev, bias_dtype):
    g = torch.Generator().manual_seed(seed)
    a = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8).to(dev)
    w = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8).to(dev)
    a_scale = (torch.rand(M, generator=g) * 1e-2 + 1e-3).to(dev)
    w_scale = (torch.rand(N, generator=g) * 1e-3 + 1e-4).to(dev)
    bias = None if bias_dtype is None else torch.randn(N, generator=g).to(bias_dtype).to(dev)
    return a, w, a_scale, w_scale, bias


def _run(name, ops, M, N, K, epilogue, out_dtype, workspace=None):
    from fms_mo_amd import _lib as L
    from fms_mo_amd.kernels import _DT

    a, w, a_scale, w_scale, bias = ops
    y = torch.full((M, N), float("nan"), dtype=out_dtype, device=a.device)
    args = [a.data_ptr(), K, w.data_ptr(), K, a_scale.data_ptr(), M, w_scale.data_ptr(), N,
            None if bias is None else bias.data_ptr(), 0 if bias is None else _DT[bias.dtype],
            epilogue, y.data_ptr(), _DT[out_dtype], N, M, N, K]
    if workspace is not None:
        args += [workspace.data_ptr(), workspace.numel()]
    L.call(name, *args, torch.cuda.current_stream(a.device).cuda_stream)
    return y


CALLS = [
    # (M, N, K, epilogue, out dtype, bias dtype); splits and scratch bytes in the comments
    (128, 4096, 14336, 0, torch.float16, torch.float16),   # 4 slices on 128 x 64 tiles, 8 MiB
    (17, 4096, 4096, 0, torch.float16, None),              # decode-batch kernel: no scratch used
    (300, 1024, 2048, 1, torch.bfloat16, torch.float32),   # 2 slices of 1024
    (2048, 512, 1024, 1, torch.float32, None),             # no split: no scratch used
    (40, 6144, 4096, 0, torch.float16, torch.bfloat16),    # decode-batch kernel: no scratch used
]


def test_noalloc_entry_point_matches_workspace_entry_point(dev):
    from fms_mo_amd import _lib as L

    lib = L.load()
    assert L.call  # the library is loaded: there is no fallback
    seen_split = 0
    for i, (M, N, K, epi, odt, bdt) in enumerate(CALLS):
        ops = _operands(M, N, K, 100 + i, dev, bdt)
        need = lib.fmsmo_gemm_workspace_bytes(M, N, K)
        assert need <= 16 << 20
        seen_split += need > 0
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device=dev)
        y_ref = _run("fmsmo_gemm_i8_dq_ws", ops, M, N, K, epi, odt, ws)
        y = _run("fmsmo_gemm_i8_dq_noalloc", ops, M, N, K, epi, odt)
        torch.cuda.synchronize()
        assert not torch.isnan(y_ref.float()).any()
        assert torch.equal(y.view(torch.uint8), y_ref.view(torch.uint8)), (M, N, K)
    assert seen_split >= 3


def test_noalloc_entry_point_takes_the_plan_that_fits(dev):
    """512 x 4096 x 14336: the preferred plan (four slices on register-staged tiles) needs 32 MiB of
    partial sums; the static array holds 16 MiB, which two slices on 128 x 128 tiles fit exactly.
    Same bits as with a caller's workspace of either size, and as the single pass."""
    from fms_mo_amd import _lib as L

    lib = L.load()
    M, N, K = 512, 4096, 14336
    need = lib.fmsmo_gemm_workspace_bytes(M, N, K)
    assert need == 32 << 20
    ops = _operands(M, N, K, 300, dev, torch.float16)
    y_big = _run("fmsmo_gemm_i8_dq_ws", ops, M, N, K, 0, torch.float16, torch.empty(need, dtype=torch.uint8, device=dev))
    y_small = _run("fmsmo_gemm_i8_dq_ws", ops, M, N, K, 0, torch.float16,
                   torch.empty(16 << 20, dtype=torch.uint8, device=dev))
    y_none = _run("fmsmo_gemm_i8_dq", ops, M, N, K, 0, torch.float16)
    y = _run("fmsmo_gemm_i8_dq_noalloc", ops, M, N, K, 0, torch.float16)
    torch.cuda.synchronize()
    for other in (y_big, y_small, y_none):
        assert torch.equal(y.view(torch.int16), other.view(torch.int16))
    # 1024 rows: a full round of 128 x 128 tiles, one pass with every entry point
    ops = _operands(1024, N, K, 301, dev, None)
    y_none = _run("fmsmo_gemm_i8_dq", ops, 1024, N, K, 0, torch.float16)
    y = _run("fmsmo_gemm_i8_dq_noalloc", ops, 1024, N, K, 0, torch.float16)
    torch.cuda.synchronize()
    assert torch.equal(y.view(torch.int16), y_none.view(torch.int16))


def test_noalloc_entry_point_allocates_nothing_and_repeats(dev):
    """Two calls in a row, the second smaller, with no device allocation in between (torch's
    allocator statistics do not move and the driver reports the same free memory), and the
    result of each equals the workspace entry point's."""
    shapes = [(128, 4096, 14336), (24, 2048, 4096)]
    prepared = []
    for i, (M, N, K) in enumerate(shapes):
        ops = _operands(M, N, K, 7 + i, dev, torch.float16)
        ws = torch.empty(16 << 20, dtype=torch.uint8, device=dev)
        y_ref = _run("fmsmo_gemm_i8_dq_ws", ops, M, N, K, 0, torch.float16, ws)
        prepared.append((ops, y_ref, torch.empty_like(y_ref)))
    # first call on the device has happened in the test above or happens here: look the array up
    _run("fmsmo_gemm_i8_dq_noalloc", prepared[1][0], *shapes[1], 0, torch.float16)
    torch.cuda.synchronize()
    from fms_mo_amd import _lib as L
    from fms_mo_amd.kernels import _DT

    free0 = torch.cuda.mem_get_info(dev)[0]
    stats0 = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
    st = torch.cuda.current_stream(dev).cuda_stream
    for (ops, _, y), (M, N, K) in zip(prepared, shapes):
        a, w, a_scale, w_scale, bias = ops
        L.call("fmsmo_gemm_i8_dq_noalloc", a.data_ptr(), K, w.data_ptr(), K, a_scale.data_ptr(), M,
               w_scale.data_ptr(), N, bias.data_ptr(), _DT[bias.dtype], 0, y.data_ptr(), L.F16, N,
               M, N, K, st)
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats(dev)["allocation.all.allocated"] == stats0
    # a hidden hipMalloc of the partial sums (2 - 16 MiB) would show here
    assert free0 - torch.cuda.mem_get_info(dev)[0] < (1 << 20)
    for (_, y_ref, y) in prepared:
        assert torch.equal(y.view(torch.int16), y_ref.view(torch.int16))


def test_noalloc_entry_point_random_sequence_of_calls(dev):
    """Twenty-four seeded calls in a row through the shared array, shapes on both sides of every
    routing boundary (decode kernels, K slices of either tile kind, plans that had to shrink to
    fit, single pass): each equals the plain entry point's result bit for bit."""
    import random

    rng = random.Random(24680)
    for case in range(24):
        M = rng.choice([rng.randint(1, 16), rng.randint(17, 128), rng.randint(129, 700), rng.randint(700, 1500)])
        N = rng.choice([8 * rng.randint(1, 64), 128 * rng.randint(1, 48), rng.randint(100, 5000)])
        K = rng.choice([128 * rng.randint(4, 128), 1024 * rng.choice([1, 2, 4, 8, 14]), 64 * rng.randint(1, 64)])
        epi = rng.choice([0, 1])
        odt = torch.float16 if epi == 0 else rng.choice([torch.float16, torch.bfloat16, torch.float32])
        bdt = rng.choice([None, torch.float16, torch.float32])
        ops = _operands(M, N, K, 500 + case, dev, bdt)
        y_ref = _run("fmsmo_gemm_i8_dq", ops, M, N, K, epi, odt)
        y = _run("fmsmo_gemm_i8_dq_noalloc", ops, M, N, K, epi, odt)
        torch.cuda.synchronize()
        assert torch.equal(y.view(torch.uint8), y_ref.view(torch.uint8)), f"case {case}: M={M} N={N} K={K} epi={epi} {odt} bias={bdt}"


def test_noalloc_entry_point_validates_like_the_others(dev):
    from fms_mo_amd import _lib as L

    lib = L.load()
    x = torch.zeros(4096, dtype=torch.int8, device=dev)
    p = x.data_ptr()
    assert lib.fmsmo_gemm_i8_dq_noalloc(None, 64, p, 64, p, 1, p, 1, None, 0, 0, p, 0, 64, 1, 1, 64, None) == 1
    assert lib.fmsmo_gemm_i8_dq_noalloc(p, 32, p, 64, p, 1, p, 1, None, 0, 0, p, 0, 64, 1, 1, 64, None) == 2
    assert lib.fmsmo_status_str(6).startswith(b"shape needs more scratch")
