"""The C-ABI library: it loads, exports every symbol the header declares, validates arguments
(no compute is launched here -- every call below is rejected before any kernel launch)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "fmsmo_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fmsmo_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    syms = declared_symbols()
    for s in ["fmsmo_quant_act_i8_pertoken", "fmsmo_quant_act_i8_static", "fmsmo_quant_act_fp8_pertoken",
              "fmsmo_quant_act_fp8_dynamic",
              "fmsmo_gemm_i8_i32", "fmsmo_gemm_i8_i32_ws", "fmsmo_gemm_i8_dq", "fmsmo_gemm_fp8_dq", "fmsmo_gemv_i8_dq",
              "fmsmo_gemv_fp8_dq", "fmsmo_matmul_chunk_i8", "fmsmo_matmul_chunk_fp",
              "fmsmo_grouped_gemm_i8_dq", "fmsmo_quant_weight_i8", "fmsmo_absmax_cols",
              "fmsmo_quant_act_i8_mulscale", "fmsmo_zero_shift_bias", "fmsmo_quant_i8_affine",
              "fmsmo_bmm_i8_dq", "fmsmo_bmm_fp8_dq", "fmsmo_gemm_i8_dq_ws", "fmsmo_gemm_fp8_dq_ws", "fmsmo_gemm_i8_dq_noalloc",
              "fmsmo_gemm_tail_columns", "fmsmo_quant_act_i8_static_t", "fmsmo_quant_act_i8_dynamic", "fmsmo_fake_quant_fp8",
              "fmsmo_gemm_workspace_bytes", "fmsmo_decode_linear_i8", "fmsmo_decode_linear_fp8", "fmsmo_decode_linear_ok", "fmsmo_decode_linear_f32s_ok", "fmsmo_debug_clock_probe", "fmsmo_debug_stream_read", "fmsmo_debug_mfma_loop", "fmsmo_matmul_chunk_i8_dq", "fmsmo_matmul_chunk_fp_dq", "fmsmo_gemm_plan", "fmsmo_abi_version", "fmsmo_status_str", "fmsmo_last_error"]:
        assert s in syms


def test_library_exports_every_declared_symbol():
    from fms_mo_amd import _lib

    lib = _lib.load()
    for s in declared_symbols():
        assert hasattr(lib, s), f"{s} declared in include/fmsmo_hip.h but not exported"
    assert set(_lib.SIGNATURES) | set(_lib.OTHER) == set(declared_symbols())
    assert lib.fmsmo_abi_version() == 2
    assert lib.fmsmo_status_str(0) == b"ok"


def test_every_declaration_cites_the_reference():
    text = open(HEADER).read()
    for name in ["fms_mo/modules/linear.py:1085-1100", "cutlass_i8i32gemm.cu:100-120",
                 "ext_kernel_cublas.cpp:103-195", "triton_kernels.py:211-302", "fp8_linear.py:275-283"]:
        assert name in text


def test_argument_validation_without_a_gpu():
    from fms_mo_amd import _lib

    lib = _lib.load()
    buf = (ctypes.c_char * 4096)()
    p = ctypes.addressof(buf)
    p = (p + 15) // 16 * 16
    # NULL pointers
    assert lib.fmsmo_gemm_i8_i32(None, 64, p, 64, p, 64, 1, 1, 64, None) == 1
    assert lib.fmsmo_quant_act_i8_pertoken(None, 0, 64, None, 0, 0, 0, p, 64, p, 1, 64, None) == 1
    # bad shapes: leading dimension smaller than K, negative M
    assert lib.fmsmo_gemm_i8_i32(p, 32, p, 64, p, 64, 1, 1, 64, None) == 2
    assert lib.fmsmo_gemm_i8_i32(p, 64, p, 64, p, 64, -1, 1, 64, None) == 2
    # alignment: K not a multiple of 16, misaligned pointer
    assert lib.fmsmo_gemm_i8_i32(p, 24, p, 24, p, 64, 1, 1, 24, None) == 3
    assert lib.fmsmo_gemm_i8_i32(p + 1, 64, p, 64, p, 64, 1, 1, 64, None) == 3
    # unsupported enum values
    assert lib.fmsmo_quant_act_i8_pertoken(p, 7, 64, None, 0, 0, 0, p, 64, p, 1, 64, None) == 4
    assert lib.fmsmo_gemv_i8_dq(p, 128, p, 128, p, 1, p, 1, None, 0, 0, p, 0, 64, 17, 64, 128, None) == 4  # M > 16
    assert lib.fmsmo_matmul_chunk_i8(p, 64, p, 64, None, p, 64, 1, 1, 64, 48, 0, 32, 1, None) == 4  # chunk not 2^n
    assert lib.fmsmo_matmul_chunk_fp(p, 64, p, 64, 1, None, p, 64, 1, 1, 64, 64, 23, 0, 1, None) == 4  # t > 22
    # empty problems are accepted without a launch
    assert lib.fmsmo_gemm_i8_i32(p, 64, p, 64, p, 64, 0, 1, 64, None) == 0
    # the later entry points validate the same way
    assert lib.fmsmo_debug_stream_read(None, 64, p, None) == 1
    assert lib.fmsmo_debug_stream_read(p, 24, p, None) == 2 and lib.fmsmo_debug_stream_read(p, 0, p, None) == 2
    assert lib.fmsmo_debug_stream_read(p + 1, 64, p, None) == 3
    assert lib.fmsmo_debug_mfma_loop(0, None, 64, 1, None, p, None) == 1
    assert lib.fmsmo_debug_mfma_loop(0, p, 64, 0, None, p, None) == 2 and lib.fmsmo_debug_mfma_loop(2, p, 64, 1, None, p, None) == 4
    # the fused chunked matmuls validate like the plain ones, plus their epilogue arguments
    assert lib.fmsmo_matmul_chunk_i8_dq(p, 64, p, 64, None, 1, p, 1, None, 0, 3, p, 0, 64, 1, 1, 64, 64, 0, 32, 1, None) == 1
    assert lib.fmsmo_matmul_chunk_i8_dq(p, 64, p, 64, p, 1, p, 1, None, 0, 7, p, 0, 64, 1, 1, 64, 64, 0, 32, 1, None) == 4  # epilogue
    assert lib.fmsmo_matmul_chunk_i8_dq(p, 64, p, 64, p, 3, p, 1, None, 0, 3, p, 0, 64, 1, 1, 64, 64, 0, 32, 1, None) == 2  # a_scale_n
    assert lib.fmsmo_matmul_chunk_fp_dq(p, 64, p, 64, 0, p, 1, p, 1, None, 0, 3, p, 0, 64, 1, 1, 64, 64, 0, 0, 1, None) == 4  # op dtype
    assert lib.fmsmo_matmul_chunk_fp_dq(p, 64, p, 64, 2, p, 1, p, 1, None, 0, 3, p, 0, 64, 1, 1, 64, 24, 0, 0, 1, None) == 4  # chunk
    assert lib.fmsmo_quant_act_i8_static_t(None, 0, 64, 0, 0, 1.0, 0.0, 0, 0.0, 0.0, p, 64, 1, 64, None) == 1
    assert lib.fmsmo_quant_act_i8_static_t(p, 0, 64, 9, 0, 1.0, 0.0, 0, 0.0, 0.0, p, 64, 1, 64, None) == 4  # mode
    assert lib.fmsmo_quant_act_i8_static_t(p, 0, 32, 0, 0, 1.0, 0.0, 0, 0.0, 0.0, p, 64, 1, 64, None) == 2  # ldx < K
    assert lib.fmsmo_quant_act_i8_dynamic(None, 0, 64, p, 0, 127, 0, p, 64, p, 1, 64, None) == 1
    assert lib.fmsmo_quant_act_i8_dynamic(p, 0, 64, p, 5, 127, 0, p, 64, p, 1, 64, None) == 4  # granularity
    assert lib.fmsmo_fake_quant_fp8(None, 0, 64, 0, None, p, 64, None, 0, None, None, 1, 64, None) == 1
    assert lib.fmsmo_fake_quant_fp8(p, 0, 64, 7, None, p, 64, None, 0, None, None, 1, 64, None) == 4  # mode
    assert lib.fmsmo_gemm_i8_dq_noalloc(None, 64, p, 64, p, 1, p, 1, None, 0, 0, p, 0, 64, 1, 1, 64, None) == 1
    assert lib.fmsmo_gemm_i8_dq_noalloc(p, 64, p, 64, p, 1, p, 1, None, 0, 9, p, 0, 64, 1, 1, 64, None) == 4  # epilogue
    # (the call above is rejected before the static scratch is looked up: no device is touched)
    F32 = 2
    assert lib.fmsmo_quant_act_fp8_dynamic(None, 0, 64, 0, 0, None, 1e-12, F32, p, 64, p, 1, 64, None) == 1
    assert lib.fmsmo_quant_act_fp8_dynamic(p, 0, 64, 0, 1, None, 1e-12, F32, p, 64, p, 1, 64, None) == 1  # no col_amax
    assert lib.fmsmo_quant_act_fp8_dynamic(p, 0, 64, 0, 0, None, 0.0, F32, p, 64, p, 1, 64, None) == 4    # floor <= 0
    assert lib.fmsmo_quant_act_fp8_dynamic(p, 0, 64, 0, 0, None, 1e-12, 0, p, 64, p, 1, 64, None) == 4    # fp16 floor -> 0
    assert lib.fmsmo_quant_act_fp8_dynamic(p, 0, 64, 0, 0, None, 1e-5, 1, p, 64, p, 1, 64, None) == 4     # not x's dtype
    assert lib.fmsmo_quant_act_fp8_dynamic(p, 0, 64, 0, 0, None, 1e-5, 0, p, 64, p, 0, 64, None) == 0     # empty


def test_python_wrapper_raises_on_cpu_tensors():
    import torch

    from fms_mo_amd import kernels

    a = torch.zeros(4, 64, dtype=torch.int8)
    with pytest.raises(RuntimeError, match="no CPU path"):
        kernels.gemm_i8_i32(a, a)
    with pytest.raises(RuntimeError, match="no CPU path"):
        kernels.quant_act_i8_pertoken(torch.zeros(4, 64, dtype=torch.float16))


def test_missing_library_fails_loudly(monkeypatch):
    from fms_mo_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libfmsmo_hip.so")
    with pytest.raises(_lib.FmsMoHipError, match="no fallback"):
        _lib.load()


def test_workspace_plan_is_host_logic():
    """Which shapes split their reduction is decided on the host: decode and large problems do
    not, a batch of tokens through a projection with few output columns does, and the slices
    divide K into multiples of 128 of at least 512."""
    from fms_mo_amd import _lib

    lib = _lib.load()
    assert lib.fmsmo_gemm_workspace_bytes(1, 4096, 14336) == 0
    assert lib.fmsmo_gemm_workspace_bytes(16, 4096, 14336) == 0
    assert lib.fmsmo_gemm_workspace_bytes(4096, 4096, 14336) == 0
    assert lib.fmsmo_gemm_workspace_bytes(64, 28672, 4096) == 0      # 224 tiles already
    assert lib.fmsmo_gemm_workspace_bytes(64, 4096, 4000) == 0       # K not a multiple of 128
    b = lib.fmsmo_gemm_workspace_bytes(64, 4096, 14336)
    assert b > 0 and b % (64 * 4096 * 4) == 0
    s = b // (64 * 4096 * 4)
    assert 2 <= s <= 8 and 14336 % (s * 128) == 0 and 14336 // s >= 512
    # slices of at least 1024 on 128 x 64 tiles, at most 256 blocks
    assert lib.fmsmo_gemm_workspace_bytes(128, 4096, 4096) == 4 * 128 * 4096 * 4    # 64 tiles x 4
    assert lib.fmsmo_gemm_workspace_bytes(128, 1000, 4096) == 4 * 128 * 1000 * 4    # 16 tiles x 4
    assert lib.fmsmo_gemm_workspace_bytes(128, 4096, 2048) == 2 * 128 * 4096 * 4
    # reductions under 2048: 128 x 128 tiles, slices of at least 512
    assert lib.fmsmo_gemm_workspace_bytes(200, 1024, 1536) == 3 * 200 * 1024 * 4


def test_gemm_plan_is_host_logic():
    """Kernel and tile choice per shape, queried without a GPU: decode kernels for skinny M,
    256 x 192 tiles where 256 x 256 would leave the last round of tiles half empty, split
    reductions only with a workspace, the generic kernel when K is not a multiple of 64."""
    from fms_mo_amd import _lib, kernels as K

    if os.environ.get("FMSMO_TILE") or os.environ.get("FMSMO_RS") or os.environ.get("FMSMO_SPLIT_K"):
        pytest.skip("tuning overrides are set")
    RS, DMA = _lib.PLAN_TILE_REGISTER_STAGED, _lib.PLAN_TILE_LDS_DMA
    # the four linears of a Llama-3-8B layer at 4096 tokens
    assert K.gemm_plan(4096, 6144, 4096) == (RS, 256, 192, 1)     # 512 tiles = 2 full rounds
    assert K.gemm_plan(4096, 4096, 4096) == (RS, 256, 256, 1)     # 256 tiles = 1 round
    assert K.gemm_plan(4096, 28672, 4096) == (RS, 256, 256, 1)    # 1792 tiles = 7 rounds
    assert K.gemm_plan(4096, 4096, 14336) == (RS, 256, 256, 1)
    # Granite-3-8B linears with 4096 output columns at 2048 tokens: 256 x 256 tiles would fill half
    # the compute units, 256 x 128 tiles of the same pipeline fill them all
    assert K.gemm_plan(2048, 4096, 4096) == (RS, 256, 128, 1)
    assert K.gemm_plan(2048, 4096, 12800) == (RS, 256, 128, 1)
    assert K.gemm_plan(2048, 6144, 4096) == (RS, 256, 192, 1)
    assert K.gemm_plan(2048, 25600, 4096) == (RS, 256, 256, 1)
    # a nearly empty last round of 256 x 256 tiles is cut off and run as a second GEMM
    tail = _lib.load().fmsmo_gemm_tail_columns
    if not os.environ.get("FMSMO_TAIL_SPLIT"):
        assert tail(2048, 25600, 4096) == 1024 and tail(2048, 25600, 128) == 1024   # 800 tiles
        assert tail(1100, 14080, 128) == 0        # 128 x 256 tiles win here: no 256 x 256 round to cut
        assert tail(4096, 28672, 4096) == 0       # 1792 tiles: full rounds
        assert tail(4096, 8448, 8192) == 0        # one column tile only: too narrow to pay
        assert tail(16, 25600, 4096) == 0         # decode kernel
    # decode and batched decode
    assert K.gemm_plan(1, 4096, 4096)[0] == _lib.PLAN_DECODE
    assert K.gemm_plan(16, 28672, 4096)[0] == _lib.PLAN_DECODE
    assert K.gemm_plan(32, 4096, 8192)[0] == _lib.PLAN_DECODE
    assert K.gemm_plan(64, 4096, 4096)[0] == _lib.PLAN_DECODE
    assert K.gemm_plan(64, 4096, 8192)[0] != _lib.PLAN_DECODE
    assert K.gemm_plan(32, 5120, 5120)[0] == _lib.PLAN_DECODE      # Llama-2-13B hidden size
    assert K.gemm_plan(33, 5120, 5120)[0] != _lib.PLAN_DECODE
    # a few tokens through a long reduction: split only when a workspace is offered
    k, tm, tn, s = K.gemm_plan(17, 4096, 14336, with_workspace=True)
    assert (k, tm, tn) == (DMA, 128, 64) and s >= 2 and 14336 % (s * 128) == 0
    assert K.gemm_plan(17, 4096, 14336, with_workspace=False)[3] == 1
    # a few hundred rows through a long reduction: the slices run on register-staged 256 x 128 tiles
    if not os.environ.get("FMSMO_RS"):
        assert K.gemm_plan(512, 4096, 14336, with_workspace=True) == (RS, 256, 128, 4)
        assert K.gemm_plan(768, 4096, 14336, with_workspace=True) == (RS, 256, 128, 2)
    # a full round of 128 x 128 tiles runs in one pass
    assert K.gemm_plan(1024, 4096, 14336, with_workspace=True) == (DMA, 128, 128, 1)
    assert K.gemm_plan(256, 4096, 14336, with_workspace=True)[:3] == (DMA, 128, 64)
    assert K.gemm_plan(200, 1024, 1536, with_workspace=True) == (DMA, 128, 128, 3)
    # half a round or more of 128 x 64 tiles and a short reduction: one pass of those, no slices
    if not os.environ.get("FMSMO_TALL"):
        for shape in ((512, 4096, 4096), (256, 4096, 4096), (256, 6144, 4096), (1024, 2048, 4096),
                      (512, 4096, 8192), (300, 4096, 2048), (100, 14336, 4096), (48, 13824, 5120)):
            assert K.gemm_plan(*shape, with_workspace=True) == (DMA, 128, 64, 1), shape
            assert _lib.load().fmsmo_gemm_workspace_bytes(*shape) == 0
        # long reductions and half-filled rounds of longer ones keep the slices
        for shape in ((512, 4096, 14336), (256, 4096, 8192), (256, 4096, 5120), (128, 4096, 4096),
                      (256, 1024, 4096)):
            assert K.gemm_plan(*shape, with_workspace=True)[3] >= 2, shape
    # K in 64-byte stages only: no register-staged kernel; K % 64 != 0: generic kernel
    assert K.gemm_plan(4096, 4096, 4160)[0] == DMA
    assert K.gemm_plan(300, 520, 1040) == (_lib.PLAN_GENERIC, 0, 0, 1)
    # small problems take small tiles
    assert K.gemm_plan(300, 520, 1024)[1:3] == (128, 128)
    with pytest.raises(_lib.FmsMoHipError):
        K.gemm_plan(0, 4096, 4096)
    with pytest.raises(_lib.FmsMoHipError):
        K.gemm_plan(128, 128, 100)


def test_plan_of_the_entry_point_that_allocates_nothing():
    """with_workspace = 2 describes fmsmo_gemm_i8_dq_noalloc: the split that fits the 16 MiB static
    scratch where the preferred one does not."""
    from fms_mo_amd import _lib

    lib = _lib.load()
    k, tm, tn, sp = (ctypes.c_int() for _ in range(4))
    # 512 x 4096 x 14336: four register-staged slices want 32 MiB; the scratch holds two 128 x 128 ones
    assert lib.fmsmo_gemm_plan(512, 4096, 14336, 1, ctypes.byref(k), ctypes.byref(tm), ctypes.byref(tn), ctypes.byref(sp)) == 0
    pref = (k.value, tm.value, tn.value, sp.value)
    assert lib.fmsmo_gemm_plan(512, 4096, 14336, 2, ctypes.byref(k), ctypes.byref(tm), ctypes.byref(tn), ctypes.byref(sp)) == 0
    fit = (k.value, tm.value, tn.value, sp.value)
    assert pref[3] * 512 * 4096 * 4 > 16 * 2 ** 20 >= fit[3] * 512 * 4096 * 4 and fit[3] >= 2
    assert fit != pref and fit[0] == _lib.PLAN_TILE_LDS_DMA
    # a shape that needs no scratch reads the same in every mode
    for mode in (0, 1, 2):
        assert lib.fmsmo_gemm_plan(4, 4096, 4096, mode, ctypes.byref(k), ctypes.byref(tm), ctypes.byref(tn), ctypes.byref(sp)) == 0
        assert k.value == _lib.PLAN_DECODE
