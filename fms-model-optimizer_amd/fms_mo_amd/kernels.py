"""Tensor-level wrappers over the C-ABI kernels: argument checks, output allocation through
torch's caching allocator, the current HIP stream of the tensors' device.  No arithmetic happens
here; torch is only the owner of device memory and streams."""
from __future__ import annotations

import torch

from . import _lib as L

_DT = {torch.float16: L.F16, torch.bfloat16: L.BF16, torch.float32: L.F32}
_OPDT = {torch.int8: L.OP_I8, torch.float8_e4m3fn: L.OP_E4M3, torch.float16: L.OP_F16,
         torch.bfloat16: L.OP_BF16, torch.float32: L.OP_F32}
_BITS = {1: torch.uint8, 2: torch.int16, 4: torch.int32}


def _need_gpu(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "fms_mo_amd kernels run on an AMD GPU only (tensor is on %s); there is no CPU path"
                % t.device
            )


_RAW_STREAM = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_CUR_DEVICE = getattr(torch._C, "_cuda_getDevice", None)


def _stream(t: torch.Tensor):
    """The current HIP stream of the tensor's device, as the integer handle the C ABI takes."""
    if _RAW_STREAM is not None:
        return _RAW_STREAM(t.get_device())
    return torch.cuda.current_stream(t.device).cuda_stream


class _NoSwitch:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _dev(t: torch.Tensor):
    """Context that makes the tensor's GPU current for a launch; nothing to do (and nothing paid:
    entering torch.cuda.device costs about a microsecond each way) when it already is."""
    idx = t.get_device()
    if _CUR_DEVICE is not None and _CUR_DEVICE() == idx:
        return _NO_SWITCH
    return torch.cuda.device(idx)


def _eager(*ts) -> bool:
    """True when the call can go straight to the implementation: plain tensors outside a compiler
    trace.  Otherwise the registered ``torch.ops.fms_mo_amd`` operator is called, whose shape-only
    twin serves tracing (going through the dispatcher costs about 3 us per call)."""
    if torch.compiler.is_compiling():
        return False
    for t in ts:
        if t is not None and type(t) is not torch.Tensor and type(t) is not torch.nn.Parameter:
            return False
    return True


def _ptr(t):
    return None if t is None else t.data_ptr()


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported floating dtype {t.dtype}") from None


def _rows(t: torch.Tensor) -> torch.Tensor:
    """2-D, unit inner stride (row stride may be larger than the row)."""
    if t.dim() != 2:
        raise ValueError("expected a 2-D tensor")
    if t.stride(1) != 1 or (t.shape[0] > 1 and t.stride(0) < t.shape[1]):
        t = t.contiguous()
    return t


def _ld(t: torch.Tensor) -> int:
    return t.stride(0) if t.shape[0] > 1 else max(t.shape[1], t.stride(0))


def _scale_vec(s, n, device, name):
    if (type(s) is torch.Tensor and s.dtype is torch.float32 and s.dim() == 1 and s.is_cuda
            and s.is_contiguous() and not s.requires_grad and s.get_device() == device.index
            and s.numel() in (1, n)):
        return s  # the usual case: already the vector the kernels take
    if not torch.is_tensor(s):
        s = torch.tensor([float(s)], dtype=torch.float32, device=device)
    s = s.detach().to(device=device, dtype=torch.float32).reshape(-1).contiguous()
    if s.numel() not in (1, n):
        raise ValueError(f"{name} must have 1 or {n} elements, got {s.numel()}")
    return s


# ------------------------------------------------------------------------------- quantizers
def quant_act_i8_pertoken(x, smooth=None, compute_dtype=None, saturate=False):
    """(q int8 [M,K], scale fp32 [M]) -- see fmsmo_quant_act_i8_pertoken."""
    _need_gpu(x, smooth)
    x = _rows(x)
    M, K = x.shape
    if smooth is not None:
        smooth = smooth.detach().reshape(-1).contiguous()
        if smooth.numel() != K:
            raise ValueError("smooth scale must have K elements")
        if smooth.data_ptr() % 16:
            smooth = smooth.clone()
    if compute_dtype is None:
        compute_dtype = x.dtype if smooth is None else torch.promote_types(x.dtype, smooth.dtype)
    q = torch.empty((M, K), dtype=torch.int8, device=x.device)
    scale = torch.empty((M,), dtype=torch.float32, device=x.device)
    with _dev(x):
        L.call("fmsmo_quant_act_i8_pertoken", x.data_ptr(), _dt(x), _ld(x), _ptr(smooth),
               _dt(smooth) if smooth is not None else 0, _DT[compute_dtype], int(bool(saturate)),
               q.data_ptr(), K, scale.data_ptr(), M, K, _stream(x))
    return q, scale


def quant_act_i8_static(x, scale: float, zp: int, sym: int):
    _need_gpu(x)
    x = _rows(x)
    M, K = x.shape
    q = torch.empty((M, K), dtype=torch.int8, device=x.device)
    with _dev(x):
        L.call("fmsmo_quant_act_i8_static", x.data_ptr(), _dt(x), _ld(x), float(scale), int(zp),
               int(sym), q.data_ptr(), K, M, K, _stream(x))
    return q


def quant_act_i8_mulscale(x, mode, clip=None, smooth=None, meta_dtype=None):
    """(q int8 [M,K], a_scale fp32 [M] or [2]) -- see fmsmo_quant_act_i8_mulscale.  clip: device
    tensor {a_clip_val, a_clip_valn}; smooth: device tensor [K]; both of one dtype.  meta_dtype:
    dtype of the metadata vector when neither is passed (it still decides the compute dtype)."""
    _need_gpu(x, clip, smooth)
    x = _rows(x)
    M, K = x.shape
    meta = smooth if smooth is not None else clip
    if clip is not None and smooth is not None and clip.dtype != smooth.dtype:
        raise TypeError("clip and smooth must share one dtype")
    if mode != L.MS_PER_TOKEN:
        if clip is None or clip.numel() != 2:
            raise ValueError("clip must hold {a_clip_val, a_clip_valn}")
        clip = clip.detach().reshape(-1).contiguous()
    if smooth is not None:
        smooth = smooth.detach().reshape(-1).contiguous()
        if smooth.numel() != K:
            raise ValueError("smooth scale must have K elements")
        if smooth.data_ptr() % 16:
            smooth = smooth.clone()
    if meta is not None:
        meta_dtype = meta.dtype
    compute_dtype = x.dtype if meta_dtype is None else torch.promote_types(x.dtype, meta_dtype)
    q = torch.empty((M, K), dtype=torch.int8, device=x.device)
    a_scale = torch.empty((M if mode == L.MS_PER_TOKEN else 2,), dtype=torch.float32,
                          device=x.device)
    with _dev(x):
        L.call("fmsmo_quant_act_i8_mulscale", x.data_ptr(), _dt(x), _ld(x), _ptr(smooth),
               _ptr(clip), _DT[meta_dtype] if meta_dtype is not None else _dt(x), _DT[compute_dtype],
               int(mode), q.data_ptr(), K, a_scale.data_ptr(), M, K, _stream(x))
    return q, a_scale


def quant_act_fp8_pertoken(x, variant=L.FP8_LINEAR, static_scale=None):
    """(q e4m3 [M,K], scale fp32 [M] or the [1] static scale)."""
    _need_gpu(x)
    x = _rows(x)
    M, K = x.shape
    q = torch.empty((M, K), dtype=torch.float8_e4m3fn, device=x.device)
    if static_scale is not None:
        scale = _scale_vec(static_scale, 1, x.device, "static_scale")[:1].contiguous()
    else:
        scale = torch.empty((M,), dtype=torch.float32, device=x.device)
    with _dev(x):
        L.call("fmsmo_quant_act_fp8_pertoken", x.data_ptr(), _dt(x), _ld(x), int(variant),
               int(static_scale is not None), q.data_ptr(), K, scale.data_ptr(), M, K, _stream(x))
    return q, scale


def quant_act_fp8_dynamic(x, variant=L.FP8_LINEAR, per_tensor=False, scale_floor=1e-12,
                          scale_in_x_dtype=False):
    """(q e4m3 [M,K], scale fp32 [M] or [1]): the e4m3 quantizer with a dynamic scale
    max(amax / 448, scale_floor) per token or for the whole tensor, the division in fp32 or in
    x's dtype (see fmsmo_quant_act_fp8_dynamic).  Per tensor it is two passes over x (column
    abs-max, quantizer) with nothing read back to the host."""
    _need_gpu(x)
    if x.dim() != 2:
        raise ValueError("expected a 2-D tensor")
    x = _rows(x)
    M, K = x.shape
    q = torch.empty((M, K), dtype=torch.float8_e4m3fn, device=x.device)
    scale = torch.empty((1 if per_tensor else M,), dtype=torch.float32, device=x.device)
    col_amax = absmax_cols(x) if per_tensor else None
    with _dev(x):
        L.call("fmsmo_quant_act_fp8_dynamic", x.data_ptr(), _dt(x), _ld(x), int(variant),
               int(bool(per_tensor)), _ptr(col_amax), float(scale_floor),
               _dt(x) if scale_in_x_dtype else L.F32, q.data_ptr(), K, scale.data_ptr(), M, K,
               _stream(x))
    return q, scale


def quant_act_i8_static_t(x, mode, compute_dtype, scale, zp, sym=0, clip_lo=0.0, clip_hi=0.0):
    """int8 [M,K]: the static per-tensor formulas evaluated in ``compute_dtype`` (see
    fmsmo_quant_act_i8_static_t; mode is one of L.SQ_*).  All parameters are host numbers."""
    _need_gpu(x)
    x = _rows(x)
    M, K = x.shape
    q = torch.empty((M, K), dtype=torch.int8, device=x.device)
    with _dev(x):
        L.call("fmsmo_quant_act_i8_static_t", x.data_ptr(), _dt(x), _ld(x), int(mode),
               _DT[compute_dtype], float(scale), float(zp), int(sym), float(clip_lo), float(clip_hi),
               q.data_ptr(), K, M, K, _stream(x))
    return q


def quant_act_i8_dynamic(x, per_column, levels, zp=0, want_amax=False):
    """(q int8 [M,K], scale fp32 [1] or [K]): dynamic symmetric quantizer with one scale for the
    whole tensor or one per column, abs-max / levels in x's dtype, codes shifted by zp (see
    fmsmo_quant_act_i8_dynamic).  Two passes over x: the column abs-max, then the quantizer; nothing
    is read back to the host.  want_amax: also return the fp32 [K] column abs-max."""
    _need_gpu(x)
    x = _rows(x)
    M, K = x.shape
    col_amax = absmax_cols(x)
    q = torch.empty((M, K), dtype=torch.int8, device=x.device)
    scale = torch.empty((K if per_column else 1,), dtype=torch.float32, device=x.device)
    with _dev(x):
        L.call("fmsmo_quant_act_i8_dynamic", x.data_ptr(), _dt(x), _ld(x), col_amax.data_ptr(),
               L.DQ_PER_COLUMN if per_column else L.DQ_PER_TENSOR, int(levels), int(zp),
               q.data_ptr(), K, scale.data_ptr(), M, K, _stream(x))
    return (q, scale, col_amax) if want_amax else (q, scale)


def fake_quant_fp8(x, mode, want_values=True, want_codes=False):
    """FP8 (e4m3) emulation quantizer of QLinear on x [M,K] (see fmsmo_fake_quant_fp8; mode is one of
    L.F8E_*).  Returns (y, q, scale, inv_scale): y the fake-quantized tensor in x's dtype (None
    unless want_values), q the e4m3 codes (None unless want_codes), scale / inv_scale fp32 [1] or
    [M] (None for the saturating cast)."""
    _need_gpu(x)
    x = _rows(x)
    M, K = x.shape
    y = torch.empty((M, K), dtype=x.dtype, device=x.device) if want_values else None
    q = torch.empty((M, K), dtype=torch.float8_e4m3fn, device=x.device) if want_codes else None
    n = {L.F8E_SAT: 0, L.F8E_PER_TENSOR: 1, L.F8E_PER_ROW: M}[mode]
    scale = torch.empty((n,), dtype=torch.float32, device=x.device) if n else None
    inv = torch.empty((n,), dtype=torch.float32, device=x.device) if n else None
    col_amax = absmax_cols(x) if mode == L.F8E_PER_TENSOR else None
    with _dev(x):
        L.call("fmsmo_fake_quant_fp8", x.data_ptr(), _dt(x), _ld(x), int(mode), _ptr(col_amax),
               _ptr(y), K, _ptr(q), K, _ptr(scale), _ptr(inv), M, K, _stream(x))
    return y, q, scale, inv


# ------------------------------------------------------------------------------------ GEMMs
_WS_BYTES: dict = {}


def _workspace(M, N, K, device):
    """Scratch for the split-K form of the *_dq GEMMs (None when the shape does not use one).  It
    comes from torch's caching allocator like every output, so it is also valid under graph
    capture; the library itself never allocates."""
    key = (M, N, K)
    nbytes = _WS_BYTES.get(key)
    if nbytes is None:  # the policy is fixed for the life of the process: ask the library once per shape
        nbytes = _WS_BYTES[key] = L.load().fmsmo_gemm_workspace_bytes(M, N, K)
    return torch.empty((nbytes,), dtype=torch.uint8, device=device) if nbytes > 0 else None


def gemm_plan(M, N, K, with_workspace=False):
    """(kernel, tile_m, tile_n, splits) the *_dq GEMMs use for a shape; no GPU needed
    (kernel is one of L.PLAN_*; see fmsmo_gemm_plan)."""
    import ctypes

    out = [ctypes.c_int(0) for _ in range(4)]
    L.call("fmsmo_gemm_plan", M, N, K, int(bool(with_workspace)), *[ctypes.byref(o) for o in out])
    return tuple(o.value for o in out)


def clock_probe(buf):
    """Diagnostic: have block 0 of the following 256-row-tile GEMM launches store its clock
    readings into `buf` (int64 [6] on the GPU), or switch the probe off with None.  See
    fmsmo_debug_clock_probe; `core_clock_mhz` turns a filled buffer into a frequency."""
    if buf is None:
        L.call("fmsmo_debug_clock_probe", None)
        return
    _need_gpu(buf)
    if buf.dtype != torch.int64 or buf.numel() < 6 or not buf.is_contiguous():
        raise ValueError("the probe buffer must be a contiguous int64 tensor of 6 elements")
    L.call("fmsmo_debug_clock_probe", buf.data_ptr())


def stream_read(t, sink):
    """Diagnostic: one launch that only reads the bytes of the contiguous tensor `t` from device
    memory (fmsmo_debug_stream_read); `sink` is an int32 tensor of one element on the same GPU.
    Timed like a decode linear over the same weights it gives the floor the launch and the
    memory system set for that linear."""
    _need_gpu(t)
    _need_gpu(sink)
    if not t.is_contiguous() or sink.dtype != torch.int32 or sink.numel() < 1:
        raise ValueError("stream_read wants a contiguous tensor and an int32 sink")
    L.call("fmsmo_debug_stream_read", t.data_ptr(), t.numel() * t.element_size(), sink.data_ptr(), _stream(t))


def mfma_loop(data, iters, clk=None):
    """Diagnostic: the GEMM kernels' matrix instructions alone, fed from registers loaded once from
    `data` (int8 or float8_e4m3fn, contiguous; see fmsmo_debug_mfma_loop).  Returns the operations
    of one launch; `clk` (int64 [2] on the GPU) receives block 0's {core cycles, 100 MHz ticks}."""
    _need_gpu(data, clk)
    if data.dtype not in (torch.int8, torch.float8_e4m3fn) or not data.is_contiguous() or data.numel() % 4:
        raise ValueError("data must be a contiguous int8 / float8_e4m3fn tensor of a multiple of 4 elements")
    sink = torch.zeros(1, dtype=torch.float32, device=data.device)
    with _dev(data):
        L.call("fmsmo_debug_mfma_loop", _OPDT[data.dtype], data.data_ptr(), data.numel(), int(iters), _ptr(clk),
               sink.data_ptr(), _stream(data))
    return 1024.0 * iters * 2 * 16 * 2 * 32 * 32 * 64


def core_clock_mhz(buf):
    """Average core clock (MHz) over the life of the probed block: core cycles per tick of the
    constant 100 MHz counter, start of the block to the end of its epilogue."""
    c = buf.cpu().tolist()
    return (c[4] - c[0]) / ((c[5] - c[1]) / 100.0)


def _check_ab(a, w, dtype):
    _need_gpu(a, w)
    if a.dtype != dtype or w.dtype != dtype:
        raise TypeError(f"operands must be {dtype}, got {a.dtype} and {w.dtype}")
    a, w = _rows(a), _rows(w)
    if a.shape[1] != w.shape[1]:
        raise ValueError(f"K mismatch: a is {tuple(a.shape)}, w is {tuple(w.shape)} ([N,K] layout)")
    return a, w


def gemm_i8_i32(a, w):
    """int32 [M,N] = a int8 [M,K] . w int8 [N,K]^T."""
    a, w = _check_ab(a, w, torch.int8)
    M, K = a.shape
    N = w.shape[0]
    c = torch.empty((M, N), dtype=torch.int32, device=a.device)
    ws = _workspace(M, N, K, a.device)
    with _dev(a):
        if ws is not None:
            L.call("fmsmo_gemm_i8_i32_ws", a.data_ptr(), _ld(a), w.data_ptr(), _ld(w), c.data_ptr(), N,
                   M, N, K, ws.data_ptr(), ws.numel(), _stream(a))
        else:
            L.call("fmsmo_gemm_i8_i32", a.data_ptr(), _ld(a), w.data_ptr(), _ld(w), c.data_ptr(), N,
                   M, N, K, _stream(a))
    return c


def gemm_i8_dq(a, w, a_scale, w_scale, bias=None, out_dtype=torch.float16, epilogue=L.EPI_REF_F16,
               force_gemv=False):
    a, w = _check_ab(a, w, torch.int8)
    M, K = a.shape
    N = w.shape[0]
    a_scale = _scale_vec(a_scale, M, a.device, "a_scale")
    w_scale = _scale_vec(w_scale, N, a.device, "w_scale")
    if bias is not None:
        _need_gpu(bias)
        bias = bias.detach().reshape(-1).contiguous()
        if bias.numel() != N:
            raise ValueError("bias must have N elements")
    y = torch.empty((M, N), dtype=out_dtype, device=a.device)
    args = (a.data_ptr(), _ld(a), w.data_ptr(), _ld(w), a_scale.data_ptr(),
            a_scale.numel(), w_scale.data_ptr(), w_scale.numel(), _ptr(bias),
            _dt(bias) if bias is not None else 0, int(epilogue),
            y.data_ptr(), _DT[out_dtype], N, M, N, K)
    ws = None if force_gemv else _workspace(M, N, K, a.device)
    with _dev(a):
        if ws is not None:
            L.call("fmsmo_gemm_i8_dq_ws", *args, ws.data_ptr(), ws.numel(), _stream(a))
        else:
            L.call("fmsmo_gemv_i8_dq" if force_gemv else "fmsmo_gemm_i8_dq", *args, _stream(a))
    return y


def gemm_fp8_dq(a, w, a_scale, w_scale, bias=None, out_dtype=torch.bfloat16, force_gemv=False):
    a, w = _check_ab(a, w, torch.float8_e4m3fn)
    M, K = a.shape
    N = w.shape[0]
    a_scale = _scale_vec(a_scale, M, a.device, "a_scale")
    w_scale = _scale_vec(w_scale, N, a.device, "w_scale")
    if bias is not None:
        _need_gpu(bias)
        bias = bias.detach().reshape(-1).contiguous()
        if bias.numel() != N:
            raise ValueError("bias must have N elements")
    y = torch.empty((M, N), dtype=out_dtype, device=a.device)
    args = (a.data_ptr(), _ld(a), w.data_ptr(), _ld(w), a_scale.data_ptr(),
            a_scale.numel(), w_scale.data_ptr(), w_scale.numel(), _ptr(bias),
            _dt(bias) if bias is not None else 0, y.data_ptr(), _DT[out_dtype], N, M, N, K)
    ws = None if force_gemv else _workspace(M, N, K, a.device)
    with _dev(a):
        if ws is not None:
            L.call("fmsmo_gemm_fp8_dq_ws", *args, ws.data_ptr(), ws.numel(), _stream(a))
        else:
            L.call("fmsmo_gemv_fp8_dq" if force_gemv else "fmsmo_gemm_fp8_dq", *args, _stream(a))
    return y


def grouped_gemm_i8_dq(a, w, offsets, a_scale, w_scale, bias=None, out_dtype=torch.float16,
                       exact_ref=True):
    """a int8 [T,K] rows sorted by expert, w int8 [E,N,K], offsets int32 [E+1] (device),
    a_scale fp32 [T], w_scale fp32 [E,N], bias [E,N] or None -> [T,N]."""
    _need_gpu(a, w, offsets)
    if a.dtype != torch.int8 or w.dtype != torch.int8 or w.dim() != 3:
        raise TypeError("a must be int8 [T,K], w int8 [E,N,K]")
    a = _rows(a)
    w = w.contiguous()
    T, K = a.shape
    E, N, K2 = w.shape
    if K2 != K or offsets.numel() != E + 1 or offsets.dtype != torch.int32:
        raise ValueError("shape mismatch (w [E,N,K], offsets int32 [E+1])")
    a_scale = _scale_vec(a_scale, T, a.device, "a_scale")
    w_scale = w_scale.detach().to(torch.float32).reshape(-1).contiguous()
    if a_scale.numel() != T or w_scale.numel() != E * N:
        raise ValueError("a_scale must be [T], w_scale [E,N]")
    if bias is not None:
        bias = bias.detach().reshape(-1).contiguous()
        if bias.numel() != E * N:
            raise ValueError("bias must be [E,N]")
    y = torch.empty((T, N), dtype=out_dtype, device=a.device)
    with _dev(a):
        L.call("fmsmo_grouped_gemm_i8_dq", a.data_ptr(), _ld(a), w.data_ptr(), K, N * K,
               offsets.contiguous().data_ptr(), E, T, a_scale.data_ptr(), w_scale.data_ptr(),
               _ptr(bias), _dt(bias) if bias is not None else 0,
               L.EPI_REF_F16 if exact_ref else L.EPI_F32, y.data_ptr(), _DT[out_dtype], N, N, K,
               _stream(a))
    return y


# ----------------------------------------------------------------------- chunked accumulation
def matmul_chunk(a, w, c=None, chunk_size=64, chunk_trun_bits=0, max_acc_bits=32,
                 truncate_then_accumulate=True, clamp_acc_to_dl16=False):
    """a [M,K], w [N,K] (int8 | float8_e4m3fn | float16 | bfloat16 | float32) -> int32 / fp32 [M,N]."""
    _need_gpu(a, w, c)
    if a.dtype != w.dtype or a.dtype not in _OPDT:
        raise TypeError(f"unsupported operand dtypes {a.dtype}, {w.dtype}")
    a, w = _rows(a), _rows(w)
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K:
        raise ValueError("K mismatch")
    esz = a.element_size()
    per16 = 16 // esz
    if K % per16 or _ld(a) % per16 or _ld(w) % per16:  # zero-pad K: contributes nothing to any chunk
        Kp = (K + 63) // 64 * 64
        a = torch.nn.functional.pad(a.view(_BITS[esz]), (0, Kp - K)).view(a.dtype)
        w = torch.nn.functional.pad(w.view(_BITS[esz]), (0, Kp - K)).view(w.dtype)
        K = Kp
    acc_dtype = torch.int32 if a.dtype == torch.int8 else torch.float32
    d = torch.empty((M, N), dtype=acc_dtype, device=a.device)
    if c is not None:
        if c.shape != (M, N):
            raise ValueError("C shape is inconsistent with A B.")
        c = c.to(acc_dtype).contiguous()
    with _dev(a):
        if a.dtype == torch.int8:
            L.call("fmsmo_matmul_chunk_i8", a.data_ptr(), _ld(a), w.data_ptr(), _ld(w), _ptr(c),
                   d.data_ptr(), N, M, N, K, int(chunk_size), int(chunk_trun_bits),
                   int(max_acc_bits), int(bool(truncate_then_accumulate)), _stream(a))
        else:
            L.call("fmsmo_matmul_chunk_fp", a.data_ptr(), _ld(a), w.data_ptr(), _ld(w),
                   _OPDT[a.dtype], _ptr(c), d.data_ptr(), N, M, N, K, int(chunk_size),
                   int(chunk_trun_bits), int(bool(clamp_acc_to_dl16)),
                   int(bool(truncate_then_accumulate)), _stream(a))
    return d


def matmul_chunk_dq(a, w, a_scale, w_scale, bias=None, epilogue=L.EPI_SEQ_OUT, out_dtype=torch.float16,
                    chunk_size=64, chunk_trun_bits=0, max_acc_bits=32, truncate_then_accumulate=True,
                    clamp_acc_to_dl16=False):
    """y [M,N] = epilogue(chunked accumulator of a [M,K] . w [N,K]^T): the chunk-truncate matmul and
    its dequantization in one launch (see fmsmo_matmul_chunk_i8_dq / _fp_dq).  a_scale fp32 [M] or
    [1], w_scale fp32 [N] or [1], bias [N] (fp16 / bf16 / fp32) or None, epilogue one of L.EPI_*."""
    _need_gpu(a, w, a_scale, w_scale, bias)
    if a.dtype != w.dtype or a.dtype not in _OPDT:
        raise TypeError(f"unsupported operand dtypes {a.dtype}, {w.dtype}")
    a, w = _rows(a), _rows(w)
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K:
        raise ValueError("K mismatch")
    esz = a.element_size()
    per16 = 16 // esz
    if K % per16 or _ld(a) % per16 or _ld(w) % per16:  # zero-pad K: contributes nothing to any chunk
        Kp = (K + 63) // 64 * 64
        a = torch.nn.functional.pad(a.view(_BITS[esz]), (0, Kp - K)).view(a.dtype)
        w = torch.nn.functional.pad(w.view(_BITS[esz]), (0, Kp - K)).view(w.dtype)
        K = Kp
    a_scale = _scale_vec(a_scale, M, a.device, "a_scale")
    w_scale = _scale_vec(w_scale, N, a.device, "w_scale")
    if bias is not None:
        if bias.numel() != N or bias.dtype not in _DT:
            raise ValueError("bias must hold N fp16 / bf16 / fp32 values")
        bias = bias.reshape(-1).contiguous()
    y = torch.empty((M, N), dtype=out_dtype, device=a.device)
    common = (a_scale.data_ptr(), a_scale.numel(), w_scale.data_ptr(), w_scale.numel(), _ptr(bias),
              _DT[bias.dtype] if bias is not None else L.F32, int(epilogue), y.data_ptr(), _DT[out_dtype],
              N, M, N, K, int(chunk_size), int(chunk_trun_bits))
    with _dev(a):
        if a.dtype == torch.int8:
            L.call("fmsmo_matmul_chunk_i8_dq", a.data_ptr(), _ld(a), w.data_ptr(), _ld(w), *common,
                   int(max_acc_bits), int(bool(truncate_then_accumulate)), _stream(a))
        else:
            L.call("fmsmo_matmul_chunk_fp_dq", a.data_ptr(), _ld(a), w.data_ptr(), _ld(w), _OPDT[a.dtype],
                   *common, int(bool(clamp_acc_to_dl16)), int(bool(truncate_then_accumulate)), _stream(a))
    return y


def quant_weight_i8(w, coef, smooth=None, mode="mul", want_row_sum=False):
    """Offline weight quantizer (see fmsmo_quant_weight_i8): w [N,K] fp16/bf16/fp32, coef [N] or [1]
    (``127 / clip_val`` for mode "mul", ``w_scale`` for mode "div"), smooth [K] or None.
    Returns int8 [N,K] (and the int32 row sums [N] when asked)."""
    _need_gpu(w, coef, smooth)
    if w.dim() != 2:
        raise ValueError("w must be [N, K]")
    if w.stride(1) != 1:
        w = w.contiguous()
    N, K = w.shape
    coef = coef.detach().reshape(-1).contiguous()
    if coef.numel() not in (1, N):
        raise ValueError("coef must have 1 or N elements")
    if smooth is not None:
        smooth = smooth.detach().reshape(-1).contiguous()
        if smooth.numel() != K:
            raise ValueError("smooth must have K elements")
        if smooth.data_ptr() % 16:
            smooth = smooth.clone()
    q = torch.empty((N, K), dtype=torch.int8, device=w.device)
    rs = torch.empty((N,), dtype=torch.int32, device=w.device) if want_row_sum else None
    with _dev(w):
        L.call("fmsmo_quant_weight_i8", w.data_ptr(), _dt(w), _ld(w), _ptr(smooth),
               _dt(smooth) if smooth is not None else 0, coef.data_ptr(), _dt(coef), coef.numel(),
               L.WQ_MUL if mode == "mul" else L.WQ_DIV, q.data_ptr(), K, _ptr(rs), N, K, _stream(w))
    return (q, rs) if want_row_sum else q


def absmax_cols(x, running=None):
    """Per-column abs-max of x [*, K] as fp32 [K]; with ``running`` (fp32 [K], >= 0) the result is
    the element-wise maximum of both, updated in place and returned."""
    _need_gpu(x, running)
    x = _rows(x.reshape(-1, x.shape[-1]))
    M, K = x.shape
    if running is None:
        running = torch.zeros((K,), dtype=torch.float32, device=x.device)
    elif running.dtype != torch.float32 or running.numel() != K or not running.is_contiguous():
        raise ValueError("running must be a contiguous fp32 tensor with K elements")
    with _dev(x):
        L.call("fmsmo_absmax_cols", x.data_ptr(), _dt(x), _ld(x), M, K, running.data_ptr(), _stream(x))
    return running


def zero_shift_bias(w, w_scale, a_meta, bias=None, offset=128.0):
    """fp32 [N] bias with the zero-point correction of asymmetric activations folded in
    (see fmsmo_zero_shift_bias).  w int8 [N,K]; w_scale fp32 [N] or [1]; a_meta fp32 [2]."""
    _need_gpu(w, w_scale, a_meta, bias)
    if w.dtype != torch.int8:
        raise TypeError("w must be int8")
    w = _rows(w)
    N, K = w.shape
    w_scale = _scale_vec(w_scale, N, w.device, "w_scale")
    if a_meta.dtype != torch.float32 or a_meta.numel() != 2:
        raise ValueError("a_meta must be fp32 {1/scale, zero point}")
    if bias is not None:
        bias = bias.detach().reshape(-1).contiguous()
        if bias.numel() != N:
            raise ValueError("bias must have N elements")
    out = torch.empty((N,), dtype=torch.float32, device=w.device)
    with _dev(w):
        L.call("fmsmo_zero_shift_bias", w.data_ptr(), _ld(w), w_scale.data_ptr(), w_scale.numel(),
               a_meta.contiguous().data_ptr(), float(offset), _ptr(bias),
               _dt(bias) if bias is not None else 0, out.data_ptr(), N, K, _stream(w))
    return out


# ---------------------------------------------------------------------------- batched matmul
def _batched3(t: torch.Tensor) -> torch.Tensor:
    """[..., R, C] -> [batch, R, C] with unit inner stride and one batch stride (a view when the
    leading dimensions collapse, a copy otherwise)."""
    t3 = t.reshape(-1, t.shape[-2], t.shape[-1])
    if t3.stride(2) != 1 or (t3.shape[1] > 1 and t3.stride(1) < t3.shape[2]):
        t3 = t3.contiguous()
    return t3


def quant_i8_affine(x, scale: float, offset: float, compute_dtype=None, transpose=False, pad_to=64):
    """int8 codes of x [..., R, C] (see fmsmo_quant_i8_affine) as [batch, R, Cp] or, transposed,
    [batch, C, Rp]; the last dimension is zero-padded to a multiple of ``pad_to``."""
    _need_gpu(x)
    x3 = _batched3(x)
    B, R, C = x3.shape
    compute_dtype = compute_dtype or x.dtype
    inner = R if transpose else C
    ldq = (inner + pad_to - 1) // pad_to * pad_to
    q = torch.empty((B, C if transpose else R, ldq), dtype=torch.int8, device=x.device)
    with _dev(x):
        L.call("fmsmo_quant_i8_affine", x3.data_ptr(), _dt(x3), x3.stride(1) if R > 1 else C,
               x3.stride(0) if B > 1 else R * C, float(scale), float(offset), _DT[compute_dtype],
               int(bool(transpose)), q.data_ptr(), ldq, q.stride(0), B, R, C, _stream(x))
    return q


def _bmm(fn, dtype, a, b, a_scale, b_scale, bias, out_dtype):
    _need_gpu(a, b, bias)
    if a.dtype != dtype or b.dtype != dtype or a.dim() != 3 or b.dim() != 3:
        raise TypeError(f"operands must be 3-D {dtype} tensors: a [batch,M,K], b [batch,N,K]")
    a = a.contiguous()
    if b.stride(2) != 1 or b.stride(1) < b.shape[2]:
        b = b.contiguous()
    B, M, K = a.shape
    if b.shape[0] != B or b.shape[2] != K:
        raise ValueError(f"shape mismatch: a {tuple(a.shape)}, b {tuple(b.shape)} ([batch,N,K] layout)")
    N = b.shape[1]
    a_scale = _scale_vec(a_scale, 1, a.device, "a_scale")
    b_scale = _scale_vec(b_scale, 1, a.device, "b_scale")
    if bias is not None:
        bias = bias.detach().to(torch.float32).reshape(-1).contiguous()
        if bias.numel() != B * N:
            raise ValueError("bias must be [batch, N]")
    y = torch.empty((B, M, N), dtype=out_dtype, device=a.device)
    with _dev(a):
        L.call(fn, a.data_ptr(), K, b.data_ptr(), b.stride(1) if N > 1 else K,
               b.stride(0) if B > 1 else N * K, a_scale.data_ptr(), b_scale.data_ptr(), _ptr(bias),
               y.data_ptr(), _DT[out_dtype], N, B, M, N, K, _stream(a))
    return y


def bmm_i8_dq(a, b, a_scale, b_scale, bias=None, out_dtype=torch.float16):
    """y [batch,M,N] = (a [batch,M,K] . b [batch,N,K]^T) * a_scale * b_scale + bias [batch,N]."""
    return _bmm("fmsmo_bmm_i8_dq", torch.int8, a, b, a_scale, b_scale, bias, out_dtype)


def bmm_fp8_dq(a, b, a_scale, b_scale, bias=None, out_dtype=torch.bfloat16):
    return _bmm("fmsmo_bmm_fp8_dq", torch.float8_e4m3fn, a, b, a_scale, b_scale, bias, out_dtype)


# ------------------------------------------------------- the hot-path wrappers as torch operators
# The five wrappers every module forward ends in are registered under ``torch.ops.fms_mo_amd`` with
# shape-only twins, so that ``torch.compile`` traces a swapped model without graph breaks (the
# reference gets the same from registering its integer matmuls as ``torch.ops.fms_mo.*``,
# fms_mo/custom_ext_kernels/utils.py:642-802).  Only GPU kernels are registered: a CPU tensor that
# gets this far fails in the dispatcher.
_OPS = torch.library.Library("fms_mo_amd", "FRAGMENT")
_quant_act_i8_pertoken_impl = quant_act_i8_pertoken
_quant_act_i8_static_impl = quant_act_i8_static
_quant_act_fp8_pertoken_impl = quant_act_fp8_pertoken
_quant_act_fp8_dynamic_impl = quant_act_fp8_dynamic
_gemm_i8_dq_impl = gemm_i8_dq
_gemm_fp8_dq_impl = gemm_fp8_dq


def _register(name, schema, impl, fake):
    _OPS.define(name + schema)
    _OPS.impl(name, impl, "CUDA")
    torch.library.register_fake("fms_mo_amd::" + name)(fake)


def _rows_shape(x):
    return (x.shape[0], x.shape[1])


_register(
    "quant_act_i8_pertoken",
    "(Tensor x, Tensor? smooth, ScalarType? compute_dtype, bool saturate) -> (Tensor, Tensor)",
    lambda x, smooth, compute_dtype, saturate: _quant_act_i8_pertoken_impl(x, smooth, compute_dtype, saturate),
    lambda x, smooth, compute_dtype, saturate: (
        torch.empty(_rows_shape(x), dtype=torch.int8, device=x.device),
        torch.empty((x.shape[0],), dtype=torch.float32, device=x.device)),
)
_register(
    "quant_act_i8_static",
    "(Tensor x, float scale, int zp, int sym) -> Tensor",
    lambda x, scale, zp, sym: _quant_act_i8_static_impl(x, scale, zp, sym),
    lambda x, scale, zp, sym: torch.empty(_rows_shape(x), dtype=torch.int8, device=x.device),
)
_register(
    "quant_act_fp8_pertoken",
    "(Tensor x, int variant, Tensor? static_scale) -> (Tensor, Tensor)",
    lambda x, variant, static_scale: _quant_act_fp8_pertoken_impl(x, variant, static_scale),
    lambda x, variant, static_scale: (
        torch.empty(_rows_shape(x), dtype=torch.float8_e4m3fn, device=x.device),
        torch.empty((1 if static_scale is not None else x.shape[0],), dtype=torch.float32,
                    device=x.device)),
)
_register(
    "quant_act_fp8_dynamic",
    "(Tensor x, int variant, bool per_tensor, float scale_floor, bool scale_in_x_dtype) -> (Tensor, Tensor)",
    lambda x, variant, per_tensor, scale_floor, scale_in_x_dtype: _quant_act_fp8_dynamic_impl(
        x, variant, per_tensor, scale_floor, scale_in_x_dtype),
    lambda x, variant, per_tensor, scale_floor, scale_in_x_dtype: (
        torch.empty(_rows_shape(x), dtype=torch.float8_e4m3fn, device=x.device),
        torch.empty((1 if per_tensor else x.shape[0],), dtype=torch.float32, device=x.device)),
)
_register(
    "gemm_i8_dq",
    "(Tensor a, Tensor w, Tensor a_scale, Tensor w_scale, Tensor? bias, ScalarType out_dtype, "
    "int epilogue, bool force_gemv) -> Tensor",
    lambda a, w, a_scale, w_scale, bias, out_dtype, epilogue, force_gemv: _gemm_i8_dq_impl(
        a, w, a_scale, w_scale, bias, out_dtype, epilogue, force_gemv),
    lambda a, w, a_scale, w_scale, bias, out_dtype, epilogue, force_gemv: torch.empty(
        (a.shape[0], w.shape[0]), dtype=out_dtype, device=a.device),
)
_register(
    "gemm_fp8_dq",
    "(Tensor a, Tensor w, Tensor a_scale, Tensor w_scale, Tensor? bias, ScalarType out_dtype, "
    "bool force_gemv) -> Tensor",
    lambda a, w, a_scale, w_scale, bias, out_dtype, force_gemv: _gemm_fp8_dq_impl(
        a, w, a_scale, w_scale, bias, out_dtype, force_gemv),
    lambda a, w, a_scale, w_scale, bias, out_dtype, force_gemv: torch.empty(
        (a.shape[0], w.shape[0]), dtype=out_dtype, device=a.device),
)


def _as_scale(s, device):
    if torch.is_tensor(s):
        return s
    return torch.tensor([float(s)], dtype=torch.float32, device=device)


# Lean forms of the three calls a decode step makes.  An eager call of a 5 us kernel is bound by
# what the host does per launch; the general wrappers above spend about 60 Python-level calls on
# argument handling.  These take the common case only -- plain, well-formed tensors on the current
# GPU, outside a compiler trace -- with the checks written inline, and return None for anything
# else, which then goes through the general path (and gets its error messages there).
_T, _P = torch.Tensor, torch.nn.Parameter
_COMPILING = torch.compiler.is_compiling
_F32, _I8 = torch.float32, torch.int8
_FN = {}


def _fn(name):
    f = _FN.get(name)
    if f is None:
        f = _FN[name] = L.entry(name)
    return f


def _mat(t, dtype):
    """(rows, cols, row stride) of a plain 2-D CUDA tensor of `dtype` with unit inner stride on
    the current GPU, else None."""
    tt = type(t)
    if (tt is not _T and tt is not _P) or t.dtype is not dtype or not t.is_cuda or t.dim() != 2:
        return None
    r, c = t.shape
    s0, s1 = t.stride()
    if s1 != 1 or (r > 1 and s0 < c):
        return None
    return r, c, (s0 if r > 1 else max(c, s0))


def _vec32(t, n):
    return (type(t) is _T and t.dtype is _F32 and t.is_cuda and t.dim() == 1 and t.is_contiguous()
            and (t.numel() == n or t.numel() == 1) and not t.requires_grad)


def _gemm_i8_dq_lean(a, w, a_scale, w_scale, bias, out_dtype, epilogue):
    if _COMPILING() or _RAW_STREAM is None:
        return None
    ma, mw = _mat(a, _I8), _mat(w, _I8)
    if ma is None or mw is None or ma[1] != mw[1] or not _vec32(a_scale, ma[0]) or not _vec32(w_scale, mw[0]):
        return None
    M, K, lda = ma
    N, _, ldw = mw
    if bias is not None:
        tb = type(bias)
        if ((tb is not _T and tb is not _P) or not bias.is_cuda or bias.dim() != 1 or bias.numel() != N
                or not bias.is_contiguous() or bias.dtype not in _DT):
            return None
        bptr, bdt = bias.data_ptr(), _DT[bias.dtype]
    else:
        bptr, bdt = None, 0
    idx = a.get_device()
    if _CUR_DEVICE() != idx or out_dtype not in _DT:
        return None
    y = torch.empty((M, N), dtype=out_dtype, device=a.device)
    nbytes = _WS_BYTES.get((M, N, K))
    if nbytes is None:
        nbytes = _WS_BYTES[(M, N, K)] = L.load().fmsmo_gemm_workspace_bytes(M, N, K)
    if nbytes > 0:
        ws = torch.empty((nbytes,), dtype=torch.uint8, device=a.device)
        rc = _fn("fmsmo_gemm_i8_dq_ws")(a.data_ptr(), lda, w.data_ptr(), ldw, a_scale.data_ptr(), a_scale.numel(),
                                        w_scale.data_ptr(), w_scale.numel(), bptr, bdt, epilogue, y.data_ptr(),
                                        _DT[out_dtype], N, M, N, K, ws.data_ptr(), nbytes, _RAW_STREAM(idx))
    else:
        rc = _fn("fmsmo_gemm_i8_dq")(a.data_ptr(), lda, w.data_ptr(), ldw, a_scale.data_ptr(), a_scale.numel(),
                                     w_scale.data_ptr(), w_scale.numel(), bptr, bdt, epilogue, y.data_ptr(),
                                     _DT[out_dtype], N, M, N, K, _RAW_STREAM(idx))
    if rc:
        L.raise_status("fmsmo_gemm_i8_dq", rc)
    return y


def _smooth_ok(smooth, K):
    ts = type(smooth)
    return ((ts is _T or ts is _P) and smooth.is_cuda and smooth.dim() == 1 and smooth.numel() == K
            and smooth.is_contiguous() and smooth.dtype in _DT and smooth.data_ptr() % 16 == 0)


def _quant_act_i8_pertoken_lean(x, smooth, compute_dtype, saturate):
    if _COMPILING() or _RAW_STREAM is None or x.dtype not in _DT:
        return None
    mx = _mat(x, x.dtype)
    if mx is None:
        return None
    M, K, ldx = mx
    if smooth is not None:
        if not _smooth_ok(smooth, K):
            return None
        sptr, sdt = smooth.data_ptr(), _DT[smooth.dtype]
        if compute_dtype is None:
            compute_dtype = x.dtype if smooth.dtype is x.dtype else torch.promote_types(x.dtype, smooth.dtype)
    else:
        sptr, sdt = None, 0
        if compute_dtype is None:
            compute_dtype = x.dtype
    idx = x.get_device()
    if _CUR_DEVICE() != idx or compute_dtype not in _DT:
        return None
    q = torch.empty((M, K), dtype=_I8, device=x.device)
    scale = torch.empty((M,), dtype=_F32, device=x.device)
    rc = _fn("fmsmo_quant_act_i8_pertoken")(x.data_ptr(), _DT[x.dtype], ldx, sptr, sdt, _DT[compute_dtype],
                                            1 if saturate else 0, q.data_ptr(), K, scale.data_ptr(), M, K,
                                            _RAW_STREAM(idx))
    if rc:
        L.raise_status("fmsmo_quant_act_i8_pertoken", rc)
    return q, scale


def _decode_linear_i8_lean(x, w, w_scale, bias, smooth, out_dtype, exact_ref, saturate):
    if _COMPILING() or _RAW_STREAM is None or x.dtype not in _DT:
        return None
    mx, mw = _mat(x, x.dtype), _mat(w, _I8)
    if mx is None or mw is None or mx[1] != mw[1] or not _vec32(w_scale, mw[0]):
        return None
    M, K, ldx = mx
    N, _, ldw = mw
    if smooth is not None:
        if not _smooth_ok(smooth, K):
            return None
        sptr, sdt = smooth.data_ptr(), _DT[smooth.dtype]
    else:
        sptr, sdt = None, 0
    if bias is not None:
        tb = type(bias)
        if ((tb is not _T and tb is not _P) or not bias.is_cuda or bias.dim() != 1 or bias.numel() != N
                or not bias.is_contiguous() or bias.dtype not in _DT):
            return None
        bptr, bdt = bias.data_ptr(), _DT[bias.dtype]
    else:
        bptr, bdt = None, 0
    idx = x.get_device()
    if _CUR_DEVICE() != idx or out_dtype not in _DT:
        return None
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    a_scale = torch.empty((M,), dtype=_F32, device=x.device)
    rc = _fn("fmsmo_decode_linear_i8")(x.data_ptr(), _DT[x.dtype], ldx, sptr, sdt, 1 if saturate else 0, w.data_ptr(),
                                       ldw, w_scale.data_ptr(), w_scale.numel(), bptr, bdt,
                                       L.EPI_REF_F16 if exact_ref else L.EPI_F32, y.data_ptr(), _DT[out_dtype], N,
                                       a_scale.data_ptr(), M, N, K, _RAW_STREAM(idx))
    if rc:
        L.raise_status("fmsmo_decode_linear_i8", rc)
    return y, a_scale


_E4M3 = torch.float8_e4m3fn


def _bias_ok(bias, N):
    tb = type(bias)
    return ((tb is _T or tb is _P) and bias.is_cuda and bias.dim() == 1 and bias.numel() == N
            and bias.is_contiguous() and bias.dtype in _DT)


def _gemm_fp8_dq_lean(a, w, a_scale, w_scale, bias, out_dtype):
    if _COMPILING() or _RAW_STREAM is None:
        return None
    ma, mw = _mat(a, _E4M3), _mat(w, _E4M3)
    if ma is None or mw is None or ma[1] != mw[1] or not _vec32(a_scale, ma[0]) or not _vec32(w_scale, mw[0]):
        return None
    M, K, lda = ma
    N, _, ldw = mw
    if bias is not None:
        if not _bias_ok(bias, N):
            return None
        bptr, bdt = bias.data_ptr(), _DT[bias.dtype]
    else:
        bptr, bdt = None, 0
    idx = a.get_device()
    if _CUR_DEVICE() != idx or out_dtype not in _DT:
        return None
    y = torch.empty((M, N), dtype=out_dtype, device=a.device)
    nbytes = _WS_BYTES.get((M, N, K))
    if nbytes is None:
        nbytes = _WS_BYTES[(M, N, K)] = L.load().fmsmo_gemm_workspace_bytes(M, N, K)
    if nbytes > 0:
        ws = torch.empty((nbytes,), dtype=torch.uint8, device=a.device)
        rc = _fn("fmsmo_gemm_fp8_dq_ws")(a.data_ptr(), lda, w.data_ptr(), ldw, a_scale.data_ptr(), a_scale.numel(),
                                         w_scale.data_ptr(), w_scale.numel(), bptr, bdt, y.data_ptr(),
                                         _DT[out_dtype], N, M, N, K, ws.data_ptr(), nbytes, _RAW_STREAM(idx))
    else:
        rc = _fn("fmsmo_gemm_fp8_dq")(a.data_ptr(), lda, w.data_ptr(), ldw, a_scale.data_ptr(), a_scale.numel(),
                                      w_scale.data_ptr(), w_scale.numel(), bptr, bdt, y.data_ptr(),
                                      _DT[out_dtype], N, M, N, K, _RAW_STREAM(idx))
    if rc:
        L.raise_status("fmsmo_gemm_fp8_dq", rc)
    return y


def _decode_linear_fp8_lean(x, w, w_scale, bias, out_dtype):
    if _COMPILING() or _RAW_STREAM is None or x.dtype not in _DT:
        return None
    mx, mw = _mat(x, x.dtype), _mat(w, _E4M3)
    if mx is None or mw is None or mx[1] != mw[1] or not _vec32(w_scale, mw[0]):
        return None
    M, K, ldx = mx
    N, _, ldw = mw
    if bias is not None:
        if not _bias_ok(bias, N):
            return None
        bptr, bdt = bias.data_ptr(), _DT[bias.dtype]
    else:
        bptr, bdt = None, 0
    idx = x.get_device()
    if _CUR_DEVICE() != idx or out_dtype not in _DT:
        return None
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    a_scale = torch.empty((M,), dtype=_F32, device=x.device)
    rc = _fn("fmsmo_decode_linear_fp8")(x.data_ptr(), _DT[x.dtype], ldx, w.data_ptr(), ldw, w_scale.data_ptr(),
                                        w_scale.numel(), bptr, bdt, y.data_ptr(), _DT[out_dtype], N,
                                        a_scale.data_ptr(), M, N, K, _RAW_STREAM(idx))
    if rc:
        L.raise_status("fmsmo_decode_linear_fp8", rc)
    return y, a_scale


def quant_act_i8_pertoken(x, smooth=None, compute_dtype=None, saturate=False):  # noqa: F811
    """(q int8 [M,K], scale fp32 [M]) -- see fmsmo_quant_act_i8_pertoken."""
    r = _quant_act_i8_pertoken_lean(x, smooth, compute_dtype, saturate)
    if r is not None:
        return r
    _need_gpu(x, smooth)
    if x.dim() != 2:
        raise ValueError("expected a 2-D tensor")
    if _eager(x, smooth):
        return _quant_act_i8_pertoken_impl(x, smooth, compute_dtype, bool(saturate))
    return torch.ops.fms_mo_amd.quant_act_i8_pertoken(x, smooth, compute_dtype, bool(saturate))


def quant_act_i8_static(x, scale: float, zp: int, sym: int):  # noqa: F811
    _need_gpu(x)
    if x.dim() != 2:
        raise ValueError("expected a 2-D tensor")
    if _eager(x):
        return _quant_act_i8_static_impl(x, float(scale), int(zp), int(sym))
    return torch.ops.fms_mo_amd.quant_act_i8_static(x, float(scale), int(zp), int(sym))


def quant_act_fp8_pertoken(x, variant=L.FP8_LINEAR, static_scale=None):  # noqa: F811
    """(q e4m3 [M,K], scale fp32 [M] or the [1] static scale)."""
    _need_gpu(x)
    if x.dim() != 2:
        raise ValueError("expected a 2-D tensor")
    if static_scale is not None:
        static_scale = _as_scale(static_scale, x.device)
    if _eager(x, static_scale):
        return _quant_act_fp8_pertoken_impl(x, int(variant), static_scale)
    return torch.ops.fms_mo_amd.quant_act_fp8_pertoken(x, int(variant), static_scale)


def quant_act_fp8_dynamic(x, variant=L.FP8_LINEAR, per_tensor=False, scale_floor=1e-12,  # noqa: F811
                          scale_in_x_dtype=False):
    """(q e4m3 [M,K], scale fp32 [M] or [1]), see fmsmo_quant_act_fp8_dynamic."""
    _need_gpu(x)
    if x.dim() != 2:
        raise ValueError("expected a 2-D tensor")
    if _eager(x):
        return _quant_act_fp8_dynamic_impl(x, int(variant), bool(per_tensor), float(scale_floor),
                                           bool(scale_in_x_dtype))
    return torch.ops.fms_mo_amd.quant_act_fp8_dynamic(x, int(variant), bool(per_tensor),
                                                      float(scale_floor), bool(scale_in_x_dtype))


def gemm_i8_dq(a, w, a_scale, w_scale, bias=None, out_dtype=torch.float16, exact_ref=True,  # noqa: F811
               force_gemv=False, epilogue=None):
    """y [M,N] = dequant(a int8 [M,K] . w int8 [N,K]^T), see fmsmo_gemm_i8_dq.  ``epilogue`` (one of
    L.EPI_*) overrides ``exact_ref`` (True = L.EPI_REF_F16, False = L.EPI_F32)."""
    if epilogue is None:
        epilogue = L.EPI_REF_F16 if exact_ref else L.EPI_F32
    if not force_gemv:
        y = _gemm_i8_dq_lean(a, w, a_scale, w_scale, bias, out_dtype, int(epilogue))
        if y is not None:
            return y
    _need_gpu(a, w, bias)
    if _eager(a, w, bias) and (not torch.is_tensor(a_scale) or _eager(a_scale)) \
            and (not torch.is_tensor(w_scale) or _eager(w_scale)):
        return _gemm_i8_dq_impl(a, w, a_scale, w_scale, bias, out_dtype, int(epilogue), bool(force_gemv))
    return torch.ops.fms_mo_amd.gemm_i8_dq(a, w, _as_scale(a_scale, a.device), _as_scale(w_scale, a.device),
                                           bias, out_dtype, int(epilogue), bool(force_gemv))


def gemm_fp8_dq(a, w, a_scale, w_scale, bias=None, out_dtype=torch.bfloat16, force_gemv=False):  # noqa: F811
    if not force_gemv:
        y = _gemm_fp8_dq_lean(a, w, a_scale, w_scale, bias, out_dtype)
        if y is not None:
            return y
    _need_gpu(a, w, bias)
    if _eager(a, w, bias) and (not torch.is_tensor(a_scale) or _eager(a_scale)) \
            and (not torch.is_tensor(w_scale) or _eager(w_scale)):
        return _gemm_fp8_dq_impl(a, w, a_scale, w_scale, bias, out_dtype, bool(force_gemv))
    return torch.ops.fms_mo_amd.gemm_fp8_dq(a, w, _as_scale(a_scale, a.device), _as_scale(w_scale, a.device),
                                            bias, out_dtype, bool(force_gemv))


# ------------------------------------------------------------------------ fused decode linear
_DECODE_OK = {}


def decode_linear_ok(x, smooth, K):
    """Can ``decode_linear_i8`` serve these activations?  fp16 / bf16, SmoothQuant divisors of the
    same dtype (or none): one token at K up to 8192 in one of the decode kernel's sizes or at
    14336 / 12800, up to four tokens at K = 4096, up to three at 14336 / 12800.  fp32 divisors
    (the quantizer then runs in fp32): K = 4096 up to two tokens, 14336 / 12800 one token."""
    if x.dim() != 2 or x.dtype not in (torch.float16, torch.bfloat16) or not x.is_cuda:
        return False
    f32s = smooth is not None and smooth.dtype == torch.float32
    if smooth is not None and ((smooth.dtype != x.dtype and not f32s) or smooth.numel() != K):
        return False
    key = (x.shape[0], K, f32s)
    if torch.compiler.is_compiling():
        # answers of earlier eager calls only (a foreign-function call cannot be traced); a shape
        # never seen eagerly takes the two-kernel path, which serves every shape
        return _DECODE_OK.get(key, False)
    if key not in _DECODE_OK:
        lib = L.load()
        ok = lib.fmsmo_decode_linear_f32s_ok if f32s else lib.fmsmo_decode_linear_ok
        _DECODE_OK[key] = bool(ok(x.shape[0], K))
    return _DECODE_OK[key]


def _decode_linear_i8_impl(x, w, w_scale, bias, smooth, out_dtype, exact_ref, saturate):
    x = _rows(x)
    w = _rows(w)
    M, K = x.shape
    N = w.shape[0]
    if w.dtype != torch.int8 or w.shape[1] != K:
        raise ValueError("w must be int8 [N, K]")
    w_scale = _scale_vec(w_scale, N, x.device, "w_scale")
    if smooth is not None:
        _need_gpu(smooth)
        smooth = smooth.detach().reshape(-1).contiguous()
        if smooth.numel() != K or smooth.dtype not in (x.dtype, torch.float32):
            raise ValueError("smooth must have K elements of x's dtype or fp32")
        if smooth.data_ptr() % 16:
            smooth = smooth.clone()
    if bias is not None:
        _need_gpu(bias)
        bias = bias.detach().reshape(-1).contiguous()
        if bias.numel() != N:
            raise ValueError("bias must have N elements")
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    a_scale = torch.empty((M,), dtype=torch.float32, device=x.device)
    with _dev(x):
        L.call("fmsmo_decode_linear_i8", x.data_ptr(), _dt(x), _ld(x), _ptr(smooth),
               _dt(smooth) if smooth is not None else 0, int(bool(saturate)),
               w.data_ptr(), _ld(w), w_scale.data_ptr(), w_scale.numel(), _ptr(bias),
               _dt(bias) if bias is not None else 0, L.EPI_REF_F16 if exact_ref else L.EPI_F32,
               y.data_ptr(), _DT[out_dtype], N, a_scale.data_ptr(), M, N, K, _stream(x))
    return y, a_scale


_register(
    "decode_linear_i8",
    "(Tensor x, Tensor w, Tensor w_scale, Tensor? bias, Tensor? smooth, ScalarType out_dtype, "
    "bool exact_ref, bool saturate) -> (Tensor, Tensor)",
    lambda x, w, w_scale, bias, smooth, out_dtype, exact_ref, saturate: _decode_linear_i8_impl(
        x, w, w_scale, bias, smooth, out_dtype, exact_ref, saturate),
    lambda x, w, w_scale, bias, smooth, out_dtype, exact_ref, saturate: (
        torch.empty((x.shape[0], w.shape[0]), dtype=out_dtype, device=x.device),
        torch.empty((x.shape[0],), dtype=torch.float32, device=x.device)),
)


def decode_linear_i8(x, w, w_scale, bias=None, smooth=None, out_dtype=torch.float16, exact_ref=True,
                     saturate=False):
    """(y [M,N], per-token scales fp32 [M]) = quantize x per token (see quant_act_i8_pertoken) and
    multiply with the int8 weights w [N,K], in one launch; check ``decode_linear_ok`` first."""
    r = _decode_linear_i8_lean(x, w, w_scale, bias, smooth, out_dtype, exact_ref, saturate)
    if r is not None:
        return r
    _need_gpu(x, w, bias, smooth)
    if _eager(x, w, bias, smooth) and (not torch.is_tensor(w_scale) or _eager(w_scale)):
        return _decode_linear_i8_impl(x, w, w_scale, bias, smooth, out_dtype, bool(exact_ref), bool(saturate))
    return torch.ops.fms_mo_amd.decode_linear_i8(x, w, _as_scale(w_scale, x.device), bias, smooth,
                                                 out_dtype, bool(exact_ref), bool(saturate))


def _decode_linear_fp8_impl(x, w, w_scale, bias, out_dtype):
    x = _rows(x)
    w = _rows(w)
    M, K = x.shape
    N = w.shape[0]
    if w.dtype != torch.float8_e4m3fn or w.shape[1] != K:
        raise ValueError("w must be float8_e4m3fn [N, K]")
    w_scale = _scale_vec(w_scale, N, x.device, "w_scale")
    if bias is not None:
        _need_gpu(bias)
        bias = bias.detach().reshape(-1).contiguous()
        if bias.numel() != N:
            raise ValueError("bias must have N elements")
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    a_scale = torch.empty((M,), dtype=torch.float32, device=x.device)
    with _dev(x):
        L.call("fmsmo_decode_linear_fp8", x.data_ptr(), _dt(x), _ld(x), w.data_ptr(), _ld(w),
               w_scale.data_ptr(), w_scale.numel(), _ptr(bias), _dt(bias) if bias is not None else 0,
               y.data_ptr(), _DT[out_dtype], N, a_scale.data_ptr(), M, N, K, _stream(x))
    return y, a_scale


_register(
    "decode_linear_fp8",
    "(Tensor x, Tensor w, Tensor w_scale, Tensor? bias, ScalarType out_dtype) -> (Tensor, Tensor)",
    lambda x, w, w_scale, bias, out_dtype: _decode_linear_fp8_impl(x, w, w_scale, bias, out_dtype),
    lambda x, w, w_scale, bias, out_dtype: (
        torch.empty((x.shape[0], w.shape[0]), dtype=out_dtype, device=x.device),
        torch.empty((x.shape[0],), dtype=torch.float32, device=x.device)),
)


def decode_linear_fp8(x, w, w_scale, bias=None, out_dtype=torch.bfloat16):
    """(y [M,N], token scales fp32 [M]): dynamic per-token e4m3 quantizer (the FP8Linear recipe) and
    the e4m3 weight-streaming matmul in one launch; check ``decode_linear_ok(x, None, K)`` first."""
    r = _decode_linear_fp8_lean(x, w, w_scale, bias, out_dtype)
    if r is not None:
        return r
    _need_gpu(x, w, bias)
    if _eager(x, w, bias) and (not torch.is_tensor(w_scale) or _eager(w_scale)):
        return _decode_linear_fp8_impl(x, w, w_scale, bias, out_dtype)
    return torch.ops.fms_mo_amd.decode_linear_fp8(x, w, _as_scale(w_scale, x.device), bias, out_dtype)
