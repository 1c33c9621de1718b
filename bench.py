#!/usr/bin/env python3
"""Benchmark of the W8A8 quantized-linear hot path on one MI355X.

A step = one pass of the path over one batch of synthetic activations already resident in HBM:
for each of the four Llama-3-8B decoder-layer linears at M = 4096 tokens (q/k/v fused 4096->6144,
o 4096->4096, gate+up 4096->28672, down 14336->4096) run the fused SmoothQuant-divide + per-token
int8 activation quantizer, then the int8 MFMA GEMM with the dequantizing epilogue (fp16 out).
Weights are quantized once, before the timed region (they are constants of the deployed module).

Prints ONE JSON line (see the keys below).  `value` is 2*M*N*K summed over the four linears
divided by the wall time of a step; `roofline` prices the GEMM kernel alone (HIP-event time of
its launches inside the timed region) against the published dense INT8 MFMA peak; `roofline_fp8`
and `roofline_decode` carry the other two parts of the metric (e4m3 GEMMs against the FP8 MFMA
peak, M <= 16 decode launches against the HBM peak); `cpu_baseline` is the CPU restatement of the
reference's QLinear forward timed on the host cores on a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "fms-model-optimizer_amd"))

PEAK_INT8_TOPS = 5000.0   # MI355X dense INT8 MFMA, published
PEAK_FP8_TFLOPS = 5000.0  # MI355X dense FP8 MFMA, published
PEAK_HBM_GBS = 8000.0     # MI355X HBM3E, published

LLAMA3_8B = [("qkv", 4096, 6144), ("o", 4096, 4096), ("gate_up", 4096, 28672), ("down", 14336, 4096)]
M_TOKENS = 4096


def make_layer(torch, dev, K, N, seed):
    """Inputs of the headline configuration: x ~ N(0,1) with 1 % of the input channels scaled x50, W ~ N(0,0.02),
    SmoothQuant alpha = 0.5 with a_k = max_m |x_mk|.  Generated on the CPU from a seeded generator
    (so the CPU baseline sees the same bits), quantized offline with the deploy-module recipe."""
    from fms_mo_amd.modules.linear import prepare_deploy_weights

    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M_TOKENS, K, generator=g)
    idx = torch.randperm(K, generator=g)[: round(0.01 * K)]
    x[:, idx] *= 50
    W = 0.02 * torch.randn(N, K, generator=g)
    b = 0.01 * torch.randn(N, generator=g)
    x, W, b = x.half(), W.half(), b.half()
    act_scale = x.float().abs().amax(dim=0)
    xd, Wd = x.to(dev), W.to(dev)
    w_i8, w_scale, smooth = prepare_deploy_weights(Wd, act_scale.to(dev), 0.5)
    # buffers as in a module cast with .half() for deployment: SmoothQuant scale in fp16, so
    # x / smoothq_scale is an fp16 division (fms_mo/modules/linear.py:1331-1332)
    return {"x": xd, "w": w_i8, "w_scale": w_scale.float(), "smooth": smooth.reshape(-1).half(),
            "bias": b.to(dev), "x_cpu": x, "W_cpu": W, "b_cpu": b, "act_scale_cpu": act_scale}


def cpu_baseline(torch, layers, budget_s=30.0):
    """The reference's CPU QLinear path (fake-quant forward with per-call weight re-quantization,
    fms_mo/modules/linear.py:248-305) restated in oracle/: all four linears of the step on the
    first 2048 of the 4096 tokens, a bounded sample of about 15 s of host time."""
    from oracle import qlinear_oracle as O

    torch.set_num_threads(os.cpu_count() or 1)
    rows = 2048

    def one_pass():
        for layer in layers:
            O.qlinear_forward(layer["x_cpu"][:rows], layer["W_cpu"], layer["b_cpu"], layer["act_scale_cpu"], 0.5)

    one_pass()  # warm-up
    times = []
    t_all = time.perf_counter()
    while len(times) < 5 and (len(times) < 2 or time.perf_counter() - t_all < budget_s):
        t0 = time.perf_counter()
        one_pass()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    ops = sum(2.0 * rows * layer["W_cpu"].shape[0] * layer["W_cpu"].shape[1] for layer in layers)
    res = {"value": ops / med / 1e12, "unit": "TOPS", "cores": torch.get_num_threads(),
           "kind": "port",
           "sample": f"QLinear fake-quant forward (act Q/dQ, per-call weight Q/dQ, fp16 F.linear) of all four "
                     f"linears, first {rows} of 4096 tokens, median of {len(times)} passes, "
                     f"{med:.2f} s each"}
    # second leg: the deployed module's CPU fallback, QLinearINT8Deploy.forward with iaddmm_FP
    # (fms_mo/modules/linear.py:1190-1211, 1309-1338): weights already int8, per-token quantizer,
    # matmul on the dequantized operands in fp16 -- needs every buffer in x's dtype
    bufs = []
    for layer in layers:
        b = O.deploy_prepare(layer["W_cpu"], layer["b_cpu"], layer["W_cpu"].abs().amax(dim=1).float(),
                             layer["act_scale_cpu"], 0.5)
        bufs.append({k: (v.half() if v.is_floating_point() else v) for k, v in b.items()})

    def fp_pass():
        for layer, b in zip(layers, bufs):
            O.deploy_forward_fp(layer["x_cpu"][:rows], b)

    fp_pass()
    t_fp = []
    for _ in range(3):
        t0 = time.perf_counter()
        fp_pass()
        t_fp.append(time.perf_counter() - t0)
    t_fp.sort()
    res["deploy_iaddmm_FP"] = {"value": ops / t_fp[1] / 1e12, "unit": "TOPS",
                               "sample": f"QLinearINT8Deploy forward with the iaddmm_FP fallback, same "
                                         f"{rows} tokens and linears, median of 3 passes, {t_fp[1]:.2f} s each"}
    return res

def gemm_sources_sha16():
    """Names the GEMM kernel sources a counter profile belongs to."""
    import hashlib

    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "fms-model-optimizer_amd", "csrc")
    for name in ("common.hpp", "gemm_tile.hpp", "gemm_rs.hpp", "gemm_launch.hpp", "gemm.hip"):
        with open(os.path.join(csrc, name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


GRANITE_8B = [("qkv", 4096, 6144), ("o", 4096, 4096), ("gate_up", 4096, 25600), ("down", 12800, 4096)]


def time_events(torch, fn, iters=30, warm=5, min_seconds=0.0):
    """Average HIP-event time (ms) of fn over iters eager calls on the current stream; with
    min_seconds the number of calls is raised so that the timed region lasts that long (the part
    settles its clock over milliseconds: a burst of twenty launches is timed at whatever clock the
    work before it left behind)."""
    for _ in range(warm):
        fn()
    if min_seconds > 0:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(5):
            fn()
        e1.record()
        torch.cuda.synchronize()
        iters = max(iters, int(min_seconds * 1e3 / max(e0.elapsed_time(e1) / 5, 1e-3)))
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters


def fp8_rooflines(torch, K, dev, min_seconds=0.15):
    """The FP8 half of the metric: e4m3 x e4m3 GEMMs with fp32 accumulation and the dequantizing
    epilogue (per-token activation scale, bf16 out) against the 5.0 PFLOP/s dense FP8 peak, on the
    Llama-3-8B shapes at M = 4096 (per-channel weight scales) and the Granite-3-8B-like shapes at
    M = 2048 (per-tensor weight scale).  Operands are real quantizer outputs (codes over the whole
    +-448 range), timed over eager launches with HIP events, the GEMM alone."""
    from fms_mo_amd import _lib as L

    g = torch.Generator().manual_seed(3)
    out = {"peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s", "bound": "mfma", "dtype": "e4m3 x e4m3 -> fp32"}
    clk = torch.zeros(6, dtype=torch.int64, device=dev)
    for label, M, shapes, per_channel in (("llama3_8b_M4096", M_TOKENS, LLAMA3_8B, True),
                                          ("granite_8b_M2048", 2048, GRANITE_8B, False)):
        per, tot_ms, tot_ops, vend = {}, 0.0, 0.0, {}
        for name, k, n in shapes:
            x = torch.randn(M, k, generator=g).bfloat16().to(dev)
            w = (0.02 * torch.randn(n, k, generator=g)).to(dev)
            ws = (w.abs().amax(dim=1) / 448).float() if per_channel else (w.abs().amax() / 448).reshape(1).float()
            w8 = (w / (ws[:, None] if per_channel else ws)).clamp(-448, 448).to(torch.float8_e4m3fn)
            q, s = K.quant_act_fp8_pertoken(x, L.FP8_LINEAR)
            K.clock_probe(clk)
            ms = time_events(torch, lambda: K.gemm_fp8_dq(q, w8, s, ws, None, out_dtype=torch.bfloat16), iters=20, warm=4,
                             min_seconds=min_seconds)
            K.clock_probe(None)
            ops = 2.0 * M * k * n
            tot_ms += ms
            tot_ops += ops
            tf = ops / (ms * 1e-3) / 1e12
            per[name] = {"ms": round(ms, 4), "tflops": round(tf, 1), "frac": round(tf / PEAK_FP8_TFLOPS, 4),
                         "core_clock_mhz": round(K.core_clock_mhz(clk))}
            # the vendor library on the SAME codes, same event timing, same run: torch._scaled_mm
            # (hipBLASLt), what the reference's FP8Linear calls on a GPU
            # (fms_mo/aiu_addons/fp8/fp8_linear.py:275-283), with row-wise scales (per token x per
            # channel, this kernel's epilogue) and with one scale per tensor
            sa_row = s.reshape(-1, 1).contiguous()
            sb_row = (ws if per_channel else ws.expand(n)).reshape(1, -1).contiguous()
            one = torch.ones((), device=dev)
            for vlabel, sa, sb in (("vendor_scaled_mm_rowwise", sa_row, sb_row), ("vendor_scaled_mm_tensorwise", one, one)):
                try:
                    vms = time_events(torch, lambda: torch._scaled_mm(q, w8.t(), scale_a=sa, scale_b=sb,
                                                                       out_dtype=torch.bfloat16), iters=20, warm=4,
                                      min_seconds=min_seconds)
                    per[name][vlabel] = {"ms": round(vms, 4), "tflops": round(ops / (vms * 1e-3) / 1e12, 1)}
                    vend[vlabel] = vend.get(vlabel, 0.0) + vms
                except Exception as e:  # the vendor path is evidence, not a dependency
                    per[name][vlabel] = {"error": str(e)[:160]}
                    vend[vlabel] = float("nan")
            del x, w, w8, q
        tf = tot_ops / (tot_ms * 1e-3) / 1e12
        out[label] = {"per_shape": per, "achieved": round(tf, 1), "frac": round(tf / PEAK_FP8_TFLOPS, 4)}
        for vlabel, vms in vend.items():
            if vms == vms:
                out[label][vlabel + "_tflops"] = round(tot_ops / (vms * 1e-3) / 1e12, 1)
    return out


def decode_rooflines(torch, K, dev, m_list=(1, 4, 16), ops=("i8", "fp8"), copies_mib=300):
    """The decode half of the metric: y = dequant(q_x . W_q^T) for M in {1, 4, 16} tokens on the four
    Llama-3-8B weight shapes, int8 and e4m3 weights, against the 8 TB/s HBM peak.  Algorithmic bytes
    per launch: N K (weights) + M K (codes) + 2 M N (bf16 out) + 4 N (scales).  Weight copies
    totalling > 256 MiB are rotated so the memory-side cache cannot hold them.  `us` is device time
    (the launches replayed from a HIP graph); `eager_us` is the time per call of the same launches
    issued one by one from Python through the operator wrapper (host launch cost included).
    `read_only_floor_<shape>`: a launch that only reads the same weight bytes (256 x 1024 threads,
    16-byte loads, nothing written), timed in the same graph over the same rotation -- what the
    launch and the memory system leave to any kernel of that size; `floor_over_us` is its share of
    the decode launch's time."""
    from fms_mo_amd import _lib as L

    out = {"peak": PEAK_HBM_GBS, "unit": "GB/s", "bound": "hbm"}
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    floors = {}
    for name, k, n in LLAMA3_8B:
        wbytes = k * n
        copies = max(3, (copies_mib * 1024 * 1024 + wbytes - 1) // wbytes)
        wsc = torch.rand(n, device=dev) * 1e-3
        for op in ops:
            if op == "i8":
                ws_q = [torch.randint(-127, 128, (n, k), dtype=torch.int8, device=dev) for _ in range(copies)]
            else:  # e4m3 weights whose codes cover the format's range (per-channel-scaled Gaussian)
                ws_q = [torch.randn(n, k, device=dev).mul_(448.0 / 4.5).clamp_(-448, 448).to(torch.float8_e4m3fn)
                        for _ in range(copies)]
            for M in (0,) * (name not in floors) + tuple(m_list):
                if M == 0:  # the floor: a launch that only reads the weight bytes (same graph, same rotation)
                    run = lambda w: K.stream_read(w, sink)  # noqa: E731
                else:
                    x = torch.randn(M, k, device=dev).bfloat16()
                if M == 0:
                    pass
                elif op == "i8":
                    q, s = K.quant_act_i8_pertoken(x)
                    run = lambda w: K.gemm_i8_dq(q, w, s, wsc, None, out_dtype=torch.bfloat16, exact_ref=True)  # noqa: E731
                else:
                    q, s = K.quant_act_fp8_pertoken(x, L.FP8_LINEAR)
                    run = lambda w: K.gemm_fp8_dq(q, w, s, wsc, None, out_dtype=torch.bfloat16)  # noqa: E731
                side = torch.cuda.Stream()
                reps, replays = 3, 5
                with torch.cuda.stream(side):
                    for w in ws_q:
                        run(w)
                    torch.cuda.synchronize()
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                    for _ in range(reps):
                        for w in ws_q:
                            run(w)
                    e1.record()
                    torch.cuda.synchronize()
                    eager_ms = e0.elapsed_time(e1) / (reps * copies)
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph, stream=side):
                        for _ in range(reps):
                            for w in ws_q:
                                run(w)
                    graph.replay()
                    torch.cuda.synchronize()
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                    for _ in range(replays):
                        graph.replay()
                    e1.record()
                    torch.cuda.synchronize()
                ms = e0.elapsed_time(e1) / (replays * reps * copies)
                del graph
                if M == 0:
                    floors[name] = ms
                    out[f"read_only_floor_{name}"] = {"us": round(ms * 1e3, 2), "GBps": round(wbytes / ms / 1e6, 1),
                                                      "frac": round(wbytes / ms / 1e6 / PEAK_HBM_GBS, 4)}
                    continue
                byts = wbytes + M * k + M * n * 2 + 4 * n
                gbs = byts / (ms * 1e-3) / 1e9
                out[f"{op}_M{M}_{name}"] = {"us": round(ms * 1e3, 2), "eager_us": round(eager_ms * 1e3, 2),
                                            "GBps": round(gbs, 1), "frac": round(gbs / PEAK_HBM_GBS, 4),
                                            "floor_over_us": round(floors[name] / ms, 3)}
            del ws_q
    fr = [v["frac"] for kk, v in out.items() if isinstance(v, dict) and not kk.startswith("read_only_floor")]
    out["frac_min"], out["frac_max"] = min(fr), max(fr)
    return out


def vendor_int_mm(torch, K, layers):
    """The vendor library's int8 GEMM (torch._int_mm -> hipBLASLt, int32 out, no epilogue) on the
    SAME quantized operands as the headline step, same event timing (each loop at least 0.15 s: a
    burst of twenty launches runs on whatever clock the work before it left behind), beside this
    library's raw int32 GEMM: how much of the distance to the published peak is the part's, not the
    kernel's."""
    res = {}
    for (name, k, n), L in zip(LLAMA3_8B, layers):
        q, _ = K.quant_act_i8_pertoken(L["x"], L["smooth"])
        wt = L["w"].t()
        ops = 2.0 * M_TOKENS * k * n
        try:
            ms_v = time_events(torch, lambda: torch._int_mm(q, wt), iters=20, warm=4, min_seconds=0.15)
            v = {"ms": round(ms_v, 4), "tops": round(ops / ms_v / 1e9, 1)}
        except Exception as e:  # the vendor path is evidence, not a dependency
            v = {"error": str(e)[:200]}
        ms_o = time_events(torch, lambda: K.gemm_i8_i32(q, L["w"]), iters=20, warm=4, min_seconds=0.15)
        res[name] = {"torch_int_mm": v, "fmsmo_gemm_i8_i32": {"ms": round(ms_o, 4), "tops": round(ops / ms_o / 1e9, 1)}}
    return res


def power_account(torch, K, dev, layers, seconds=1.2):
    """Evidence for how far the power limit, not the schedule, holds the GEMMs back: each loop below
    runs for about `seconds` while a thread polls the amdgpu driver's hwmon sensors (power1_input:
    socket power; freq1_input: the core clock the driver reports).  Loops: the four headline GEMMs through
    fmsmo_gemm_i8_i32 and through torch._int_mm (hipBLASLt), each on the step's quantized operands
    and on all-zero operands of the same shape; and the GEMM kernels' matrix instructions alone
    (fmsmo_debug_mfma_loop: registers only, every SIMD busy) on Gaussian codes and on zeros -- the
    ceiling of any schedule of those instructions on such operand bits."""
    import glob
    import threading

    power_files = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input")
                         + glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_average"))
    freq_files = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/freq1_input"))

    def sample_while(fn):
        samples, stop = [], [False]

        def poll():
            # the amdgpu driver's own sensors: socket power in microwatts, core clock in Hz
            while not stop[0]:
                try:
                    w = float(open(power_files[0]).read()) / 1e6 if power_files else None
                    mhz = float(open(freq_files[0]).read()) / 1e6 if freq_files else None
                    samples.append((w, mhz))
                except Exception as e:  # the sensors are evidence, not a dependency
                    samples.append(("error: " + str(e)[:80], None))
                    return
                time.sleep(0.02)

        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        th = threading.Thread(target=poll)
        th.start()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0, n = time.perf_counter(), 0
        e0.record()
        while time.perf_counter() - t0 < seconds:
            for _ in range(20):
                fn()
            n += 20
            torch.cuda.synchronize()
        e1.record()
        torch.cuda.synchronize()
        stop[0] = True
        th.join()
        ms = e0.elapsed_time(e1) / n
        good = [s_ for s_ in samples[len(samples) // 4:] if isinstance(s_[0], float)]   # after the ramp
        out = {"ms": round(ms, 4), "sensor_samples": len(good)}
        if good:
            out["socket_power_w"] = round(sum(s_[0] for s_ in good) / len(good), 1)
            sc = [s_[1] for s_ in good if s_[1]]
            if sc:
                out["driver_sclk_mhz"] = round(sum(sc) / len(sc))
        elif samples:
            out["sensors"] = str(samples[0][0])
        return out

    res = {}
    for (name, k, n), L_ in zip(LLAMA3_8B, layers):
        ops = 2.0 * M_TOKENS * k * n
        q, _ = K.quant_act_i8_pertoken(L_["x"], L_["smooth"])
        zq, zw = torch.zeros_like(q), torch.zeros_like(L_["w"])
        for label, a, w in (("step_operands", q, L_["w"]), ("zero_operands", zq, zw)):
            wt = w.t()
            for kname, fn in (("fmsmo_gemm_i8_i32", lambda: K.gemm_i8_i32(a, w)), ("torch_int_mm", lambda: torch._int_mm(a, wt))):
                try:
                    r = sample_while(fn)
                    r["tops"] = round(ops / r["ms"] / 1e9, 1)
                except Exception as e:
                    r = {"error": str(e)[:160]}
                res[f"{name}_{label}_{kname}"] = r
        del zq, zw
    g = torch.Generator(device=dev).manual_seed(11)
    clk = torch.zeros(2, dtype=torch.int64, device=dev)
    gauss = torch.randn(1 << 25, device=dev, generator=g)
    datas = {"i8_gaussian_sigma29": (gauss * 29).clamp_(-127, 127).round_().to(torch.int8),
             "i8_zeros": torch.zeros(1 << 25, dtype=torch.int8, device=dev),
             "e4m3_gaussian_full_range": (gauss * (448.0 / 4.5)).clamp_(-448, 448).to(torch.float8_e4m3fn),
             "e4m3_zeros": torch.zeros(1 << 25, dtype=torch.int8, device=dev).view(torch.float8_e4m3fn)}
    for label, d in datas.items():
        ops = [0.0]

        def fn():
            ops[0] = K.mfma_loop(d, 2000, clk)

        r = sample_while(fn)
        c = clk.cpu().tolist()
        r["tops"] = round(ops[0] / r["ms"] / 1e9, 1)
        r["frac_peak"] = round(ops[0] / r["ms"] / 1e9 / PEAK_INT8_TOPS, 4)
        r["core_clock_mhz"] = round(c[0] / (c[1] / 100.0)) if c[1] else None
        res["mfma_only_" + label] = r
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-fp8-decode", action="store_true",
                    help="skip the FP8 GEMM and decode rooflines (profiling runs of the INT8 step)")
    ap.add_argument("--no-decode", action="store_true", help="skip the decode rooflines only (counter runs of the FP8 GEMMs)")
    ap.add_argument("--burst", action="store_true",
                    help="time the FP8 GEMMs over twenty launches instead of 0.15 s (counter runs: every launch is slow there)")
    ap.add_argument("--no-power-account", action="store_true",
                    help="--extras without its power account (counter runs: its loops make tens of thousands of launches)")
    ap.add_argument("--extras", action="store_true",
                    help="also time the vendor GEMM, mid-size batches, MoE, chunk-truncate, side kernels")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives are part of it); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from fms_mo_amd import kernels as K

    dev = torch.device("cuda:0")
    layers = [make_layer(torch, dev, k, n, seed=1 + i) for i, (_, k, n) in enumerate(LLAMA3_8B)]
    total_ops = sum(2.0 * M_TOKENS * k * n for _, k, n in LLAMA3_8B)

    clk = [torch.zeros(6, dtype=torch.int64, device=dev) for _ in layers]

    def step(events=None):
        for i, L in enumerate(layers):
            q, s = K.quant_act_i8_pertoken(L["x"], L["smooth"])
            if events is not None:
                # block 0 of this launch stores its clock readings (core clock the GEMM ran at)
                K.clock_probe(clk[i])
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
            y = K.gemm_i8_dq(q, L["w"], s, L["w_scale"], L["bias"], out_dtype=torch.float16,
                             exact_ref=True)
            if events is not None:
                e1.record()
                events[i].append((e0, e1))
        return y

    # Counter calibration: one plain device-to-device copy of known size (256 MiB read + 256 MiB
    # written), outside the timed region.  A counter run of this same command scales the GEMM's
    # FETCH_SIZE / WRITE_SIZE readings by what the counters report for this copy.
    calib_src = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device=dev).random_(0, 255)
    calib_dst = torch.empty_like(calib_src)
    calib_dst.copy_(calib_src)
    torch.cuda.synchronize()
    del calib_src, calib_dst

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    events = [[] for _ in layers]
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(events)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    K.clock_probe(None)
    ms_per_step = dt / args.steps * 1e3
    value = total_ops / (dt / args.steps) / 1e12

    gemm_ms = [sum(a.elapsed_time(b) for a, b in ev) / len(ev) for ev in events]
    gemm_ops = [2.0 * M_TOKENS * k * n for _, k, n in LLAMA3_8B]
    per_shape = {name: round(o / (ms * 1e-3) / 1e12, 1) for (name, _, _), o, ms in zip(LLAMA3_8B, gemm_ops, gemm_ms)}
    achieved = sum(gemm_ops) / (sum(gemm_ms) * 1e-3) / 1e12
    # Core clock of block 0 of the last timed launch of each shape.  The published peak is
    # 2400 MHz x the MFMA rate; the operands' switching activity decides how far below that the
    # power cap lets the clock settle, so the peak at the measured clock is reported beside it.
    mhz = [K.core_clock_mhz(c) for c in clk]
    peak_at_clock = sum(gemm_ops) / sum(o / (PEAK_INT8_TOPS * m / 2400.0) for o, m in zip(gemm_ops, mhz))
    # HBM traffic per launch is a counter figure (two rocprofv3 --pmc runs of this command), not
    # something this process can measure: it is read from the committed profile and reported only
    # while the GEMM sources are the ones that profile was collected with
    traffic, traffic_source = None, None
    tfile = os.path.join(ROOT, "profiles", "gemm_i8_traffic.json")
    if os.path.exists(tfile):
        with open(tfile) as f:
            tj = json.load(f)
        if tj.get("gemm_sources_sha16") == gemm_sources_sha16():
            traffic = tj.get("hbm_bytes_per_launch_avg")
            traffic_source = "profiles/gemm_i8_traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of " \
                             "this command; GEMM sources unchanged since: sha16 " + tj["gemm_sources_sha16"] + ")"
        else:
            traffic_source = "profiles/gemm_i8_traffic.json is older than the GEMM sources: not reported"

    out = {
        "metric": "W8A8 INT8 linear (SmoothQuant act-quant + int8 MFMA GEMM + dequant) throughput, "
                  "Llama-3-8B decoder-layer linears, M=4096",
        "value": round(value, 2), "unit": "TOPS", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": "Llama-3-8B decoder-layer linears W8A8 INT8 + SmoothQuant(alpha=0.5), "
                               "M=4096 tokens: qkv 4096->6144, o 4096->4096, gate+up 4096->28672, "
                               "down 14336->4096; fp16 in/out, per-token act / per-channel weight scales",
                   "tokens": M_TOKENS},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 1), "peak": PEAK_INT8_TOPS,
                     "unit": "TFLOP/s", "frac": round(achieved / PEAK_INT8_TOPS, 4),
                     "traffic": traffic, "traffic_source": traffic_source, "kernel": "gemm_rs_kernel<int8, dequant epilogue> (4 launches per step)",
                     "per_shape_tops": per_shape,
                     "avg_launch_ms": {n: round(ms, 4) for (n, _, _), ms in zip(LLAMA3_8B, gemm_ms)},
                     "core_clock_mhz": {n: round(m) for (n, _, _), m in zip(LLAMA3_8B, mhz)},
                     "peak_at_measured_clock": round(peak_at_clock, 1),
                     "frac_at_measured_clock": round(achieved / peak_at_clock, 4)},
    }
    if not args.no_fp8_decode:
        out["roofline_fp8"] = fp8_rooflines(torch, K, dev, 0.0 if args.burst else 0.15)
        if not args.no_decode:
            out["roofline_decode"] = decode_rooflines(torch, K, dev)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(torch, layers)
    if args.extras:
        out["extras"] = extras(torch, K, dev, layers, power=not args.no_power_account)
    print(json.dumps(out))


def extras(torch, K, dev, layers, power=True):
    """The vendor GEMM on the same operands, mid-size batches (M in 32 .. 128), the Mixtral-style
    grouped expert GEMMs, the chunk-truncate emulation and the side kernels; reported in addition
    to the headline value and the FP8 / decode rooflines of the default run."""
    from fms_mo_amd import _lib as L

    res = {}

    def timeit(fn, iters=30, warm=5):
        return time_events(torch, fn, iters, warm)

    # the reference's CPU-runnable configuration (512 tokens through a 4096 -> 4096 linear) on the
    # GPU: SmoothQuant act-quant + int8 GEMM + dequant (512 x 4096 x 4096 splits its reduction in two)
    o_layer = layers[1]
    x512 = o_layer["x"][:512]

    def c1_step():
        q, sc = K.quant_act_i8_pertoken(x512, o_layer["smooth"])
        return K.gemm_i8_dq(q, o_layer["w"], sc, o_layer["w_scale"], o_layer["bias"], out_dtype=torch.float16,
                            exact_ref=True)

    def graph_time(fn, reps=20, replays=5):  # device time: launches replayed from a HIP graph
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            fn()
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                for _ in range(reps):
                    fn()
            graph.replay()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(replays):
                graph.replay()
            e1.record()
            torch.cuda.synchronize()
        return e0.elapsed_time(e1) / (reps * replays)

    ms_eager, ms = timeit(c1_step), graph_time(c1_step)
    res["c1_o_proj_M512"] = {"us": round(ms * 1e3, 1), "eager_us": round(ms_eager * 1e3, 1),
                             "tops": round(2.0 * 512 * 4096 * 4096 / ms / 1e9, 1)}

    # the sample the CPU baseline is timed on (first 2048 tokens through all four linears), on the GPU
    def cpu_sample_step():
        for L in layers:
            q, sc = K.quant_act_i8_pertoken(L["x"][:2048], L["smooth"])
            K.gemm_i8_dq(q, L["w"], sc, L["w_scale"], L["bias"], out_dtype=torch.float16, exact_ref=True)

    ms = timeit(cpu_sample_step)
    sample_ops = sum(2.0 * 2048 * k * n for _, k, n in LLAMA3_8B)
    res["cpu_baseline_sample_on_gpu_M2048"] = {"ms": round(ms, 4), "tops": round(sample_ops / ms / 1e9, 1)}
    res["vendor"] = vendor_int_mm(torch, K, layers)
    if power:
        res["power_account"] = power_account(torch, K, dev, layers)
    # batches of a few hundred rows (split-K territory) beside the vendor GEMM, launches replayed
    # from a HIP graph, weights rotated over > 300 MB: this library's fused-dequant GEMM, its raw
    # int32 GEMM and torch._int_mm (int32 out, no dequantization) on the same operands
    for (name, k, n), L_ in ((LLAMA3_8B[1], layers[1]), (LLAMA3_8B[3], layers[3])):
        copies = max(3, (300 * 1024 * 1024) // (k * n) + 1)
        ws = [L_["w"]] + [torch.randint(-127, 128, (n, k), dtype=torch.int8, device=dev) for _ in range(copies - 1)]
        for M in (128, 512, 1024):
            q, sc = K.quant_act_i8_pertoken(L_["x"][:M], L_["smooth"])
            row = {}
            for label, fn in (("fmsmo_gemm_i8_dq", lambda w: K.gemm_i8_dq(q, w, sc, L_["w_scale"], L_["bias"],
                                                                              out_dtype=torch.float16, exact_ref=True)),
                              ("fmsmo_gemm_i8_i32", lambda w: K.gemm_i8_i32(q, w)),
                              ("torch_int_mm", lambda w: torch._int_mm(q, w.t()))):
                try:
                    it = iter(range(10 ** 9))
                    ms = graph_time(lambda: fn(ws[next(it) % copies]), reps=2 * copies, replays=5)
                    row[label + "_us"] = round(ms * 1e3, 1)
                except Exception as e:  # the vendor path is evidence, not a dependency
                    row[label + "_us"] = str(e)[:120]
            res[f"mid_batch_M{M}_{name}"] = row
        del ws
    # batches between decode and the large GEMMs (decode kernels up to 64 tokens at K <= 4096,
    # tiled / split-K above), int8, same protocol as the decode rooflines
    mid = decode_rooflines(torch, K, dev, m_list=(32, 64, 128), ops=("i8",))
    res.update({f"decode_{k_}": v for k_, v in mid.items() if isinstance(v, dict)})
    # the four int8 GEMMs of the headline workload on all-zero operands: nothing toggles in the
    # multipliers, the clock stays up, and the figure shows how far the kernel's instruction
    # stream goes when the power limit does not hold it back
    zero_ms, zero_ops = 0.0, 0.0
    for name, k, n in LLAMA3_8B:
        qz = torch.zeros((M_TOKENS, k), dtype=torch.int8, device=dev)
        wz = torch.zeros((n, k), dtype=torch.int8, device=dev)
        sz = torch.ones(M_TOKENS, device=dev)
        wsz = torch.ones(n, device=dev)
        ms = timeit(lambda: K.gemm_i8_dq(qz, wz, sz, wsz, None, out_dtype=torch.float16, exact_ref=True), iters=10, warm=3)
        clkz = torch.zeros(6, dtype=torch.int64, device=dev)
        K.clock_probe(clkz)  # one more launch with the probe on: the clock these operands leave the part
        K.gemm_i8_dq(qz, wz, sz, wsz, None, out_dtype=torch.float16, exact_ref=True)
        K.clock_probe(None)
        torch.cuda.synchronize()
        zero_ms += ms
        zero_ops += 2.0 * M_TOKENS * k * n
        res[f"gemm_i8_zero_operands_M4096_{name}"] = {"ms": round(ms, 4), "tops": round(2.0 * M_TOKENS * k * n / ms / 1e9, 1),
                                                       "core_clock_mhz": round(K.core_clock_mhz(clkz))}
        del qz, wz
    res["gemm_i8_zero_operands_M4096_all"] = {"tops": round(zero_ops / zero_ms / 1e9, 1),
                                             "frac_peak": round(zero_ops / zero_ms / 1e9 / PEAK_INT8_TOPS, 4)}
    # a whole decode-step linear from fp16 activations (SmoothQuant divide, per-token quantizer,
    # weight-streaming matmul, dequantizing epilogue): two launches against the fused one
    for name, k, n in LLAMA3_8B:
        wbytes = k * n
        copies = max(3, (300 * 1024 * 1024 + wbytes - 1) // wbytes)
        ws_i8 = [torch.randint(-127, 128, (n, k), dtype=torch.int8, device=dev) for _ in range(copies)]
        wsc = torch.rand(n, device=dev) * 1e-3
        sm = (torch.rand(k, device=dev) + 0.5).half()
        for M in (1, 2, 4):
            x = torch.randn(M, k, device=dev).half()

            def two(w):
                q, s = K.quant_act_i8_pertoken(x, sm)
                return K.gemm_i8_dq(q, w, s, wsc, None, out_dtype=torch.float16, exact_ref=True)

            def one(w):  # the fused launch where it is served, else the same two
                if not K.decode_linear_ok(x, sm, k):
                    return two(w)
                return K.decode_linear_i8(x, w, wsc, None, sm, out_dtype=torch.float16, exact_ref=True)[0]

            us = {}
            for label, fn in (("two_launches", two), ("fused", one)):
                side = torch.cuda.Stream()
                with torch.cuda.stream(side):
                    for w in ws_i8:
                        fn(w)
                    torch.cuda.synchronize()
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph, stream=side):
                        for _ in range(3):
                            for w in ws_i8:
                                fn(w)
                    graph.replay()
                    torch.cuda.synchronize()
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                    for _ in range(5):
                        graph.replay()
                    e1.record()
                    torch.cuda.synchronize()
                us[label] = e0.elapsed_time(e1) / (5 * 3 * copies) * 1e3
                del graph
            res[f"decode_linear_fp16_in_M{M}_{name}"] = {
                "two_launches_us": round(us["two_launches"], 2), "fused_us": round(us["fused"], 2),
                "fused_GBps": round(wbytes / us["fused"] / 1e3, 1),
                "frac_hbm": round(wbytes / us["fused"] / 1e3 / PEAK_HBM_GBS, 4)}
        del ws_i8
    # Mixtral-style MoE (8 experts, 4096 tokens routed top-2 with uniform-random logits) in one
    # grouped launch per projection, and the chunk-truncate emulation on one expert's w2
    E, T, H, I = 8, 4096, 4096, 14336
    g = torch.Generator().manual_seed(4)
    flat = torch.rand(T, E, generator=g).topk(2, dim=-1).indices.reshape(-1)
    counts = torch.bincount(flat, minlength=E)
    offsets = torch.zeros(E + 1, dtype=torch.int32)
    offsets[1:] = counts.cumsum(0)
    rows = int(offsets[-1])
    off_d = offsets.to(dev)
    def codes(*shape):
        # what the quantizers emit for bell-shaped data: abs-max scaling of a few thousand Gaussian
        # values puts sigma near 127 / 4 (uniform random bytes toggle more bits than any real
        # operand and lower the clock further)
        return torch.randn(*shape, device=dev).mul_(30.0).round_().clamp_(-127, 127).to(torch.int8)

    for name, k, n in (("w1_w3", H, I), ("w2", I, H)):
        a = codes(rows, k)
        w = codes(E, n, k)
        a_s = torch.rand(rows, device=dev) * 1e-2
        w_s = torch.rand(E, n, device=dev) * 1e-3
        ms = timeit(lambda: K.grouped_gemm_i8_dq(a, w, off_d, a_s, w_s, None, out_dtype=torch.float16), iters=30, warm=5)
        tops = 2.0 * rows * k * n / (ms * 1e-3) / 1e12
        res[f"moe_grouped_i8_{name}"] = {"ms": round(ms, 4), "tops": round(tops, 1), "frac_peak": round(tops / PEAK_INT8_TOPS, 4),
                                         "rows_per_expert": counts.tolist()}
        del a, w
    m_e = int(counts[0])
    a = codes(m_e, I)
    w = codes(H, I)
    for t in (7, 16):
        ms = timeit(lambda: K.matmul_chunk(a, w, chunk_size=64, chunk_trun_bits=t), iters=10, warm=3)
        tops = 2.0 * m_e * I * H / (ms * 1e-3) / 1e12
        res[f"chunk64_trunc{t}_i8_w2_M{m_e}"] = {"ms": round(ms, 4), "tops": round(tops, 1), "frac_peak": round(tops / PEAK_INT8_TOPS, 4)}
    # the same on 4096 rows (1024 tiles of 128 x 128: whole rounds over the compute units, where one
    # expert's 1069 rows make 288 tiles for 256 units), chunk sizes 32 / 64 / 128
    a4 = codes(4096, I)
    for cs in (32, 64, 128):
        ms = timeit(lambda: K.matmul_chunk(a4, w, chunk_size=cs, chunk_trun_bits=7), iters=10, warm=3)
        tops = 2.0 * 4096 * I * H / (ms * 1e-3) / 1e12
        res[f"chunk{cs}_trunc7_i8_w2_M4096"] = {"ms": round(ms, 4), "tops": round(tops, 1), "frac_peak": round(tops / PEAK_INT8_TOPS, 4)}
    del a4
    # the steps either side of the hot path: offline weight quantizer, SmoothQuant statistics, the
    # accelerator op's quantizer (HBM bound; inputs rotated so the Infinity Cache cannot hold them)
    # and the accelerator op end to end
    n, k = 28672, 4096
    ws = [(0.02 * torch.randn(n, k, device=dev)).half() for _ in range(2)]
    coef = (127.0 / ws[0].float().abs().amax(dim=1)).float()
    smooth = (torch.rand(k, device=dev) + 0.5).half()
    it = iter(range(10 ** 9))
    ms = timeit(lambda: K.quant_weight_i8(ws[next(it) % 2], coef, smooth=smooth, mode="mul", want_row_sum=True), iters=10, warm=2)
    gbs = n * k * 3 / (ms * 1e-3) / 1e9
    res["offline_weight_quant_fp16_gate_up"] = {"ms": round(ms, 4), "GBps": round(gbs, 1), "frac_hbm": round(gbs / PEAK_HBM_GBS, 4)}
    del ws
    M, k = 4096, 14336
    xs = [torch.randn(M, k, device=dev).half() for _ in range(3)]
    run = torch.zeros(k, device=dev)
    ms = timeit(lambda: K.absmax_cols(xs[next(it) % 3], run), iters=12, warm=3)
    gbs = M * k * 2 / (ms * 1e-3) / 1e9
    res["smoothquant_stats_absmax_cols_M4096_K14336"] = {"us": round(ms * 1e3, 1), "GBps": round(gbs, 1), "frac_hbm": round(gbs / PEAK_HBM_GBS, 4)}
    sm = (torch.rand(k, device=dev) + 0.5).half()
    clip = torch.tensor([3.0, -2.0], device=dev).half()
    for mode, label in ((L.MS_PER_TOKEN, "per_token"), (L.MS_ASYMM, "per_tensor_asymm")):
        ms = timeit(lambda: K.quant_act_i8_mulscale(xs[next(it) % 3], mode, clip=None if mode == L.MS_PER_TOKEN else clip, smooth=sm), iters=12, warm=3)
        gbs = M * k * 3 / (ms * 1e-3) / 1e9
        res[f"aiu_act_quant_{label}_smooth_M4096_K14336"] = {"us": round(ms * 1e3, 1), "GBps": round(gbs, 1), "frac_hbm": round(gbs / PEAK_HBM_GBS, 4)}
    # the deploy module's static quantizers in the module's 16-bit dtype (clip values from
    # calibration: qa_fmo_mo_qfunc, the default when the dynamic quantizer is not asked for,
    # and qa_raw_qfunc)
    step = float(torch.tensor(5.0 / 255).half())
    for mode, label, args in ((L.SQ_FMO, "fmo_mo", (step, -102.0, 0, -2.0, 3.0)), (L.SQ_RAW, "raw", (step, 102.0, 0))):
        ms = timeit(lambda: K.quant_act_i8_static_t(xs[next(it) % 3], mode, torch.float16, *args), iters=12, warm=3)
        gbs = M * k * 3 / (ms * 1e-3) / 1e9
        res[f"static_act_quant_{label}_fp16_M4096_K14336"] = {"us": round(ms * 1e3, 1), "GBps": round(gbs, 1), "frac_hbm": round(gbs / PEAK_HBM_GBS, 4)}
    from fms_mo_amd.aiu_addons.i8i8.i8i8_aiu_op import i8i8_aiu
    n = 4096
    w = torch.randint(-127, 128, (n, k), dtype=torch.int8, device=dev)
    bias = torch.zeros(n, device=dev).half()
    for act in ("per_token", "per_tensor_asymm"):
        zs = torch.zeros(n if act == "per_tensor_asymm" else 1, device=dev).half()
        qdata = torch.cat((torch.full((n,), 0.3, device=dev).half(), torch.full((n,), -0.3, device=dev).half(), clip, zs, sm))
        ms = timeit(lambda: i8i8_aiu(xs[0], w, bias, qdata, "per_channel", act, True), iters=10, warm=3)
        tops = 2.0 * M * k * n / (ms * 1e-3) / 1e12
        res[f"i8i8_aiu_op_{act}_down_M4096"] = {"ms": round(ms, 4), "tops": round(tops, 1), "frac_peak": round(tops / PEAK_INT8_TOPS, 4)}
    # attention matmuls of one Llama-3-8B sequence (32 heads, head dimension 128, 4096 tokens):
    # with K or N of 128 these are HBM bound (the score matrix dominates the bytes)
    h, sq, d = 32, 4096, 128
    qi = torch.randint(-128, 128, (h, sq, d), dtype=torch.int8, device=dev)
    ki = torch.randint(-128, 128, (h, sq, d), dtype=torch.int8, device=dev)
    one = torch.full((1,), 1e-3, device=dev)
    ms = timeit(lambda: K.bmm_i8_dq(qi, ki, one, one, out_dtype=torch.float16), iters=10, warm=3)
    byts = 2 * h * sq * d + h * sq * sq * 2
    res["attn_bmm_i8_qk_S4096"] = {"ms": round(ms, 4), "tops": round(2.0 * h * sq * sq * d / ms / 1e9, 1),
                                   "GBps": round(byts / ms / 1e6, 1), "frac_hbm": round(byts / ms / 1e6 / PEAK_HBM_GBS, 4)}
    pi = torch.randint(0, 128, (h, sq, sq), dtype=torch.int8, device=dev)
    vt = torch.randint(-128, 128, (h, d, sq), dtype=torch.int8, device=dev)
    ms = timeit(lambda: K.bmm_i8_dq(pi, vt, one, one, out_dtype=torch.float16), iters=10, warm=3)
    byts = h * sq * sq + h * sq * d + h * sq * d * 2
    res["attn_bmm_i8_pv_S4096"] = {"ms": round(ms, 4), "tops": round(2.0 * h * sq * sq * d / ms / 1e9, 1),
                                   "GBps": round(byts / ms / 1e6, 1), "frac_hbm": round(byts / ms / 1e6 / PEAK_HBM_GBS, 4)}
    del pi
    pf = torch.rand(h, sq, sq, device=dev).half()
    # the quantizer's scale is a tensor of the compute dtype in the module, i.e. an fp16 value here
    s_p = float(torch.tensor(1.0 / 127).half())
    s_v = float(torch.tensor(0.03).half())
    ms = timeit(lambda: K.quant_i8_affine(pf, s_p, -64.0, torch.float16), iters=5, warm=2)
    byts = h * sq * sq * 3
    res["attn_quant_scores_fp16_S4096"] = {"ms": round(ms, 4), "GBps": round(byts / ms / 1e6, 1), "frac_hbm": round(byts / ms / 1e6 / PEAK_HBM_GBS, 4)}
    vf = torch.randn(h, sq, d, device=dev).half()
    ms = timeit(lambda: K.quant_i8_affine(vf, s_v, 0.0, torch.float16, transpose=True), iters=10, warm=3)
    byts = h * sq * d * 3
    res["attn_quant_v_transposed_fp16_S4096"] = {"us": round(ms * 1e3, 1), "GBps": round(byts / ms / 1e6, 1), "frac_hbm": round(byts / ms / 1e6 / PEAK_HBM_GBS, 4)}
    return res


if __name__ == "__main__":
    main()
