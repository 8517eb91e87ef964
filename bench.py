#!/usr/bin/env python3
"""Headline benchmark: W4A16 g128 fused dequant-GEMM on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras]

A step is one decode pass (M = 1) through the 224 quantised linears of a 32-layer Llama-2-7B-shaped decoder
(per layer q/k/v/o 4096x4096, gate/up 4096->11008, down 11008->4096; 4-bit, group 128), inputs resident in
HBM: --layers distinct layers' weights (8: 860 MB, more than the 256 MiB Infinity Cache holds) are run through
32 / layers times.  `value` is algorithmic bytes per step (packed weights + scales + zero points + activations
in + out) over the time per step, in GB/s.  A step is one HIP graph of 224 launches, so the Python
interpreter is not what is being timed; the default 100 steps (after 20 warm-ups) last about 110 ms.

Also reported on the same JSON line: the roofline of the decode kernel (overall and per layer shape, next to
this board's measured stream-copy rate), the CPU path timed on the host cores, and (unless --no-extras)
per-M decode rates, prefill TFLOP/s next to same-run fp16 hipBLASLt, quantiser rates and the end-to-end decoder.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
MODEL_LAYERS = 32          # decoder layers a headline step stands for (Llama-2-7B)
MFMA_F16_PEAK_TFLOPS = 2500.0
LLAMA7B_LINEARS = [("q_proj", 4096, 4096), ("k_proj", 4096, 4096), ("v_proj", 4096, 4096), ("o_proj", 4096, 4096),
                   ("gate_proj", 4096, 11008), ("up_proj", 4096, 11008), ("down_proj", 11008, 4096)]   # name, K, N


def decode_bytes(m, k, n, bits, g):
    """Algorithmic bytes of one fused forward: packed weights + scale + zero point + x + y (no bias)."""
    return n * k * bits // 8 + 2 * n * (k // g) * 2 + m * k * 2 + m * n * 2


def make_layer(torch, QuantizedLinear, k, n, bits, g, seed, outliers=False):
    gen = torch.Generator(device="cuda").manual_seed(seed)
    w = torch.randn(n, k, device="cuda", generator=gen) * 0.02
    if outliers:
        w = torch.where(torch.rand(n, k, device="cuda", generator=gen) < 0.001, w * 10, w)
    lin = torch.nn.Linear(k, n, bias=False, device="cuda", dtype=torch.float16)
    lin.weight.data = w.half()
    q = QuantizedLinear.from_float(lin, bits, g)
    del lin, w
    return q


def time_calls(torch, fn, iters, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / iters      # us per call


def time_alternating(torch, fns, iters, warmup, rounds=3):
    """Median over `rounds` of time_calls for each of `fns`, the functions taking turns within a round: clocks and
    power state drift over a run of large GEMMs, and a figure and the one it is compared with should see the same drift."""
    for fn in fns:
        for _ in range(warmup):
            fn()
    runs = [[time_calls(torch, fn, iters, 2) for fn in fns] for _ in range(rounds)]
    return [sorted(r[i] for r in runs)[rounds // 2] for i in range(len(fns))]


def graph_of(torch, fn):
    g = torch.cuda.CUDAGraph()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        fn()                                       # warm the launch path outside capture
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    with torch.cuda.graph(g):
        fn()
    return g


def _cpu_info():
    model, cores = "unknown", set()
    try:
        phys = core = None
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name") and model == "unknown":
                model = line.split(":", 1)[1].strip()
            elif line.startswith("physical id"):
                phys = line.split(":", 1)[1].strip()
            elif line.startswith("core id"):
                core = line.split(":", 1)[1].strip()
            elif not line.strip():
                if core is not None:
                    cores.add((phys, core))
                phys = core = None
    except OSError:
        pass
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = os.cpu_count() or 1
    return model, len(cores) or (os.cpu_count() or 1), usable


def cpu_baseline():
    """The reference's CPU path on this host: oracle/torch_cpu_path.py, the eager-torch restatement of
    bitween/functional.py:3-71 + the module's float16 stores + main.py:462-466, on the one configuration that runs on
    the CPU (an OPT-125m fc1: 768 -> 3072, 4-bit g128, M = 1 and 16), timed as the reference times things
    (bitween/benchmark.py:191-218: 10 warm-ups, 50 runs, perf_counter) with torch's default thread count and with 1
    thread.  `value` = algorithmic bytes of the M = 1 forward over its time at the default thread count.  A second
    entry times the scalar C port (oracle/rtn_oracle.c, OpenMP) on one 4096 x 4096 layer."""
    import numpy as np
    import torch
    from oracle import c_oracle, rtn_oracle as orc, torch_cpu_path as tcp
    k, n, bits, g = 768, 3072, 4, 128
    gen = torch.Generator().manual_seed(0)
    w16 = (torch.randn(n, k, generator=gen) * 0.02).half()
    xs = {m: torch.randn(m, k, generator=gen).half() for m in (1, 16)}
    qw, s16, z16 = tcp.module_buffers(w16, bits, g)

    def timed(fn):
        for _ in range(10):
            fn()
        t0 = time.perf_counter()
        for _ in range(50):
            fn()
        return (time.perf_counter() - t0) / 50 * 1e3

    model, physical, usable = _cpu_info()
    default_threads = torch.get_num_threads()
    legs = {}
    for label, threads in (("default_threads", default_threads), ("1_thread", 1)):
        torch.set_num_threads(threads)
        legs[label] = {"torch_threads": torch.get_num_threads(),
                       "quantize_pack_ms": round(timed(lambda: tcp.module_buffers(w16, bits, g)), 3),
                       "forward_M1_ms": round(timed(lambda: tcp.forward(xs[1], qw, s16, z16, None, bits, g)), 3),
                       "forward_M16_ms": round(timed(lambda: tcp.forward(xs[16], qw, s16, z16, None, bits, g)), 3)}
    torch.set_num_threads(default_threads)
    # the scalar C port on one Llama-sized layer (what the GPU headline runs 224 of per step)
    kk = nn = 4096
    rng = np.random.default_rng(0)
    wl = (rng.standard_normal((nn, kk)) * 0.02).astype(np.float16).astype(np.float32)
    qwl, sl, zl = c_oracle.quantize_rtn_f32(wl, bits, g)
    sl16, zl16 = orc.store_module_buffers(sl, zl)
    xl = rng.standard_normal((1, kk)).astype(np.float16)
    c_oracle.qlinear_forward(xl, qwl, sl16, zl16, None, bits, g)
    t0, reps = time.perf_counter(), 0
    while time.perf_counter() - t0 < 4.0:
        c_oracle.qlinear_forward(xl, qwl, sl16, zl16, None, bits, g)
        reps += 1
    c_ms = (time.perf_counter() - t0) / reps * 1e3
    omp = int(os.environ.get("OMP_NUM_THREADS", usable))
    # the eager-torch path on the same Llama-sized layer (one of the 224 launches of a GPU step): 3 warm-ups + 20 runs
    wl16 = torch.from_numpy(wl).half()
    qwt, st16, zt16 = tcp.module_buffers(wl16, bits, g)
    xt = torch.from_numpy(xl)
    for _ in range(3):
        tcp.forward(xt, qwt, st16, zt16, None, bits, g)
    t0 = time.perf_counter()
    for _ in range(20):
        tcp.forward(xt, qwt, st16, zt16, None, bits, g)
    llama_ms = (time.perf_counter() - t0) / 20 * 1e3
    return {"value": round(decode_bytes(1, kk, nn, bits, g) / (llama_ms * 1e-3) / 1e9, 3), "unit": "GB/s",
            "cores": default_threads, "kind": "port",
            "sample": "one Llama-2-7B q_proj (4096 x 4096, W4 g128, M = 1: the most frequent launch of a GPU step), the "
                      "reference's forward as eager torch on the host (oracle/torch_cpu_path.py: dequantize_rtn -> "
                      "float16 -> matmul), 3 warm-ups + 20 runs at torch's default thread count; value = algorithmic "
                      "bytes of that forward over its time.  Extra entries: the OPT-125m fc1 configuration (768 -> 3072, "
                      "10 warm-ups + 50 runs of quantize+pack and of the forward at M = 1 / 16, default threads and 1 "
                      "thread) and the scalar C restatement (OpenMP) on the same 4096 x 4096 layer",
            "llama7b_q_proj_torch_cpu_forward_ms": round(llama_ms, 2),
            "cpu_model": model, "physical_cores": physical, "usable_cpus": usable,
            "opt125m_fc1_torch_cpu": legs,
            "c_port_4096x4096_M1": {"forward_ms": round(c_ms, 2), "GBps": round(decode_bytes(1, kk, nn, bits, g) / c_ms / 1e6, 3),
                                    "omp_threads": omp, "runs": reps}}


TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "qgemv_w4g128_llama7b_decode_M1_hbm_traffic.txt")


def profiled_traffic(kernels, m):
    """HBM bytes per launch of the headline step from the committed rocprofv3 counter summary, or None (with the
    reason) when that summary was taken on other kernels than the ones dispatched now, or for another M."""
    if m != 1:
        return None, "the counter profile covers M = 1 only"
    try:
        text = open(TRAFFIC_PROFILE).read()
    except OSError:
        return None, "profiles/qgemv_w4g128_llama7b_decode_M1_hbm_traffic.txt is not present"
    fields = {}
    for line in text.splitlines():
        if line.startswith("machine:"):
            key, _, value = line[len("machine:"):].strip().partition("=")
            fields[key.strip()] = value.strip()
    profiled = sorted(v.strip() for v in fields.get("kernels", "").split(";") if v.strip())
    if profiled != sorted(set(kernels.values())):
        return None, "the counter profile covers %s, the library now dispatches %s: re-profile" % (profiled, sorted(set(kernels.values())))
    return int(fields["traffic_bytes_per_launch"]), "rocprofv3 FETCH_SIZE / WRITE_SIZE, scaled by a device copy of known size (profiles/)"


def copy_probe(torch):
    """This board's stream-copy rate: a 1 GiB device-to-device copy (read + write bytes over device time)."""
    src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").fill_(1)
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    us = time_calls(torch, lambda: dst.copy_(src), 10, 2)
    del src, dst
    return round(2 * (1 << 30) / us / 1e3, 1)


# ---- extras: every section takes (torch, hip, QuantizedLinear, layers) and returns a JSON-able dict; `layers`
# are the headline's rotating W4 g128 layer copies --------------------------------------------------------------

def extras_decode(torch, hip, QuantizedLinear, layers):
    """Decode for every Llama-2-7B shape and M (graph replay, device time per call), rotating over enough copies
    of the one shape to exceed the 256 MiB Infinity Cache."""
    bits, g, out = 4, 128, {}
    for idx, (name, k, n) in enumerate(LLAMA7B_LINEARS):
        if name in ("k_proj", "v_proj", "o_proj", "up_proj"):
            continue
        copies = [layer[idx] for layer in layers]
        while len(copies) * n * k * bits // 8 < (320 << 20):
            copies.append(make_layer(torch, QuantizedLinear, k, n, bits, g, seed=1000 + len(copies)))
        for mm in (1, 2, 4, 8, 16):
            x = torch.randn(mm, k, device="cuda", dtype=torch.float16)
            reps = max(1, 96 // len(copies))                  # >= 96 launches per replay: graph launch cost amortised
            gr = graph_of(torch, lambda: [hip.quantized_gemv_hip(x, q.qweight, q.scale, q.zero_point, None, bits, g)
                                          for _ in range(reps) for q in copies])
            us = time_calls(torch, gr.replay, 10, 2) / (reps * len(copies))
            out[f"{name}_{k}x{n}_M{mm}"] = {"us": round(us, 2), "GBps": round(decode_bytes(mm, k, n, bits, g) / us / 1e3, 1)}
        del copies
    return out


def extras_decode_hot(torch, hip, QuantizedLinear, layers):
    """The same launches on one layer copy over and over: weights come from the 256 MiB Infinity Cache, not HBM."""
    bits, g, out = 4, 128, {}
    for idx, (name, k, n) in enumerate(LLAMA7B_LINEARS):
        if name in ("k_proj", "v_proj", "o_proj", "up_proj"):
            continue
        x = torch.randn(1, k, device="cuda", dtype=torch.float16)
        q = layers[0][idx]
        gr = graph_of(torch, lambda: [hip.quantized_gemv_hip(x, q.qweight, q.scale, q.zero_point, None, bits, g) for _ in range(96)])
        us = time_calls(torch, gr.replay, 10, 2) / 96
        out[f"{name}_{k}x{n}_M1"] = {"us": round(us, 2), "GBps": round(decode_bytes(1, k, n, bits, g) / us / 1e3, 1)}
    return out


def extras_decode_other_formats(torch, hip, QuantizedLinear, layers):
    """K=4096 -> N=11008 at 8-bit g128, 4-bit g64, 2-bit g32 (weights with 0.1 % outliers x10), M = 1 and 16; and the
    8-bit attention linears of the mixed recipe: 4096 x 4096 and the fused q/k/v launch (N = 12288)."""
    out = {}
    for bits, g, k, n in ((8, 128, 4096, 11008), (4, 64, 4096, 11008), (2, 32, 4096, 11008), (8, 128, 4096, 4096), (8, 128, 4096, 12288)):
        copies = (320 << 20) // (n * k * bits // 8) + 1          # > 256 MiB of packed weights in rotation
        qs = [make_layer(torch, QuantizedLinear, k, n, bits, g, seed=31 * bits + i, outliers=True) for i in range(copies)]
        for mm in (1, 16):
            x = torch.randn(mm, k, device="cuda", dtype=torch.float16)
            reps = 96 // copies
            gr = graph_of(torch, lambda: [hip.quantized_gemv_hip(x, q.qweight, q.scale, q.zero_point, None, bits, g)
                                          for _ in range(reps) for q in qs])
            us = time_calls(torch, gr.replay, 10, 2) / (reps * copies)
            out[f"w{bits}g{g}_{k}x{n}_M{mm}"] = {"us": round(us, 2), "GBps": round(decode_bytes(mm, k, n, bits, g) / us / 1e3, 1)}
        del qs
    return out


def extras_hipblaslt_decode(torch, hip, QuantizedLinear, layers):
    """Same-run fp16 hipBLASLt GEMV on dequantised weights (reads 4x the bytes)."""
    out = {}
    for name, k, n in (("q_proj", 4096, 4096), ("gate_proj", 4096, 11008)):
        ws = [torch.randn(n, k, device="cuda", dtype=torch.float16) for _ in range(12)]
        x = torch.randn(1, k, device="cuda", dtype=torch.float16)
        gr = graph_of(torch, lambda: [torch.matmul(x, w.T) for _ in range(8) for w in ws])
        us = time_calls(torch, gr.replay, 10, 2) / (8 * len(ws))
        out[f"{name}_{k}x{n}_M1"] = {"us": round(us, 2), "fp16_GBps": round(2 * n * k / us / 1e3, 1)}
        del ws
    return out


def sclk_under_load(torch, fn, seconds=0.4, batch=200):
    """Mean / min of the driver's current shader clock (sysfs pp_dpm_sclk, MHz) sampled while batches of `fn` are in
    flight; None where the file is absent or unreadable.  A slow average that includes the gaps between launches:
    it ranks loads, the in-kernel counters of board_probes measure one."""
    import glob
    import re
    import time
    files = glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk")
    if len(files) != 1:
        return None            # no file, or several cards and no way to tell which one is this process's
    def read():
        try:
            for line in open(files[0]).read().split("\n"):
                if "*" in line:
                    m = re.search(r"(\d+)\s*[Mm]hz", line)
                    if m:
                        return int(m.group(1))
        except OSError:
            pass
        return None
    torch.cuda.synchronize()
    samples, t_end = [], time.time() + seconds
    while time.time() < t_end:
        for _ in range(batch):
            fn()
        v = read()                                     # taken with the batch still in flight
        torch.cuda.synchronize()
        if v is None:
            return None
        samples.append(v)
    samples = samples[2:] or samples
    return {"mean_MHz": round(sum(samples) / len(samples)), "min_MHz": min(samples), "samples": len(samples)}


def extras_prefill(torch, hip, QuantizedLinear, layers):
    """Prefill on the Llama-3-8B MLP shapes, W4 g128, next to fp16 hipBLASLt on the dequantised weights.  `us` is
    the kernel on float16 x; `bf16_x_us` the forward on bfloat16 x (cast + split-K workspace + kernel); `tile_rows` the
    output tile the library picked (128 or 256 rows).  Every figure is the median of three rounds in which the kernels
    take turns."""
    bits, g, out = 4, 128, {}
    for k, n in ((4096, 14336), (14336, 4096)):
        q = make_layer(torch, QuantizedLinear, k, n, bits, g, seed=7)
        w16 = hip.dequantize(q.qweight, q.scale, q.zero_point, g, bits, torch.float16)
        for mm in (128, 512, 2048):
            x = torch.randn(mm, k, device="cuda", dtype=torch.float16)
            # the configuration names bfloat16 activations: the reference's forward casts them to float16
            # (bitween/modules.py:74) and so does this one, in a pass of its own ahead of the prefill kernel
            xb = x.to(torch.bfloat16)
            us_q, us_b, us_qb = time_alternating(torch, [
                lambda: hip.quantized_gemm_hip(x, q.qweight, q.scale, q.zero_point, None, bits, g),
                lambda: torch.matmul(x, w16.T),
                lambda: hip.quantized_matmul_hip(xb, q.qweight, q.scale, q.zero_point, None, bits, g)], 20, 10)
            fl = 2.0 * mm * n * k
            out[f"{k}x{n}_M{mm}"] = {"us": round(us_q, 1), "bf16_x_us": round(us_qb, 1), "TFLOPs": round(fl / us_q / 1e6, 1),
                                     "tile_rows": hip.load().bw_qgemm_tile_rows(mm, n, k, bits, g),
                                     "pct_mfma_f16_peak": round(100 * fl / us_q / 1e6 / MFMA_F16_PEAK_TFLOPS, 1),
                                     "hipblaslt_fp16_us": round(us_b, 1), "hipblaslt_fp16_TFLOPs": round(fl / us_b / 1e6, 1),
                                     "frac_of_hipblaslt": round(us_b / us_q, 3)}
            if (k, n, mm) == (4096, 14336, 2048):
                # both kernels run this shape at the part's power limit: the clock each is allowed
                out["sclk_under_load_4096x14336_M2048"] = {
                    "this_kernel": sclk_under_load(torch, lambda: hip.quantized_gemm_hip(x, q.qweight, q.scale, q.zero_point, None, bits, g)),
                    "hipblaslt_fp16": sclk_under_load(torch, lambda: torch.matmul(x, w16.T))}
        del q, w16
    return out


def extras_prefill_clock(torch, hip, QuantizedLinear, layers):
    """The shader clock inside the prefill kernel.  The measurement build of the library (python -m
    bitween_amd.csrc.build --tune) lets workgroups 0..255 of a launch leave the core-clock ticks and the real-time
    ticks of their K loop in a buffer; ticks / ticks x the real-time rate is the clock the part allowed under that
    load, cycles / MFMAs how close the loop is to the bare MFMA stream (board_probes: 18.4 cycles per MFMA and wave
    at 2.27 GHz with nothing else going on).  `us` is the whole call of the measurement build, for orientation."""
    import ctypes
    from bitween_amd.csrc import build as hip_build
    if not os.path.exists(hip_build.TUNE_LIB):
        return {"skipped": "libbitween_hip_tune.so is not built (python -m bitween_amd.csrc.build --tune)"}
    lib = ctypes.CDLL(hip_build.TUNE_LIB)
    vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    lib.bw_abi_version.restype = i32
    if lib.bw_abi_version() != hip.ABI_VERSION:
        return {"skipped": "libbitween_hip_tune.so is stale (ABI %d): rebuild it" % lib.bw_abi_version()}
    lib.bw_qgemm_ws.argtypes = [vp, i32, i64, i64, i64, vp, vp, vp, vp, i64, i32, i32, vp, i64, vp, ctypes.c_size_t, vp]
    lib.bw_qgemm_ws.restype = i32
    lib.bw_qgemm_workspace_bytes.argtypes, lib.bw_qgemm_workspace_bytes.restype = [i64, i64, i64, i32, i32], ctypes.c_size_t
    lib.bw_qgemm_tile_rows.argtypes, lib.bw_qgemm_tile_rows.restype = [i64, i64, i64, i32, i32], i32
    lib.bw_tune_clock_buffer.argtypes = [vp]
    # the real-time counter's rate: 100 MHz on this part (hipDeviceAttributeWallClockRate); torch does not expose it
    tick_hz = 100e6
    clk = torch.zeros(512, device="cuda", dtype=torch.int64)
    out = {}
    stream = torch.cuda.current_stream().cuda_stream
    for bits, g, k, n, mm in ((4, 128, 4096, 8192, 2048), (4, 128, 4096, 14336, 2048), (4, 128, 14336, 4096, 2048), (4, 128, 4096, 14336, 512),
                              (4, 128, 4096, 14336, 128), (8, 128, 4096, 14336, 2048), (2, 32, 4096, 14336, 2048)):
        q = make_layer(torch, QuantizedLinear, k, n, bits, g, seed=7)
        x = torch.randn(mm, k, device="cuda", dtype=torch.float16)
        y = torch.empty(mm, n, device="cuda", dtype=torch.float16)
        ws = torch.empty(max(16, lib.bw_qgemm_workspace_bytes(mm, n, k, bits, g)), device="cuda", dtype=torch.uint8)
        def call():
            st = lib.bw_qgemm_ws(x.data_ptr(), 0, mm, k, k, q.qweight.data_ptr(), q.scale.data_ptr(), q.zero_point.data_ptr(), None, n, bits, g,
                                 y.data_ptr(), n, ws.data_ptr(), ws.numel(), stream)
            assert st == 0, st
        lib.bw_tune_clock_buffer(None)
        us = min(time_calls(torch, call, 20, 30) for _ in range(2))    # (the first large GEMMs of a fresh process run slow)
        clk.zero_()
        lib.bw_tune_clock_buffer(clk.data_ptr())
        for _ in range(30):
            call()
        torch.cuda.synchronize()
        lib.bw_tune_clock_buffer(None)
        d = clk.cpu().view(256, 2).double()
        d = d[d[:, 1] > 0]
        rows = lib.bw_qgemm_tile_rows(mm, n, k, bits, g)
        # MFMAs of one wave in a whole-K loop: (rows / 16) x 4 tiles x K / 32
        mfmas = rows // 16 * 4 * k // 32
        cycles = d[:, 0].mean().item()
        out[f"w{bits}g{g}_{k}x{n}_M{mm}"] = {"us": round(us, 1), "tile_rows": rows, "k_loop_us": round(d[:, 1].mean().item() / tick_hz * 1e6, 1),
                                           "shader_clock_GHz": round((d[:, 0] / d[:, 1]).mean().item() * tick_hz / 1e9, 3),
                                           "k_loop_kcycles": round(cycles / 1e3, 1), "cycles_per_mfma": round(cycles / mfmas, 1)}
        del q, x, y, ws
    out["note"] = ("workgroups of split tiles run a slice of K: their cycles_per_mfma reads low where the first 256 workgroups "
                   "include them (M = 128)")
    return out


def extras_prefill_other_formats(torch, hip, QuantizedLinear, layers):
    """Prefill at the other widths of the mixed-precision recipe (attention int8 g128, four down_proj int2 g32) and
    int4 g64, 4096 -> 14336, against the same fp16 hipBLASLt GEMM."""
    out, k, n = {}, 4096, 14336
    for bits, g in ((8, 128), (4, 64), (2, 32)):
        q = make_layer(torch, QuantizedLinear, k, n, bits, g, seed=7)
        w16 = hip.dequantize(q.qweight, q.scale, q.zero_point, g, bits, torch.float16)
        for mm in (512, 2048):
            x = torch.randn(mm, k, device="cuda", dtype=torch.float16)
            # 30 untimed calls of each first: the first large GEMMs of a fresh process run ~18 % slow (clocks, first touch
            # of the workspace), whichever kernel they are
            us_q, us_b = time_alternating(torch, [lambda: hip.quantized_gemm_hip(x, q.qweight, q.scale, q.zero_point, None, bits, g),
                                                  lambda: torch.matmul(x, w16.T)], 20, 30)
            fl = 2.0 * mm * n * k
            out[f"w{bits}g{g}_{k}x{n}_M{mm}"] = {"us": round(us_q, 1), "TFLOPs": round(fl / us_q / 1e6, 1),
                                                 "tile_rows": hip.load().bw_qgemm_tile_rows(mm, n, k, bits, g),
                                                 "hipblaslt_fp16_us": round(us_b, 1), "frac_of_hipblaslt": round(us_b / us_q, 3)}
        del q, w16
    return out


def extras_quantize(torch, hip, QuantizedLinear, layers):
    """Quantiser: fp16 weights in, packed words + fp16 scale / zero point out (the from_float path)."""
    out = {}
    for bits, g in ((4, 128), (8, 128), (2, 32)):
        k, n = 4096, 11008
        ws = [(torch.randn(n, k, device="cuda") * 0.02).half() for _ in range(6)]
        # graph replay: the Python call (three output allocations, ctypes) costs as much as the kernel
        gr = graph_of(torch, lambda: [hip.quantize_pack(w, bits, g, torch.float32, torch.float16, torch.float16)
                                      for _ in range(4) for w in ws])
        us = time_calls(torch, gr.replay, 10, 2) / 24
        by = n * k * (2 + bits / 8 + 4 / g)
        out[f"w{bits}g{g}_{k}x{n}_f16_in"] = {"us": round(us, 1), "GBps": round(by / us / 1e3, 1),
                                             "pct_hbm_peak": round(100 * by / us / 1e3 / HBM_PEAK_GBPS, 1),
                                             "Gweights_per_s": round(n * k / us / 1e3, 1)}
        del ws
    return out


def extras_mixed_precision_model(torch, hip, QuantizedLinear, layers):
    """The linears of a 32-layer, hidden-4096, MLP-11008 decoder with the mixed recipe: attention 8-bit g128,
    gate/up/down 4-bit g128, down_proj of layers 0, 1, 30, 31 2-bit g32.  Reports the time to quantise all of
    them (13 GB of fp16 in) and the time of one decode token through all of them (M = 1, one HIP graph, nothing but the
    quantised linears: no attention, norms, embeddings or lm_head), next to fp16 hipBLASLt on the same shapes."""
    nlayers, low = 32, (0, 1, 30, 31)
    gen = torch.Generator(device="cuda").manual_seed(5)
    plan = []
    for li in range(nlayers):
        for name, k, n in LLAMA7B_LINEARS:
            if name in ("q_proj", "k_proj", "v_proj", "o_proj"):
                plan.append((k, n, 8, 128))
            elif name == "down_proj" and li in low:
                plan.append((k, n, 2, 32))
            else:
                plan.append((k, n, 4, 128))
    # quantise: one launch per linear, every linear its own fp16 weights (13 GB in all: nothing is cache-resident).
    # The first pass only warms torch's allocator (4.3 GB of fresh hipMalloc would otherwise be what is timed).
    srcs = [torch.empty(n, k, device="cuda", dtype=torch.float16).normal_(0, 0.02, generator=gen) for k, n, _, _ in plan]
    for timed in (False, True):
        packed = None
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        packed = [hip.quantize_pack(w, b, g, torch.float32, torch.float16, torch.float16) for w, (k, n, b, g) in zip(srcs, plan)]
        e1.record()
        torch.cuda.synchronize()
        quant_ms = e0.elapsed_time(e1)
    del srcs
    weights = sum(k * n for k, n, _, _ in plan)
    xs = {k: torch.randn(1, k, device="cuda", dtype=torch.float16) for k in (4096, 11008)}
    gr = graph_of(torch, lambda: [hip.quantized_gemv_hip(xs[k], qw, s, z, None, b, g)
                                  for (k, n, b, g), (qw, s, z) in zip(plan, packed)])
    tok_us = time_calls(torch, gr.replay, 20, 3)
    by = sum(decode_bytes(1, k, n, b, g) for k, n, b, g in plan)
    del gr
    # the same token with q/k/v and gate/up sharing a launch (fuse_sibling_linears): 7 module calls, 4 launches per layer
    import bitween_amd
    names = [nm for nm, _, _ in LLAMA7B_LINEARS]
    blocks = []
    for li in range(nlayers):
        blk = torch.nn.Module()
        for j, nm in enumerate(names):
            k, n, b, g = plan[li * 7 + j]
            q = QuantizedLinear(k, n, bits=b, group_size=g, bias=False)
            q._buffers["qweight"], q._buffers["scale"], q._buffers["zero_point"] = packed[li * 7 + j]
            setattr(blk, nm, q)
        bitween_amd.fuse_sibling_linears(blk)
        blocks.append(blk)
    del packed

    def fused_token():
        with torch.no_grad():
            for blk in blocks:
                xa, xo, xm, xd = xs[4096][:], xs[4096][:], xs[4096][:], xs[11008][:]
                blk.q_proj(xa), blk.k_proj(xa), blk.v_proj(xa)
                blk.o_proj(xo)
                blk.gate_proj(xm), blk.up_proj(xm)
                blk.down_proj(xd)

    gr = graph_of(torch, fused_token)
    fused_us = time_calls(torch, gr.replay, 20, 3)
    del gr, blocks
    # fp16 hipBLASLt over the same shapes: one set of fp16 weights per layer would be 13 GB; rotate 4 layers' worth
    w16 = [[torch.randn(n, k, device="cuda", dtype=torch.float16) for _, k, n in LLAMA7B_LINEARS] for _ in range(4)]
    gr = graph_of(torch, lambda: [torch.matmul(xs[w.shape[1]], w.T) for li in range(nlayers) for w in w16[li % 4]])
    blas_us = time_calls(torch, gr.replay, 10, 2)
    return {"linears": len(plan), "weights_G": round(weights / 1e9, 3), "quantize_all_ms": round(quant_ms, 2),
            "quantize_Gweights_per_s": round(weights / quant_ms / 1e6, 1),
            "decode_token_us_linears_only": round(tok_us, 1), "decode_tokens_per_s_linears_only": round(1e6 / tok_us, 1),
            "decode_GBps": round(by / tok_us / 1e3, 1), "decode_bytes_per_token": by,
            "decode_token_us_fused_siblings": round(fused_us, 1),
            "decode_tokens_per_s_fused_siblings": round(1e6 / fused_us, 1),
            "hipblaslt_fp16_token_us_linears_only": round(blas_us, 1)}


def extras_decode_fused_siblings(torch, hip, QuantizedLinear, layers):
    """The headline step again with q/k/v and gate/up grouped by fuse_sibling_linears: the model still calls seven
    modules per layer, four launches run (a launch costs ~2.5 us before its first byte arrives).  Not the headline:
    the caller has to opt in.  Runs after every section that uses `layers`: it re-points their buffers at concatenated copies."""
    import bitween_amd
    names = [n for n, _, _ in LLAMA7B_LINEARS]
    blocks = []
    for layer in layers:
        blk = torch.nn.Module()
        for n, q in zip(names, layer):
            setattr(blk, n, q)
        blocks.append(blk)
    groups = sum(bitween_amd.fuse_sibling_linears(b) for b in blocks)
    xs = {k: torch.randn(1, k, device="cuda", dtype=torch.float16) for k in (4096, 11008)}

    def run():
        with torch.no_grad():
            for _ in range(2):
                for blk in blocks:
                    # a new tensor object per block and pass, as in a real model: a group only re-uses its result
                    # for the very tensor it was computed from
                    x_attn, x_o, x_mlp, x_down = xs[4096][:], xs[4096][:], xs[4096][:], xs[11008][:]
                    blk.q_proj(x_attn), blk.k_proj(x_attn), blk.v_proj(x_attn)
                    blk.o_proj(x_o)
                    blk.gate_proj(x_mlp), blk.up_proj(x_mlp)
                    blk.down_proj(x_down)

    gr = graph_of(torch, run)
    us = time_calls(torch, gr.replay, 20, 3) / (2 * len(blocks))
    by = sum(decode_bytes(1, k, n, 4, 128) for _, k, n in LLAMA7B_LINEARS)
    return {"groups_per_layer": groups // len(blocks), "launches_per_layer": len(names) - 3, "us_per_layer": round(us, 2),
            "GBps": round(by / us / 1e3, 1), "pct_hbm_peak": round(100 * by / us / 1e3 / HBM_PEAK_GBPS, 1)}


def extras_eager_call(torch, hip, QuantizedLinear, layers):
    """Host side of the drop-in: wall time per QuantizedLinear.forward call issued eagerly from Python (no graph),
    M = 1, next to torch's own fp16 nn.Linear of the same shape.  The kernel itself runs for ~4 us."""
    q = layers[0][0]
    x = torch.randn(1, q.in_features, device="cuda", dtype=torch.float16)
    lin = torch.nn.Linear(q.in_features, q.out_features, bias=False, device="cuda", dtype=torch.float16)

    def wall(fn, n=3000):
        for _ in range(300):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n * 1e6

    with torch.no_grad():
        return {"quantized_linear_forward_us": round(wall(lambda: q(x)), 1),
                "torch_fp16_linear_forward_us": round(wall(lambda: lin(x)), 1)}


def extras_llama7b_end_to_end(torch, hip, QuantizedLinear, layers):
    """The reference's use end to end: a transformers Llama of Llama-2-7B shape (random weights, fp16, no network
    for a checkpoint), Bitween(...).quantize(rtn=True, ignore_layers=[lm_head, embed_tokens], layer_config=the mixed
    recipe), then a 512-token prompt and 256 greedy tokens at batch 1, eager PyTorch (no graph), next to the fp16
    model in the same loop.  Attention, norms, rotary embedding, the KV cache and lm_head are transformers' own
    kernels and Python; only the 224 linears are this library's."""
    try:
        from transformers import LlamaConfig, LlamaForCausalLM
    except Exception as exc:                                   # noqa: BLE001
        return {"skipped": "transformers not importable: %s" % exc}
    import bitween_amd
    cfg = LlamaConfig(hidden_size=4096, intermediate_size=11008, num_hidden_layers=32, num_attention_heads=32,
                      num_key_value_heads=32, vocab_size=32000, max_position_embeddings=2048, tie_word_embeddings=False)
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.float16)
    try:
        with torch.device("cuda"):
            model = LlamaForCausalLM(cfg)
    finally:
        torch.set_default_dtype(old)
    model = model.half().cuda().eval()
    recipe = {}
    for i in range(32):
        recipe["model.layers.%d.self_attn" % i] = (8, 128)
        recipe["model.layers.%d.mlp" % i] = (4, 128)
    for i in (0, 1, 30, 31):
        recipe["model.layers.%d.mlp.down_proj" % i] = (2, 32)
    ids = torch.randint(0, 32000, (1, 512), device="cuda", generator=torch.Generator(device="cuda").manual_seed(0))

    def run(m, new_tokens=64):
        with torch.no_grad():
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            out = m(input_ids=ids, use_cache=True)
            past = out.past_key_values
            tok = out.logits[:, -1].argmax(-1, keepdim=True)
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            for _ in range(new_tokens - 1):
                out = m(input_ids=tok, past_key_values=past, use_cache=True)
                past = out.past_key_values
                tok = out.logits[:, -1].argmax(-1, keepdim=True)
            torch.cuda.synchronize()
            t2 = time.perf_counter()
        return (t1 - t0) * 1e3, (new_tokens - 1) / (t2 - t1)

    res = {}
    run(model, 8)
    pre, tps = run(model)
    res["fp16_prefill512_ms"], res["fp16_decode_tokens_per_s"] = round(pre, 1), round(tps, 1)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    qmodel = bitween_amd.Bitween(model, bits=4, group_size=128).quantize(
        rtn=True, ignore_layers=["lm_head", "embed_tokens"], layer_config=recipe, verbose=False)
    torch.cuda.synchronize()
    res["bitween_quantize_call_s"] = round(time.perf_counter() - t0, 2)      # includes the deep copy of the model
    del model
    res["quantized_linears"] = sum(isinstance(m, QuantizedLinear) for m in qmodel.modules())
    run(qmodel, 8)
    pre, tps = run(qmodel)
    res["quantized_prefill512_ms"], res["quantized_decode_tokens_per_s"] = round(pre, 1), round(tps, 1)
    bitween_amd.fuse_sibling_linears(qmodel)
    run(qmodel, 8)
    pre, tps = run(qmodel)
    res["fused_siblings_prefill512_ms"], res["fused_siblings_decode_tokens_per_s"] = round(pre, 1), round(tps, 1)
    res["note"] = ("drop-in check only: an eager transformers loop, 64 new tokens, host-bound (about a thousand small "
                   "launches per token); the measured end-to-end configuration is llama7b_decoder_graph")
    return res


def extras_llama7b_decoder_graph(torch, hip, QuantizedLinear, layers):
    """BASELINE's end-to-end configuration: a 32-layer Llama-7B-shaped decoder (bench_decoder.py: hidden 4096, 32
    heads, MLP 11008, vocab 32000, random weights), Bitween(...).quantize(rtn=True, ignore_layers=[lm_head,
    embed_tokens], layer_config = attention 8-bit g128, MLP 4-bit g128, down_proj of layers 0, 1, 30, 31 2-bit g32),
    then a 512-token random prompt and 256 greedy tokens at batch 1 with one decode step captured in a HIP graph
    and replayed.  The glue (RMSNorm, rotary, cache update, attention, SwiGLU) is plain torch - about 17 small
    launches per layer next to the 4-7 of the linears - or, in the *_hip_glue entries, the five fused kernels of
    bench_decoder_glue.hip (6 launches per layer)."""
    import bitween_amd
    import bench_decoder as bd
    nlayers, prompt, new_tokens = 32, 512, 256
    with torch.device("cuda"):
        model = bd.Decoder(layers=nlayers, max_len=prompt + new_tokens).half()
    model.init_weights(seed=0)
    ids = torch.randint(0, 32000, (prompt,), device="cuda", generator=torch.Generator(device="cuda").manual_seed(0))
    res = {}
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    qmodel = bitween_amd.Bitween(model, bits=4, group_size=128).quantize(
        rtn=True, ignore_layers=["lm_head", "embed_tokens"], layer_config=bd.mixed_recipe(nlayers), verbose=False)
    torch.cuda.synchronize()
    res["bitween_quantize_call_s"] = round(time.perf_counter() - t0, 3)
    del model
    qlin = [mod for mod in qmodel.modules() if isinstance(mod, QuantizedLinear)]
    res["quantized_linears"] = len(qlin)
    by = sum(decode_bytes(1, q.in_features, q.out_features, q.bits, q.group_size) for q in qlin)
    by_all = by + 2 * 32000 * 4096                                   # + the float16 lm_head
    res["bytes_per_token_quantized_linears"] = by
    res["byte_ceiling_tokens_per_s"] = round(HBM_PEAK_GBPS * 1e9 / by_all, 1)
    qmodel.alloc_state()
    fused = False
    # "per_module_launches" is the configuration as the reference would run it (one launch per module, torch glue) and
    # is the stated end-to-end figure; the opt_in_* entries need the caller to ask for sibling fusion and / or use this
    # benchmark's own glue kernels
    for label, fuse, hip_glue in (("per_module_launches", False, False), ("opt_in_hip_glue", False, True),
                                  ("opt_in_fused_siblings", True, False), ("opt_in_fused_siblings_hip_glue", True, True)):
        if fuse and not fused:
            bitween_amd.fuse_sibling_linears(qmodel)
            fused = True
        if hip_glue:
            qmodel.use_hip_glue(splits=12)
        else:
            qmodel.glue = None
        bd.generate(qmodel, ids, 4)                                   # warm every kernel and the allocator
        graph = bd.capture_step(qmodel)
        pre_ms, dec_s, toks = bd.generate(qmodel, ids, new_tokens, graph)
        _, eager_s, toks_eager = bd.generate(qmodel, ids, 32)
        res[label] = {"prefill512_ms": round(pre_ms, 2), "decode_tokens_per_s": round((new_tokens - 1) / dec_s, 1),
                      "decode_ms_per_token": round(dec_s / (new_tokens - 1) * 1e3, 3),
                      "fraction_of_byte_ceiling": round((new_tokens - 1) / dec_s * by_all / (HBM_PEAK_GBPS * 1e9), 3),
                      "eager_loop_tokens_per_s": round(31 / eager_s, 1),
                      "graph_tokens_equal_eager_tokens": bool(torch.equal(toks[:32], toks_eager))}
        del graph
    res["decode_tokens_per_s"] = res["per_module_launches"]["decode_tokens_per_s"]
    res["stated_configuration"] = "per_module_launches (the reference's form: every QuantizedLinear launches its own kernel, plain torch between them)"
    return res


def build_probes():
    """hipcc bench_probes.hip for gfx950 into bench_probes.so next to this file (works without a GPU)."""
    import subprocess
    here = os.path.dirname(os.path.abspath(__file__))
    lib = os.path.join(here, "bench_probes.so")
    cmd = [os.environ.get("HIPCC", "/opt/rocm/bin/hipcc"), "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-o", lib, os.path.join(here, "bench_probes.hip")]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + proc.stderr)
    return lib


def extras_board_probes(torch, hip, QuantizedLinear, layers):
    """The constants of this board that the decode and prefill ceilings are derived from (bench_probes.hip): device
    time per launch of an empty kernel under graph replay, the rate of a kernel that only reads, and how many
    instructions a single wave can issue per MFMA."""
    import ctypes
    lib_path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "bench_probes.so")
    if not os.path.exists(lib_path):
        return {"skipped": "bench_probes.so is not built (run __graft_entry__.build())"}
    lib = ctypes.CDLL(lib_path)
    vp, i32, dbl = ctypes.c_void_p, ctypes.c_int32, ctypes.c_double
    lib.probe_launch_floor.argtypes, lib.probe_launch_floor.restype = [i32, i32, i32, i32], dbl
    lib.probe_read_rate.argtypes, lib.probe_read_rate.restype = [vp, ctypes.c_size_t, vp, i32, i32, i32, i32, i32], dbl
    lib.probe_mfma_issue.argtypes, lib.probe_mfma_issue.restype = [i32, i32, vp], dbl
    torch.cuda.synchronize()
    out = {"empty_kernel_us_per_launch_graph_replay": {
        "grid256_block512": round(lib.probe_launch_floor(200, 256, 512, 10), 3),
        "grid688_block1024": round(lib.probe_launch_floor(200, 688, 1024, 10), 3)}}
    src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").fill_(1)
    scratch = torch.zeros(4, dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    # the rate depends on how the requests of the moment are spread over memory and on the cache hint: a small sweep,
    # the best entry is the board's streaming-read ceiling (labels: grid x block, loads in flight per lane, hint)
    sweep = {}
    for grid, block, unroll in ((4096, 256, 4), (256, 512, 4), (512, 256, 4), (256, 256, 8), (8192, 512, 8)):
        for nt in (0, 1):
            sweep["%dx%d_u%d_%s" % (grid, block, unroll, "nt" if nt else "default")] = round(
                lib.probe_read_rate(src.data_ptr(), src.numel(), scratch.data_ptr(), grid, block, unroll, nt, 4), 1)
    out["read_only_kernel_sweep_GBps_1GiB"] = sweep
    out["read_only_kernel_GBps_1GiB"] = max(sweep.values())
    del src
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    ns = [lib.probe_mfma_issue(v, cus, scratch.data_ptr()) for v in range(4)]
    out["mfma_16x16x32_f16_ns_per_wave"] = {"mfma_only": round(ns[0], 2), "plus_1_valu": round(ns[1], 2), "plus_2_valu": round(ns[2], 2),
                                            "plus_3_valu": round(ns[3], 2)}
    out["mfma_only_TFLOPs"] = round(cus * 4 * 16384 / ns[0] / 1e3, 1)
    # the shader clock inside the same kernels (20 launches back to back, about 10 ms of load): what part of "ns per
    # MFMA" is the clock the part allows under that load
    lib.probe_mfma_clock.argtypes, lib.probe_mfma_clock.restype = [i32, i32, i32, vp], dbl
    clk_buf = torch.zeros(8 + 16 * cus, dtype=torch.uint8, device="cuda")
    ghz = [lib.probe_mfma_clock(v, cus, 20, clk_buf.data_ptr()) for v in range(4)]
    out["mfma_kernel_shader_clock_GHz"] = {"mfma_only": round(ghz[0], 3), "plus_1_valu": round(ghz[1], 3), "plus_2_valu": round(ghz[2], 3),
                                           "plus_3_valu": round(ghz[3], 3)}
    out["mfma_16x16x32_f16_cycles_per_wave"] = {"mfma_only": round(ns[0] * ghz[0], 1), "plus_1_valu": round(ns[1] * ghz[1], 1),
                                                "plus_2_valu": round(ns[2] * ghz[2], 1), "plus_3_valu": round(ns[3] * ghz[3], 1)}
    return out


def extras_backward(torch, hip, QuantizedLinear, layers):
    """grad_input of QuantizedLinearFunction.backward, 4096 -> 14336 W4 g128: the fused kernel (bw_qdgrad; which of
    its kernels a row count gets is `kernel_tile_rows`), the path it replaces (HIP dequantise to float16 + library GEMM)
    and that GEMM alone on resident fp16 weights."""
    k, n = 4096, 14336
    q = make_layer(torch, QuantizedLinear, k, n, 4, 128, seed=11)
    w16 = hip.dequantize(q.qweight, q.scale, q.zero_point, 128, 4, torch.float16)
    out = {}
    for m in (128, 512, 2048):
        go = torch.randn(m, n, device="cuda", dtype=torch.float16)

        def ours():
            w = hip.dequantize(q.qweight, q.scale, q.zero_point, 128, 4, torch.float16)
            return go @ w

        def fused():
            return hip.quantized_input_grad(go, q.qweight, q.scale, q.zero_point, 4, 128)

        t_fused = time_calls(torch, fused, 30, 5)
        t_ours = time_calls(torch, ours, 30, 5)
        t_deq = time_calls(torch, lambda: hip.dequantize(q.qweight, q.scale, q.zero_point, 128, 4, torch.float16), 30, 5)
        t_gemm = time_calls(torch, lambda: go @ w16, 30, 5)
        out["4096x14336_M%d" % m] = {"fused_dgrad_us": round(t_fused, 1), "fused_TFLOPs": round(2.0 * m * n * k / t_fused / 1e6, 1),
                                     # 128 / 256: the kernel that walks N in steps of 32 rows; 129 / 257: the 256 x 256 kernel
                                     "kernel_tile_rows": hip.load().bw_qdgrad_tile_rows(m, n, k, 4, 128),
                                     "dequantize_plus_gemm_us": round(t_ours, 1), "dequantize_us": round(t_deq, 1),
                                     "fp16_gemm_us": round(t_gemm, 1)}
        # bfloat16 gradients: the same kernel with the weight rounded to bfloat16 in registers, against the
        # dequantise-to-bfloat16 + library GEMM path of the module's unfused backward
        gb = go.to(torch.bfloat16)
        t_fused_b = time_calls(torch, lambda: hip.quantized_input_grad(gb, q.qweight, q.scale, q.zero_point, 4, 128), 30, 5)
        t_ours_b = time_calls(torch, lambda: gb @ hip.dequantize(q.qweight, q.scale, q.zero_point, 128, 4, torch.bfloat16), 30, 5)
        out["4096x14336_M%d" % m].update({"bf16_fused_dgrad_us": round(t_fused_b, 1), "bf16_dequantize_plus_gemm_us": round(t_ours_b, 1)})
    return out


def extras_opt125m_fc1(torch, hip, QuantizedLinear, layers):
    """The one configuration that also runs on the CPU path: an OPT-125m fc1 (768 -> 3072), W4 g128, quantize + pack,
    then the forward at M = 1 and 16 - on the GPU (graph replay, weights cache-resident at this size) and through the
    C restatement of the reference arithmetic on this host's cores."""
    import numpy as np
    from oracle import c_oracle, rtn_oracle as orc
    k, n, bits, g = 768, 3072, 4, 128
    gen = torch.Generator(device="cuda").manual_seed(0)
    w = (torch.randn(n, k, device="cuda", generator=gen) * 0.02).half()
    out = {}
    us_q = time_calls(torch, lambda: hip.quantize_pack(w, bits, g, math_dtype=torch.float32, scale_dtype=torch.float16,
                                                      zp_dtype=torch.float16), 50, 10)
    qw, sc, zp = hip.quantize_pack(w, bits, g, math_dtype=torch.float32, scale_dtype=torch.float16, zp_dtype=torch.float16)
    w_np = w.float().cpu().numpy()
    t0 = time.perf_counter()
    for _ in range(10):
        qw_c, s_c, z_c = c_oracle.quantize_rtn_f32(w_np, bits, g)
    cpu_q_ms = (time.perf_counter() - t0) / 10 * 1e3
    s16, z16 = orc.store_module_buffers(s_c, z_c)
    out["quantize_pack"] = {"gpu_us": round(us_q, 2), "cpu_ms": round(cpu_q_ms, 3),
                            "bit_identical": bool(np.array_equal(qw.cpu().numpy(), qw_c))}
    for m in (1, 16):
        x = torch.randn(m, k, device="cuda", dtype=torch.float16, generator=gen)
        gr = graph_of(torch, lambda: [hip.quantized_matmul_hip(x, qw, sc, zp, None, bits, g) for _ in range(64)])
        us = time_calls(torch, gr.replay, 20, 3) / 64
        x_np = x.cpu().numpy()
        c_oracle.qlinear_forward(x_np, qw_c, s16, z16, None, bits, g)
        t0 = time.perf_counter()
        for _ in range(20):
            c_oracle.qlinear_forward(x_np, qw_c, s16, z16, None, bits, g)
        cpu_ms = (time.perf_counter() - t0) / 20 * 1e3
        out["forward_M%d" % m] = {"gpu_us": round(us, 2), "cpu_ms": round(cpu_ms, 3)}
    return out


EXTRAS = {"opt125m_fc1": extras_opt125m_fc1, "decode": extras_decode, "decode_infinity_cache_hot": extras_decode_hot,
          "decode_other_formats": extras_decode_other_formats, "hipblaslt_fp16_decode": extras_hipblaslt_decode,
          "prefill": extras_prefill, "prefill_clock": extras_prefill_clock, "prefill_other_formats": extras_prefill_other_formats, "quantize": extras_quantize, "mixed_precision_model": extras_mixed_precision_model, "eager_call": extras_eager_call,
          "decode_fused_siblings": extras_decode_fused_siblings, "board_probes": extras_board_probes,
          # the heavy sections last: the GEMMs and the 7B model leave the board warm, which shows in the decode timings
          "backward": extras_backward, "llama7b_decoder_graph": extras_llama7b_decoder_graph,
          "transformers_drop_in_check": extras_llama7b_end_to_end}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--layers", type=int, default=8, help="distinct weight sets rotated through")
    ap.add_argument("--m", type=int, default=1, help="decode batch of the headline number")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--only", choices=sorted(EXTRAS), default=None,
                    help="run just this section of the extras and print it (used for profiling one kernel)")
    ap.add_argument("--probe", default=None, metavar="K,N,M,BITS,GROUP",
                    help="run only eager decode launches of this one shape over 12 rotating layer copies (one dispatch per "
                         "launch, for rocprofv3 counter runs) and print their device time")
    ap.add_argument("--copy-probe", action="store_true",
                    help="run only a plain 256 MiB device copy a few times (calibrates rocprof FETCH_SIZE/WRITE_SIZE)")
    ap.add_argument("--decoder-probe", action="store_true",
                    help="run only the end-to-end decoder (sibling launches fused, HIP glue): quantize, 512-token prompt, then "
                         "64 replays of the captured decode step (for rocprofv3 kernel traces of a whole token)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this path is a single-device operator and every box here has one GPU; "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from bitween_amd import QuantizedLinear
    from bitween_amd.kernels import hip_loader as hip
    assert torch.cuda.is_available(), "bench.py needs the GPU"
    hip.load()
    torch.cuda.set_device(0)
    bits, g, m = 4, 128, args.m
    if args.copy_probe:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_probe_bytes": 256 << 20, "launches": 5, "copy_gbps_1GiB": copy_probe(torch)}))
        return

    if args.decoder_probe:
        import bitween_amd
        import bench_decoder as bd
        with torch.device("cuda"):
            model = bd.Decoder(layers=32, max_len=768).half()
        model.init_weights(seed=0)
        qmodel = bitween_amd.Bitween(model, bits=4, group_size=128).quantize(
            rtn=True, ignore_layers=["lm_head", "embed_tokens"], layer_config=bd.mixed_recipe(32), verbose=False)
        qmodel.alloc_state()
        bitween_amd.fuse_sibling_linears(qmodel)
        qmodel.use_hip_glue()
        ids = torch.randint(0, 32000, (512,), device="cuda", generator=torch.Generator(device="cuda").manual_seed(0))
        bd.generate(qmodel, ids, 4)
        graph = bd.capture_step(qmodel)
        _, dec_s, _ = bd.generate(qmodel, ids, 65, graph)
        print(json.dumps({"decoder_probe": "32 layers, fused siblings, HIP glue", "replays": 64, "decode_ms_per_token": round(dec_s / 64 * 1e3, 3)}))
        return

    if args.probe:
        pk, pn, pm, pb, pg = (int(v) for v in args.probe.split(","))
        qs = [make_layer(torch, QuantizedLinear, pk, pn, pb, pg, seed=i, outliers=True) for i in range(12)]
        x = torch.randn(pm, pk, device="cuda", dtype=torch.float16)
        us = time_calls(torch, lambda: [hip.quantized_matmul_hip(x, q.qweight, q.scale, q.zero_point, None, pb, pg) for q in qs], 3, 1) / 12
        print(json.dumps({"probe": args.probe, "launches": 48, "eager_us_per_launch": round(us, 2),
                          "bytes": decode_bytes(pm, pk, pn, pb, pg)}))
        return

    layers = [[make_layer(torch, QuantizedLinear, k, n, bits, g, seed=100 * li + i)
               for i, (_, k, n) in enumerate(LLAMA7B_LINEARS)] for li in range(args.layers)]
    if args.only:
        print(json.dumps({args.only: EXTRAS[args.only](torch, hip, QuantizedLinear, layers)}))
        return
    xs = {k: torch.randn(m, k, device="cuda", dtype=torch.float16) for k in (4096, 11008)}
    passes = max(1, MODEL_LAYERS // args.layers)           # a step = one token through MODEL_LAYERS decoder layers
    layer_bytes = sum(decode_bytes(m, k, n, bits, g) for _, k, n in LLAMA7B_LINEARS)
    step_bytes = layer_bytes * passes * args.layers
    launches_per_step = len(LLAMA7B_LINEARS) * passes * args.layers

    def run_linears(select):
        for _ in range(passes):
            for layer in layers:
                for q in layer:
                    if select(q):
                        hip.quantized_gemv_hip(xs[q.in_features], q.qweight, q.scale, q.zero_point, None, bits, g)

    if args.no_graph:
        def one_step():
            run_linears(lambda q: True)
    else:
        one_step = graph_of(torch, lambda: run_linears(lambda q: True)).replay

    for _ in range(args.warmup):
        one_step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        one_step()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    dev_ms = e0.elapsed_time(e1)
    ms_per_step = dev_ms / args.steps
    gbps = step_bytes / (ms_per_step * 1e-3) / 1e9
    us_per_launch = ms_per_step * 1e3 / launches_per_step
    bytes_per_launch = step_bytes / launches_per_step

    # the same launches shape by shape (each shape's launches of a step as a graph of their own): where the step's
    # time goes, and what fraction of the HBM peak each shape reaches
    per_shape = {}
    if not args.no_graph:
        for (kk, nn) in sorted({(k, n) for _, k, n in LLAMA7B_LINEARS}):
            count = sum(1 for _, k, n in LLAMA7B_LINEARS if (k, n) == (kk, nn)) * passes * args.layers
            gr = graph_of(torch, lambda: run_linears(lambda q: (q.in_features, q.out_features) == (kk, nn)))
            us = time_calls(torch, gr.replay, max(3, args.steps // 2), 2) / count
            by = decode_bytes(m, kk, nn, bits, g)
            per_shape["%dx%d" % (kk, nn)] = {"launches_per_step": count, "us": round(us, 3), "bytes": by,
                                             "GBps": round(by / us / 1e3, 1), "frac": round(by / us / 1e3 / HBM_PEAK_GBPS, 4)}
            del gr

    # which kernel each shape's launch runs (asked of the library), and the HBM traffic per launch that was measured
    # with rocprofv3 counters for exactly those kernels (profiles/...hbm_traffic.txt): a profile taken on other
    # kernels is not quoted
    kernels = {}
    for _, kk, nn in LLAMA7B_LINEARS:
        q = next(q for q in layers[0] if (q.in_features, q.out_features) == (kk, nn))
        hip.quantized_gemv_hip(xs[kk], q.qweight, q.scale, q.zero_point, None, bits, g)
        kernels["%dx%d" % (kk, nn)] = hip.last_decode_kernel()
    torch.cuda.synchronize()
    traffic, traffic_note = profiled_traffic(kernels, m)

    result = {
        "metric": "W4A16 g128 dequant-GEMM: decode HBM GB/s (% peak); prefill TFLOP/s",
        "value": round(gbps, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": "Llama-2-7B decoder-layer linears (q/k/v/o 4096x4096, gate/up 4096->11008, down "
                               "11008->4096), 4-bit g128 RTN, fp16 activations, decode M=%d; one step = one token "
                               "through the %d linears of %d decoder layers (%d distinct layers' weights, %d MB, "
                               "run through %d times)" % (m, launches_per_step, passes * args.layers, args.layers,
                                                          layer_bytes * args.layers // 1000000, passes),
                   "M": m, "bits": bits, "group_size": g, "layers_rotated": args.layers, "launches_per_step": launches_per_step,
                   "bytes_per_step": step_bytes, "launch": "eager" if args.no_graph else "hip_graph"},
        "pct_hbm_peak": round(100 * gbps / HBM_PEAK_GBPS, 2),
        "wall_ms_total": round(wall_ms, 3),
        "roofline": {"bound": "hbm", "achieved": round(bytes_per_launch / (us_per_launch * 1e-6) / 1e9, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(bytes_per_launch / (us_per_launch * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
                     # HBM bytes per launch from rocprofv3 FETCH_SIZE / WRITE_SIZE, scaled by the same counters on
                     # a plain copy (profiles/qgemv_w4g128_llama7b_decode_M1_hbm_traffic.txt); not measurable live
                     "traffic": traffic, "traffic_source": traffic_note, "kernel": kernels.get("4096x4096"), "kernels": kernels,
                     "avg_launch_us": round(us_per_launch, 3),
                     "bytes_per_launch": round(bytes_per_launch),
                     "per_shape": per_shape,
                     # what this board's memory system delivers to a plain device-to-device copy of 1 GiB (read + write)
                     "copy_gbps": copy_probe(torch)},
    }

    if not args.no_extras:
        del one_step
        result["extras"] = {name: fn(torch, hip, QuantizedLinear, layers) for name, fn in EXTRAS.items()}

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
