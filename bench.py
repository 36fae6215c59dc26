#!/usr/bin/env python3
"""Benchmark of the quantized-Linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Headline workload (the one the metric is quoted on): the INT4 AWQ-style W4 GEMV,
M=1, K=4096, N=4096, group size 128, f32 activations, f32 scale + f32
zero-point per group (the reference's storage).  A step is one pass over the
batch of synthetic input: 64 GEMV launches, one per distinct weight set
(> 600 MB in all, so that the 256 MB Infinity Cache cannot serve the weights),
replayed from one HIP graph, with all inputs resident in HBM before the timed
region.  --steps K times exactly K such passes, each between its own pair of
HIP events on the launch stream; the figure of record is the median pass.  The
INT8 prefill GEMM
(2048 x 4096 x 11008 on the i8 matrix cores) is timed in the same run and
reported under "secondary".  One JSON line is printed on stdout.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
I8_PEAK_TOPS = 5000.0        # MI355X dense int8 MFMA, published
F16_PEAK_TFLOPS = 2500.0     # MI355X dense f16 MFMA, published

M, K, N, G = 1, 4096, 4096, 128
GROUPS = K // G
# algorithmic bytes of one GEMV: packed nibbles + scales + zero-points + x + y, each once
BYTES_F32_ZP = K * N // 2 + 2 * GROUPS * N * 4 + K * 4 + N * 4           # 9,469,952 (layout executed)
BYTES_U4_ZP = K * N // 2 + GROUPS * N * 4 + GROUPS * N // 2 + K * 4 + N * 4  # 9,011,200 (u4 zero-points)
WEIGHT_SETS = 64
# HBM bytes per GEMV launch from rocprofv3 FETCH_SIZE + WRITE_SIZE, each scaled by a 256 MiB copy
# (profiles/w4_gemv_dot8_1x4096x4096_hbm_traffic.txt); a counter result, not measured by this script
GEMV_TRAFFIC_BYTES = 9659300
# the same for the INT8 GEMM 2048 x 4096 x 11008 (112,742,523 B read + 90,177,536 B written), same file
I8_GEMM_TRAFFIC_BYTES = 202920059
# untimed replays before a long matrix-core kernel is timed (see time_graph)
SETTLE_S = 0.06


def log(msg):
    print(msg, file=sys.stderr, flush=True)


def time_graph(torch, launch_all, launches_per_replay, replays, warmup_replays, settle_s=0.0):
    """Capture `launch_all` (a burst of `launches_per_replay` launches) in a HIP graph and time exactly
    `replays` replays after `warmup_replays` untimed ones, every replay between its own pair of HIP
    events on the stream the kernels run on.  Returns a dict: seconds per LAUNCH as median / mean / min /
    max over the replays, the replay count and whether a graph was used.
    `settle_s`: the untimed replays go on for at least this long.  A kernel that loads the matrix cores runs its
    first few hundred launches after a quieter phase 10-25 % slower (the board's power management settles over
    about 40 ms: 2048 x 4096 x 11008 int8 measured 107, 131, 121, 114, 107 ... 103 us per launch in successive
    bursts of ten), so the long kernels are timed once that has passed."""
    stream = torch.cuda.current_stream()
    graph = None
    try:
        side = torch.cuda.Stream()
        side.wait_stream(stream)
        with torch.cuda.stream(side):
            launch_all()                       # warm the capture stream
        stream.wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):     # the stream warmed above: its workspace exists already
            launch_all()
        graph = g
    except Exception as e:  # capture is an optimisation of the launch path only
        log(f"[bench] HIP graph capture unavailable ({e!r}); timing direct launches")
        torch.cuda.synchronize()
    run = graph.replay if graph is not None else launch_all
    replays = max(1, int(replays))
    for _ in range(max(0, int(warmup_replays))):
        run()
    torch.cuda.synchronize()
    t_settle = time.perf_counter()
    while time.perf_counter() - t_settle < settle_s:
        for _ in range(4):
            run()
        torch.cuda.synchronize()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(replays + 1)]
    marks[0].record()
    for i in range(replays):
        run()
        marks[i + 1].record()
    torch.cuda.synchronize()
    per = np.array([marks[i].elapsed_time(marks[i + 1]) for i in range(replays)]) * 1e-3 / launches_per_replay
    return {"median": float(np.median(per)), "mean": float(marks[0].elapsed_time(marks[replays]) * 1e-3
                                                              / (replays * launches_per_replay)),
            "min": float(per.min()), "max": float(per.max()), "replays": replays,
            "launches_per_replay": launches_per_replay, "graph": graph is not None}


def spread(t):
    """The per-replay statistics of time_graph, in microseconds per launch, for the JSON line."""
    return {"replays": t["replays"], "launches_per_replay": t["launches_per_replay"],
            "us_median": t["median"] * 1e6, "us_mean": t["mean"] * 1e6, "us_min": t["min"] * 1e6, "us_max": t["max"] * 1e6}


def bench_gemv(torch, ops, steps, warmup):
    from rumus_amd import workloads
    dev = torch.device("cuda:0")
    w0, x0 = workloads.w4_gemv(0)
    x = torch.from_numpy(x0).to(dev)
    # reference storage (f32 zero-points); its tile-major decode layout; AWQ storage (u4 zero-points)
    sets, sets_dl, sets_awq = [], [], []
    gen = torch.Generator(device=dev).manual_seed(0)
    for i in range(WEIGHT_SETS):
        if i == 0:
            w = torch.from_numpy(w0).to(dev)
        else:
            w = torch.randn((K, N), generator=gen, device=dev, dtype=torch.float32) * 0.02
        sets.append(ops.w4_quantize_pack(w, G))
        sets_dl.append(ops.w4_decode_layout(*sets[-1], G))
        sets_awq.append(ops.w4_decode_layout_zp4(*ops.w4_quantize_pack_awq(w, G), G))
        del w
    ys = [torch.empty((M, N), dtype=torch.float32, device=dev) for _ in range(WEIGHT_SETS)]
    torch.cuda.synchronize()

    # what QLinear.forward launches for a decode row: the decode-layout entry point
    def burst_rotating():
        for (p, s, z), y in zip(sets_dl, ys):
            ops.qmatmul_int4_decode(x, p, s, z, K, G, out=y)

    def burst_resident():
        p, s, z = sets_dl[0]
        for y in ys:
            ops.qmatmul_int4_decode(x, p, s, z, K, G, out=y)

    # the same GEMV through the reference-layout entry point (64-byte segments 16 KB apart)
    def burst_rotating_ref():
        for (p, s, z), y in zip(sets, ys):
            ops.qmatmul_int4(x, p, s, z, K, G, out=y)

    def burst_rotating_awq():
        for (p, s, qz), y in zip(sets_awq, ys):
            ops.qmatmul_int4_decode_zp4(x, p, s, qz, K, G, out=y)

    # the timed region of record: EXACTLY `steps` passes over the 64 weight sets
    t = time_graph(torch, burst_rotating, WEIGHT_SETS, steps, warmup)
    t_res = time_graph(torch, burst_resident, WEIGHT_SETS, steps, warmup)
    y0 = ys[0].cpu().numpy()
    t_awq = time_graph(torch, burst_rotating_awq, WEIGHT_SETS, steps, warmup)
    t_ref = time_graph(torch, burst_rotating_ref, WEIGHT_SETS, steps, warmup)
    return {"t": t, "t_resident": t_res, "t_awq": t_awq, "t_ref": t_ref, "x": x0, "w": w0, "y0": y0}


def bench_i8_gemm(torch, ops, replays=12, warmup=3):
    m, k, n = 2048, 4096, 11008
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(1)
    x = torch.randn((m, k), generator=gen, device=dev)
    w = torch.randn((k, n), generator=gen, device=dev) * 0.02
    xq, sx = ops.i8_quantize_rows(x)
    wq, sw = ops.i8_quantize_cols_t(w)
    del w
    y = torch.empty((m, n), dtype=torch.float32, device=dev)
    per_graph = 10

    def burst():
        for _ in range(per_graph):
            ops.i8_gemm(xq, wq, sx, sw, None, out=y)

    t = time_graph(torch, burst, per_graph, replays, warmup, SETTLE_S)
    sec = t["median"]
    ops_per = 2.0 * m * k * n

    # dynamic activation quantizer, timed separately (it precedes every GEMM in a forward)
    xq2, sx2 = torch.empty_like(xq), torch.empty_like(sx)

    def burst_q():
        for _ in range(per_graph):
            ops.i8_quantize_rows(x, out=(xq2, sx2))

    sec_q = time_graph(torch, burst_q, per_graph, replays, warmup)["median"]
    tops = ops_per / sec / 1e12
    # Two yardsticks measured in the same run, on the same operands where it applies:
    # the matrix cores alone (MFMA from registers, random operand bits, no memory traffic:
    # what the board's power limit lets them sustain), and the vendor library's int8 GEMM
    # (hipBLASLt through torch._int_mm: i32 output, no rescale) on the same xq, wq.
    ceiling = probe_mfma_ceiling()
    vendor = None
    try:
        wt = wq.t()

        def burst_vendor():
            for _ in range(per_graph):
                torch._int_mm(xq, wt)

        vendor = ops_per / time_graph(torch, burst_vendor, per_graph, replays, warmup, SETTLE_S)["median"] / 1e12
    except Exception as exc:   # informational only
        log(f"[bench] vendor int8 GEMM not timed: {exc}")
    # The same kernel on operands without bit activity (all ones: every product and sum is still computed, the
    # instruction stream and the memory traffic are those of the timed run above): what the kernel's schedule
    # reaches when the board's power management does not hold the shader clock down.  Not a throughput claim.
    quiet = None
    try:
        xq1, wq1 = torch.ones_like(xq), torch.ones_like(wq)

        def burst_quiet():
            for _ in range(per_graph):
                ops.i8_gemm(xq1, wq1, sx, sw, None, out=y)

        tq = time_graph(torch, burst_quiet, per_graph, replays, warmup, SETTLE_S)["median"]
        quiet = {"operands": "all ones", "ms_per_launch": tq * 1e3, "tops": ops_per / tq / 1e12,
                 "frac": ops_per / tq / 1e12 / I8_PEAK_TOPS}
        wt1 = wq1.t()

        def burst_vendor_quiet():
            for _ in range(per_graph):
                torch._int_mm(xq1, wt1)

        quiet["vendor_int_mm_tops"] = ops_per / time_graph(torch, burst_vendor_quiet, per_graph, replays, warmup, SETTLE_S)["median"] / 1e12
        del xq1, wq1, wt1
    except Exception as exc:   # informational only
        log(f"[bench] constant-operand run not timed: {exc}")
    return {
        "workload": "int8_gemm_2048x4096x11008", "ms_per_launch": sec * 1e3, "tops": tops, "hip_graph": t["graph"],
        "operands": "int8 from absmax-quantized normal samples (random bits)",
        "same_kernel_constant_operands": quiet,
        "timing": spread(t),
        "roofline": {"bound": "mfma", "achieved": tops, "peak": I8_PEAK_TOPS, "unit": "TOP/s",
                     "frac": tops / I8_PEAK_TOPS, "traffic": I8_GEMM_TRAFFIC_BYTES,
                     "traffic_from": "profiles/w4_gemv_dot8_1x4096x4096_hbm_traffic.txt (rocprofv3 FETCH_SIZE + WRITE_SIZE "
                                     "of a counter run of this kernel, not measured by this script)"},
        "mfma_only_random_operands": ceiling,
        "frac_of_mfma_only": (tops / ceiling["tops"]) if ceiling else None,
        "vendor_int_mm_tops": vendor,
        "act_quantize_rows_ms": sec_q * 1e3,
        "act_quantize_rows_gbs": (m * k * 5 + m * 4) / sec_q / 1e9,
    }


def probe_launch_floor():
    """What a single launch of the GEMV's size can reach on this GPU: an empty kernel, and a
    kernel that only reads 8 MiB (the packed weights) from 64 rotating buffers, both replayed
    from a HIP graph (bench/probe_mfma.hip).  None when the probe library is absent."""
    import ctypes
    path = os.path.join(ROOT, "bench", "librumus_probe.so")
    if not os.path.exists(path):
        return None
    lib = ctypes.CDLL(path)
    lib.rumus_probe_read_launch.restype = ctypes.c_int
    lib.rumus_probe_read_launch.argtypes = [ctypes.c_uint64, ctypes.c_int, ctypes.POINTER(ctypes.c_double)]
    empty, read = ctypes.c_double(), ctypes.c_double()
    nbytes = K * N // 2
    if lib.rumus_probe_read_launch(0, 1, ctypes.byref(empty)) != 0:
        return None
    if lib.rumus_probe_read_launch(nbytes, WEIGHT_SETS, ctypes.byref(read)) != 0:
        return None
    return {"empty_kernel_us": empty.value, "read_only_us": read.value, "read_only_bytes": nbytes,
            "read_only_gbs": nbytes / read.value / 1e3}


def probe_mfma_ceiling():
    """int8 TOP/s of v_mfma_i32_32x32x32_i8 issued back to back from registers with random
    operand bits (bench/probe_mfma.hip, its own small library), or None."""
    import ctypes
    path = os.path.join(ROOT, "bench", "librumus_probe.so")
    if not os.path.exists(path):
        return None
    lib = ctypes.CDLL(path)
    lib.rumus_probe_i8_mfma.restype = ctypes.c_int
    lib.rumus_probe_i8_mfma.argtypes = [ctypes.c_int, ctypes.POINTER(ctypes.c_double),
                                        ctypes.POINTER(ctypes.c_double)]
    tops, mhz = ctypes.c_double(), ctypes.c_double()
    if lib.rumus_probe_i8_mfma(1, ctypes.byref(tops), ctypes.byref(mhz)) != 0:
        return None
    return {"tops": tops.value, "shader_mhz": mhz.value}


def probe_f16_mfma_ceiling():
    """f16 TFLOP/s of v_mfma_f32_32x32x16_f16 issued back to back from registers (bench/probe_mfma.hip): with
    random f16 operands, with random activations against small-integer weights (what the W4 kernels multiply),
    and with ones; or None."""
    import ctypes
    path = os.path.join(ROOT, "bench", "librumus_probe.so")
    if not os.path.exists(path):
        return None
    lib = ctypes.CDLL(path)
    if not hasattr(lib, "rumus_probe_f16_mfma"):
        return None
    lib.rumus_probe_f16_mfma.restype = ctypes.c_int
    lib.rumus_probe_f16_mfma.argtypes = [ctypes.c_int, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]
    out = {}
    for name, mode in (("random_operands", 1), ("random_times_nibbles", 2), ("ones", 0)):
        tf, mhz = ctypes.c_double(), ctypes.c_double()
        if lib.rumus_probe_f16_mfma(mode, ctypes.byref(tf), ctypes.byref(mhz)) != 0:
            return None
        out[name] = {"tflops": tf.value, "shader_mhz": mhz.value}
    return out


def bench_gemv_shapes(torch, ops, replays=10, warmup=2):
    """The same decode kernel on the wider projections of a Llama-7B block (q|k|v, gate|up, down),
    each rotating over enough weight sets (> 600 MB) to defeat the Infinity Cache.  The longer a
    launch, the smaller the share of its fixed start-up and drain."""
    import ctypes
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(5)
    probe = None
    path = os.path.join(ROOT, "bench", "librumus_probe.so")
    if os.path.exists(path):
        probe = ctypes.CDLL(path)
        probe.rumus_probe_read_launch.restype = ctypes.c_int
        probe.rumus_probe_read_launch.argtypes = [ctypes.c_uint64, ctypes.c_int, ctypes.POINTER(ctypes.c_double)]
    rows = []
    for k, n in ((4096, 12288), (4096, 22016), (11008, 4096)):
        nbytes = k * n // 2 + 2 * (k // G) * n * 4 + k * 4 + n * 4
        nsets = -(-640_000_000 // nbytes)
        sets = []
        for _ in range(nsets):
            w = torch.randn((k, n), generator=gen, device=dev, dtype=torch.float32) * 0.02
            q = ops.w4_quantize_pack(w, G)
            sets.append(ops.w4_decode_layout(*q, G))
            del w, q
        x = torch.randn((1, k), generator=gen, device=dev)
        y = torch.empty((1, n), dtype=torch.float32, device=dev)

        def burst():
            for p, s, z in sets:
                ops.qmatmul_int4_decode(x, p, s, z, k, G, out=y)

        per = time_graph(torch, burst, nsets, replays, warmup)["median"]
        row = {"workload": f"w4_gemv_1x{k}x{n}_g128", "weight_sets_rotated": nsets, "bytes_per_step": nbytes,
               "ms_per_step": per * 1e3, "gbs": nbytes / per / 1e9, "hbm_frac": nbytes / per / 1e9 / HBM_PEAK_GBS}
        if probe is not None:
            us = ctypes.c_double()
            if probe.rumus_probe_read_launch(k * n // 2, nsets, ctypes.byref(us)) == 0:
                row["read_only_launch_us"] = us.value
                row["frac_of_read_only_launch"] = us.value * 1e-6 * (nbytes / (k * n // 2)) / per
        rows.append(row)
        del sets
    return rows


def bench_w4_gemm(torch, ops, m, replays=10, warmup=2, symmetric=True):
    """W4 GEMM with act-order (GPTQ style), K=4096, N=11008, g128, symmetric zp=8 (stored as f32, as the reference
    holds it; symmetric=False: the reference quantizer's own fractional zero-points, for which the large-batch kernel
    keeps its extra pass).  The weights rotate over
    copies (> 600 MB in total, more than the 256 MB Infinity Cache) so that every launch reads them from HBM;
    the time on a single, cache-resident copy is reported beside it."""
    k, n = 4096, 11008
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(2)
    w = torch.randn((k, n), generator=gen, device=dev) * 0.02
    packed, scales, zp = ops.w4_quantize_pack(w, G, symmetric=symmetric)
    del w
    g_idx = (torch.randperm(k, generator=gen, device=dev) // G).to(torch.int32)
    packed_sorted, perm = ops.w4_actorder_prepare(packed, g_idx, G)
    x = torch.randn((m, k), generator=gen, device=dev)
    y = torch.empty((m, n), dtype=torch.float32, device=dev)
    nbytes = k * n // 2 + 2 * (k // G) * n * 4 + k * 4 + m * k * 4 + m * n * 4
    # large batches re-read the weights per row tile out of the caches anyway: one copy is enough there
    ncopy = max(2, 600_000_000 // (k * n // 2)) if m <= 256 else 1
    copies = [(packed_sorted.clone(), scales.clone(), zp.clone()) for _ in range(ncopy - 1)] + [(packed_sorted, scales, zp)]

    def burst():
        for p, s_, z in copies:
            ops.qmatmul_int4_perm(x, p, s_, z, k, G, perm=perm, out=y)

    def burst_resident():
        for _ in range(10):
            ops.qmatmul_int4_perm(x, packed_sorted, scales, zp, k, G, perm=perm, out=y)

    settle = SETTLE_S if m >= 512 else 0.0
    sec = time_graph(torch, burst, len(copies), replays, warmup, settle)["median"]
    sec_res = time_graph(torch, burst_resident, 10, replays, warmup, settle)["median"]
    del copies
    flops = 2.0 * m * k * n
    return {"workload": f"w4_gemm_actorder_{m}x4096x11008_g128", "zero_points": "8.0 (f32)" if symmetric else "fractional (f32)",
            "hip_graph": True, "weight_copies_rotated": ncopy,
            "ms_per_launch": sec * 1e3, "cache_resident_ms_per_launch": sec_res * 1e3,
            "gbs": nbytes / sec / 1e9, "hbm_frac": nbytes / sec / 1e9 / HBM_PEAK_GBS,
            "tflops": flops / sec / 1e12, "f16_mfma_frac": flops / sec / 1e12 / F16_PEAK_TFLOPS}


def bench_i8_small(torch, ops, replays=10, warmup=2):
    """W8A8 at decode batch sizes, 4096 x 11008, rotating over 8 copies of the weights (361 MB: HBM,
    not the Infinity Cache); graph-timed."""
    k, n = 4096, 11008
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(5)
    wq, sw = ops.i8_quantize_cols_t(torch.randn((k, n), generator=gen, device=dev) * 0.02)
    copies = [wq] + [wq.clone() for _ in range(7)]
    rows = []
    for m in (1, 4, 8, 32):
        xq, sx = ops.i8_quantize_rows(torch.randn((m, k), generator=gen, device=dev))

        def burst():
            for c in copies:
                ops.i8_gemm(xq, c, sx, sw, None)

        sec = time_graph(torch, burst, len(copies), replays, warmup)["median"]
        rows.append({"workload": f"int8_gemm_{m}x4096x11008", "ms_per_launch": sec * 1e3, "weight_gbs": k * n / sec / 1e9,
                     "hbm_frac": k * n / sec / 1e9 / HBM_PEAK_GBS})
    return rows


def bench_i8_mid(torch, ops, replays=10, warmup=2):
    """W8A8 GEMM between the decode and the prefill shapes (1024 rows on the square and the down-projection
    weights): the 128 x 128 tile kernel; graph-timed, the vendor library's i32-output GEMM beside it."""
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(6)
    rows = []
    for (m, k, n) in ((1024, 4096, 4096), (1024, 11008, 4096), (256, 4096, 11008)):
        wq, sw = ops.i8_quantize_cols_t(torch.randn((k, n), generator=gen, device=dev) * 0.02)
        xq, sx = ops.i8_quantize_rows(torch.randn((m, k), generator=gen, device=dev))
        y = torch.empty((m, n), dtype=torch.float32, device=dev)

        def burst():
            for _ in range(4):
                ops.i8_gemm(xq, wq, sx, sw, None, out=y)

        sec = time_graph(torch, burst, 4, replays, warmup, SETTLE_S)["median"]
        row = {"workload": f"int8_gemm_{m}x{k}x{n}", "ms_per_launch": sec * 1e3, "tops": 2.0 * m * k * n / sec / 1e12}
        try:
            wt = wq.t()

            def vendor():
                for _ in range(4):
                    torch._int_mm(xq, wt)

            row["vendor_int_mm_tops"] = 2.0 * m * k * n / time_graph(torch, vendor, 4, replays, warmup, SETTLE_S)["median"] / 1e12
        except Exception as e:                      # not every torch build can capture it
            row["vendor_int_mm_tops"] = None
            log(f"vendor int_mm skipped: {e}")
        rows.append(row)
    return rows


def bench_grad_x(torch, ops, replays=10, warmup=2):
    """grad_x of the INT4 Linear (QLinearBackward: grad_y . dequant(W)^T), K=4096, N=11008, g128:
    whole call, graph-timed."""
    k, n = 4096, 11008
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(4)
    w = torch.randn((k, n), generator=gen, device=dev) * 0.02
    packed, scales, zp = ops.w4_quantize_pack(w, G)
    del w
    rows = []
    # small batches: weights from HBM (rotating copies, > 600 MB in total); large ones re-read them from the caches anyway
    ncopy = max(2, 600_000_000 // (k * n // 2))
    copies = [(packed.clone(), scales.clone(), zp.clone()) for _ in range(ncopy - 1)] + [(packed, scales, zp)]
    for m in (1, 16, 128, 2048):
        gy = torch.randn((m, n), generator=gen, device=dev)
        out = torch.empty((m, k), dtype=torch.float32, device=dev)
        sets = copies if m <= 128 else copies[-1:] * 4

        def burst():
            for p, s_, z in sets:
                ops.qmatmul_int4_t(gy, p, s_, z, k, G, out=out)

        sec = time_graph(torch, burst, len(sets), replays, warmup, SETTLE_S if m >= 512 else 0.0)["median"]
        rows.append({"workload": f"w4_grad_x_{m}x4096x11008_g128", "ms_per_call": sec * 1e3,
                     "weight_copies_rotated": len(sets) if m <= 128 else 1,
                     "tflops": 2.0 * m * k * n / sec / 1e12,
                     "weight_gbs": (k * n // 2 + 2 * (k // G) * n * 4) / sec / 1e9})
    return rows


def bench_q8_matmul(torch, ops, replays=10, warmup=2):
    """The reference's f32 x Q8 matmul (Tensor::matmul with a Q8 right-hand side), K=4096, N=11008,
    at the block sizes that take different kernels: whole call, graph-timed."""
    k, n = 4096, 11008
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(3)
    wt = ops.transpose_f32(torch.randn((k, n), generator=gen, device=dev) * 0.02).reshape(-1)
    rows = []
    for bs in (32, 128, 4096):
        words = ops.q8_quantize(wt, bs)
        # few rows: the 45 MB buffer from HBM (rotating copies, > 600 MB in total)
        copies = [words.clone() for _ in range(600_000_000 // (k * n))] + [words]
        for m in (1, 32, 2048):
            a = torch.randn((m, k), generator=gen, device=dev)
            c = torch.empty((m, n), dtype=torch.float32, device=dev)
            sets = copies if m <= 32 else [words] * 4

            def burst():
                for wds in sets:
                    ops.matmul_q8(a, wds, k, n, bs, out=c)

            sec = time_graph(torch, burst, len(sets), replays, warmup, SETTLE_S if m >= 512 else 0.0)["median"]
            rows.append({"workload": f"matmul_q8_{m}x4096x11008_bs{bs}", "ms_per_call": sec * 1e3,
                         "weight_copies_rotated": len(sets) if m <= 32 else 1,
                         "tflops": 2.0 * m * k * n / sec / 1e12,
                         "weight_gbs": (k * n + 4 * n * (k // bs)) / sec / 1e9})
        if bs >= k:                                        # per output channel: also against a dense copy made once
            wq, sw = ops.q8_dense_layout(words, k, n, bs)
            for m in (512, 2048):
                a = torch.randn((m, k), generator=gen, device=dev)
                c = torch.empty((m, n), dtype=torch.float32, device=dev)

                def burst():
                    for _ in range(4):
                        ops.matmul_q8_dense(a, wq, sw, out=c)

                sec = time_graph(torch, burst, 4, replays, warmup, SETTLE_S)["median"]
                rows.append({"workload": f"matmul_q8_dense_{m}x4096x11008", "ms_per_call": sec * 1e3,
                             "tflops": 2.0 * m * k * n / sec / 1e12, "weight_gbs": (k * n + 4 * n) / sec / 1e9})
            del wq, sw
        del words, copies
    return rows


def bench_decoder_block(torch, ops):
    """Llama-7B-shaped block, all seven projections INT4 g128 with the reference's f32 zero-points:
    one decode step (batch 1, position 2047 of a 2048-entry cache) and one prefill of 8 x 512
    tokens.  Times include every kernel of the block (norms, projections, attention, SwiGLU,
    residuals) and the Python launch path.  The graph-timed decode step rotates over four copies of the
    block and of its cache (720 MB read per round: a model's layers come from HBM, one block replayed
    alone would sit in the 256 MB Infinity Cache); the single-copy figure is reported beside it."""
    from rumus_amd import nn, workloads
    dev = torch.device("cuda:0")
    dim, heads = 4096, 32
    w = workloads.decoder_block()
    blk = nn.DecoderBlockW4.from_f32({k: torch.from_numpy(v).to(dev) for k, v in w.items()}, G, heads)
    del w
    x, kc, vc = workloads.decoder_block_inputs(1, 1, dim, cache_len=2048, heads=heads)
    x, kc, vc = (torch.from_numpy(t).to(dev) for t in (x, kc, vc))
    xp = torch.from_numpy(workloads.decoder_block_inputs(8, 512, dim, seed=9)[0]).to(dev)

    def timed(fn, steps, warmup):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(steps):
            fn()
        end.record()
        torch.cuda.synchronize()
        return start.elapsed_time(end) * 1e-3 / steps

    t_dec_resident = None
    t_dec = timed(lambda: blk(x, kc, vc, pos=2047), 50, 5)
    t_pre = timed(lambda: blk(xp), 5, 2)
    # the same decode step replayed from a HIP graph (what a serving loop would do): the capture
    # stream's workspace is reserved first, the library does not allocate while capturing
    t_dec_graph = None
    try:
        from rumus_amd import _lib
        side = torch.cuda.Stream()
        _lib.call("rumus_hip_workspace_reserve", side.cuda_stream, 1 << 22)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            blk(x, kc, vc, pos=2047)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(10):
                blk(x, kc, vc, pos=2047)
        t_dec_resident = timed(graph.replay, 20, 3) / 10
        # the same step over four copies of the block, each with a cache of its own
        copies = [(blk, kc, vc)]
        for _ in range(3):
            proj = {name: nn.QLinear(nn.QuantizedTensor(lin.weight.k, lin.weight.n, lin.weight.padded_k,
                                                       lin.weight.group_size, lin.weight.num_groups,
                                                       lin.weight.packed_tensor.clone(), lin.weight.scales_tensor.clone(),
                                                       lin.weight.zp_tensor.clone()), None)
                    for name, lin in blk.proj.items()}
            copies.append((nn.DecoderBlockW4(proj, blk.norm1, blk.norm2, heads, blk.eps), kc.clone(), vc.clone()))
        with torch.cuda.stream(side):
            for c, k_, v_ in copies:
                c(x, k_, v_, pos=2047)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph4 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph4, stream=side):
            for _ in range(3):
                for c, k_, v_ in copies:
                    c(x, k_, v_, pos=2047)
        t_dec_graph = timed(graph4.replay, 20, 3) / 12
        del copies, graph4
    except Exception as exc:
        log(f"[bench] decoder-block graph capture unavailable: {exc!r}")
    # the block's seven layers through the on-disk form: written once, then loaded (file -> pinned
    # staging -> device, tile-major copies rebuilt); the file sits in the page cache
    ckpt = None
    try:
        import tempfile
        import time
        from rumus_amd import checkpoint
        with tempfile.TemporaryDirectory() as tmp:
            path = os.path.join(tmp, "block.safetensors")
            checkpoint.save_w4(path, {f"blk.{name}": lin for name, lin in blk.proj.items()})
            size = os.path.getsize(path)
            checkpoint.load_w4(path, dev)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            loaded = checkpoint.load_w4(path, dev)
            torch.cuda.synchronize()
            t_load = time.perf_counter() - t0
            same = all(torch.equal(loaded[f"blk.{n}"].weight.packed_tensor, blk.proj[n].weight.packed_tensor)
                       for n in blk.proj)
            del loaded
        ckpt = {"file_bytes": size, "load_ms": t_load * 1e3, "gbs": size / t_load / 1e9, "bits_identical": same}
    except Exception as exc:
        log(f"[bench] checkpoint leg failed: {exc!r}")
    weight_bytes = 4 * (dim * dim // 2 + 2 * (dim // G) * dim * 4) + \
        2 * (dim * 11008 // 2 + 2 * (dim // G) * 11008 * 4) + (11008 * dim // 2 + 2 * (11008 // G) * dim * 4)
    kv_bytes = 2 * 2048 * dim * 4
    flops = 2.0 * 8 * 512 * (4 * dim * dim + 3 * dim * 11008)
    t_best = t_dec_graph if t_dec_graph else t_dec
    return {"workload": "llama7b_block_w4_g128", "decode_ms": t_dec * 1e3,
            "decode_hip_graph_ms": None if t_dec_graph is None else t_dec_graph * 1e3,
            "decode_hip_graph_cache_resident_ms": None if t_dec_resident is None else t_dec_resident * 1e3,
            "decode_copies_rotated": 4,
            "decode_weight_and_cache_gbs": (weight_bytes + kv_bytes) / t_best / 1e9,
            "prefill_8x512_ms": t_pre * 1e3, "prefill_tokens_per_s": 8 * 512 / t_pre,
            "prefill_projection_tflops": flops / t_pre / 1e12, "checkpoint_load": ckpt}


def cpu_baseline(x, w, budget_s=12.0):
    """The CPU restatement of the reference kernels on the host cores: single thread (the
    reference CpuBackend's contract) for `value`, all cores as an extra figure.  Runs before the process touches
    the GPU: the runtime's helper threads otherwise share the cores with the timed loops (the all-core figure
    then scattered between 1.4 and 12 ms)."""
    import oracle
    t0 = time.perf_counter()
    packed, scales, zp = oracle.w4_from_f32(w, G)
    t_pack = time.perf_counter() - t0
    times = []
    t_start = time.perf_counter()
    while len(times) < 5 and (time.perf_counter() - t_start) < budget_s:
        t0 = time.perf_counter()
        y = oracle.qmatmul_int4(x, packed, scales, zp, K, G, threads=1)
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    # every core the job may use: the GPU box gives a one-GPU job 16 threads whatever the host shows
    visible = os.cpu_count() or 1
    try:
        allowed = len(os.sched_getaffinity(0))
    except AttributeError:
        allowed = visible
    cores = max(1, min(allowed, int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or 16))
    mt = []
    for _ in range(7):
        t0 = time.perf_counter()
        oracle.qmatmul_int4(x, packed, scales, zp, K, G, threads=cores)
        mt.append(time.perf_counter() - t0)
    t_mt = float(np.median(mt))
    return {
        "value": BYTES_F32_ZP / med / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
        "sample": f"{len(times)} full 1x4096x4096 g128 GEMVs, median, scalar C restatement of "
                  "qmatmul_int4.wgsl (reference has no CPU kernel for this op)",
        "ms_per_gemv": med * 1e3,
        "host_cpus_visible": visible, "host_cpus_allowed": allowed,
        "all_cores": {"value": BYTES_F32_ZP / t_mt / 1e9, "cores": cores, "ms_per_gemv": t_mt * 1e3,
                      "samples": len(mt), "ms_min": min(mt) * 1e3, "ms_max": max(mt) * 1e3,
                      "note": "the same C restatement, OpenMP over output columns, median"},
        "quantize_pack_from_f32_s": t_pack,
    }, y


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100,
                    help="timed passes over the 64 weight sets (64 GEMV launches each)")
    ap.add_argument("--warmup", type=int, default=10, help="untimed passes before them")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only-gemv", action="store_true", help="skip the secondary workloads")
    ap.add_argument("--with-i8-gemm", action="store_true",
                    help="with --only-gemv: run the INT8 GEMM leg as well (the two kernels whose HBM traffic is "
                         "taken from counters)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run plain 256 MiB device copies (reference kernel of known traffic for "
                         "scaling FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build targets one GPU; --gpus above 1 is not supported "
                 "(no collectives or sharding are part of it)")

    cb = y_cpu = None
    if not args.no_cpu:
        from rumus_amd import workloads
        w_cpu, x_cpu = workloads.w4_gemv(0)
        cb, y_cpu = cpu_baseline(x_cpu, w_cpu)
        del w_cpu, x_cpu

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP path has no CPU fallback")
    from rumus_amd import _lib, ops
    _lib.call("rumus_hip_init", 0)
    torch.cuda.set_device(0)

    if args.steps < 1 or args.warmup < 0:
        sys.exit("bench.py: --steps must be at least 1 and --warmup at least 0")
    steps, warmup = args.steps, args.warmup

    torch.cuda.synchronize()
    wall0 = time.perf_counter()
    r = bench_gemv(torch, ops, steps, warmup)
    wall = time.perf_counter() - wall0
    log(f"[bench] gemv leg wall {wall:.1f}s (includes building {WEIGHT_SETS} weight sets)")

    t = r["t"]
    per_launch = t["median"]                        # seconds per GEMV launch, median over the timed passes
    gbs = BYTES_F32_ZP / per_launch / 1e9
    per_launch_res, per_launch_ref, per_launch_awq = r["t_resident"]["median"], r["t_ref"]["median"], r["t_awq"]["median"]

    out = {
        "metric": "W4 GEMV GB/s (%HBM peak) @1x4096x4096; INT8 GEMM TOPS (%MFMA peak)",
        "value": gbs, "unit": "GB/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": per_launch * WEIGHT_SETS * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "w4_gemv_1x4096x4096_g128_awq_f32zp", "weight_layout": "tile-major copy (16 columns)",
                   "step": "one pass over 64 distinct weight sets = 64 GEMV launches replayed from one HIP graph",
                   "launches_per_step": WEIGHT_SETS, "weight_sets_rotated": WEIGHT_SETS,
                   "hip_graph": t["graph"], "bytes_per_launch": BYTES_F32_ZP, "bytes_per_step": BYTES_F32_ZP * WEIGHT_SETS,
                   "arithmetic": "f32 in, f32 out; inside, each 32-row chunk of x is 20-bit fixed point relative to the "
                                 "chunk's largest magnitude and meets the u4 weights in v_dot8_u32_u4 (exact integer "
                                 "sums), then scale, zero-point and the sum over chunks in f32; within rel 1e-3 / "
                                 "abs 1e-4 of the f32 reference loop (parity_vs_cpu)"},
        "us_per_launch": per_launch * 1e6,
        "timing": {"statistic": "median over the timed steps, each between its own pair of HIP events on the launch stream",
                   **spread(t)},
        "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": gbs / HBM_PEAK_GBS, "traffic": GEMV_TRAFFIC_BYTES,
                     "achieved_from": "9,469,952 algorithmic bytes / median launch time of this run",
                     "traffic_from": "profiles/w4_gemv_dot8_1x4096x4096_hbm_traffic.txt (rocprofv3 counters of an "
                                     "earlier run of this kernel, not measured by this script)"},
        "gbs_at_u4_zero_point_bytes": BYTES_U4_ZP / per_launch / 1e9,
        "reference_layout_entry": {
            "us_per_launch": per_launch_ref * 1e6,
            "gbs": BYTES_F32_ZP / per_launch_ref / 1e9,
            "note": "rumus_hip_qmatmul_int4 on the reference's row-major arrays; the headline uses the "
                    "tile-major copy QuantizedTensor builds once (same words, same bytes)"},
        "awq_storage_u4_zero_points": {
            "us_per_launch": per_launch_awq * 1e6, "bytes_per_launch": BYTES_U4_ZP,
            "gbs": BYTES_U4_ZP / per_launch_awq / 1e9,
            "note": "same shape with integer zero-points packed eight per word, tile-major copy "
                    "(rumus_hip_qmatmul_int4_decode_zp4)"},
        "cache_resident": {"gbs": BYTES_F32_ZP / per_launch_res / 1e9,
                           "us_per_launch": per_launch_res * 1e6,
                           "note": "single weight set, served by Infinity Cache / L2; not HBM"},
    }

    floor = probe_launch_floor()
    if floor:
        out["single_launch_floor"] = floor
        out["frac_of_read_only_launch"] = floor["read_only_us"] * 1e-6 / per_launch

    if args.calibrate_copy:
        src = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device="cuda:0").normal_()
        dst = torch.empty_like(src)
        for _ in range(10):
            dst.copy_(src)              # reads 256 MiB, writes 256 MiB per launch
        torch.cuda.synchronize()
        del src, dst

    if args.only_gemv and args.with_i8_gemm:
        out["secondary"] = bench_i8_gemm(torch, ops)
    if not args.only_gemv:
        out["secondary"] = bench_i8_gemm(torch, ops)
        out["w4_gemv_wider"] = bench_gemv_shapes(torch, ops)
        out["w4_gemm"] = [bench_w4_gemm(torch, ops, 16), bench_w4_gemm(torch, ops, 128), bench_w4_gemm(torch, ops, 256),
                          bench_w4_gemm(torch, ops, 512),
                          bench_w4_gemm(torch, ops, 1024), bench_w4_gemm(torch, ops, 2048),
                          bench_w4_gemm(torch, ops, 2048, symmetric=False)]
        out["f16_mfma_only"] = probe_f16_mfma_ceiling()
        out["q8_matmul"] = bench_q8_matmul(torch, ops)
        out["w4_grad_x"] = bench_grad_x(torch, ops)
        out["int8_decode"] = bench_i8_small(torch, ops)
        out["int8_mid"] = bench_i8_mid(torch, ops)
        out["decoder_block"] = bench_decoder_block(torch, ops)

    if not args.no_cpu:
        out["cpu_baseline"] = cb
        err = np.abs(r["y0"] - y_cpu)
        tol = 1e-4 + 1e-3 * np.abs(y_cpu)
        out["parity_vs_cpu"] = {"max_abs_err": float(err.max()), "within_tol": bool((err <= tol).all())}
    else:
        out["cpu_baseline"] = None

    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
