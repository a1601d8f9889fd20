#!/usr/bin/env python3
"""Benchmark of the int8 hot path on one MI355X.

Default workload: the standalone int8 Gemm M=N=K=4096 (A fp32 N(0,1) quantised per row on the device,
constant int8 B, fp32 bias, fp32 output).  One step = per-row quantisation of A + the MFMA Gemm with its
fused dequantise/bias epilogue, all operands resident in HBM before the timed region.

Prints ONE JSON line: whole-step int8 TOPS (`value`), the roofline of the dominant kernel measured with HIP
events around every launch inside the timed region, and a CPU baseline (the scalar oracle, OpenMP) timed on
this host on a bounded sample.  Other workloads (--workload) report the remaining configurations.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

INT8_MFMA_PEAK_TOPS = 5000.0  # MI355X dense int8, published
HBM_PEAK_GBS = 8000.0         # MI355X HBM3E, published


def _events(lib, check, n):
    evs = []
    for _ in range(n):
        e = C.c_void_p()
        check(lib.ncnnhip_event_create(C.byref(e)))
        evs.append(e)
    return evs


def _elapsed(lib, check, a, b):
    ms = C.c_float()
    check(lib.ncnnhip_event_elapsed_ms(a, b, C.byref(ms)))
    return ms.value


def cpu_baseline_gemm(n, k, per_col, budget_s=12.0):
    """The same Gemm on this host's cores, on a row sample: the x86 VNNI restatement of how the reference's CPU path
    computes it (oracle/cpu_vnni_gemm.c, checked bit for bit against the scalar oracle); the scalar OpenMP oracle when
    the host has no AVX512-VNNI."""
    from oracle import cpubaseline, oracle
    if cpubaseline.available():
        threads = min(os.cpu_count() or 1, 16)
        os.environ.setdefault("OMP_NUM_THREADS", str(threads))
        rng = np.random.default_rng(0)
        bq = rng.integers(-127, 128, (n, k)).astype(np.int8)
        sb = rng.uniform(40, 60, n if per_col else 1).astype(np.float32)
        bias = np.zeros(n, np.float32)
        packed = cpubaseline.pack_b(bq)  # constant weights: packed once, outside the timed region, as at create_pipeline
        rows = min(n, 1024)
        a = rng.standard_normal((rows, k), dtype=np.float32)
        cpubaseline.gemm(a, packed, n, sb, bias)  # warm-up (threads, page faults)
        times, t_start = [], time.perf_counter()
        while len(times) < 3 or (time.perf_counter() - t_start < budget_s and len(times) < 10000):
            t0 = time.perf_counter()
            cpubaseline.gemm(a, packed, n, sb, bias)
            times.append(time.perf_counter() - t0)
        dt = float(np.mean(times))
        # the same on one thread, on an eighth of the rows
        cpubaseline.set_num_threads(1)
        a1 = a[: max(16, rows // 8)]
        cpubaseline.gemm(a1, packed, n, sb, bias)
        t1 = []
        while len(t1) < 2 or (sum(t1) < budget_s / 4 and len(t1) < 1000):
            t0 = time.perf_counter()
            cpubaseline.gemm(a1, packed, n, sb, bias)
            t1.append(time.perf_counter() - t0)
        cpubaseline.set_num_threads(threads)
        return dict({"value": 2.0 * rows * n * k / dt / 1e12, "unit": "TOPS", "cores": threads, "kind": "port",
                     "value_1_thread": 2.0 * a1.shape[0] * n * k / min(t1) / 1e12,
                     "sample": "%d of %d rows of the same Gemm (N=%d, K=%d): per-row quantise + AVX512-VNNI int8 GEMM + dequantise/bias, OpenMP, mean of %d runs "
                               "(%.1f s in all); one thread: %d rows, best of %d" % (rows, n, n, k, len(times), sum(times), a1.shape[0], len(t1))}, **host_cpu_info())
    threads = min(oracle.num_threads(), 16)
    oracle.set_num_threads(threads)
    rng = np.random.default_rng(0)
    bq = rng.integers(-127, 128, (n, k)).astype(np.int8)
    rows = 2 * threads
    while True:
        a = rng.standard_normal((rows, k), dtype=np.float32)
        t0 = time.perf_counter()
        aq, sa = oracle.gemm_quantize_rows(a)
        oracle.gemm_int8(aq, bq, sa, [50.0], np.zeros(n, np.float32), 4)
        dt = time.perf_counter() - t0
        if dt * 4 > budget_s or rows >= 4096:
            break
        rows = min(4096, int(rows * max(2.0, min(8.0, budget_s / 2 / max(dt, 1e-3)))))
    tops = 2.0 * rows * n * k / dt / 1e12
    return {"value": tops, "unit": "TOPS", "cores": threads, "kind": "port",
            "sample": "%d of %d rows of the same Gemm (N=%d, K=%d), scalar OpenMP oracle, %.1f s" % (rows, n, n, k, dt)}


def host_cpu_info():
    """CPU model, logical CPUs and the ISA flags that matter for an int8 path, from /proc/cpuinfo."""
    model, flags, n = "unknown", set(), 0
    try:
        with open("/proc/cpuinfo") as f:
            for ln in f:
                if ln.startswith("model name") and model == "unknown":
                    model = ln.split(":", 1)[1].strip()
                elif ln.startswith("flags") and not flags:
                    flags = set(ln.split(":", 1)[1].split())
                elif ln.startswith("processor"):
                    n += 1
    except OSError:
        pass
    keep = [f for f in ("sse4_2", "avx2", "fma", "avx512f", "avx512bw", "avx512_vnni", "avx_vnni", "amx_int8") if f in flags]
    return {"cpu_model": model, "logical_cpus": n or (os.cpu_count() or 1), "isa_flags": keep}


def cpu_baseline_blockquant(n, k, m, bits, block, budget_s=12.0):
    """The reference's only block-quant implementation is the naive fp32 loop (src/layer/gemm.cpp:425-483), OpenMP over the M
    activation rows only: restated in the oracle, timed here on a bounded number of weight rows with min(M, threads) threads
    (one thread at M = 1, as the reference runs it), and again with every thread over the weight rows for comparison."""
    from oracle import oracle
    from ncnn_amd import synth
    info = host_cpu_info()
    all_threads = min(oracle.num_threads(), 16)
    rows = min(n, 2048)
    a, packed, scales = synth.blockquant_operands(7, m, rows, k, bits, block)
    res = {}
    for label, threads in (("reference_threads", max(1, min(m, all_threads))), ("all_threads", all_threads)):
        oracle.set_num_threads(threads)
        oracle.gemm_blockquant(a, packed, scales, bits, block)
        times, t_start = [], time.perf_counter()
        while len(times) < 2 or (time.perf_counter() - t_start < budget_s / 2 and len(times) < 1000):
            t0 = time.perf_counter()
            oracle.gemm_blockquant(a, packed, scales, bits, block)
            times.append(time.perf_counter() - t0)
        nbytes = packed.nbytes + scales.nbytes + a.nbytes + m * rows * 4
        res[label] = (nbytes / min(times) / 1e9, threads, len(times), sum(times))
    oracle.set_num_threads(all_threads)
    v, threads, reps, total = res["reference_threads"]
    return dict({"value": v, "unit": "GB/s", "cores": threads, "kind": "port", "value_all_threads": res["all_threads"][0], "cores_all_threads": res["all_threads"][1],
                 "sample": "%d of %d weight rows of the same Gemm (K=%d, M=%d), naive fp32 block-quant loop as in the reference (OpenMP over M only: %d thread%s), "
                           "best of %d runs (%.1f s); all_threads = the same loop with the weight rows spread over %d threads"
                           % (rows, n, k, m, threads, "" if threads == 1 else "s", reps, total, res["all_threads"][1])}, **info)


def measured_traffic(key):
    """bytes per launch past L2 (read + write) from the committed counter summary, or None"""
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            e = json.load(f).get(key)
        return None if e is None else e["read_bytes"] + e["write_bytes"]
    except (OSError, ValueError, KeyError):
        return None


def bench_gemm(args, size, shape=None):
    import ncnn_amd
    from ncnn_amd.hip import check, lib as load
    from ncnn_amd import synth
    lib = load()
    rt = ncnn_amd.Runtime(0)
    m, n, k = shape if shape else (size, size, size)
    a, bq, sb, bias = synth.gemm_operands(size, m, n, k, per_col=args.b_scale == "per_column")
    d_a, d_bq, d_sb, d_bias = rt.up(a), rt.up(bq), rt.up(sb), rt.up(bias)
    d_aq = ncnn_amd.DeviceBuffer.empty((m, k), np.int8)
    d_sa = ncnn_amd.DeviceBuffer.empty((m,), np.float32)
    d_out = ncnn_amd.DeviceBuffer.empty((m, n), np.float32)
    st = rt.stream
    # From 128 tiles of 256 x 256 up the constant B is laid out once, before the timed region, in the 256x256 kernel's
    # tiled operand layout (what the Gemm layer does at create_pipeline) and the quantiser writes A in that layout.
    tiled = m % 256 == 0 and n % 256 == 0 and k % 64 == 0 and k <= 8192 and m * n >= 256 * 256 * 128
    if tiled:
        d_bt = ncnn_amd.DeviceBuffer.empty((n * k,), np.int8)
        check(lib.ncnnhip_gemm_int8_tile_operand(d_bq.ptr, k, n, k, 1, d_bt.ptr, st))
        rt.sync()

    def step(ev=None, ev_quant=None):
        # ev: the event pair around the Gemm launch (every timed step); ev_quant: a pair around the quantise pass, only in the
        # few extra steps after the timed region (each event record costs about 2 us of stream time)
        if ev_quant:
            check(lib.ncnnhip_event_record(ev_quant[0], st))
        if tiled:
            check(lib.ncnnhip_gemm_quantize_rows_tiled(d_a.ptr, k, m, k, d_aq.ptr, d_sa.ptr, st))
        else:
            check(lib.ncnnhip_gemm_quantize_rows(d_a.ptr, k, m, k, d_aq.ptr, k, d_sa.ptr, st))
        if ev_quant:
            check(lib.ncnnhip_event_record(ev_quant[1], st))
        if ev:
            check(lib.ncnnhip_event_record(ev[0], st))
        if tiled:
            check(lib.ncnnhip_gemm_int8_tiled(d_aq.ptr, d_bt.ptr, m, n, k, d_sa.ptr, d_sb.ptr, sb.size, d_bias.ptr, 4, 1.0, 1.0, d_out.ptr, n, st))
        else:
            check(lib.ncnnhip_gemm_int8(d_aq.ptr, k, d_bq.ptr, k, m, n, k, d_sa.ptr, d_sb.ptr, sb.size, d_bias.ptr, 4, 1.0, 1.0, 0,
                                        d_out.ptr, n, None, st))
        if ev:
            check(lib.ncnnhip_event_record(ev[1], st))

    if args.calib_copy:
        # one device-to-device copy of known size: gives counter runs (FETCH_SIZE / WRITE_SIZE) a dispatch to calibrate against
        check(lib.ncnnhip_memcpy_d2d(d_out.ptr, d_a.ptr, m * k * 4, st))
    for _ in range(args.warmup):
        step()
    rt.sync()
    evs = [_events(lib, check, 2) for _ in range(args.steps)]
    check(lib.ncnnhip_device_synchronize())
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(evs[i])
    check(lib.ncnnhip_device_synchronize())
    wall = time.perf_counter() - t0
    qevs = [_events(lib, check, 2) for _ in range(10)]
    for e in qevs:
        step(None, e)
    check(lib.ncnnhip_device_synchronize())

    gemm_ms = float(np.mean([_elapsed(lib, check, e[0], e[1]) for e in evs]))
    quant_ms = float(np.mean([_elapsed(lib, check, e[0], e[1]) for e in qevs]))
    ops = 2.0 * m * n * k
    ms_per_step = wall * 1e3 / args.steps
    achieved = ops / (gemm_ms * 1e-3) / 1e12

    line = {
        "metric": "int8 TOPS", "value": ops / (ms_per_step * 1e-3) / 1e12, "unit": "TOPS", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": ("standalone int8 Gemm M=N=K=%d" % size if not shape else "standalone int8 Gemm M=%d N=%d K=%d" % (m, n, k)) + ": per-row quantise A (fp32->int8) + int8 MFMA Gemm + fused dequantise/bias to fp32",
                   "b_scale": args.b_scale,
                   "parity": ("per-column B scales are a generalisation ncnn's Gemm cannot express: parity unpinned by the reference (own formula, "
                              "((float)acc*(1/sA_i))*(1/sB_j)); --b-scale per_tensor is the reference's form" if args.b_scale == "per_column"
                              else "the reference's per-tensor B scale: bit-exact against the oracle"), "operand_layout": "tiled" if tiled else "row-major",
                   "kernel_ms": {"gemm_int8": gemm_ms, "quantize_rows": quant_ms}},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": INT8_MFMA_PEAK_TOPS, "unit": "TOPS", "frac": achieved / INT8_MFMA_PEAK_TOPS,
                     "traffic": measured_traffic("gemm%d" % size), "kernel": "gemm_int8", "ops_per_launch": ops},
    }
    if m <= 48:
        # a few rows of A: the work is reading B once, so the line is priced against the memory system
        algo = n * k + m * k + m * n * 4
        gbs = algo / (gemm_ms * 1e-3) / 1e9
        line["roofline"] = {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS, "traffic": None,
                            "kernel": "gemm_int8 (few rows: gemm_skinny_int8_kernel where the shape allows)", "bytes_per_launch": algo,
                            "note": "B is the same buffer in every step and may be served by the memory-side cache: an upper bound on what a pass over cold weights reaches"}
        if not args.no_cpu:
            line["cpu_baseline"] = cpu_baseline_gemm(n, k, args.b_scale == "per_column")
        return line
    # what the matrix pipe of THIS chip sustains on operands like these (register-only spin, random bytes), beside the published peak
    mp = measure_peak_mfma_i8(lib, check, rt, True, iters=8000, reps=3)
    line["roofline"].update(measured_peak=mp["tops"], frac_of_measured=achieved / mp["tops"],
                            measured_peak_how="v_mfma_i32_32x32x32_i8 from registers on all %d SIMDs, pseudo-random operands: %.0f MHz, %.0f ops/clk/CU"
                                              % (mp["compute_units"] * 4, mp["shader_mhz"], mp["ops_per_clk_per_cu"]))
    if not args.no_cpu:
        # the CPU leg: first the checker (a row sample of the timed output buffer against the oracle), then the baseline timing
        from oracle import oracle
        rows = np.arange(0, m, max(1, m // 8))[:8]
        aq_ref, sa_ref = oracle.gemm_quantize_rows(a[rows])
        ref = oracle.gemm_int8(aq_ref, bq, sa_ref, sb, bias, 4)
        got = d_out.to_numpy(st)[rows]
        if not np.array_equal(got, ref):
            raise SystemExit("bench: GPU output differs from the oracle on the sampled rows")
        line["cpu_baseline"] = cpu_baseline_gemm(n, k, args.b_scale == "per_column")
    return line


def bench_blockquant(args, n, k, m, bits=8, block=64):
    """LLM-decode block-quant Gemm: weights int8 in blocks of 64 with one fp32 scale per block, streamed from a
    rotating set of weight copies larger than the 256 MB last-level cache so that the rate is an HBM rate."""
    import ncnn_amd
    from ncnn_amd.hip import check, lib as load
    from ncnn_amd import synth
    lib = load()
    rt = ncnn_amd.Runtime(0)
    a, packed, scales = synth.blockquant_operands(n + k + m, m, n, k, bits, block)
    wbytes = packed.nbytes + scales.nbytes
    copies = int(np.ceil(512e6 / wbytes)) + 1
    half = args.act == "fp16"
    packed_form = half or (args.act == "fp32" and k % 16 == 0 and (m >= 32 or lib.ncnnhip_gemm_blockquant_packed_supported(k)))
    # fp32 activations as the layers dispatch them: up to 4 rows (2 where K is beyond 4096) the few-row kernel, else the kernels that
    # split the activations in a pass of their own into a workspace
    rows_entry = packed_form and not half and (m >= 5 or (m >= 3 and k > 4096))
    if packed_form:  # constant weights are repacked once into matrix-core tiles, as create_pipeline does
        pw, pd = rt.blockquant_pack(packed, scales, block, bits=bits, k=k)
        d_w = [rt.up(pw) for _ in range(copies)]  # algorithmic bytes stay those of the .bin: the fields and one fp32 scale per block
        d_s = [rt.up(pd) for _ in range(copies)]
    else:
        d_w = [rt.up(packed) for _ in range(copies)]
        d_s = [rt.up(scales) for _ in range(copies)]
    d_a = rt.up(a.astype(np.float16) if half else a)
    d_out = ncnn_amd.DeviceBuffer.empty((m, n), np.float32)
    st = rt.stream
    rows_ws_bytes = C.c_size_t(0)
    if rows_entry:
        check(lib.ncnnhip_gemm_blockquant_packed_rows_workspace_bytes(m, k, C.byref(rows_ws_bytes)))
        d_rows_ws = ncnn_amd.DeviceBuffer.empty((rows_ws_bytes.value,), np.uint8)

    def launch(i):
        j = i % copies
        if half:
            check(lib.ncnnhip_gemm_blockquant_packed_f16a(d_a.ptr, k, m, n, k, d_w[j].ptr, d_s[j].ptr, bits, block, None, -1, 1.0, 1.0, d_out.ptr, n, st))
        elif rows_entry:
            check(lib.ncnnhip_gemm_blockquant_packed_rows(d_a.ptr, k, m, n, k, d_w[j].ptr, d_s[j].ptr, bits, block, None, None, -1, 1.0, 1.0, d_out.ptr, n,
                                                          d_rows_ws.ptr, rows_ws_bytes.value, st))
        elif packed_form:
            check(lib.ncnnhip_gemm_blockquant_packed(d_a.ptr, k, m, n, k, d_w[j].ptr, d_s[j].ptr, bits, block, None, None, -1, 1.0, 1.0, d_out.ptr, n, st))
        else:
            check(lib.ncnnhip_gemm_blockquant(d_a.ptr, k, m, n, k, d_w[j].ptr, bits, block, d_s[j].ptr, None, None, -1, 1.0, 1.0, d_out.ptr, n, st))

    for i in range(args.warmup):
        launch(i)
    rt.sync()
    evs = _events(lib, check, 2)
    check(lib.ncnnhip_device_synchronize())
    t0 = time.perf_counter()
    check(lib.ncnnhip_event_record(evs[0], st))
    for i in range(args.steps):
        launch(i)
    check(lib.ncnnhip_event_record(evs[1], st))
    check(lib.ncnnhip_device_synchronize())
    wall = time.perf_counter() - t0
    k_ms = _elapsed(lib, check, evs[0], evs[1]) / args.steps
    abytes = m * k * (2 if half else 4)
    algo = wbytes + abytes + m * n * 4
    achieved = algo / (k_ms * 1e-3) / 1e9
    ms_per_step = wall * 1e3 / args.steps
    del d_w, d_s
    floor = measure_peak_hbm_read(lib, check, rt, int(algo), 8, launches=200)  # a kernel that only READS as many bytes, same launch pattern
    line = {
        "metric": "HBM GB/s", "value": algo / (ms_per_step * 1e-3) / 1e9, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "block-quant Gemm M=%d N=%d K=%d, %d-bit weights in blocks of %d, fp32 block scales, %s activations" % (m, n, k, bits, block, args.act),
                   "weight_copies_rotated": copies},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "traffic": measured_traffic("blockquant:%dx%dx%d%s%s" % (n, k, m, "" if (bits, block) == (8, 64) else ":%d:%d" % (bits, block),
                                                                              "" if half else ":" + args.act)) if packed_form else None,
                     "kernel": ("blockquant_rows16_bf16x3_kernel" if (m <= 128 and 5.0 + ((m + 15) // 16) * (n * k * bits / 8.0 / 1.0e6) / 2.0 <= 6.0 + k / 85.0) else "blockquant_rows_bf16x3_kernel") if rows_entry else "blockquant8_upfront_kernel" if packed_form else ("blockquant8_f32_mfma_kernel" if m >= 32 else "blockquant8_stream_kernel"),
                     "bytes_per_launch": algo,
                     "measured_peak": floor["gbs"], "frac_of_measured": achieved / floor["gbs"],
                     "measured_peak_how": "read-only kernel over the same number of bytes, back-to-back launches over rotating copies: %.2f us per launch"
                                          % floor["us_per_launch"]},
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline_blockquant(n, k, m, bits, block)
    return line


def bench_blockquant_multi(args, ns, k, m, bits=8, block=64):
    """Sibling block-quant Gemms of a decoder layer (gate + up, q + k + v) on the same activation rows: all matrices in ONE launch
    (ncnnhip_gemm_blockquant_packed_multi), against one launch per matrix, weights rotated over more copies than the last-level
    cache holds.  One step = every matrix of the group once."""
    import ncnn_amd
    from ncnn_amd.hip import check, lib as load
    from ncnn_amd import synth
    lib = load()
    rt = ncnn_amd.Runtime(0)
    half = args.act == "fp16"
    if not half and args.act != "fp32":
        raise SystemExit("blockquant-multi runs on the packed weights: --act fp16 or fp32")
    a = None
    packs, wbytes = [], 0
    for i, n in enumerate(ns):
        ai, packed, scales = synth.blockquant_operands(n + k + m + i, m, n, k, bits, block)
        a = ai if a is None else a
        wbytes += packed.nbytes + scales.nbytes
        packs.append(rt.blockquant_pack(packed, scales, block, bits=bits, k=k))
    copies = int(np.ceil(512e6 / wbytes)) + 1
    dev = [[(rt.up(pw), rt.up(pd), n, None, -1, 1.0, 1.0) for (pw, pd), n in zip(packs, ns)] for _ in range(copies)]
    d_a = rt.up(a.astype(np.float16) if half else a)
    douts = [ncnn_amd.DeviceBuffer.empty((m, n), np.float32) for n in ns]
    multi_args = [rt.blockquant_multi_args(mats, douts) for mats in dev]
    st = rt.stream
    esize = 2 if half else 4

    def launch_multi(i):
        nn, ws, ds, cs, bts, als, bes, outs, strides = multi_args[i % copies]
        check(lib.ncnnhip_gemm_blockquant_packed_multi(d_a.ptr, esize, k, m, k, len(ns), nn, ws, ds, bits, block, None, cs, bts, als, bes, outs, strides, st))

    def launch_singles(i):
        for (dw, dd, n, _, _, _, _), do in zip(dev[i % copies], douts):
            if half:
                check(lib.ncnnhip_gemm_blockquant_packed_f16a(d_a.ptr, k, m, n, k, dw.ptr, dd.ptr, bits, block, None, -1, 1.0, 1.0, do.ptr, n, st))
            else:
                check(lib.ncnnhip_gemm_blockquant_packed(d_a.ptr, k, m, n, k, dw.ptr, dd.ptr, bits, block, None, None, -1, 1.0, 1.0, do.ptr, n, st))

    def timed(fn):
        for i in range(args.warmup):
            fn(i)
        rt.sync()
        evs = _events(lib, check, 2)
        t0 = time.perf_counter()
        check(lib.ncnnhip_event_record(evs[0], st))
        for i in range(args.steps):
            fn(i)
        check(lib.ncnnhip_event_record(evs[1], st))
        check(lib.ncnnhip_device_synchronize())
        return _elapsed(lib, check, evs[0], evs[1]) / args.steps, (time.perf_counter() - t0) * 1e3 / args.steps

    singles_ms, _ = timed(launch_singles)
    k_ms, ms_per_step = timed(launch_multi)
    algo = wbytes + m * k * esize + sum(m * n * 4 for n in ns)
    achieved = algo / (k_ms * 1e-3) / 1e9
    del dev, multi_args
    floor = measure_peak_hbm_read(lib, check, rt, int(algo), 8, launches=200)
    line = {
        "metric": "HBM GB/s", "value": algo / (ms_per_step * 1e-3) / 1e9, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "block-quant Gemms %s x K=%d on the same M=%d activation rows in one launch, %d-bit weights in blocks of %d, fp32 block scales, %s activations"
                               % ("+".join(str(n) for n in ns), k, m, bits, block, args.act),
                   "weight_copies_rotated": copies, "one_launch_per_matrix_us": singles_ms * 1e3, "one_launch_us": k_ms * 1e3},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": None,
                     "kernel": "blockquant8_upfront_kernel (several matrices per launch)", "bytes_per_launch": algo,
                     "measured_peak": floor["gbs"], "frac_of_measured": achieved / floor["gbs"],
                     "measured_peak_how": "read-only kernel over the same number of bytes, back-to-back launches over rotating copies: %.2f us per launch"
                                          % floor["us_per_launch"]},
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline_blockquant(sum(ns), k, m, bits, block)
    return line


def measure_peak_mfma_i8(lib, check, rt, random_operands, iters=20000, reps=5):
    """int8 matrix-core rate with nothing else going on: (POP/s, shader MHz, operations per clock per compute unit)."""
    import ncnn_amd
    scratch = ncnn_amd.DeviceBuffer.empty((8,), np.int64)
    scratch.fill_bytes(0, rt.stream)
    name = C.create_string_buffer(128)
    cus = C.c_int()
    check(lib.ncnnhip_device_info(name, 128, C.byref(cus), None))
    check(lib.ncnnhip_peak_mfma_i8(iters, int(random_operands), scratch.ptr, rt.stream))  # warm-up (clocks ramp)
    rt.sync()
    ev = _events(lib, check, 2)
    best = None
    for _ in range(reps):
        check(lib.ncnnhip_event_record(ev[0], rt.stream))
        check(lib.ncnnhip_peak_mfma_i8(iters, int(random_operands), scratch.ptr, rt.stream))
        check(lib.ncnnhip_event_record(ev[1], rt.stream))
        check(lib.ncnnhip_event_synchronize(ev[1]))
        ms = _elapsed(lib, check, ev[0], ev[1])
        clocks = scratch.to_numpy(rt.stream)
        ops = cus.value * 4.0 * iters * 8 * 65536
        r = (ops / (ms * 1e-3) / 1e12, float(clocks[0]) / max(float(clocks[1]), 1.0) * 100.0, 4.0 * iters * 8 * 65536 / max(float(clocks[0]), 1.0))
        if best is None or r[0] > best[0]:
            best = r
    return {"tops": best[0], "shader_mhz": best[1], "ops_per_clk_per_cu": best[2], "compute_units": cus.value,
            "operands": "random" if random_operands else "zeros", "instruction": "v_mfma_i32_32x32x32_i8", "mfma_per_wavefront": iters * 8}


def measure_peak_hbm_read(lib, check, rt, nbytes, loads_per_lane=16, launches=200):
    """GB/s of a kernel that only reads `nbytes`, back-to-back launches over rotating copies larger than the last-level cache."""
    import ncnn_amd
    nbytes = max(4096, nbytes // 16 * 16)
    copies = int(np.ceil(600e6 / nbytes)) + 1
    bufs = []
    for _ in range(copies):
        b = ncnn_amd.DeviceBuffer(nbytes)
        b.fill_bytes(1, rt.stream)
        bufs.append(b)
    sink = ncnn_amd.DeviceBuffer.zeros(64, rt.stream)
    for i in range(20):
        check(lib.ncnnhip_peak_hbm_read(bufs[i % copies].ptr, nbytes, loads_per_lane, sink.ptr, rt.stream))
    rt.sync()
    ev = _events(lib, check, 2)
    check(lib.ncnnhip_event_record(ev[0], rt.stream))
    for i in range(launches):
        check(lib.ncnnhip_peak_hbm_read(bufs[i % copies].ptr, nbytes, loads_per_lane, sink.ptr, rt.stream))
    check(lib.ncnnhip_event_record(ev[1], rt.stream))
    check(lib.ncnnhip_event_synchronize(ev[1]))
    us = _elapsed(lib, check, ev[0], ev[1]) * 1e3 / launches
    return {"gbs": nbytes / us / 1e3, "us_per_launch": us, "bytes": nbytes, "loads_per_lane": loads_per_lane, "copies_rotated": copies}


def measure_peak_launch(lib, check, rt, nodes, reps):
    """us per dependent one-wavefront launch: `nodes` launches enqueued on a stream, and the same captured once into a
    graph and replayed; events around `reps` repetitions of each, plus the host's time to enqueue them."""
    import ncnn_amd
    counter = ncnn_amd.DeviceBuffer.empty((16,), np.int32)
    counter.fill_bytes(0, rt.stream)
    ev = _events(lib, check, 2)
    out = {"nodes": nodes, "reps": reps}
    for r in range(3):
        check(lib.ncnnhip_peak_launch_chain(nodes, counter.ptr, rt.stream))
    rt.sync()
    t0 = time.perf_counter()
    check(lib.ncnnhip_event_record(ev[0], rt.stream))
    for r in range(reps):
        check(lib.ncnnhip_peak_launch_chain(nodes, counter.ptr, rt.stream))
    check(lib.ncnnhip_event_record(ev[1], rt.stream))
    host = time.perf_counter() - t0
    check(lib.ncnnhip_event_synchronize(ev[1]))
    out["stream_us_per_launch"] = _elapsed(lib, check, ev[0], ev[1]) * 1e3 / (nodes * reps)
    out["stream_host_enqueue_us_per_launch"] = host * 1e6 / (nodes * reps)
    exe = C.c_void_p()
    check(lib.ncnnhip_stream_begin_capture(rt.stream))
    check(lib.ncnnhip_peak_launch_chain(nodes, counter.ptr, rt.stream))
    check(lib.ncnnhip_stream_end_capture(rt.stream, C.byref(exe)))
    for r in range(3):
        check(lib.ncnnhip_graph_launch(exe, rt.stream))
    rt.sync()
    t0 = time.perf_counter()
    check(lib.ncnnhip_event_record(ev[0], rt.stream))
    for r in range(reps):
        check(lib.ncnnhip_graph_launch(exe, rt.stream))
    check(lib.ncnnhip_event_record(ev[1], rt.stream))
    host = time.perf_counter() - t0
    check(lib.ncnnhip_event_synchronize(ev[1]))
    out["graph_us_per_node"] = _elapsed(lib, check, ev[0], ev[1]) * 1e3 / (nodes * reps)
    out["graph_host_enqueue_us_per_node"] = host * 1e6 / (nodes * reps)
    check(lib.ncnnhip_graph_destroy(exe))
    total = int(counter.to_numpy(rt.stream)[0])
    if total != nodes * (2 * reps + 6):
        raise SystemExit("bench.py: the launch chain counted %d, expected %d" % (total, nodes * (2 * reps + 6)))
    return out


def bench_peak(args, what, arg):
    """The chip's own ceilings, measured: `peak:mfma_i8[:zeros|random]`, `peak:hbm_read:<bytes>[:<loads per lane>]` and
    `peak:launch[:<nodes>]` (what one dependent kernel launch costs, on a stream and as a node of a replayed graph)."""
    import ncnn_amd
    from ncnn_amd.hip import check, lib as load
    lib = load()
    rt = ncnn_amd.Runtime(0)
    base = {"n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "data": "synthetic"}
    if what == "mfma_i8":
        kinds = [arg == "random"] if arg in ("zeros", "random") else [False, True]
        res = [measure_peak_mfma_i8(lib, check, rt, k, iters=max(1000, args.steps * 400)) for k in kinds]
        top = res[-1]
        return dict(base, metric="int8 TOPS", value=top["tops"], unit="TOPS", ms_per_step=None, dtype="int8",
                    config={"workload": "register-only spin of v_mfma_i32_32x32x32_i8 on every SIMD: the matrix pipe's sustained rate", "runs": res},
                    roofline={"bound": "mfma", "achieved": top["tops"], "peak": INT8_MFMA_PEAK_TOPS, "unit": "TOPS", "frac": top["tops"] / INT8_MFMA_PEAK_TOPS,
                              "traffic": None, "kernel": "peak_mfma_i8_kernel"})
    if what == "hbm_read":
        parts = arg.split(":") if arg else []
        nbytes = int(float(parts[0])) if parts else 256 << 20
        lpl = int(parts[1]) if len(parts) > 1 else 16
        r = measure_peak_hbm_read(lib, check, rt, nbytes, lpl, launches=max(50, args.steps * 4))
        return dict(base, metric="HBM GB/s", value=r["gbs"], unit="GB/s", ms_per_step=r["us_per_launch"] * 1e-3, dtype="u8",
                    config={"workload": "read-only kernel over %d bytes, %d 16-byte loads in flight per lane, weight-stream rotation as in the block-quant workload"
                                        % (r["bytes"], lpl), "run": r},
                    roofline={"bound": "hbm", "achieved": r["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": r["gbs"] / HBM_PEAK_GBS, "traffic": None,
                              "kernel": "peak_hbm_read_kernel", "bytes_per_launch": r["bytes"]})
    if what == "launch":
        r = measure_peak_launch(lib, check, rt, int(arg) if arg else 57, reps=max(20, args.steps))
        best = min(r["stream_us_per_launch"], r["graph_us_per_node"])
        return dict(base, metric="us per dependent launch", value=best, unit="us", ms_per_step=best * r["nodes"] * 1e-3, dtype="none", higher_is_better=False,
                    config={"workload": "chain of %d one-wavefront kernels, each reading what the one before wrote: stream launches against one replayed graph"
                                        % r["nodes"], "run": r},
                    roofline={"bound": "launch", "achieved": best, "peak": None, "unit": "us", "frac": None, "traffic": None, "kernel": "peak_launch_chain_kernel"})
    raise SystemExit("unknown peak workload " + what)


def bench_mha(args, embed, heads, src, past):
    """Self-attention layer with 8-bit block-quantised weights (blocks of 64) on device-resident operands: the launches of
    MultiHeadAttention_hip::forward without its host copies.  src new tokens are appended to a cache of `past` tokens."""
    import ncnn_amd
    from ncnn_amd.hip import check, lib as load
    from ncnn_amd import synth
    lib = load()
    rt = ncnn_amd.Runtime(0)
    st = rt.stream
    rng = np.random.default_rng(0)
    dst = past + src
    ws, host = [], []
    for _ in range(4):
        w = rng.normal(0, 1.0 / np.sqrt(embed), (embed, embed)).astype(np.float32)
        packed, scales = synth.blockquant_weights(w, 8, 64)
        bias = rng.uniform(-0.1, 0.1, embed).astype(np.float32)
        host.append((packed, scales, bias))
        pw, pd = rt.blockquant_pack(packed, scales, 64)  # the second form create_pipeline uploads: matrix-core tiles
        ws.append((rt.up(packed), rt.up(scales), rt.up(bias), packed.nbytes + scales.nbytes, rt.up(pw), rt.up(pd)))
    packed, scales, bias = [np.concatenate([h[i] for h in host[:3]]) for i in range(3)]
    pw, pd = rt.blockquant_pack(packed, scales, 64)
    w_qkv = (rt.up(packed), rt.up(scales), rt.up(bias), packed.nbytes + scales.nbytes, rt.up(pw), rt.up(pd))
    d_x = rt.up(rng.normal(0, 1, (src, embed)).astype(np.float32))
    d_kt = rt.up(rng.normal(0, 1, (embed, dst)).astype(np.float32))
    d_vt = rt.up(rng.normal(0, 1, (embed, dst)).astype(np.float32))
    d_ctx, d_out = [ncnn_amd.DeviceBuffer.empty((src, embed), np.float32) for _ in range(2)]
    d_qkv = ncnn_amd.DeviceBuffer.empty((src, 3 * embed), np.float32)
    scale = float(1.0 / np.sqrt(embed // heads))
    wsb = C.c_size_t()
    check(lib.ncnnhip_attention_workspace_bytes(heads, embed // heads, src, dst, C.byref(wsb)))
    d_ws = ncnn_amd.DeviceBuffer.empty((max(wsb.value, 4),), np.uint8)

    # the projections as the layer dispatches them (blockquant_gemm_device): fewer than 32 rows on the packed tiles four rows per pass,
    # 32 and more through the tiled bf16 kernel with its workspace; `--act fp32-bin` keeps the kernels of the .bin layout
    packed_ok = args.act != "fp32-bin" and lib.ncnnhip_gemm_blockquant_packed_supported(embed)
    rows_ws = None
    if packed_ok and src >= 32:
        rb = C.c_size_t()
        check(lib.ncnnhip_gemm_blockquant_packed_rows_workspace_bytes(src, embed, C.byref(rb)))
        rows_ws = (ncnn_amd.DeviceBuffer.empty((rb.value,), np.uint8), rb.value)

    def project(x, w, n, out, out_stride):
        if rows_ws is not None:
            check(lib.ncnnhip_gemm_blockquant_packed_rows(x.ptr, embed, src, n, embed, w[4].ptr, w[5].ptr, 8, 64, None, w[2].ptr, 4, 1.0, 1.0, out.ptr, out_stride,
                                                          rows_ws[0].ptr, rows_ws[1], st))
        elif packed_ok:
            check(lib.ncnnhip_gemm_blockquant_packed(x.ptr, embed, src, n, embed, w[4].ptr, w[5].ptr, 8, 64, None, w[2].ptr, 4, 1.0, 1.0, out.ptr, out_stride, st))
        else:
            check(lib.ncnnhip_gemm_blockquant(x.ptr, embed, src, n, embed, w[0].ptr, 8, 64, w[1].ptr, None, w[2].ptr, 4, 1.0, 1.0, out.ptr, out_stride, st))

    def step():
        # self-attention: q, k and v out of one Gemm over the three weight matrices as one (what create_pipeline keeps for this case),
        # its k and v columns appended to the cache and the query's scale applied by the attention call
        project(d_x, w_qkv, 3 * embed, d_qkv, 3 * embed)
        check(lib.ncnnhip_attention_f32_append(d_qkv.ptr, 3 * embed, scale, d_kt.ptr, d_vt.ptr, dst, past, None, 0, heads, embed // heads, src, d_ctx.ptr, d_ws.ptr,
                                               wsb.value, st))
        project(d_ctx, ws[3], embed, d_out, embed)

    for _ in range(args.warmup):
        step()
    rt.sync()
    evs = _events(lib, check, 2)
    t0 = time.perf_counter()
    check(lib.ncnnhip_event_record(evs[0], st))
    for _ in range(args.steps):
        step()
    check(lib.ncnnhip_event_record(evs[1], st))
    check(lib.ncnnhip_device_synchronize())
    wall = time.perf_counter() - t0
    k_ms = _elapsed(lib, check, evs[0], evs[1]) / args.steps
    # bytes that must move: the four weight matrices with their scales, the keys and values of the cache, activations in and out
    algo = sum(w[3] for w in ws) + 2 * embed * dst * 4 + 2 * src * embed * 4
    ops = 2.0 * src * embed * embed * 4 + 4.0 * src * dst * embed
    ms_per_step = wall * 1e3 / args.steps
    achieved = algo / (k_ms * 1e-3) / 1e9
    return {
        "metric": "HBM GB/s", "value": algo / (ms_per_step * 1e-3) / 1e9, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "self-attention layer, embed %d, %d heads, %d new tokens on a cache of %d, 8-bit block-quantised weights (blocks of 64)"
                               % (embed, heads, src, past), "launches_per_step": (6 if rows_ws is not None else 3) + (1 if wsb.value else 0), "projections": "tiled bf16x3 kernel" if rows_ws is not None else ("packed tiles" if packed_ok else ".bin layout"), "device_ms_per_step": k_ms, "gflop": ops / 1e9},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": None,
                     "kernel": "whole layer (q/k/v projection, cache append, attention core, output projection)", "bytes_per_launch": algo},
    }


def _timed(fn, budget_s, min_reps=3, max_reps=100000):
    fn()  # warm-up: threads, page faults, buffers that later calls write again
    times, t_start = [], time.perf_counter()
    while len(times) < min_reps or (time.perf_counter() - t_start < budget_s and len(times) < max_reps):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    return times


def cpu_baseline_conv(c, h, w, cout, k, pad, batch=1, budget_s=10.0):
    """The same layer on this host's cores the way the reference's x86 path computes it (oracle/cpu_vnni_conv.c: quantise,
    im2col, AVX512-VNNI, vector epilogue; bit-exact against the scalar oracle), on all threads and on one; the scalar
    OpenMP oracle when the host has no AVX512-VNNI."""
    from oracle import cpubaseline as cb, oracle
    rng = np.random.default_rng(0)
    wq = rng.integers(-127, 128, (cout, c, k, k)).astype(np.int8)
    ws = rng.uniform(50, 100, cout).astype(np.float32)
    b = rng.uniform(-0.1, 0.1, cout).astype(np.float32)
    oh, ow = h + 2 * pad - k + 1, w + 2 * pad - k + 1
    ops = 2.0 * batch * cout * oh * ow * c * k * k
    if cb.available():
        threads = min(os.cpu_count() or 1, 16)
        x = rng.uniform(-1, 1, (batch, h, w, c)).astype(np.float32)
        d = cb.ConvDesc(w, h, c, batch, cout, k, k, 1, 1, 1, 1, pad, pad, pad, pad, 0.0)
        packed, scale_in = cb.pack_conv_weights(wq), cb.fold_scales(ws, np.float32(127.0))  # load-time work, outside the timed region
        res = {}
        for label, th in (("all", threads), ("one", 1)):
            cb.set_num_threads(th)
            keep = [None]

            def once():
                keep[0] = cb.conv_nhwc(d, x, 127.0, packed, scale_in, b, None, 1, (0.0, 0.0), out=keep[0])
            res[label] = _timed(once, budget_s if label == "all" else budget_s / 3)
        cb.set_num_threads(threads)
        dt = float(np.mean(res["all"]))
        return dict({"value": ops / dt / 1e12, "unit": "TOPS", "cores": threads, "kind": "port", "value_1_thread": ops / min(res["one"]) / 1e12,
                     "sample": "%d whole forward passes of the same layer, batch %d (quantise + im2col + AVX512-VNNI int8 GEMM + dequantise/bias/ReLU, OpenMP), "
                               "mean %.3f ms each; one thread: best of %d, %.3f ms" % (len(res["all"]), batch, dt * 1e3, len(res["one"]), min(res["one"]) * 1e3)},
                    **host_cpu_info())
    threads = min(oracle.num_threads(), 16)
    oracle.set_num_threads(threads)
    x = rng.uniform(-1, 1, (c, h, w)).astype(np.float32)
    d = oracle.make_desc((c, h, w), cout, (k, k), (1, 1), (1, 1), (pad,) * 4, 0.0, 1, 1, 1, 1, (0.0, 0.0))
    times = _timed(lambda: oracle.convolution_int8(d, x, wq, b, ws, np.float32(127.0), None), budget_s, max_reps=200)
    dt = float(np.mean(times))
    return dict({"value": ops / batch / dt / 1e12, "unit": "TOPS", "cores": threads, "kind": "port",
                 "sample": "%d whole forward passes of the same layer at batch 1 (quantise + convolution + epilogue), scalar OpenMP oracle, %.2f ms each"
                           % (len(times), dt * 1e3)}, **host_cpu_info())


def cpu_baseline_net(param, blob, input_shape, batch, ops, budget_s=12.0):
    """The same model on this host's cores: the whole-model pass of oracle/cpunet.py (VNNI convolution, depthwise and
    inner-product layers plus the glue loops, bit-exact against the scalar oracle's executor), on a bounded batch, on all
    threads and on one.  None when the host has no AVX512-VNNI (the scalar executor would take minutes per image)."""
    from oracle import cpubaseline as cb, cpunet
    if not cb.available():
        return None
    threads = min(os.cpu_count() or 1, 16)
    nb = min(batch, 4)
    x = np.random.default_rng(0).uniform(0, 1, (nb,) + tuple(input_shape)).astype(np.float32)
    model = cpunet.load(param, blob)  # load-time work, outside the timed region
    res = {}
    for label, th, xs in (("all", threads, x), ("one", 1, x[:1])):
        cb.set_num_threads(th)
        keep = [None]

        def once():
            keep[0] = cpunet.run(model, xs, keep=keep[0])
        res[label] = _timed(once, budget_s if label == "all" else budget_s / 2, min_reps=2)
    cb.set_num_threads(threads)
    dt = float(np.mean(res["all"]))
    per_image = ops / batch
    return dict({"value": per_image * nb / dt / 1e12, "unit": "TOPS", "cores": threads, "kind": "port", "images_per_s": nb / dt,
                 "value_1_thread": per_image / min(res["one"]) / 1e12, "images_per_s_1_thread": 1.0 / min(res["one"]),
                 "sample": "%d whole forward passes of the same model at batch %d (of the workload's %d), every layer on the CPU: mean %.2f ms per pass; "
                           "one thread, batch 1: best of %d, %.2f ms" % (len(res["all"]), nb, batch, dt * 1e3, len(res["one"]), min(res["one"]) * 1e3)},
                **host_cpu_info())


def bench_conv(args, spec):
    """One Convolution layer, fp32 in -> fp32 out with ReLU (int8_scale_term 1), batch 1 unless stated: the single-layer
    configuration.  spec = <cin>x<h>x<w>:<cout>:k<k>[:b<batch>].  A step is the layer as it runs inside a device-resident
    net: Quantize of the fp32 blob + the implicit-GEMM kernel with its fused dequantise/bias/ReLU epilogue, back to back
    on one stream (the layer is launch/latency bound: about 0.1 us of matrix work)."""
    import ncnn_amd
    from ncnn_amd.hip import Activation, ConvDesc, check, lib as load
    lib = load()
    rt = ncnn_amd.Runtime(0)
    st = rt.stream
    parts = spec.split(":")
    c, h, w = (int(v) for v in parts[0].split("x"))
    cout, k = int(parts[1]), int(parts[2][1:])
    batch = int(parts[3][1:]) if len(parts) > 3 else 1
    pad = k // 2
    cp = lib.ncnnhip_padded_channels
    rng = np.random.default_rng(0)
    desc = ConvDesc(w, h, c, batch, cout, k, k, 1, 1, 1, 1, pad, pad, pad, pad, 0.0, 1)
    nb, wb, sb = C.c_size_t(), C.c_size_t(), C.c_size_t()
    check(lib.ncnnhip_conv_nhwc_sizes(C.byref(desc), C.byref(nb), C.byref(wb), C.byref(sb)))
    wq = rng.integers(-127, 128, cout * c * k * k).astype(np.int8)
    pk = np.empty(wb.value, np.int8)
    check(lib.ncnnhip_conv_pack_weights(C.byref(desc), wq.ctypes.data, pk.ctypes.data))
    xf = np.zeros((batch, h * w, cp(c)), np.float32)
    xf[:, :, :c] = rng.uniform(-1, 1, (batch, h * w, c))
    d_x, d_xq = rt.up(xf), ncnn_amd.DeviceBuffer.empty((batch, h * w, cp(c)), np.int8)
    d_s = rt.up(np.array([127.0], np.float32))
    d_pk, d_si, d_b = rt.up(pk), rt.up(rng.uniform(1e-4, 1e-3, cout).astype(np.float32)), rt.up(rng.uniform(-0.1, 0.1, cout).astype(np.float32))
    d_out = ncnn_amd.DeviceBuffer.empty((batch, h * w, cp(cout)), np.float32)
    d_ws = ncnn_amd.DeviceBuffer.zeros(sb.value, st)
    act = Activation.make(1)

    def quantise():
        check(lib.ncnnhip_quantize_nhwc(d_x.ptr, d_xq.ptr, batch * h * w, c, d_s.ptr, 1, st))

    def conv():
        check(lib.ncnnhip_conv_int8_nhwc(C.byref(desc), d_xq.ptr, d_pk.ptr, d_si.ptr, d_b.ptr, None, act, d_out.ptr, 1, 0, 0, d_ws.ptr, sb.value, st))

    def two_launches():
        quantise()
        conv()

    def one_launch():  # the Quantize pass inside the convolution's loader
        check(lib.ncnnhip_conv_int8_nhwc_from_float(C.byref(desc), d_x.ptr, 4, d_s.ptr, d_pk.ptr, d_si.ptr, d_b.ptr, None, act, d_out.ptr, None, d_fws.ptr, fws.value, st))

    fused_quantise = bool(lib.ncnnhip_conv_from_float_supported(C.byref(desc)))
    fws = C.c_size_t(0)
    if fused_quantise:
        check(lib.ncnnhip_conv_from_float_workspace_bytes(C.byref(desc), C.byref(fws)))
    d_fws = ncnn_amd.DeviceBuffer.zeros(fws.value, st)
    step = one_launch if fused_quantise else two_launches
    kernel = one_launch if fused_quantise else conv
    small_tile = bool(lib.ncnnhip_conv_small_tile_selected(C.byref(desc), 4 if fused_quantise else 1))

    def wall_ms(fn):
        check(lib.ncnnhip_device_synchronize())
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn()
        check(lib.ncnnhip_device_synchronize())
        return (time.perf_counter() - t0) * 1e3 / args.steps

    for _ in range(args.warmup):
        two_launches()
        step()
    rt.sync()
    ev = _events(lib, check, 2)
    check(lib.ncnnhip_event_record(ev[0], st))
    for _ in range(args.steps):
        kernel()
    check(lib.ncnnhip_event_record(ev[1], st))
    check(lib.ncnnhip_event_synchronize(ev[1]))
    kernel_ms = _elapsed(lib, check, ev[0], ev[1]) / args.steps
    ms_per_step = wall_ms(step)
    two_launch_ms = wall_ms(two_launches)
    ops = 2.0 * batch * cout * h * w * c * k * k
    achieved = ops / (kernel_ms * 1e-3) / 1e12
    line = {
        "metric": "int8 TOPS", "value": ops / (ms_per_step * 1e-3) / 1e12, "unit": "TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": "Convolution %dx%d %d->%d on %dx%d, batch %d, fp32 in -> quantise -> int8 implicit GEMM -> fp32 out with ReLU; "
                               "back-to-back launches, channels-last resident blobs" % (k, k, c, cout, h, w, batch), "kernel_us": kernel_ms * 1e3,
                   "launches_per_step": 1 if fused_quantise else 2,
                   "submission": "one launch, the Quantize pass inside the convolution's loader" if fused_quantise else "Quantize kernel, then the convolution kernel",
                   "quantize_then_convolution_us": two_launch_ms * 1e3},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": INT8_MFMA_PEAK_TOPS, "unit": "TOPS", "frac": achieved / INT8_MFMA_PEAK_TOPS,
                     "traffic": measured_traffic("conv:" + spec), "kernel": "conv_patch_kernel" if small_tile else "conv_nhwc_pipelined_kernel", "ops_per_launch": ops},
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline_conv(c, h, w, cout, k, pad, batch)
    return line


def bench_layers(args, which, batch):
    """The quantised layers of a ResNet-50 / MobileNetV2-shaped int8 net, each alone through the C ABI on device-resident
    channels-last blobs of its real shape (the form the layers see inside a running net): fp32 inputs are quantised
    first, int8 inputs feed the kernel directly, outputs are requantised int8 or fp32 as the generated model asks.
    One step = one pass over all quantised layers; the table lists each layer's time with and without its quantise pass."""
    import ncnn_amd
    from ncnn_amd.hip import Activation, ConvDesc, check, lib as load
    from ncnn_amd import zoo
    lib = load()
    rt = ncnn_amd.Runtime(0)
    st = rt.stream
    g = getattr(zoo, which)()
    rows = zoo.quantised_layer_table(g)
    rng = np.random.default_rng(0)
    cp = lib.ncnnhip_padded_channels
    plans = []
    for r in rows:
        if r["type"] == "InnerProduct":
            k, n = int(np.prod(r["in_shape"])), r["out_shape"][0]
            x = rng.uniform(-1, 1, (batch, k)).astype(np.float32)
            plan = dict(row=r, kind="fc", k=k, n=n, d_x=rt.up(x), d_xq=ncnn_amd.DeviceBuffer.empty((batch, k), np.int8),
                        d_w=rt.up(rng.integers(-127, 128, (n, k)).astype(np.int8)), d_si=rt.up(rng.uniform(1e-4, 1e-3, n).astype(np.float32)),
                        d_b=rt.up(rng.uniform(-0.1, 0.1, n).astype(np.float32)), d_s=rt.up(np.array([50.0], np.float32)),
                        d_out=ncnn_amd.DeviceBuffer.empty((batch, n), np.float32))
            wsb = C.c_size_t()
            check(lib.ncnnhip_innerproduct_workspace_bytes(batch, k, n, C.byref(wsb)))
            plan.update(d_ws=ncnn_amd.DeviceBuffer.zeros(wsb.value, st), ws_bytes=wsb.value)
        else:
            c, h, w = r["in_shape"]
            cout, oh, ow = r["out_shape"]
            desc = ConvDesc(w, h, c, batch, cout, r["k"], r["k"], 1, 1, r["stride"], r["stride"], r["pad"], r["pad"], r["pad"], r["pad"], 0.0, r["group"])
            plan = dict(row=r, kind="conv", desc=desc, npix=batch * h * w,
                        d_xq=rt.up(rng.integers(-127, 128, (batch, h * w, cp(c))).astype(np.int8)),
                        d_si=rt.up(rng.uniform(1e-4, 1e-3, cout).astype(np.float32)), d_b=rt.up(rng.uniform(-0.1, 0.1, cout).astype(np.float32)),
                        d_so=rt.up(np.full(cout, 20.0, np.float32)) if r["int8_out"] else None,
                        d_out=ncnn_amd.DeviceBuffer.empty((batch, oh * ow, cp(cout)), np.int8 if r["int8_out"] else np.float32),
                        act=Activation.make(r["act"], r["act_params"]))
            if not r["int8_in"]:
                plan["d_x"] = rt.up(rng.uniform(-1, 1, (batch, h * w, cp(c))).astype(np.float32))
                plan["d_s"] = rt.up(np.array([100.0], np.float32))
            taps = r["k"] * r["k"]
            if r["group"] == 1 and lib.ncnnhip_conv_stem_supported(C.byref(desc)):
                # at most 4 input channels: the narrow-input form the layer takes inside a net (fp32 image at 4 floats per pixel,
                # quantised into the bordered 4-byte-per-pixel image, 4 neighbouring pixels per K chunk)
                ib, wb, sb = C.c_size_t(), C.c_size_t(), C.c_size_t()
                check(lib.ncnnhip_conv_stem_sizes(C.byref(desc), C.byref(ib), C.byref(wb), C.byref(sb)))
                wq = rng.integers(-127, 128, cout * c * taps).astype(np.int8)
                pk = np.empty(wb.value, np.int8)
                check(lib.ncnnhip_conv_stem_pack_weights(C.byref(desc), wq.ctypes.data, pk.ctypes.data))
                plan.update(kind="stem", d_pk=rt.up(pk), d_ws=ncnn_amd.DeviceBuffer.zeros(sb.value, st), ws_bytes=sb.value,
                            d_img=ncnn_amd.DeviceBuffer.zeros(ib.value, st), d_x=rt.up(rng.uniform(-1, 1, (batch, h * w, 4)).astype(np.float32)),
                            d_s=rt.up(np.array([100.0], np.float32)))
            elif r["group"] == 1:
                nb, wb, sb = C.c_size_t(), C.c_size_t(), C.c_size_t()
                check(lib.ncnnhip_conv_nhwc_sizes(C.byref(desc), C.byref(nb), C.byref(wb), C.byref(sb)))
                wq = rng.integers(-127, 128, cout * c * taps).astype(np.int8)
                pk = np.empty(wb.value, np.int8)
                check(lib.ncnnhip_conv_pack_weights(C.byref(desc), wq.ctypes.data, pk.ctypes.data))
                plan.update(d_pk=rt.up(pk), d_ws=ncnn_amd.DeviceBuffer.zeros(sb.value, st), ws_bytes=sb.value)
            else:
                assert r["group"] == c == cout, "the benchmark nets only hold plain and depthwise convolutions"
                wq = rng.integers(-127, 128, c * taps).astype(np.int8)
                nbytes = C.c_size_t()
                check(lib.ncnnhip_dwconv_packed_bytes(c, r["k"], r["k"], C.byref(nbytes)))
                pk = np.empty(nbytes.value, np.int8)
                check(lib.ncnnhip_dwconv_pack_weights(c, r["k"], r["k"], wq.ctypes.data, pk.ctypes.data))
                plan.update(d_pk=rt.up(pk))
        plans.append(plan)

    def run_layer(p, prepass=True):
        r = p["row"]
        if p["kind"] == "fc":
            if prepass:
                check(lib.ncnnhip_quantize(p["d_x"].ptr, p["k"], 0, p["d_xq"].ptr, p["k"], 0, batch, p["k"], 1, p["d_s"].ptr, 1, st))
            check(lib.ncnnhip_innerproduct_int8_ws(p["d_xq"].ptr, p["k"], batch, p["k"], p["n"], p["d_w"].ptr, p["d_si"].ptr, p["d_b"].ptr,
                                                   Activation.make(0), p["d_out"].ptr, p["n"], p["d_ws"].ptr, p["ws_bytes"], st))
            return
        so = p["d_so"].ptr if p["d_so"] else None
        if p["kind"] == "stem":
            if prepass:
                check(lib.ncnnhip_quantize_stem(C.byref(p["desc"]), p["d_x"].ptr, 4, 4, p["d_s"].ptr, p["d_img"].ptr, st))
            check(lib.ncnnhip_conv_int8_stem(C.byref(p["desc"]), p["d_img"].ptr, p["d_pk"].ptr, p["d_si"].ptr, p["d_b"].ptr, so, p["act"], p["d_out"].ptr, None,
                                             p["d_ws"].ptr, p["ws_bytes"], st))
            return
        if prepass and not r["int8_in"]:
            check(lib.ncnnhip_quantize_nhwc(p["d_x"].ptr, p["d_xq"].ptr, p["npix"], r["in_shape"][0], p["d_s"].ptr, 1, st))
        so = p["d_so"].ptr if p["d_so"] else None
        if r["group"] == 1:
            check(lib.ncnnhip_conv_int8_nhwc(C.byref(p["desc"]), p["d_xq"].ptr, p["d_pk"].ptr, p["d_si"].ptr, p["d_b"].ptr, so, p["act"], p["d_out"].ptr,
                                             1, 0, 0, p["d_ws"].ptr, p["ws_bytes"], st))
        else:
            check(lib.ncnnhip_dwconv_int8_nhwc(C.byref(p["desc"]), p["d_xq"].ptr, p["d_pk"].ptr, p["d_si"].ptr, p["d_b"].ptr, so, p["act"], p["d_out"].ptr, st))

    def step():
        for p in plans:
            run_layer(p)

    for _ in range(args.warmup):
        step()
    rt.sync()

    def timed(p, prepass, reps=10):
        ev = _events(lib, check, 2)
        check(lib.ncnnhip_event_record(ev[0], st))
        for _ in range(reps):
            run_layer(p, prepass)
        check(lib.ncnnhip_event_record(ev[1], st))
        check(lib.ncnnhip_event_synchronize(ev[1]))
        return _elapsed(lib, check, ev[0], ev[1]) * 1e3 / reps

    table = []
    for p in plans:
        r = p["row"]
        us, us_kernel = timed(p, True), timed(p, False)
        cin, cout = r["in_shape"][0], r["out_shape"][0]
        in_px = batch * r["in_shape"][1] * r["in_shape"][2] if len(r["in_shape"]) == 3 else batch
        out_px = batch * r["out_shape"][1] * r["out_shape"][2] if len(r["out_shape"]) == 3 else batch
        # bytes the layer has to move at least once: int8 input, weights, output as stored
        nbytes = in_px * cin + r["macs"] // max(out_px // batch, 1) + out_px * cout * (1 if r.get("int8_out") else 4)
        table.append((r["name"], r["type"], r["in_shape"], r["out_shape"], r["k"], r["stride"], r["group"], 2.0 * r["macs"] * batch, us, us_kernel, nbytes))
    evs = _events(lib, check, 2)
    check(lib.ncnnhip_device_synchronize())
    t0 = time.perf_counter()
    check(lib.ncnnhip_event_record(evs[0], st))
    for _ in range(args.steps):
        step()
    check(lib.ncnnhip_event_record(evs[1], st))
    check(lib.ncnnhip_device_synchronize())
    wall = time.perf_counter() - t0
    dev_ms = _elapsed(lib, check, evs[0], evs[1]) / args.steps
    ops = sum(t[7] for t in table)
    ms_per_step = wall * 1e3 / args.steps
    if args.layer_table:
        with open(args.layer_table, "w") as f:
            f.write("%-22s %-22s %-18s %-18s k s group %12s %9s %9s %8s %8s\n" % ("layer", "type", "in", "out", "ops", "us", "us_kernel", "TOPS", "GB/s"))
            for t in sorted(table, key=lambda t: -t[8]):
                f.write("%-22s %-22s %-18s %-18s %d %d %5d %12.0f %9.2f %9.2f %8.2f %8.0f\n"
                        % (t[0], t[1], t[2], t[3], t[4], t[5], t[6], t[7], t[8], t[9], t[7] / t[9] / 1e6, t[10] / t[9] / 1e3))
            f.write("sum of per-layer times %.1f us (kernels alone %.1f us); whole pass %.1f us (device events)\n"
                    % (sum(t[8] for t in table), sum(t[9] for t in table), dev_ms * 1e3))
    worst = max(table, key=lambda t: t[8])
    achieved = ops / (dev_ms * 1e-3) / 1e12
    return {
        "metric": "int8 TOPS", "value": ops / (ms_per_step * 1e-3) / 1e12, "unit": "TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": "%s-shaped int8 net, the %d quantised layers (conv/depthwise/fc) one by one on channels-last resident blobs, batch %d"
                               % (which, len(plans), batch),
                   "images_per_s": batch / (ms_per_step * 1e-3), "slowest_layer": [worst[0], worst[8]]},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": INT8_MFMA_PEAK_TOPS, "unit": "TOPS", "frac": achieved / INT8_MFMA_PEAK_TOPS,
                     "traffic": None, "kernel": "conv_nhwc_pipelined_kernel and the depthwise / pointwise / InnerProduct kernels (all layers of the pass)", "ops_per_launch": ops},
    }


def bench_net(args, which, batch):
    """A whole ResNet-50 / MobileNetV2-shaped int8 model through the product path: generated .param/.bin, Net with the
    HIP layers registered and use_hip_compute on, one Extractor per inference.  The input batch is uploaded once
    (resident in HBM, channels-last) before the timed region; a step enqueues every layer of one forward pass and
    leaves the logits in HBM; the region ends with a stream synchronise."""
    from ncnn_amd import host, zoo
    g, param, blob, info = zoo.build(which, n_calib=1)
    rows = zoo.quantised_layer_table(g)
    ops = 2.0 * sum(r["macs"] for r in rows) * batch
    net = host.Net()
    if net.register_int8_layers() != 0 or net.load_param_mem(param) != 0:
        raise SystemExit("bench.py: could not load the generated model")
    net.set_use_hip_compute(True)
    if net.load_model_mem(blob) != 0:
        raise SystemExit("bench.py: load_model failed (no GPU?)")
    out_name = "fc1000" if which == "resnet50" else "fc"
    x = np.random.default_rng(0).uniform(0, 1, (batch,) + tuple(g.input_shape)).astype(np.float32)
    xin = net.upload(x)

    graph = net.record("data", xin, out_name) if args.graph else None

    def step():
        if graph is not None:
            graph.launch()  # the recorded pass: one launch
            return graph, None
        ex = net.create_extractor(own_stream=False)
        ex.input_resident("data", xin)
        return ex, ex.extract_resident(out_name)

    # --streams N keeps the last N Extractors alive, so N passes are in flight on N of the net's streams (each live
    # Extractor borrows its own command); 1 = one pass after the other on one stream.  --threads T: T host threads, each
    # with such a ring of its own, enqueue their share of the steps side by side (the C calls release the interpreter
    # lock): one thread cannot describe a batch-1 pass as fast as the GPU runs it.
    threads = max(1, args.threads) if graph is None else 1
    rings = [[None] * max(1, args.streams) for _ in range(threads)]
    outs = [None] * threads

    def run(t, count):
        ring = rings[t]
        for i in range(count):
            ex, out = step()
            ring[i % len(ring)] = ex
            outs[t] = out

    def run_all(total):
        share = [total // threads + (1 if t < total % threads else 0) for t in range(threads)]
        if threads == 1:
            run(0, share[0])
            return
        import threading
        ts = [threading.Thread(target=run, args=(t, share[t])) for t in range(threads)]
        for th in ts:
            th.start()
        for th in ts:
            th.join()

    def drain():
        for ring in rings:
            for e in ring:
                if e is not None:
                    e.synchronize()

    run_all(max(args.warmup, threads))
    drain()
    t0 = time.perf_counter()
    run_all(args.steps)
    enqueue = time.perf_counter() - t0  # the host is done describing the work; the GPU may still be running it
    drain()
    wall = time.perf_counter() - t0
    out = outs[0]
    logits = (graph.output() if graph is not None else out).to_numpy()
    if not np.isfinite(logits).all():
        raise SystemExit("bench.py: non-finite logits")
    ms_per_step = wall * 1e3 / args.steps
    achieved = ops / (ms_per_step * 1e-3) / 1e12
    line = {
        "metric": "int8 TOPS", "value": achieved, "unit": "TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": "%s-shaped int8 model (%d layers, %d quantised), whole forward pass through Net/Extractor with device-resident blobs, batch %d"
                               % (which, len(g.layers), len(rows), batch),
                   "images_per_s": batch / (ms_per_step * 1e-3), "host_enqueue_ms_per_step": enqueue * 1e3 / args.steps,
                   "submission": "recorded pass replayed as one graph launch" if graph is not None else "layer by layer through an Extractor",
                   "passes_in_flight": threads * len(rings[0]), "host_threads": threads},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": INT8_MFMA_PEAK_TOPS, "unit": "TOPS", "frac": achieved / INT8_MFMA_PEAK_TOPS,
                     "traffic": None, "kernel": "whole pass (conv_nhwc_pipelined_kernel dominates)", "ops_per_launch": ops},
    }
    if not args.no_cpu:
        cpu = cpu_baseline_net(param, blob, g.input_shape, batch, ops)
        if cpu is not None:
            line["cpu_baseline"] = cpu
    return line


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="gemm4096",
                    help="gemm<size> | gemm:<M>x<N>x<K> | conv:<cin>x<h>x<w>:<cout>:k<k>[:b<batch>] | blockquant:<N>x<K>x<M>[:<bits>[:<block>]] | net:<resnet50|mobilenetv2>:<batch> (whole model through Net/Extractor) | "
                         "mha:<embed>x<heads>:<new tokens>:<cached tokens> | "
                         "layers:<resnet50|mobilenetv2>:<batch> (each quantised layer alone through the C ABI) | "
                         "peak:mfma_i8[:zeros|random] | peak:hbm_read:<bytes>[:<loads per lane>] | peak:launch[:<nodes>] (the chip's measured ceilings)")
    ap.add_argument("--streams", type=int, default=1, help="net workloads: forward passes kept in flight, each on its own stream of the net")
    ap.add_argument("--threads", type=int, default=1, help="net workloads: host threads that enqueue passes side by side, each on streams of its own")
    ap.add_argument("--graph", type=int, default=0,
                    help="net workloads: 0 = one Extractor per pass, layer by layer on a stream (faster on this ROCm: a replayed graph costs more per kernel node "
                         "on the GPU than a stream launch does); 1 = replay the recorded pass (HipGraph), which takes the host out of the loop")
    ap.add_argument("--b-scale", dest="b_scale", default="per_column", choices=["per_column", "per_tensor"],
                    help="per_column is the benchmark configuration; per_tensor is what ncnn's Gemm layer can express")
    ap.add_argument("--act", default="fp16", choices=["fp16", "fp32", "fp32-bin"],
                    help="activation type of the block-quant workload; fp32 = the layer's contract on packed weights where they have a kernel, "
                         "fp32-bin = always the kernel that streams the .bin layout")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--layer-table", default=None, help="layers workloads: write the per-layer timing table to this file")
    ap.add_argument("--calib-copy", action="store_true", help="issue one D2D copy of M*K*4 bytes first (calibrates HBM byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py: this build runs on one GPU only (--gpus 1); multi-GPU figures are not produced")
    if args.workload.startswith("gemm:"):
        line = bench_gemm(args, 0, tuple(int(v) for v in args.workload[5:].split("x")))
    elif args.workload.startswith("gemm"):
        line = bench_gemm(args, int(args.workload[4:] or 4096))
    elif args.workload.startswith("blockquant-multi:"):
        parts = args.workload.split(":")
        nspec, k, m = parts[1].split("x")
        line = bench_blockquant_multi(args, [int(v) for v in nspec.split("+")], int(k), int(m), int(parts[2]) if len(parts) > 2 else 8,
                                      int(parts[3]) if len(parts) > 3 else 64)
    elif args.workload.startswith("blockquant:"):
        parts = args.workload.split(":")
        n, k, m = (int(v) for v in parts[1].split("x"))
        line = bench_blockquant(args, n, k, m, int(parts[2]) if len(parts) > 2 else 8, int(parts[3]) if len(parts) > 3 else 64)
    elif args.workload.startswith("mha:"):
        dims, src, past = args.workload.split(":")[1:]
        embed, heads = [int(v) for v in dims.split("x")]
        line = bench_mha(args, embed, heads, int(src), int(past))
    elif args.workload.startswith("conv:"):
        line = bench_conv(args, args.workload[5:])
    elif args.workload.startswith("net:"):
        _, which, batch = args.workload.split(":")
        line = bench_net(args, which, int(batch))
    elif args.workload.startswith("peak:"):
        parts = args.workload.split(":", 2)
        line = bench_peak(args, parts[1], parts[2] if len(parts) > 2 else "")
    elif args.workload.startswith("layers:"):
        _, which, batch = args.workload.split(":")
        line = bench_layers(args, which, int(batch))
    else:
        raise SystemExit("unknown workload " + args.workload)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
