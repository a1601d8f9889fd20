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


def cpu_baseline_gemm(n, k, budget_s=12.0):
    """Scalar oracle (ncnn's naive loop restated, OpenMP over rows) on a row sample of the same Gemm."""
    from oracle import oracle
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


def measured_traffic(key):
    """bytes per launch past L2 (read + write) from the committed counter summary, or None"""
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            e = json.load(f).get(key)
        return None if e is None else e["read_bytes"] + e["write_bytes"]
    except (OSError, ValueError, KeyError):
        return None


def bench_gemm(args, size):
    import ncnn_amd
    from ncnn_amd.hip import check, lib as load
    from ncnn_amd import synth
    lib = load()
    rt = ncnn_amd.Runtime(0)
    m = n = k = size
    a, bq, sb, bias = synth.gemm_operands(size, m, n, k, per_col=args.b_scale == "per_column")
    d_a, d_bq, d_sb, d_bias = rt.up(a), rt.up(bq), rt.up(sb), rt.up(bias)
    d_aq = ncnn_amd.DeviceBuffer.empty((m, k), np.int8)
    d_sa = ncnn_amd.DeviceBuffer.empty((m,), np.float32)
    d_out = ncnn_amd.DeviceBuffer.empty((m, n), np.float32)
    st = rt.stream

    def step(ev=None):
        if ev:
            check(lib.ncnnhip_event_record(ev[0], st))
        check(lib.ncnnhip_gemm_quantize_rows(d_a.ptr, k, m, k, d_aq.ptr, k, d_sa.ptr, st))
        if ev:
            check(lib.ncnnhip_event_record(ev[1], st))
        check(lib.ncnnhip_gemm_int8(d_aq.ptr, k, d_bq.ptr, k, m, n, k, d_sa.ptr, d_sb.ptr, sb.size, d_bias.ptr, 4, 1.0, 1.0, 0,
                                    d_out.ptr, n, None, st))
        if ev:
            check(lib.ncnnhip_event_record(ev[2], st))

    if args.calib_copy:
        # one device-to-device copy of known size: gives counter runs (FETCH_SIZE / WRITE_SIZE) a dispatch to calibrate against
        check(lib.ncnnhip_memcpy_d2d(d_out.ptr, d_a.ptr, m * k * 4, st))
    for _ in range(args.warmup):
        step()
    rt.sync()
    evs = [_events(lib, check, 3) for _ in range(args.steps)]
    check(lib.ncnnhip_device_synchronize())
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(evs[i])
    check(lib.ncnnhip_device_synchronize())
    wall = time.perf_counter() - t0

    gemm_ms = float(np.mean([_elapsed(lib, check, e[1], e[2]) for e in evs]))
    quant_ms = float(np.mean([_elapsed(lib, check, e[0], e[1]) for e in evs]))
    ops = 2.0 * m * n * k
    ms_per_step = wall * 1e3 / args.steps
    achieved = ops / (gemm_ms * 1e-3) / 1e12

    # correctness spot check of the timed buffers against the oracle on a row sample
    from oracle import oracle
    rows = np.arange(0, m, max(1, m // 8))[:8]
    aq_ref, sa_ref = oracle.gemm_quantize_rows(a[rows])
    ref = oracle.gemm_int8(aq_ref, bq, sa_ref, sb, bias, 4)
    got = d_out.to_numpy(st)[rows]
    if not np.array_equal(got, ref):
        raise SystemExit("bench: GPU output differs from the oracle on the sampled rows")

    line = {
        "metric": "int8 TOPS", "value": ops / (ms_per_step * 1e-3) / 1e12, "unit": "TOPS", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": "standalone int8 Gemm M=N=K=%d: per-row quantise A (fp32->int8) + int8 MFMA Gemm + fused dequantise/bias to fp32" % size,
                   "b_scale": args.b_scale, "kernel_ms": {"gemm_int8": gemm_ms, "quantize_rows": quant_ms}},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": INT8_MFMA_PEAK_TOPS, "unit": "TOPS", "frac": achieved / INT8_MFMA_PEAK_TOPS,
                     "traffic": measured_traffic("gemm%d" % size), "kernel": "gemm_int8", "ops_per_launch": ops},
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline_gemm(n, k)
    return line


def bench_blockquant(args, n, k, m):
    """LLM-decode block-quant Gemm: weights int8 in blocks of 64 with one fp32 scale per block, streamed from a
    rotating set of weight copies larger than the 256 MB last-level cache so that the rate is an HBM rate."""
    import ncnn_amd
    from ncnn_amd.hip import check, lib as load
    from ncnn_amd import synth
    lib = load()
    rt = ncnn_amd.Runtime(0)
    a, packed, scales = synth.blockquant8_operands(n + k + m, m, n, k)
    wbytes = packed.nbytes + scales.nbytes
    copies = int(np.ceil(512e6 / wbytes)) + 1
    half = args.act == "fp16"
    if half:  # constant weights are repacked once into matrix-core tiles, as create_pipeline does
        pw, pd = rt.blockquant_pack(packed, scales, 64)
        wbytes = n * k + scales.nbytes  # algorithmic bytes: the int8 weights and one fp32 scale per block
        d_w = [rt.up(pw) for _ in range(copies)]
        d_s = [rt.up(pd) for _ in range(copies)]
    else:
        d_w = [rt.up(packed) for _ in range(copies)]
        d_s = [rt.up(scales) for _ in range(copies)]
    d_a = rt.up(a.astype(np.float16) if half else a)
    d_out = ncnn_amd.DeviceBuffer.empty((m, n), np.float32)
    st = rt.stream

    def launch(i):
        j = i % copies
        if half:
            check(lib.ncnnhip_gemm_blockquant_packed_f16a(d_a.ptr, k, m, n, k, d_w[j].ptr, d_s[j].ptr, None, -1, 1.0, 1.0, d_out.ptr, n, st))
        else:
            check(lib.ncnnhip_gemm_blockquant(d_a.ptr, k, m, n, k, d_w[j].ptr, 8, 64, d_s[j].ptr, None, None, -1, 1.0, 1.0, d_out.ptr, n, st))

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
    return {
        "metric": "HBM GB/s", "value": algo / (ms_per_step * 1e-3) / 1e9, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "block-quant Gemm M=%d N=%d K=%d, int8 weights in blocks of 64, fp32 block scales, %s activations" % (m, n, k, args.act),
                   "weight_copies_rotated": copies},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": None,
                     "kernel": "blockquant8_mfma_kernel" if half else "blockquant8_stream_kernel", "bytes_per_launch": algo},
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="gemm4096",
                    help="gemm<size> | blockquant:<N>x<K>x<M>")
    ap.add_argument("--b-scale", dest="b_scale", default="per_column", choices=["per_column", "per_tensor"],
                    help="per_column is the benchmark configuration; per_tensor is what ncnn's Gemm layer can express")
    ap.add_argument("--act", default="fp16", choices=["fp16", "fp32"], help="activation type of the block-quant workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--calib-copy", action="store_true", help="issue one D2D copy of M*K*4 bytes first (calibrates HBM byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py: this build runs on one GPU only (--gpus 1); multi-GPU figures are not produced")
    if args.workload.startswith("gemm"):
        line = bench_gemm(args, int(args.workload[4:] or 4096))
    elif args.workload.startswith("blockquant:"):
        n, k, m = (int(v) for v in args.workload.split(":")[1].split("x"))
        line = bench_blockquant(args, n, k, m)
    else:
        raise SystemExit("unknown workload " + args.workload)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
