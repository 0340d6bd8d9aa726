#!/usr/bin/env python3
"""Headline benchmark: the bf16 8192^3 GEMM (A MxK row-major, B NxK K-major, fp32 accumulate and output) through
the C ABI of libmi_gemm.so on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3|c3f16|c2|c4|c5|skinny] [--no-cpu] [--no-vendor]
                    [--no-configs]

A "step" is one GEMM launch on inputs already resident in HBM.  Prints ONE JSON line: whole-job TFLOP/s over exactly
K timed steps (host clock, synchronised on both sides), the per-launch roofline figure measured with HIP events on
the launch stream (mean of the inter-quartile samples, the reference's statistic: gemm/gemm_test.cu:394-404), and the
reference CPU GEMM (docs/nyc25.py:16-55) timed on a bounded sample of the same workload on this host's cores (all of
them, and one thread).  With the headline workload the line also carries a `configs` object: the other BASELINE
configurations (fp16 4096^3, 16384x128x8192, 2048x2048x65536) measured the same way with fewer launches.
PyTorch only provides device memory and the stream.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS = 2500.0  # MI355X dense bf16/fp16 MFMA, published
PEAK_HBM_GBS = 8000.0
SETTLE_MS = 40.0      # untimed launches before the warm-up steps, see main()

# HBM bytes per launch of the dominant kernel from rocprofv3 --pmc (FETCH_SIZE + WRITE_SIZE, KiB per dispatch,
# scaled by the factor a plain copy kernel of known size reads on the same counters); summaries in profiles/.
MEASURED_TRAFFIC_BYTES = {"c3": 1.880e9, "c2": 2.687e8, "c4": 2.997e8, "c5": 1.224e9, "skinny": 5.329e8}
# ... and where each figure was recorded (rocprofv3 runs of this same command, not something measured in this run)
TRAFFIC_SOURCE = {"c3": "profiles/gemm_tn_256x256_bf16_8192_pmc.md",
                  "c2": "profiles/gemm_tn_256x256_f16_4096_kernel_stats_pmc_timeline.md",
                  "c4": "profiles/gemm_tn_64x128_f16_16384x128x8192_kernel_stats_pmc_timeline.md",
                  "c5": "profiles/gemm_split_k_workspace_sum_f16_2048x2048x65536_kernel_stats_pmc_timeline.md",
                  "skinny": "profiles/gemm_tn_256x128_read_once_bf16_256x8192x28672_kernel_stats_and_pmc.md"}
OTHER_CONFIGS = ("c2", "c4", "c5")  # the other BASELINE configurations that need a GPU, reported beside the headline

WORKLOADS = {
    # name: (M, N, K, dtype, data_code, param_fn, description)
    "c2": (4096, 4096, 4096, "f16", 3, lambda K: 1.0, "fp16 GEMM M=N=K=4096, uniform[-1,1] (BASELINE configs[1])"),
    "c3": (8192, 8192, 8192, "bf16", 4, lambda K: K ** -0.5,
           "bf16 GEMM M=N=K=8192, normal(0,1)/sqrt(K), A MxK row-major, B NxK K-major, fp32 C (BASELINE configs[2], headline)"),
    "c3f16": (8192, 8192, 8192, "f16", 4, lambda K: K ** -0.5,
              "fp16 GEMM M=N=K=8192, normal(0,1)/sqrt(K) (the headline shape with fp16 operands)"),
    "c4": (16384, 128, 8192, "f16", 3, lambda K: 1.0, "fp16 GEMM M=16384 N=128 K=8192, uniform[-1,1] (BASELINE configs[3])"),
    "c5": (2048, 2048, 65536, "f16", 3, lambda K: 0.5, "fp16 GEMM M=N=2048 K=65536, uniform[-0.5,0.5] (BASELINE configs[4])"),
    # not a BASELINE configuration: a few rows against a weight matrix larger than the memory-side cache (HBM-bound)
    "skinny": (256, 8192, 28672, "bf16", 4, lambda K: K ** -0.5,
               "bf16 GEMM M=256 N=8192 K=28672, normal(0,1)/sqrt(K): B is 470 MB and read once"),
}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c3", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-vendor", action="store_true", help="skip the hipBLASLt comparator leg")
    ap.add_argument("--no-configs", action="store_true", help="skip the other BASELINE configurations (headline workload only)")
    ap.add_argument("--cpu-rows", type=int, default=0, help="rows of the workload the CPU baseline computes (0 = auto)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device-to-device copy so that a rocprofv3 --pmc run of this command "
                         "shows what FETCH_SIZE / WRITE_SIZE read for a kernel of known traffic")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build drives one GPU; --gpus N with N > 1 is not supported (the GEMM shards over M or N "
              "with no communication, each GPU running this same kernel on its slab).", file=sys.stderr)
        return 2

    # The child process that times the system hipBLASLt runs first, before this process has touched the GPU (a process
    # that holds GPU state starts no other program), and alone on the device.
    system_comparator = None
    if not args.no_vendor:
        wl = WORKLOADS[args.workload]
        system_comparator = system_vendor_comparator(wl[0], wl[1], wl[2], wl[3], wl[4], wl[5](wl[2]))

    import torch

    import spork_amd as S

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    L = S.lib()
    torch.cuda.set_device(0)
    stream = torch.cuda.current_stream().cuda_stream

    m = measure(S, L, stream, args.workload, args.steps, args.warmup, SETTLE_MS, args.calibrate_copy)
    M, N, K, dtype_name, dtype, code, param = m["M"], m["N"], m["K"], m["dtype_name"], m["dtype"], m["code"], m["param"]
    desc, plan, flops, value, ms_per_step = m["desc"], m["plan"], m["flops"], m["value"], m["ms_per_step"]
    roofline, achieved, settle_launches = m["roofline"], m["achieved"], m["settle_launches"]
    max_rel_err_vs_device_baseline = m["max_rel_err_vs_device_baseline"]
    a, b, c, t = m["a"], m["b"], m["c"], m["t"]
    seed_a, seed_b = SEED_A, SEED_B

    out = {
        "metric": "TFLOP/s (2*M*N*K / t) of the bf16/fp16 -> fp32 GEMM at M=N=K=8192, and max rel err" if args.workload in ("c3", "c3f16")
        else f"TFLOP/s (2*M*N*K / t), workload {args.workload}",
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype_name,
        "data": "synthetic",
        "settle": {"ms": SETTLE_MS, "untimed_launches_before_warmup": settle_launches},
        "config": {"workload": desc, "M": M, "N": N, "K": K, "layout": "A row-major MxK, B stored NxK (K-major), C row-major fp32",
                   "tile": plan["tile"], "k_mode": plan["k_mode"], "k_splits": plan["k_splits"]},
        "frac_of_mfma_peak": round(value / PEAK_TFLOPS, 4),
        "max_rel_err_vs_device_baseline": max_rel_err_vs_device_baseline,
        "roofline": roofline,
    }

    # (the probe wants a few tens of MB of operand values: A, unless the workload's A is the small operand)
    out["mfma_ceiling"] = mfma_ceiling(S, L, a if a.numel() >= b.numel() else b, dtype, stream)
    if out["mfma_ceiling"] and "value" in out["mfma_ceiling"]:
        out["roofline"]["frac_of_sustained_ceiling"] = round(achieved / out["mfma_ceiling"]["value"], 4)
    if roofline["bound"] == "hbm":
        out["hbm_ceiling"] = hbm_ceiling(S, L, a if a.numel() >= b.numel() else b, stream)
        if "value" in out["hbm_ceiling"]:
            out["roofline"]["frac_of_streaming_ceiling"] = round(roofline["achieved"] / out["hbm_ceiling"]["value"], 4)
        if "lds_dma_rows_64_per_workgroup" in out["hbm_ceiling"]:
            out["roofline"]["frac_of_row_pattern_ceiling"] = round(roofline["achieved"] / out["hbm_ceiling"]["lds_dma_rows_64_per_workgroup"], 4)

    if not args.no_vendor:
        out["vendor_comparator"] = vendor_comparator(S, L, t, stream, flops, min(args.steps, 30))
        out["vendor_comparator_system_library"] = system_comparator

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(M, N, K, dtype, code, param, seed_a, seed_b, c, args.cpu_rows, out)
        # the single-thread leg: the reference CPU GEMM as its authors run it, on a smaller sample of rows
        out["cpu_baseline_1t"] = cpu_baseline(M, N, K, dtype, code, param, seed_a, seed_b, c, 0, None, threads=1, seconds=15.0)

    if args.workload == "c3" and not args.no_configs:
        # the other BASELINE configurations, one after the other on the same device: fewer launches, same protocol
        del a, b, c, t, m
        import torch

        torch.cuda.empty_cache()
        out["configs"] = {}
        for name in OTHER_CONFIGS:
            try:
                r = measure(S, L, stream, name, 20, 5, 30.0)
                out["configs"][name] = {
                    "workload": r["desc"], "launch_ms": round(r["launch_ms"], 5),
                    "tflops": round(r["flops"] / (r["launch_ms"] * 1e-3) * 1e-12, 1),
                    "roofline": {k: r["roofline"][k] for k in ("bound", "achieved", "peak", "unit", "frac", "traffic")},
                    "max_rel_err": r["max_rel_err_vs_device_baseline"], "plan": r["roofline"]["launches"], "steps": 20}
                if r["roofline"]["bound"] == "hbm":
                    big = r["a"] if r["a"].numel() >= r["b"].numel() else r["b"]
                    out["configs"][name]["hbm_ceiling"] = hbm_ceiling(S, L, big, stream)
                    if "value" in out["configs"][name]["hbm_ceiling"]:
                        out["configs"][name]["roofline"]["frac_of_streaming_ceiling"] = round(
                            r["roofline"]["achieved"] / out["configs"][name]["hbm_ceiling"]["value"], 4)
                    if "lds_dma_rows_64_per_workgroup" in out["configs"][name]["hbm_ceiling"]:
                        out["configs"][name]["roofline"]["frac_of_row_pattern_ceiling"] = round(
                            r["roofline"]["achieved"] / out["configs"][name]["hbm_ceiling"]["lds_dma_rows_64_per_workgroup"], 4)
            except Exception as e:  # a side measurement must never take the benchmark line down
                out["configs"][name] = {"error": str(e)[:200]}
            r = None
            torch.cuda.empty_cache()

    print(json.dumps(out), flush=True)
    return 0


SEED_A, SEED_B = 20010106, 19980724  # the reference generator's constants (gemm/gemm_test.cu:76,87)


def measure(S, L, stream, workload, steps, warmup, settle_ms, calibrate_copy=False) -> dict:
    """One workload: seeded operands generated on the device, the planner's launch checked over the whole matrix against
    the on-device baseline kernel, `settle_ms` of untimed launches, `warmup` more, then exactly `steps` timed ones."""
    import torch

    M, N, K, dtype_name, code, param_fn, desc = WORKLOADS[workload]
    dtype = S.BF16 if dtype_name == "bf16" else S.F16
    param = param_fn(K)
    seed_a, seed_b = SEED_A, SEED_B

    a = torch.empty((M, K), dtype=torch.int16, device="cuda")
    b = torch.empty((N, K), dtype=torch.int16, device="cuda")
    c = torch.empty((M, N), dtype=torch.float32, device="cuda")
    c_check = torch.empty((M, N), dtype=torch.float32, device="cuda")
    S.init_test_data(a.data_ptr(), M, K, code, False, dtype, param, seed_a, stream)
    S.init_test_data(b.data_ptr(), N, K, code, True, dtype, param, seed_b, stream)
    c.view(torch.uint8).fill_(0x7D)  # poison, gemm/gemm_test.cu:244-247
    t = S.GpuTensors.make(M, N, K, a.data_ptr(), b.data_ptr(), c.data_ptr(), dtype, 0, 1, 0)
    plan = S.matmul_mfma_plan(t)
    # Deep-K workloads: with the workspace the library prefers, K partitions are summed from copies of C instead of
    # through atomics.  Allocated once, outside the timed region; 0 bytes (and the plain entry point) for the rest.
    _, ws_bytes = S.matmul_mfma_workspace_bytes_for(t)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda") if ws_bytes else None
    if ws is not None:
        # what K_AUTO picks when it is given that room: copies of C summed by a second kernel, or a stream-K tail
        text = S.matmul_mfma_describe(t, workspace_bytes=ws_bytes)
        if "stream k" in text:
            plan = S.matmul_mfma_plan(t, S.K_STREAM)
        elif "workspace sum" in text:
            plan = S.matmul_mfma_plan(t, S.K_SPLIT_REDUCE)

        def launch():
            S.matmul_mfma_ws(t, ws.data_ptr(), ws_bytes, S.K_AUTO, S.TILE_AUTO, stream)
    else:
        def launch():
            S.matmul_mfma(t, S.K_AUTO, S.TILE_AUTO, stream)

    # correctness of what is being timed: full-matrix compare against the on-device baseline kernel
    launch()
    tb = S.GpuTensors.make(M, N, K, a.data_ptr(), b.data_ptr(), c_check.data_ptr(), dtype, 0, 1, 0)
    S.matmul_baseline(tb, stream)
    res = torch.zeros(4, dtype=torch.int64, device="cuda")
    S.compare_tensors(c_check.data_ptr(), c.data_ptr(), M, N, res.data_ptr(), stream)
    torch.cuda.synchronize()
    r = res.cpu().numpy().view("uint64")
    import numpy as np

    max_diff = float(np.array([r[1]]).view(np.float64)[0])
    max_ref = float(np.array([r[2]]).view(np.float64)[0])
    max_rel_err_vs_device_baseline = max_diff / max_ref if max_ref > 0 else float("inf")

    if calibrate_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").fill_(1.0)  # 1 GiB
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # Settle the clocks first: measured on MI355X, after an idle spell the same launch runs 4 to 20 % slower for 25 to
    # 30 ms before it reaches its steady rate, and a small --warmup / --steps would be timed inside that window.
    settle_start = torch.cuda.Event(enable_timing=True)
    settle_now = torch.cuda.Event(enable_timing=True)
    settle_start.record()
    settle_launches = 0
    while settle_launches < 4096:
        for _ in range(8):
            launch()
        settle_launches += 8
        settle_now.record()
        settle_now.synchronize()
        if settle_start.elapsed_time(settle_now) >= settle_ms:
            break

    for _ in range(warmup):
        launch()
    torch.cuda.synchronize()

    # HIP events between launches, on the stream the kernel is launched on
    events = []
    for _ in range(steps + 1):
        e = C.c_void_p()
        S.capi.check(L.mi_rt_event_create(C.byref(e)), "event create")
        events.append(e)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    L.mi_rt_event_record(events[0], stream)
    for i in range(steps):
        launch()
        L.mi_rt_event_record(events[i + 1], stream)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    per_launch_ms = []
    for i in range(steps):
        ms = C.c_float()
        S.capi.check(L.mi_rt_event_elapsed_ms(C.byref(ms), events[i], events[i + 1]), "event elapsed")
        per_launch_ms.append(ms.value)
    for e in events:
        L.mi_rt_event_destroy(e)

    flops = 2.0 * M * N * K
    alg_bytes = 2.0 * (M * K + N * K) + 4.0 * M * N
    total_s = t1 - t0
    ms_per_step = total_s * 1e3 / steps
    value = flops * steps / total_s * 1e-12
    srt = sorted(per_launch_ms)
    n = len(srt)
    iqr = srt[n // 4: n // 4 + (n + 1) // 2]
    launch_ms = sum(iqr) / len(iqr)  # gemm/gemm_test.cu:394-404
    achieved = flops / (launch_ms * 1e-3) * 1e-12
    ai = flops / alg_bytes
    hbm_bound = ai * PEAK_HBM_GBS * 1e-3 < PEAK_TFLOPS  # TFLOP/s reachable at HBM peak
    if hbm_bound:
        ach_gbs = alg_bytes / (launch_ms * 1e-3) * 1e-9
        roofline = {"bound": "hbm", "achieved": round(ach_gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                    "frac": round(ach_gbs / PEAK_HBM_GBS, 4), "traffic": MEASURED_TRAFFIC_BYTES.get(workload)}
    else:
        roofline = {"bound": "mfma", "achieved": round(achieved, 1), "peak": PEAK_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(achieved / PEAK_TFLOPS, 4), "traffic": MEASURED_TRAFFIC_BYTES.get(workload)}
    roofline.update({"kernel": f"gemm_tn_kernel tile {plan['tile']}, {plan['k_mode']}, k_splits {plan['k_splits']}",
                     "launches": S.matmul_mfma_describe(t, workspace_bytes=ws_bytes),
                     "launch_ms": round(launch_ms, 5), "algorithmic_flops": flops, "algorithmic_bytes": alg_bytes})

    roofline["traffic_source"] = TRAFFIC_SOURCE.get(workload)
    return {"M": M, "N": N, "K": K, "dtype_name": dtype_name, "dtype": dtype, "code": code, "param": param, "desc": desc,
            "plan": plan, "flops": flops, "value": value, "ms_per_step": ms_per_step, "roofline": roofline,
            "achieved": achieved, "settle_launches": settle_launches, "launch_ms": launch_ms,
            "max_rel_err_vs_device_baseline": max_rel_err_vs_device_baseline, "a": a, "b": b, "c": c, "t": t}


def mfma_ceiling(S, L, a, dtype, stream):
    """What a register-only loop of the kernel's MFMA instruction sustains on this workload's own operand values (the
    A matrix): the matrix cores are power-limited, so this, not the published peak, is the ceiling the GEMM works under."""
    import torch

    try:
        nbytes = a.numel() * a.element_size()
        clocks = torch.zeros(2 * 1024, dtype=torch.int64, device="cuda")
        sink = torch.zeros(1, dtype=torch.float32, device="cuda")
        wgs, flop = C.c_uint32(), C.c_double()
        ev0, ev1 = C.c_void_p(), C.c_void_p()
        S.capi.check(L.mi_rt_event_create(C.byref(ev0)), "event create")
        S.capi.check(L.mi_rt_event_create(C.byref(ev1)), "event create")
        iters = 4000
        for rep in range(6):  # the clocks settle over a few milliseconds of load; the last launch is the one timed
            if rep == 5:
                L.mi_rt_event_record(ev0, stream)
            S.capi.check(L.mi_mfma_ceiling(a.data_ptr(), nbytes, dtype, 16, iters, clocks.data_ptr(), sink.data_ptr(),
                                           C.byref(wgs), C.byref(flop), stream), "mi_mfma_ceiling")
        L.mi_rt_event_record(ev1, stream)
        torch.cuda.synchronize()
        ms = C.c_float()
        S.capi.check(L.mi_rt_event_elapsed_ms(C.byref(ms), ev0, ev1), "event elapsed")
        L.mi_rt_event_destroy(ev0)
        L.mi_rt_event_destroy(ev1)
        h = clocks.cpu().numpy()[: 2 * wgs.value].reshape(-1, 2)
        mhz = float((100.0 * h[:, 0] / h[:, 1]).mean())
        return {"value": round(flop.value / (ms.value * 1e-3) * 1e-12, 1), "unit": "TFLOP/s", "core_clock_mhz": round(mhz),
                "what": "register-only v_mfma_f32_16x16x32 loop, one wave per SIMD on every CU, on this workload's A operand (B where B is the larger one)"}
    except Exception as e:  # a measurement aid must never take the benchmark line down
        return {"error": str(e)[:200]}


def hbm_ceiling(S, L, operand, stream):
    """What kernels that only stream this workload's large operand sustain (16-byte vector loads, the GEMM's own LDS DMA
    with one and with two workgroups per CU, and a read-and-write copy of it): the yardstick for a memory-bound shape,
    measured in the same process on the same buffer.  GB/s of bytes moved; median of 9 launches after 10 untimed ones."""
    import torch

    try:
        nbytes = operand.numel() * operand.element_size()
        dst = torch.empty_like(operand)
        sink = torch.zeros(4, dtype=torch.int32, device="cuda")
        out = {"bytes": nbytes, "unit": "GB/s"}
        for name, mode, per_cu in (("vector_loads_8_per_cu", S.STREAM_READ, 8), ("lds_dma_1_per_cu", S.STREAM_DMA, 1),
                                   ("lds_dma_2_per_cu", S.STREAM_DMA, 2), ("copy_8_per_cu", S.STREAM_COPY, 8)):
            def launch():
                S.hbm_stream_ceiling(operand.data_ptr(), dst.data_ptr(), nbytes, mode, per_cu, sink.data_ptr(), stream)
            for _ in range(10):
                launch()
            ev = [torch.cuda.Event(enable_timing=True) for _ in range(10)]
            ev[0].record()
            for i in range(9):
                launch()
                ev[i + 1].record()
            torch.cuda.synchronize()
            ms = sorted(ev[i].elapsed_time(ev[i + 1]) for i in range(9))[4]
            out[name] = round((2 if mode == S.STREAM_COPY else 1) * nbytes / (ms * 1e-3) * 1e-9, 1)
        # the same DMA with the access pattern of a tile's operand panel: 128-byte pieces of 64 (128) rows per workgroup
        rows, row_bytes = operand.shape[0], operand.shape[1] * operand.element_size()
        for per_wg in (64, 128):
            if rows % per_wg or row_bytes % 128:
                continue
            def launch():
                S.hbm_stream_rows_ceiling(operand.data_ptr(), rows, row_bytes, per_wg, stream)
            for _ in range(10):
                launch()
            ev = [torch.cuda.Event(enable_timing=True) for _ in range(10)]
            ev[0].record()
            for i in range(9):
                launch()
                ev[i + 1].record()
            torch.cuda.synchronize()
            ms = sorted(ev[i].elapsed_time(ev[i + 1]) for i in range(9))[4]
            out[f"lds_dma_rows_{per_wg}_per_workgroup"] = round(nbytes / (ms * 1e-3) * 1e-9, 1)
        out["value"] = max(out["vector_loads_8_per_cu"], out["lds_dma_1_per_cu"], out["lds_dma_2_per_cu"])
        out["what"] = ("read-only streaming of this workload's largest operand; value = the best of the contiguous read-only "
                       "ways; lds_dma_rows_*: the DMA reading 128-byte pieces row by row, as a GEMM tile reads its panel")
        return out
    except Exception as e:  # a measurement aid must never take the benchmark line down
        return {"error": str(e)[:200]}


def vendor_comparator(S, L, t, stream, flops, steps):
    """hipBLASLt (fp32 output) on the same operand buffers, after the timed region; a reported yardstick, not a target.
    Writes into a C buffer of its own so the result checked above is left alone."""
    import torch

    try:
        from spork_amd import vendor as V

        if not V.enabled():
            return None
        c2 = torch.empty((t.M, t.N), dtype=torch.float32, device="cuda")
        ws = torch.empty(128 << 20, dtype=torch.uint8, device="cuda")
        tv = S.GpuTensors.make(t.M, t.N, t.K, t.a, t.b, c2.data_ptr(), t.ab_dtype, 0, 1, 0)
        for _ in range(5):
            V.matmul(tv, ws.data_ptr(), ws.numel(), stream)
        torch.cuda.synchronize()
        events = []
        for _ in range(steps + 1):
            e = C.c_void_p()
            S.capi.check(L.mi_rt_event_create(C.byref(e)), "event create")
            events.append(e)
        L.mi_rt_event_record(events[0], stream)
        for i in range(steps):
            V.matmul(tv, ws.data_ptr(), ws.numel(), stream)
            L.mi_rt_event_record(events[i + 1], stream)
        torch.cuda.synchronize()
        ms = []
        for i in range(steps):
            v = C.c_float()
            S.capi.check(L.mi_rt_event_elapsed_ms(C.byref(v), events[i], events[i + 1]), "event elapsed")
            ms.append(v.value)
        for e in events:
            L.mi_rt_event_destroy(e)
        srt = sorted(ms)
        n = len(srt)
        iqr = srt[n // 4: n // 4 + (n + 1) // 2]
        launch_ms = sum(iqr) / len(iqr)
        # after `import torch` the process is bound to the hipBLASLt inside the torch wheel, not to /opt/rocm's
        return {"library": "hipBLASLt (hipblasLtMatmul, fp32 output, same operand buffers)",
                "bound_to": V.library(), "version": V.version(),
                "value": round(flops / (launch_ms * 1e-3) * 1e-12, 1), "unit": "TFLOP/s", "launch_ms": round(launch_ms, 5),
                "steps": steps}
    except Exception as e:  # the comparator must never take the benchmark line down
        return {"library": "hipBLASLt", "error": str(e)[:200]}


def system_vendor_comparator(M, N, K, dtype_name, code, param) -> dict:
    """The same problem through the plain-C++ host driver in a process of its own: that process is bound to the system
    hipBLASLt, not to the older copy inside the torch wheel that this one got with `import torch`.  The driver
    generates the same seeded operands and times 25 launches per algorithm with HIP events after 30 ms of warm-up
    (gemm/gemm_test.cu:394-404); reported next to the driver's own figure for this library from the same process."""
    import re
    import subprocess

    try:
        exe = os.path.join(ROOT, "spork_amd", "csrc", "gemm")
        if not os.path.exists(exe):
            return {"error": "host driver not built"}
        style = {3: "4", 4: "5"}[code]  # uniform[-param, param] / normal(0,1)/sqrt(K)
        r = subprocess.run([exe, "--one", str(M), str(N), str(K), dtype_name, style, repr(float(param))],
                           capture_output=True, text=True, timeout=300)
        if r.returncode != 0:
            return {"error": f"host driver exit {r.returncode}: {r.stderr[-160:]}"}
        bound = re.search(r"^hipBLASLt: (\S+) \(version (-?\d+)\)", r.stderr, re.M)
        tf = {}
        for m in re.finditer(r"\} ([\d.e+-]+) ms ([\d.e+-]+) .*?max_rel_err \S+ .*?\((hipBLASLt|mi355 \(auto\)|mi355 \(auto, workspace\))\)\s*$",
                             r.stdout, re.M):
            tf[m.group(3)] = (float(m.group(2)), float(m.group(1)))
        if "hipBLASLt" not in tf:
            return {"error": "no hipBLASLt line in the driver's output"}
        ours = max(tf.get("mi355 (auto)", (0.0, 0.0)), tf.get("mi355 (auto, workspace)", (0.0, 0.0)))
        return {"library": "hipBLASLt in the host driver's process (hipblasLtMatmul, fp32 output, same seeded operands)",
                "bound_to": bound.group(1) if bound else None, "version": int(bound.group(2)) if bound else None,
                "value": tf["hipBLASLt"][0], "unit": "TFLOP/s", "launch_ms": tf["hipBLASLt"][1],
                "this_library_in_the_same_process": ours[0], "this_library_launch_ms": ours[1]}
    except Exception as e:  # the comparator must never take the benchmark line down
        return {"error": str(e)[:200]}


def cpu_baseline(M, N, K, dtype, code, param, seed_a, seed_b, c_gpu, rows, out, threads=0, seconds=15.0) -> dict:
    """The reference CPU GEMM (oracle port of nyc25_gemm_cpu) on the first `rows` rows of the same workload, OpenMP
    over m on this host's cores.  The oracle is only the thing timed and the checker here, never the product."""
    import numpy as np

    import oracle as O

    if threads <= 0:
        threads = min(O.max_threads(), 16)  # the GPU box grants 16 cores per GPU whatever nproc says
    if rows <= 0:
        # aim for roughly `seconds` of CPU work at ~1.5 GFLOP/s per thread for the scalar fp32 loop
        rows = int(seconds * 1.5e9 * threads / (2.0 * N * K))
        rows = max(16, min(M, rows // 16 * 16))
    a = O.fill(rows, K, code, False, dtype, param, seed_a)  # rows 0..rows-1 of A (row-major: a prefix)
    b = O.fill(N, K, code, True, dtype, param, seed_b)
    t0 = time.perf_counter()
    c_cpu = O.gemm_ref_f32(rows, N, K, a, b, dtype, 0, 1, 0, 0, rows, threads)
    dt = time.perf_counter() - t0
    c_dev = c_gpu[:rows].cpu().numpy()
    denom = float(np.abs(c_cpu).max())
    err = float(np.abs(c_dev.astype(np.float64) - c_cpu.astype(np.float64)).max() / denom)
    if out is not None:
        out["max_rel_err_vs_cpu_sample"] = err
    return {"max_rel_err_of_gpu_vs_this_sample": err, "value": round(2.0 * rows * N * K / dt * 1e-12, 6), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "seconds": round(dt, 2),
            "sample": f"rows 0..{rows - 1} of M={M} (all N={N}, K={K}) of the same seeded workload; fp32 accumulate, "
                      f"sequential k, {'OpenMP over m' if threads > 1 else 'one thread'}, gcc -O2"}


if __name__ == "__main__":
    sys.exit(main())
