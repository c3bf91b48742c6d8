#!/usr/bin/env python3
"""Benchmark of the tiled GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one launch of the headline workload: the FP16 x FP16 -> FP32 GEMM C = A*B + C with
M = N = K = 4096, column-major, 'N','N' (benchmark config 2), through gemmkernels.matmul -> C ABI ->
HIP kernel, inputs resident in HBM.  The other three transposes and the other benchmark configs
are timed after the timed region and reported in extra fields of the same JSON line.
Prints exactly one JSON line on stdout.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "gemmkernels.jl_amd"))
sys.path.insert(0, ROOT)

METRIC = "TFLOP/s + % FP16 MFMA peak, 4096^3 FP16->FP32 GEMM on 1 MI355X"
PEAK_FP16_TFLOPS = 2516.6     # MI355X dense FP16/BF16 matrix peak (256 CU x 4 SIMD x 1024 flop/clk x 2.4 GHz)
PEAK_HBM_GBS = 8000.0
HEADLINE_SETTLE_SECONDS = 0.4
# HBM bytes per launch of the headline kernel from the rocprofv3 FETCH_SIZE / WRITE_SIZE passes
# summarised in profiles/ (None until measured)
MEASURED_TRAFFIC_BYTES = 336_739_328   # profiles/mfma_gemm_config2_hbm_traffic.txt: (131655.5 * 2.0 + 65536.0) KiB
TRAFFIC_SOURCE = "profiles/mfma_gemm_config2_hbm_traffic.txt (a constant from the committed rocprofv3 FETCH_SIZE / WRITE_SIZE passes, not a reading of this run)"


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    # defaults: 2000 warm-up launches (0.27 s) because the clock and power management of the device needs
    # a tenth of a second of load to settle after the idle time in which the inputs are generated (measured:
    # 1029 TFLOP/s after 20 warm-up launches, 1045 after 200, 1051 after 2000 and after 5000); 1000 timed launches
    p.add_argument("--steps", type=int, default=1000)
    p.add_argument("--warmup", type=int, default=2000)
    p.add_argument("--no-extras", action="store_true", help="skip the secondary configs and the CPU baseline")
    p.add_argument("--workload", default="2", choices=["1", "2", "3", "4a", "4a-planar", "4b", "4b-rotating", "5", "skinny", "mul4000", "size"],
                   help="benchmark config to time as the step (default: 2, the headline; the others are for profiling one "
                        "kernel at a time and imply --no-extras)")
    p.add_argument("--dims", default="3072,3072,3072", help="M,N,K of --workload size: mul!(C, A, B, 1, 1) as in the sizes sweep")
    p.add_argument("--variant", default="NN", choices=["NN", "NT", "TN", "TT"], help="transposes of config 2")
    p.add_argument("--copy-calibration", action="store_true",
                   help="instead of the benchmark, run a plain 256 MiB device-to-device copy 10 times: the reference "
                        "reading for the FETCH_SIZE / WRITE_SIZE counters of rocprofv3")
    return p.parse_args()


def gk_f32():
    from gemmkernels import Float32
    return Float32


def gk_name(conf):
    from gemmkernels import Kernel, kernel_name
    return kernel_name(conf, Kernel.matmul_pipelined)


def matrix_core_ceiling():
    """What a register-only loop of the kernels' MFMA instruction delivers on this device, under its power cap, on FP16
    values spread over [-1, 1) and on zeros (gk_probe_matrix_rate: no memory access at all; a fifth of a second of launches
    each after as much to settle).  Context for roofline.frac, whose denominator is the data-sheet peak."""
    import ctypes
    import torch
    from gemmkernels import _lib
    lib = _lib.lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = {}
    for key, rnd in (("random_fp16_tflops", 1), ("zeros_tflops", 0)):
        t = ctypes.c_double(0.0)
        for _ in range(2):       # (the first call settles clock and power)
            rc = lib.gk_probe_matrix_rate(25, 2000, rnd, stream, ctypes.byref(t))
            if rc != 0:
                raise RuntimeError(_lib.last_error())
        out[key] = round(t.value, 1)
    out["frac_of_peak_on_random_fp16"] = round(out["random_fp16_tflops"] / PEAK_FP16_TFLOPS, 4)
    out["what"] = "v_mfma_f32_16x16x32_f16 from registers only, one wave per SIMD, 64 accumulator blocks per wave; HIP events"
    return out


def observe_device(fn, bursts=100, launches_per_burst=100):
    """Shader clock, power and temperature the driver reports (sysfs of the first card) while `fn` runs
    back to back for a good second (the power reading is a moving average: the second half of the
    samples is what is reported); outside every timed region.  None where the files are not there."""
    import glob
    import statistics
    import torch
    dev = "/sys/class/drm/card0/device"

    def read(path):
        try:
            with open(path) as f:
                return f.read()
        except OSError:
            return None

    hwmon = (glob.glob(dev + "/hwmon/hwmon*") or [None])[0]
    clocks, watts, temps = [], [], []
    for _ in range(bursts):
        for _ in range(launches_per_burst):
            fn()
        torch.cuda.synchronize()
        text = read(dev + "/pp_dpm_sclk")
        if text:
            for line in text.splitlines():
                if line.rstrip().endswith("*"):
                    clocks.append(int("".join(ch for ch in line.split(":")[1] if ch.isdigit())))
        if hwmon:
            w = read(hwmon + "/power1_input") or read(hwmon + "/power1_average")
            if w:
                watts.append(int(w) / 1e6)
            t = read(hwmon + "/temp2_input") or read(hwmon + "/temp1_input")
            if t:
                temps.append(int(t) / 1e3)
    torch.cuda.synchronize()
    if not clocks and not watts:
        return None
    clocks, watts = clocks[len(clocks) // 2:], watts[len(watts) // 2:]
    cap = read(hwmon + "/power1_cap") if hwmon else None
    return {"sclk_mhz_median": statistics.median(clocks) if clocks else None, "sclk_mhz_min": min(clocks) if clocks else None,
            "power_w_median": round(statistics.median(watts), 1) if watts else None,
            "power_cap_w": round(int(cap) / 1e6, 1) if cap else None,
            "temperature_c_max": max(temps) if temps else None, "samples": max(len(clocks), len(watts)),
            "note": "driver readings while the headline kernel runs back to back (spec clock 2400 MHz)"}


def time_launches(fn, steps, warmup, settle_seconds=0.0):
    """Average duration in microseconds of `steps` back-to-back launches, HIP events on the launch stream.
    settle_seconds: keep launching for at least this long before timing (on top of `warmup`), so that a
    secondary workload is not timed while the device clock is still coming up from idle."""
    import torch
    for _ in range(warmup):
        fn()
    if settle_seconds > 0:
        t_end = time.perf_counter() + settle_seconds
        while time.perf_counter() < t_end:
            for _ in range(50):
                fn()
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return start.elapsed_time(stop) * 1e3 / steps, wall


def settle_then_time(fn, steps, warmup, settle_seconds):
    """time_launches, and the number of untimed launches of the settle phase."""
    count = {"n": 0}

    def counted():
        count["n"] += 1
        fn()
    us, wall = time_launches(counted, steps, warmup, settle_seconds)
    return us, wall, count["n"] - steps - warmup


def verify_slab(wl, run, cols=256):
    """Outside every timed region: the output the timed launches of the headline workload ('N','N') left in `run.d`, its
    first and its last `cols` columns, against the float64 product D = A*B + C of the same seeded inputs.
    Returns (ok, relative Frobenius error)."""
    import numpy as np
    import gemmkernels as gk
    h = wl.host()
    a, b, c = h["a"].astype(np.float64), h["b"], h["c"]
    d = gk.to_numpy(run.d)
    num = den = 0.0
    for sl in (slice(0, cols), slice(c.shape[1] - cols, c.shape[1])):
        ref = a @ b[:, sl].astype(np.float64) + c[:, sl]
        num += float(((d[:, sl] - ref) ** 2).sum())
        den += float((ref ** 2).sum())
    err = (num / den) ** 0.5
    return bool(err <= 1e-3), err


def launch_distribution(fn, launches=40):
    """Min and median duration in microseconds of single launches, each bracketed by its own pair of events."""
    import torch
    times = []
    for _ in range(launches):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        fn()
        stop.record()
        stop.synchronize()
        times.append(start.elapsed_time(stop) * 1e3)
    times.sort()
    return times[0], times[len(times) // 2]


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    import gemmkernels as gk
    from gemmkernels import configs

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP library has no CPU fallback", file=sys.stderr)
        sys.exit(3)
    torch.cuda.set_device(0)

    if args.copy_calibration:
        src = torch.ones(64 << 20, dtype=torch.float32, device="cuda")     # 256 MiB
        dst = torch.empty_like(src)
        for _ in range(10):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration": {"bytes_read": src.numel() * 4, "bytes_written": src.numel() * 4, "launches": 10}}))
        return

    if args.workload == "size":
        # one size of the sweep below as the step, for profiling its kernel: mul!(C, A, B, 1, 1), default tile choice
        from gemmkernels.matmul import matmatmul_plan
        m, n, k = (int(x) for x in args.dims.split(","))
        gen = torch.Generator(device="cuda")
        gen.manual_seed(m * 31 + n * 17 + k)
        a_ = (torch.rand(k, m, device="cuda", generator=gen) * 2 - 1).to(torch.float16).t()
        b_ = (torch.rand(n, k, device="cuda", generator=gen) * 2 - 1).to(torch.float16).t()
        c_ = (torch.rand(n, m, device="cuda", generator=gen) * 2 - 1).t()
        plan = matmatmul_plan(c_, "N", "N", a_, b_, 1.0, 1.0)
        us, _ = time_launches(plan, args.steps, args.warmup, HEADLINE_SETTLE_SECONDS)
        tf = 2.0 * m * n * k / us / 1e6
        print(json.dumps({
            "metric": "TFLOP/s", "value": round(tf, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(us / 1e3, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "f16 multiplicands, f32 accumulate", "data": "synthetic (torch.rand on the device, seeded)",
            "config": {"workload": f"mul!(C, A, B, 1, 1), {m} x {n} x {k}, FP16 A/B, FP32 C read and written", "kernels": sorted(set(plan.kernel_names))},
            "roofline": {"bound": "mfma", "achieved": round(tf, 2), "peak": PEAK_FP16_TFLOPS, "unit": "TFLOP/s", "frac": round(tf / PEAK_FP16_TFLOPS, 4),
                         "traffic": None, "avg_launch_us": round(us, 2), "flop_per_launch": 2 * m * n * k}}))
        return

    if args.workload != "2" or args.variant != "NN":
        # one of the other workloads as the step: same JSON shape, for profiling a single kernel
        rotating = args.workload == "4b-rotating"
        key = "4b" if rotating else (int(args.workload) if args.workload.isdigit() else args.workload)
        wl = configs.benchmark_config(key, variant=args.variant if key == 2 else None)
        run = wl.prepare()
        if rotating:
            # four buffer sets (384 MiB, more than the last-level cache) in rotation: no launch finds its operands cached
            runs = [run] + [wl.prepare() for _ in range(3)]
            turn = {"i": 0}

            def run():
                runs[turn["i"] & 3]()
                turn["i"] += 1
        us, _ = time_launches(run, args.steps, args.warmup, HEADLINE_SETTLE_SECONDS)
        hbm = wl.bound == "hbm"
        achieved = wl.bytes / us / 1e3 if hbm else wl.flops / us / 1e6
        peak = PEAK_HBM_GBS if hbm else PEAK_FP16_TFLOPS
        print(json.dumps({
            "metric": "GB/s" if hbm else "TFLOP/s", "value": round(achieved, 2), "unit": "GB/s" if hbm else "TFLOP/s", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(us / 1e3, 6), "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "f16 multiplicands, f32 accumulate" if key != 1 else "f32", "data": "synthetic (counter-based splitmix64 streams)",
            "config": {"workload": wl.description + (", four buffer sets in rotation" if rotating else ""), "kernel": wl.kernel_name},
            "roofline": {"bound": "hbm" if hbm else "mfma", "achieved": round(achieved, 2), "peak": peak, "unit": "GB/s" if hbm else "TFLOP/s",
                         "frac": round(achieved / peak, 4), "traffic": None, "kernel": wl.kernel_name, "avg_launch_us": round(us, 2),
                         "bytes_per_launch": wl.bytes, "flop_per_launch": wl.flops}}))
        return

    # ---------------- headline: config 2, NN ----------------
    wl = configs.benchmark_config(2, variant="NN")
    run = wl.prepare()          # uploads the seeded inputs, returns a zero-argument launcher
    # the W warm-up launches are followed by a time-based settle phase (untimed, like the warm-up): a short run
    # such as --steps 20 --warmup 5 would otherwise time the first milliseconds after idle, while the shader
    # clock is still coming up (the secondary figures below have always been taken after such a phase)
    us, wall, settle_launches = settle_then_time(run, args.steps, args.warmup, HEADLINE_SETTLE_SECONDS)
    tflops = wl.flops / us / 1e6
    ok, err = verify_slab(wl, run)
    result = {
        "metric": METRIC,
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "settle_s": HEADLINE_SETTLE_SECONDS,
        "settle_launches": settle_launches,
        "ms_per_step": round(us / 1e3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16 multiplicands, f32 accumulate",
        "data": "synthetic (counter-based splitmix64 streams, seeds 2001-2003)",
        "config": {"workload": wl.description, "kernel": wl.kernel_name},
        "verified": ok,
        "verified_rel_frobenius_error": float(f"{err:.3e}"),
        "verified_against": "float64 product of the same inputs on the first and the last 256 columns of the D the timed launches wrote",
        "pct_of_fp16_mfma_peak": round(100.0 * tflops / PEAK_FP16_TFLOPS, 2),
        "roofline": {"bound": "mfma", "achieved": round(tflops, 2), "peak": PEAK_FP16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tflops / PEAK_FP16_TFLOPS, 4), "traffic": MEASURED_TRAFFIC_BYTES,
                     "traffic_source": TRAFFIC_SOURCE, "kernel": wl.kernel_name, "avg_launch_us": round(us, 2), "flop_per_launch": wl.flops},
    }

    if not args.no_extras:
        lo, med = launch_distribution(run)
        result["single_launch_us"] = {"min": round(lo, 2), "median": round(med, 2), "launches": 40}
        try:
            result["observed_device"] = observe_device(run)
        except Exception as e:      # readings are for orientation; never fail the benchmark over them
            result["observed_device"] = {"error": f"{type(e).__name__}: {e}"}
        try:
            result["matrix_core_ceiling"] = matrix_core_ceiling()
            result["matrix_core_ceiling"]["headline_frac_of_random_fp16_ceiling"] = round(tflops / result["matrix_core_ceiling"]["random_fp16_tflops"], 4)
        except Exception as e:
            result["matrix_core_ceiling"] = {"error": f"{type(e).__name__}: {e}"}
        # ---------------- the other transposes and configs (outside the timed region) ----------------
        extras = {}
        for cfg, variant in [(2, "NT"), (2, "TN"), (2, "TT"), (1, None), (3, None), ("4a", None), ("4a-planar", None), ("4b", None), (5, None), ("skinny", None)]:
            try:
                w = configs.benchmark_config(cfg, variant=variant)
                r = w.prepare()
                u, _ = time_launches(r, 50, 10, 0.15)
                entry = {"us": round(u, 2), "kernel": w.kernel_name}
                if w.bound == "hbm":
                    entry["GB/s"] = round(w.bytes / u / 1e3, 1)
                    entry["frac_of_hbm_peak"] = round(w.bytes / u / 1e3 / PEAK_HBM_GBS, 4)
                else:
                    entry["TFLOP/s"] = round(w.flops / u / 1e6, 2)
                extras[w.name] = entry
                del r, w
                torch.cuda.empty_cache()
            except Exception as e:  # a config that is not built yet must not hide the headline number
                extras[f"config {cfg}{' ' + variant if variant else ''}"] = {"error": f"{type(e).__name__}: {e}"}
        # config 4b is bandwidth bound: a second figure with four buffer sets (384 MiB, more than the
        # 256 MiB of last-level cache) used in rotation, so that no launch finds its operands cached
        try:
            w = configs.benchmark_config("4b")
            runs = [w.prepare() for _ in range(4)]
            state = {"i": 0}

            def rotate():
                runs[state["i"] & 3]()
                state["i"] += 1
            u, _ = time_launches(rotate, 48, 8, 0.15)
            extras["config 4b"]["rotating_buffers"] = {"us": round(u, 2), "GB/s": round(w.bytes / u / 1e3, 1),
                                                       "frac_of_hbm_peak": round(w.bytes / u / 1e3 / PEAK_HBM_GBS, 4)}
            del runs
            torch.cuda.empty_cache()
            # orientation: torch's converting copy FP16 -> FP32 of a 4096 x 4096 matrix moves exactly the same
            # bytes per launch (32 MiB read, 64 MiB written); four buffer pairs in rotation as well
            pairs = [(torch.ones(4096, 4096, dtype=torch.float16, device="cuda"), torch.empty(4096, 4096, dtype=torch.float32, device="cuda"))
                     for _ in range(4)]

            def copy_rotate():
                src, dst = pairs[state["i"] & 3]
                dst.copy_(src)
                state["i"] += 1
            u, _ = time_launches(copy_rotate, 48, 8, 0.15)
            extras["config 4b"]["converting_copy_same_bytes_rotating"] = {"us": round(u, 2), "GB/s": round(w.bytes / u / 1e3, 1),
                                                                          "frac_of_hbm_peak": round(w.bytes / u / 1e3 / PEAK_HBM_GBS, 4)}
            del pairs
            torch.cuda.empty_cache()
        except Exception as e:
            extras.setdefault("config 4b", {})["rotating_buffers"] = {"error": f"{type(e).__name__}: {e}"}
        # the headline shape with the other element types of the MFMA kernels: BF16 multiplicands, and FP16 C / D
        try:
            from gemmkernels import BFloat16, Float16, Kernel, Layout, Operator, plan
            w = configs.benchmark_config(2, variant="NN")
            r = w.prepare()
            M = N = K = 4096
            acm = Layout.UnsafeAlignedColMajor
            conf_bf = configs.mfma_config(M, N, K, operator=Operator.MFMAOp[32, 32, 16, BFloat16, gk_f32()], global_a_layout=acm[BFloat16],
                                          global_b_layout=acm[BFloat16])
            a_bf, b_bf = r.a.to(torch.bfloat16), r.b.to(torch.bfloat16)
            run_bf = plan(conf_bf, a_bf, b_bf, r.c, r.d, kernel=Kernel.matmul_pipelined)
            u, _ = time_launches(run_bf, 50, 10, 0.15)
            extras["config 2 NN, BF16 A/B"] = {"us": round(u, 2), "kernel": gk_name(conf_bf), "TFLOP/s": round(w.flops / u / 1e6, 2)}
            conf_h = configs.mfma_config(M, N, K, global_c_layout=acm[Float16], global_d_layout=acm[Float16])
            c_h = r.c.to(torch.float16)
            d_h = torch.empty_like(c_h)
            run_h = plan(conf_h, r.a, r.b, c_h, d_h, kernel=Kernel.matmul_pipelined)
            u, _ = time_launches(run_h, 50, 10, 0.15)
            extras["config 2 NN, FP16 C/D"] = {"us": round(u, 2), "kernel": gk_name(conf_h), "TFLOP/s": round(w.flops / u / 1e6, 2)}
            del r, w, run_bf, run_h, a_bf, b_bf, c_h, d_h
            torch.cuda.empty_cache()
        except Exception as e:
            extras["config 2 NN, other element types"] = {"error": f"{type(e).__name__}: {e}"}
        # the skinny product in place (mul!(C, A, B, 1, 1): d is c), which the K-split kind runs as one launch
        try:
            from gemmkernels import Kernel, plan
            w = configs.benchmark_config("skinny")
            r = w.prepare()
            in_place = plan(r.conf, r.a, r.b, r.c, r.c, kernel=Kernel.matmul_split_k)
            u, _ = time_launches(in_place, 50, 10, 0.15)
            extras["skinny"]["in_place"] = {"us": round(u, 2), "GB/s": round(w.bytes / u / 1e3, 1),
                                            "frac_of_hbm_peak": round(w.bytes / u / 1e3 / PEAK_HBM_GBS, 4)}
            del r, w, in_place
        except Exception as e:
            extras.setdefault("skinny", {})["in_place"] = {"error": f"{type(e).__name__}: {e}"}
        # the BLAS-level front end on sizes that are not whole tiles: mul!(C, A, B) with M = N = K = 4000
        # (bounds-checked layouts with 16-byte aligned columns: the aligned kernel masks the tiles over the edge)
        try:
            from gemmkernels import rng
            from gemmkernels.matmul import matmatmul_plan
            n = 4000
            a4 = gk.colmajor(rng.matrix("upm1_f16", 9001, (n, n)))
            b4 = gk.colmajor(rng.matrix("upm1_f16", 9002, (n, n)))
            c4 = gk.colmajor_empty((n, n), torch.float32)
            cut = matmatmul_plan(c4, "N", "N", a4, b4, 1.0, 0.0)
            u, _ = time_launches(cut, 50, 10, 0.15)
            extras["mul! 4000^3 (not whole tiles)"] = {"us": round(u, 2), "TFLOP/s": round(2.0 * n ** 3 / u / 1e6, 2), "launches": 1,
                                                       "kernels": sorted(set(cut.kernel_names))}
            del a4, b4, c4, cut
            torch.cuda.empty_cache()
            # sizes that are not multiples of 8 either: odd leading dimensions, every column at another offset from
            # a 16-byte boundary, 16-byte chunks that straddle the last row of A and the last column of B
            m5, n5, k5 = 4001, 4003, 4005
            a5 = gk.colmajor(rng.matrix("upm1_f16", 9003, (m5, k5)))
            b5 = gk.colmajor(rng.matrix("upm1_f16", 9004, (k5, n5)))
            c5 = gk.colmajor_empty((m5, n5), torch.float32)
            odd = matmatmul_plan(c5, "N", "N", a5, b5, 1.0, 0.0)
            u, _ = time_launches(odd, 50, 10, 0.15)
            extras["mul! 4001x4003x4005 (odd sizes)"] = {"us": round(u, 2), "TFLOP/s": round(2.0 * m5 * n5 * k5 / u / 1e6, 2), "kernels": sorted(set(odd.kernel_names))}
            del a5, b5, c5, odd
            torch.cuda.empty_cache()
        except Exception as e:
            extras["mul! 4000^3 (not whole tiles)"] = {"error": f"{type(e).__name__}: {e}"}
        # the BLAS-level front end over the sizes of the reference's performance curve (media/performance-wmma-gemm.png sweeps
        # N = 128 ... 16384): mul!(C, A, B, 1, 1) on FP16 A, B and an FP32 C that is read and written, default tile choice.
        # Each size is checked once, before it is timed: 128 columns of the result of one launch against the float64 product
        # of the same operands (generated on the device: the largest C alone is 1 GiB).  "vendor" is torch.mm on the same
        # A and B with FP16 output and no C, for orientation.
        try:
            from gemmkernels.matmul import matmatmul_plan
            sizes = {}
            for (m, n, k) in [(128, 128, 128), (256, 256, 256), (512, 512, 512), (1024, 1024, 1024), (2048, 2048, 2048), (3072, 3072, 3072), (4096, 4096, 4096), (6144, 6144, 6144),
                              (8192, 8192, 8192), (4096, 4096, 16384), (8192, 8192, 4096), (16384, 16384, 4096)]:
                gen = torch.Generator(device="cuda")
                gen.manual_seed(m * 31 + n * 17 + k)
                a_ = (torch.rand(k, m, device="cuda", generator=gen) * 2 - 1).to(torch.float16).t()      # column-major m x k
                b_ = (torch.rand(n, k, device="cuda", generator=gen) * 2 - 1).to(torch.float16).t()
                c_ = (torch.rand(n, m, device="cuda", generator=gen) * 2 - 1).t()
                c0 = c_[:, :128].to(torch.float64).cpu().numpy()
                p_ = matmatmul_plan(c_, "N", "N", a_, b_, 1.0, 1.0)
                p_()
                torch.cuda.synchronize()
                got = c_[:, :128].to(torch.float64).cpu().numpy()
                ref = a_.to(torch.float64).cpu().numpy() @ b_[:, :128].to(torch.float64).cpu().numpy() + c0
                err_ = float(np.linalg.norm(got - ref) / np.linalg.norm(ref))
                u, _ = time_launches(p_, 30 if m * n * k > 2 ** 37 else 50, 5, 0.15)
                out_ = torch.empty(m, n, device="cuda", dtype=torch.float16)
                am, bm_ = a_.contiguous(), b_.contiguous()
                uv, _ = time_launches(lambda: torch.mm(am, bm_, out=out_), 30 if m * n * k > 2 ** 37 else 50, 5, 0.15)
                sizes[f"{m}x{n}x{k}"] = {"us": round(u, 2), "TFLOP/s": round(2.0 * m * n * k / u / 1e6, 1), "rel_error_128_columns": float(f"{err_:.2e}"),
                                         "verified": bool(err_ <= 1e-3), "kernels": sorted(set(p_.kernel_names)),
                                         "vendor_fp16_out_no_c_us": round(uv, 2)}
                del a_, b_, c_, p_, out_, am, bm_
                torch.cuda.empty_cache()
            extras["sizes: mul!(C, A, B, 1, 1), FP16 x FP16 + FP32 C"] = sizes
        except Exception as e:
            extras["sizes: mul!(C, A, B, 1, 1), FP16 x FP16 + FP32 C"] = {"error": f"{type(e).__name__}: {e}"}
        # the vendor library on the headline shape, for orientation only: FP16 in, FP16 out, no C read
        # (torch.mm -> hipBLASLt), so it moves 96 MiB less per launch than config 2 does
        try:
            x = torch.randn(4096, 4096, device="cuda").to(torch.float16)
            y = torch.randn(4096, 4096, device="cuda").to(torch.float16)
            out = torch.empty(4096, 4096, device="cuda", dtype=torch.float16)
            u, _ = time_launches(lambda: torch.mm(x, y, out=out), 50, 10, 0.15)
            extras["vendor_library_fp16_out_no_c"] = {"us": round(u, 2), "TFLOP/s": round(wl.flops / u / 1e6, 2)}
            del x, y, out
        except Exception as e:
            extras["vendor_library_fp16_out_no_c"] = {"error": f"{type(e).__name__}: {e}"}
        result["other_configs"] = extras

        # ---------------- CPU baseline: the reference's own CPU path is BLAS sgemm on host arrays ----------------
        from oracle import oracle
        a, b, c = wl.host_inputs()
        a32, b32 = a.astype(np.float32), b.astype(np.float32)
        times = []
        for _ in range(3):
            t0 = time.perf_counter()
            oracle.gemm_blas_f32(a32, b32, c, 1.0, 1.0)
            times.append(time.perf_counter() - t0)
        cpu_s = sorted(times)[1]
        threads = int(os.environ.get("OPENBLAS_NUM_THREADS") or os.environ.get("OMP_NUM_THREADS") or os.cpu_count())
        result["cpu_baseline"] = {"value": round(wl.flops / cpu_s / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
                                  "sample": "3 full 4096^3 GEMMs on the FP32-converted inputs (numpy -> OpenBLAS sgemm, the "
                                            "routine behind the reference's LinearAlgebra.mul! oracle), median",
                                  "seconds": round(cpu_s, 4)}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
