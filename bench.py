#!/usr/bin/env python3
"""Benchmark of the FP8 flash-attention forward hot path on one MI355X.

A step is one call of `attention_cutlass_fp8.flash_attention_v2_cutlass(q, k, v, is_causal, softmax_scale)` on the
headline workload (B=2, H=32, N=4096, d=128, non-causal, e4m3 inputs drawn N(0,1), fp16 output) with q/k/v already
resident in HBM.  Prints ONE JSON line: TFLOP/s = 4*B*H*N^2*d / t (halved for causal workloads), the fraction of the
MI355X dense FP8 MFMA peak, and a CPU baseline (the reference's naive attention restated in PyTorch, timed on the host
cores of the same machine on a bounded sample of heads).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg3] [--no-cpu-baseline]
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FP8_MFMA_PEAK_TFLOPS = 5000.0  # MI355X dense FP8 matrix peak (5.0 PFLOP/s)
HBM_PEAK_GBPS = 8000.0

# HBM bytes per launch of the headline workload read by rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE), each scaled by
# what the same counter reads for a plain copy kernel of known size; see profiles/.  None until measured.
MEASURED_TRAFFIC_BYTES = {"cfg3": 168.0e6,  # profiles/fa8_fwd_kernel_d128_cfg3_headline.md, section 3
                          "cfg2": 21.12e6, "cfg4": 364.2e6, "cfg5": 104.2e6}  # profiles/fa8_fwd_kernel_cfg2_cfg4_cfg5.md


TRAFFIC_SOURCE = {"cfg3": "profiles/fa8_fwd_kernel_d128_cfg3_headline.md", "cfg2": "profiles/fa8_fwd_kernel_cfg2_cfg4_cfg5.md",
                  "cfg4": "profiles/fa8_fwd_kernel_cfg2_cfg4_cfg5.md", "cfg5": "profiles/fa8_fwd_kernel_cfg2_cfg4_cfg5.md"}

# cutlass fp8 milliseconds published by the reference (benchmark.png, rows in the order of test.py:95-100; Ada sm_89,
# GPU model unstated; host wall clock with a device sync per iteration)
REFERENCE_MS = {(16, 1024, 64): 0.0352, (16, 1024, 128): 0.0500, (16, 2048, 64): 0.0833, (16, 2048, 128): 0.1169,
                (16, 4096, 64): 0.1937, (16, 4096, 128): 0.3094, (32, 1024, 64): 0.0452, (32, 1024, 128): 0.0617,
                (32, 2048, 64): 0.1024, (32, 2048, 128): 0.1653, (32, 4096, 64): 0.3044, (32, 4096, 128): 0.5358,
                (64, 1024, 64): 0.0601, (64, 1024, 128): 0.0926, (64, 2048, 64): 0.1632, (64, 2048, 128): 0.2774,
                (64, 4096, 64): 0.5336, (64, 4096, 128): 0.9701}


# "official fp16" milliseconds of the same table (vllm_flash_attn on the reference's Ada GPU)
REFERENCE_FP16_MS = {(16, 1024, 64): 0.0546, (16, 1024, 128): 0.0807, (16, 2048, 64): 0.1389, (16, 2048, 128): 0.1917,
                     (16, 4096, 64): 0.3271, (16, 4096, 128): 0.5482, (32, 1024, 64): 0.0770, (32, 1024, 128): 0.1026,
                     (32, 2048, 64): 0.1844, (32, 2048, 128): 0.2900, (32, 4096, 64): 0.5487, (32, 4096, 128): 0.9789,
                     (64, 1024, 64): 0.1093, (64, 1024, 128): 0.1613, (64, 2048, 64): 0.2951, (64, 2048, 128): 0.5131,
                     (64, 4096, 64): 0.9820, (64, 4096, 128): 1.8645}


def reference_sweep(ext, torch):
    """The reference's benchmark loop (test.py:36-46, 49-91) on this GPU: same shapes, same input recipe, causal,
    scale 1/sqrt(N); v is passed as [B,H,N,d] (this build needs no caller-side transpose)."""
    import math
    rows = []
    for (H, N, d), ref_ms in REFERENCE_MS.items():
        g = torch.Generator(device="cpu").manual_seed(180)
        q, k, v = (torch.empty((1, H, N, d)).normal_(0.0, 0.5, generator=g).clamp_(-0.1, 0.1).to(torch.float8_e4m3fn).cuda()
                   for _ in range(3))
        scale = 1.0 / math.sqrt(N)
        for _ in range(20):
            ext.flash_attention_v2_cutlass(q, k, v, True, scale)
        torch.cuda.synchronize()
        n = 100
        t0 = time.perf_counter()
        for _ in range(n):
            ext.flash_attention_v2_cutlass(q, k, v, True, scale)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / n
        # the reference's "official fp16" column (test.py:76-80 times a flash-attention library on the fp16 upcasts):
        # here PyTorch's own fused fp16 attention on the same GPU
        q16, k16, v16 = q.half(), k.half(), v.half()
        sdpa = torch.nn.functional.scaled_dot_product_attention
        for _ in range(5):
            sdpa(q16, k16, v16, is_causal=True, scale=scale)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(20):
            sdpa(q16, k16, v16, is_causal=True, scale=scale)
        torch.cuda.synchronize()
        fp16_ms = (time.perf_counter() - t0) * 1e3 / 20
        rows.append({"heads": H, "seq_len": N, "head_dim": d, "ms": round(ms, 4), "official_fp16_ms": round(fp16_ms, 4),
                     "speedup_vs_official_fp16": round(fp16_ms / ms, 2), "reference_ada_ms": ref_ms,
                     "reference_ada_official_fp16_ms": REFERENCE_FP16_MS[(H, N, d)],
                     "speedup_vs_reference": round(ref_ms / ms, 2),
                     "tflops": round(2.0 * H * N * N * d / (ms * 1e-3) / 1e12, 1)})
    print(json.dumps({"metric": "reference_benchmark_table_ms", "unit": "ms", "config": "B=1 causal e4m3, scale=1/sqrt(N), "
                      "inputs N(0,0.5) clamped to +-0.1 (reference test.py:13-23,56-57)", "rows": rows}), flush=True)


def shape_sweep(ext, fa, torch):
    """Kernel time over a grid of shapes at a fixed token count (B*H*N = 262144, the headline's): head dims 64 / 128 / 256,
    N from 1024 to 16384, full and causal; N(0,1) inputs, scale 1/sqrt(d); 40 event-timed launches per shape after a short
    settle phase.  One JSON line."""
    import math
    rows = []
    for d in (64, 128, 256):
        for n, bsz, heads in ((1024, 8, 32), (2048, 4, 32), (4096, 2, 32), (8192, 1, 32), (16384, 1, 16)):
            g = torch.Generator(device="cpu").manual_seed(7)
            q, k, v = (torch.randn((bsz, heads, n, d), generator=g).to(torch.float8_e4m3fn).cuda() for _ in range(3))
            for causal in (False, True):
                scale = 1.0 / math.sqrt(d)
                plan = fa.lib().fa8_fwd_schedule(ctypes.byref(fa.make_params(
                    q, k, v, ext.flash_attention_v2_cutlass(q, k, v, causal, scale)[0], causal, scale)))
                t0 = time.perf_counter()
                while time.perf_counter() - t0 < 0.1:
                    for _ in range(10):
                        ext.flash_attention_v2_cutlass(q, k, v, causal, scale)
                    torch.cuda.synchronize()
                evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(40)]
                for e0, e1 in evs:
                    e0.record()
                    ext.flash_attention_v2_cutlass(q, k, v, causal, scale)
                    e1.record()
                torch.cuda.synchronize()
                ms = sorted(e0.elapsed_time(e1) for e0, e1 in evs)
                avg = sum(ms) / len(ms)
                flops = 4.0 * bsz * heads * n * n * d * (0.5 if causal else 1.0)
                rows.append({"batch": bsz, "heads": heads, "seq_len": n, "head_dim": d, "causal": causal,
                             "main_loop": MAIN_LOOPS.get(plan, str(plan)), "kernel_ms_avg": round(avg, 5),
                             "tflops": round(flops / (avg * 1e-3) / 1e12, 1),
                             "pct_fp8_mfma_peak": round(100.0 * flops / (avg * 1e-3) / 1e12 / FP8_MFMA_PEAK_TFLOPS, 2)})
    print(json.dumps({"metric": "fp8_attention_fwd_shape_sweep", "unit": "TFLOP/s", "rows": rows}), flush=True)


def read_sclk_mhz():
    """Current shader clock from the amdgpu sysfs node (the level marked '*' in pp_dpm_sclk), or None."""
    import glob
    import re
    for path in sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk")):
        try:
            with open(path) as f:
                for line in f:
                    if line.rstrip().endswith("*"):
                        m = re.search(r"(\d+)\s*Mhz", line, re.IGNORECASE)
                        if m:
                            return int(m.group(1))
        except OSError:
            pass
    return None


def read_power_w():
    """(board power now, power cap) in watts from the amdgpu hwmon node, None where a file is missing."""
    import glob

    def first(pattern):
        for path in sorted(glob.glob(pattern)):
            try:
                with open(path) as f:
                    return int(f.read().strip()) / 1e6
            except (OSError, ValueError):
                pass
        return None
    base = "/sys/class/drm/card*/device/hwmon/hwmon*/"
    now = first(base + "power1_average")
    if now is None:
        now = first(base + "power1_input")
    return now, first(base + "power1_cap")


def measure_traffic(workload):
    """HBM bytes per launch of one workload, measured now: four rocprofv3 --pmc child runs of this script (FETCH_SIZE and
    WRITE_SIZE, each for the kernel and for a plain 256 MiB device copy that gives the counter's scale).  This process must not
    have touched the GPU yet (it only starts children).  Prints one JSON line."""
    import csv
    import glob
    import shutil
    import subprocess
    import tempfile
    rocprof = shutil.which("rocprofv3") or os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "bin", "rocprofv3")
    tmp = tempfile.mkdtemp(prefix="fa8_traffic_", dir=os.environ.get("TMPDIR", "/tmp"))

    def counter(name, args, kernel_substr):
        out = os.path.join(tmp, name + "_" + str(len(os.listdir(tmp))))
        cmd = [rocprof, "--pmc", name, "--output-format", "csv", "-d", out, "--", sys.executable, os.path.abspath(__file__)] + args
        subprocess.run(cmd, check=True, cwd=tmp, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL, timeout=170)
        vals = []
        for f in glob.glob(os.path.join(out, "**", "*_counter_collection.csv"), recursive=True):
            with open(f) as fh:
                vals += [float(r["Counter_Value"]) for r in csv.DictReader(fh)
                         if kernel_substr in r["Kernel_Name"] and r["Counter_Name"] == name]
        if not vals:
            raise RuntimeError(f"no {name} rows for {kernel_substr}")
        return sum(vals) / len(vals), len(vals)
    kern_args = ["--workload", workload, "--no-cpu-baseline", "--no-other-workloads", "--steps", "5", "--warmup", "2",
                 "--settle-seconds", "0"]
    copy_kib = float(256 << 10)
    res = {}
    for name in ("FETCH_SIZE", "WRITE_SIZE"):
        cal, _ = counter(name, ["--copy-calibration"], "copyBuffer")
        kib, n = counter(name, kern_args, "fa8_fwd_kernel")
        res[name] = {"kib_per_launch": round(kib, 1), "launches": n, "copy_256MiB_reads": round(cal, 1),
                     "scale": round(copy_kib / cal, 3), "bytes_per_launch": kib * 1024.0 * copy_kib / cal}
    shutil.rmtree(tmp, ignore_errors=True)
    from cutlass_flash_atten_fp8_amd import inputs
    alg = inputs.algorithmic_bytes(inputs.CONFIGS[workload])
    total = res["FETCH_SIZE"]["bytes_per_launch"] + res["WRITE_SIZE"]["bytes_per_launch"]
    print(json.dumps({"workload": workload, "hbm_bytes_per_launch": round(total), "algorithmic_bytes": alg,
                      "traffic_ratio": round(total / alg, 3), "counters": res}), flush=True)


def time_other_workload(name, ext, fa, inputs, torch, launches=20, settle_seconds=0.15):
    """Kernel time of one more BASELINE workload, measured like the headline: clock-settle launches, then one HIP-event pair
    per launch on torch's current stream.  Returns the entry of config.other_workloads."""
    cfg = inputs.CONFIGS[name]
    scale, causal = inputs.softmax_scale(cfg), cfg["causal"]
    q, k, v = (t.to("cuda:0") for t in inputs.make_qkv(cfg))

    def step():
        return ext.flash_attention_v2_cutlass(q, k, v, causal, scale)[0]
    plan = fa.lib().fa8_fwd_schedule(ctypes.byref(fa.make_params(q, k, v, step(), causal, scale)))
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < settle_seconds:
        for _ in range(20):
            step()
        torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(launches)]
    for e0, e1 in evs:
        e0.record()
        step()
        e1.record()
    torch.cuda.synchronize()
    ms = sorted(e0.elapsed_time(e1) for e0, e1 in evs)
    avg = sum(ms) / len(ms)
    flops, alg = inputs.flops(cfg), inputs.algorithmic_bytes(cfg)
    traffic = MEASURED_TRAFFIC_BYTES.get(name)
    return {"workload": f"{name}: B={cfg['B']} H={cfg['H']} N={cfg['N']} d={cfg['d']} {'causal' if causal else 'non-causal'}",
            "main_loop": MAIN_LOOPS.get(plan, f"error {plan}"),
            "kernel_ms_avg": round(avg, 5), "kernel_ms_min": round(ms[0], 5),
            "tflops": round(flops / (avg * 1e-3) / 1e12, 1),
            "pct_fp8_mfma_peak": round(100.0 * flops / (avg * 1e-3) / 1e12 / FP8_MFMA_PEAK_TFLOPS, 2),
            "algorithmic_hbm_gbps": round(alg / (avg * 1e-3) / 1e9, 1),
            "pct_hbm_peak": round(100.0 * alg / (avg * 1e-3) / 1e9 / HBM_PEAK_GBPS, 2),
            # HBM bytes per launch from the committed rocprofv3 --pmc runs over the algorithmic bytes (not measured in this run)
            "traffic_ratio": round(traffic / alg, 2) if traffic else None}


MAIN_LOOPS = {1: "rolling", 2: "pipelined", 3: "dense"}  # FA8_SCHEDULE_* (include/fa8_api.h)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="cfg3", help="cfg1..cfg5 (cfg3 is the headline)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--schedule", default="auto", choices=["auto", "rolling", "pipelined", "dense"],
                    help="main loop hint passed to the operator (include/fa8_api.h, FA8_SCHEDULE_*); the results do not depend on it")
    ap.add_argument("--v-transposed", action="store_true",
                    help="hand v over as [B,H,d,N], the reference's calling convention (reference test.py:71): the kernel then "
                         "reads V^T fragments with plain 16-byte LDS reads instead of the transposing ones")
    ap.add_argument("--inputs", default="workload", choices=["workload", "v-ones", "zeros"],
                    help="what the timed tensors hold: the workload's own seeded draw; the same with v all ones; all zeros.  "
                         "Same instructions (zeros: no rescale), fewer toggling bits: shows how far board power sets the clock")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="skip the kernel times of the other BASELINE workloads (config.other_workloads; headline runs only)")
    ap.add_argument("--settle-seconds", type=float, default=0.25,
                    help="untimed launches for this long after the warm-up, so that the shader clock has settled")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="target CPU time of the baseline sample")
    ap.add_argument("--reference-sweep", action="store_true",
                    help="instead of the headline step, time the 18 shapes of the reference's own benchmark table "
                         "(reference test.py:95-100: B=1, causal, scale=1/sqrt(N), inputs clamped to +-0.1) and print "
                         "one JSON line holding the table next to the reference's published Ada numbers")
    ap.add_argument("--shape-sweep", action="store_true",
                    help="instead of the headline step, time a grid of shapes at the headline's token count (head dims 64, 128, "
                         "256; N 1024 ... 16384; full and causal) and print one JSON line")
    ap.add_argument("--instruction-mix", action="store_true",
                    help="run only the instruction-mix probe (bench_mix_probe.hip beside this file, built with hipcc on first "
                         "use): what a SIMD needs for the vector and matrix instructions of one KV block, then with the LDS "
                         "operand reads, the tile copies and the barrier of the loop added; prints its JSON lines")
    ap.add_argument("--measure-traffic", action="store_true",
                    help="measure the HBM bytes per launch of --workload now: runs rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on "
                         "child runs of this script and of its --copy-calibration (the figure roofline.traffic quotes)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run only a plain 256 MiB device-to-device copy (10 times): the known-size kernel that the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (every (batch, head) is independent: more GPUs would each take a "
              "range of heads and run this same kernel, with no communication); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    if args.measure_traffic:
        measure_traffic(args.workload)
        return
    if args.instruction_mix:
        import subprocess
        src, exe = os.path.join(ROOT, "bench_mix_probe.hip"), os.path.join(ROOT, "bench_mix_probe")
        if not os.path.exists(exe) or os.path.getmtime(exe) < os.path.getmtime(src):
            subprocess.run([os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "bin", "hipcc"), "--offload-arch=gfx950", "-O3",
                            "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-o", exe, src], check=True)
        sys.exit(subprocess.run([exe]).returncode)
    import torch
    import cutlass_flash_atten_fp8_amd as fa
    from cutlass_flash_atten_fp8_amd import inputs
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda:0").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(10):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration_bytes_read": 256 << 20, "copy_calibration_bytes_written": 256 << 20, "launches": 10}))
        return
    ext = fa.load_extension()  # raises if the native code has not been built: there is no fallback path
    if args.reference_sweep:
        reference_sweep(ext, torch)
        return
    if args.shape_sweep:
        shape_sweep(ext, fa, torch)
        return
    cfg = inputs.CONFIGS[args.workload]
    scale = inputs.softmax_scale(cfg)
    causal = cfg["causal"]
    dev = torch.device("cuda:0")
    q8, k8, v8 = inputs.make_qkv(cfg)
    q, k, v = q8.to(dev), k8.to(dev), v8.to(dev)
    flops = inputs.flops(cfg)

    if args.inputs == "v-ones":
        v = torch.ones_like(v, dtype=torch.float32).to(v.dtype)
    elif args.inputs == "zeros":
        q, k, v = torch.zeros_like(q), torch.zeros_like(k), torch.zeros_like(v)
    hint = {"auto": 0, "rolling": 1, "pipelined": 2, "dense": 3}[args.schedule]
    if args.v_transposed:
        v = v.transpose(2, 3).contiguous()

    def step():
        return ext.flash_attention_v2_cutlass(q, k, v, causal, scale, v_transposed=args.v_transposed, schedule=hint)[0]

    # which of the kernel's main loops the library runs for this launch (include/fa8_api.h, FA8_SCHEDULE_*)
    plan = fa.lib().fa8_fwd_schedule(ctypes.byref(fa.make_params(q, k, v, step(), causal, scale, v_transposed=args.v_transposed,
                                                                 schedule=hint)))
    main_loop = MAIN_LOOPS.get(plan, f"error {plan}")
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # Clock settle (untimed, disclosed as config.settle_launches): after an idle period the first launches run at a
    # lower shader clock, whatever --warmup says; keep the GPU busy for a fixed time before anything is timed.
    settle_launches = 0
    t_settle = time.perf_counter()
    while time.perf_counter() - t_settle < args.settle_seconds:
        for _ in range(50):
            step()
        torch.cuda.synchronize()
        settle_launches += 50
    # whole-step wall clock: exactly `steps` steps between two device synchronisations
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps

    # kernel duration: HIP events on the stream the kernel is launched on (torch's current stream), one pair per launch
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    for e0, e1 in evs:
        e0.record()
        step()
        e1.record()
    torch.cuda.synchronize()
    kern_ms = sorted(e0.elapsed_time(e1) for e0, e1 in evs)
    # shader clock while the kernel is running (power management lowers it under dense matrix work): sampled in the
    # middle of untimed bursts of launches long enough to keep the queue full whatever --steps is, median of 16 readings
    burst = max(25, int(0.008 / max(kern_ms[len(kern_ms) // 2] * 1e-3, 1e-6)))  # about 8 ms of kernel time per burst
    samples, watts = [], []
    for _ in range(20):
        for _ in range(burst):
            step()
        time.sleep(0.004)  # the queue stays full: the launches above take about twice as long as this
        samples.append(read_sclk_mhz())
        watts.append(read_power_w()[0])
    torch.cuda.synchronize()
    samples = sorted(x for x in samples[4:] if x is not None)
    sclk = samples[len(samples) // 2] if samples else None
    watts = sorted(x for x in watts[4:] if x is not None)
    power_w = round(watts[len(watts) // 2]) if watts else None
    power_cap_w = read_power_w()[1]
    kern_avg_ms = sum(kern_ms) / len(kern_ms)

    tflops = flops / (wall_ms * 1e-3) / 1e12
    kern_tflops = flops / (kern_avg_ms * 1e-3) / 1e12
    alg_bytes = inputs.algorithmic_bytes(cfg)

    out = {
        "metric": "fp8_attention_fwd_tflops",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3",
        "data": "synthetic",
        "config": {
            "workload": f"{args.workload}: B={cfg['B']} H={cfg['H']} N={cfg['N']} d={cfg['d']} "
                        f"{'causal' if causal else 'non-causal'}, e4m3 q/k/v ~ {cfg['dist']}, fp16 O, scale=1/sqrt(d)",
            "flops_per_step": flops,
            "pct_fp8_mfma_peak": round(100.0 * tflops / FP8_MFMA_PEAK_TFLOPS, 2),
            "algorithmic_hbm_gbps": round(alg_bytes / (kern_avg_ms * 1e-3) / 1e9, 1),
            "kv_block": fa.query(fa.FA8_QUERY_KV_BLOCK),
            "main_loop": main_loop,
            "v_layout": "[B,H,d,N]" if args.v_transposed else "[B,H,N,d]",
            "inputs": args.inputs,
            "sclk_mhz_under_load": sclk,
            "board_power_w_under_load": power_w,
            "board_power_cap_w": round(power_cap_w) if power_cap_w is not None else None,
            "settle_launches": settle_launches,
        },
        "roofline": {
            "bound": "mfma",
            "achieved": round(kern_tflops, 2),
            "peak": FP8_MFMA_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(kern_tflops / FP8_MFMA_PEAK_TFLOPS, 4),
            "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload),
            "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a plain copy: " + TRAFFIC_SOURCE[args.workload]
                              if args.workload in TRAFFIC_SOURCE else None,
            "kernel_ms_avg": round(kern_avg_ms, 5),
            "kernel_ms_min": round(kern_ms[0], 5),
            "kernel_ms_median": round(kern_ms[len(kern_ms) // 2], 5),
        },
    }

    if args.workload == "cfg3" and not args.no_other_workloads and not args.v_transposed and hint == 0 and args.inputs == "workload":
        # the other BASELINE workloads in the same process: kernel time, TFLOP/s and algorithmic HBM rate (value, ms_per_step and
        # roofline above stay the headline's)
        out["config"]["other_workloads"] = [time_other_workload(w, ext, fa, inputs, torch) for w in ("cfg2", "cfg4", "cfg5")]

    if not args.no_cpu_baseline and args.inputs == "workload":
        # The reference's CPU-runnable path (naive attention, reference test.py:25-33) restated in oracle/ and timed
        # on this machine's host cores, on the first heads of the same workload.
        from oracle.naive_attention import naive_attention_cpu
        host_cores = os.cpu_count() or 1
        threads = min(host_cores, 16)  # a one-GPU box shares its host: 16 cores are this job's share
        torch.set_num_threads(threads)
        naive_attention_cpu(q8, k8, v8, scale, causal, heads_limit=1)  # warm-up, also sizes the sample
        t0 = time.perf_counter()
        naive_attention_cpu(q8, k8, v8, scale, causal, heads_limit=1)
        per_head = time.perf_counter() - t0
        n_heads_total = cfg["B"] * cfg["H"]
        n = max(1, min(n_heads_total, int(args.cpu_seconds / max(per_head, 1e-6))))
        reps = max(1, min(8, int(args.cpu_seconds / max(per_head * n, 1e-6))))  # small workloads: several passes
        t0 = time.perf_counter()
        for _ in range(reps):
            naive_attention_cpu(q8, k8, v8, scale, causal, heads_limit=n)
        cpu_s = (time.perf_counter() - t0) / reps
        cpu_tflops = flops * (n / n_heads_total) / cpu_s / 1e12
        out["cpu_baseline"] = {
            "value": round(cpu_tflops, 4),
            "unit": "TFLOP/s",
            "cores": threads,  # threads actually used
            "host_cores": host_cores,  # os.cpu_count() of the machine
            "kind": "port",
            "sample": f"first {n} of {n_heads_total} (batch*head) slices of the same workload, {reps} pass(es) of "
                      f"{cpu_s:.2f} s, torch CPU naive attention with P re-quantised to e4m3",
        }
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
