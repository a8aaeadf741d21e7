#!/usr/bin/env python3
"""bench.py -- headline benchmark: bf16 GEMM TFLOP/s at M=N=K=8192 on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--config NAME] [--no-configs]

One "step" is one launch of the GEMM (A 8192x8192 row-major, B 8192x8192 K-major, both
U[-1,1) seeded bf16, C bf16, fp32 accumulate) with the inputs already resident in HBM.
Prints ONE JSON line.  `value` = 2*M*N*K / time per launch, in TFLOP/s.  The `roofline`
object prices the kernel against MI355X's published dense bf16 MFMA peak (2.5 PFLOP/s);
for the HBM-bound skinny workloads it is priced against 8 TB/s instead.  `cpu_baseline` is
the CPU restatement of the reference's reference_cpu_gemm (reference.h:5-46) timed on this
box's host cores on a bounded sample of 64x64 output tiles of the same problem.  After the
headline's timed region the other seven shapes of the benchmark definition (512^3, the two MLP
shapes, the three decode shapes, 4095x6143x3073) are timed with the library's own kernel choice
and reported as `configs`, one row each with its roofline fraction and tolerance check.

The timed region is bracketed by device synchronisation and measured with HIP events
recorded on the stream the kernel is launched on (the null stream, as the reference's
launchers use).  The library is loaded from h100_gemm_amd/lib; there is no fallback path.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

PEAK_BF16_TFLOPS = 2500.0     # MI355X published dense bf16 MFMA peak
PEAK_HBM_GBS = 8000.0         # MI355X published HBM3E bandwidth

# name -> (M, N, K, fill); fills as in the benchmark definition
WORKLOADS = {
    "square512": (512, 512, 512, "uniform"),
    "square8192": (8192, 8192, 8192, "uniform"),
    "mlp_up": (8192, 28672, 8192, "normal"),
    "mlp_down": (8192, 8192, 28672, "normal"),
    "skinny16": (16, 8192, 8192, "normal"),
    "skinny64": (64, 8192, 8192, "normal"),
    "skinny128": (128, 8192, 8192, "normal"),
    "unaligned": (4095, 6143, 3073, "uniform"),
    # outputs of few tiles (not BASELINE configurations; for the profiles of the small-tile kernel)
    "fewtile512": (512, 512, 4096, "uniform"),
    "fewtile1024": (1024, 1024, 4096, "uniform"),
    # 144 and 256 tiles of 128x128: one workgroup per CU at most (the kernel with two K groups)
    # 225 tiles of 96x96, one per CU at most, K too short to split over the waves (the shared-ring kernel)
    "mid1440": (1440, 1440, 1472, "uniform"),
    "square1536": (1536, 1536, 1536, "uniform"),
    "square2048": (2048, 2048, 2048, "uniform"),
    # 48 tiles of 32x32 with a very long K: K cut into pieces over workgroups in the small-tile kernel
    "longk128": (128, 384, 13376, "uniform"),
}
# HBM-side bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (the summaries
# under profiles/ give the commands), scaled by the same counters on a copy kernel of known size:
# FETCH_SIZE counts KiB and reads half of what a plain 256 MiB device copy moves (131087 for
# 262144 KiB read), so it is scaled by 2.0; WRITE_SIZE reads the copy's writes exactly (1.0).
# workload -> (kernel configuration the counters were read on, profile that holds the figures,
# FETCH_SIZE KiB of each kernel of the launch, WRITE_SIZE KiB of each).  Profile constants, not
# something this run measures: reported only while the run uses that same kernel; the figures are
# the ones the named profile shows (tests/test_host_api.py compares them).
FETCH_SCALE, WRITE_SCALE = 2.0, 1.0
MEASURED_TRAFFIC_KIB = {
    "square8192": ("m256x256_w2x2_g4_b3", "gemm_mfma16_kernel_square8192.md", (786705,), (131081,)),   # 1.75 GB against 0.40 GB algorithmic
    "skinny16": ("s16x32_n3", "gemm_stream_kernel_skinny16.md", (66585,), (256,)),                     # 0.137 GB: B is read exactly once
    "unaligned": ("m256x192_w2x2_g4_b3", "gemm_mfma16_kernel_unaligned.md", (130054,), (49665,)),      # 0.317 GB against 0.113 GB algorithmic
    "mlp_up": ("m256x256_w2x2_g4_b3", "gemm_mfma16_kernel_mlp_up.md", (2753369,), (458767,)),          # 6.1 GB against 1.34 GB algorithmic
    "mlp_down": ("m256x256_w2x2_g8_b1", "gemm_mfma16_kernel_mlp_down.md", (2752957,), (131159,)),      # 5.8 GB against 1.07 GB algorithmic
    "square512": ("k32x32_s4", "gemm_shared_ring_kernel_square512.md", (1587,), (512,)),                     # 3.7 MB against 1.5 MB algorithmic: a copy of the rows per L2
    "fewtile512": ("k32x32_n2", "gemm_wavek_kernel_fewtile.md", (12317,), (512,)),                     # 25.8 MB against 8.9 MB algorithmic
    "fewtile1024": ("k64x64_n2", "gemm_wavek_kernel_fewtile.md", (24627,), (2048,)),                   # 52.5 MB against 18.9 MB algorithmic
    "skinny64": ("d64x128_n4", "gemm_decode_kernel_skinny128_skinny64.md", (69689, 4114), (8192, 1024)),      # main + reduce kernels
    "skinny128": ("d128x128_n3", "gemm_decode_kernel_skinny128_skinny64.md", (73797, 8210), (16384, 2048)),   # main + reduce kernels
}
MEASURED_TRAFFIC_BYTES = {w: (cfg, (sum(f) * FETCH_SCALE + sum(wr) * WRITE_SCALE) * 1024)
                          for w, (cfg, _, f, wr) in MEASURED_TRAFFIC_KIB.items()}
# The eight shapes of the benchmark definition, in its order: every run of the headline workload
# also times the other seven (after the headline's timed region) and reports them as `configs`.
BASELINE_WORKLOADS = ("square512", "square8192", "mlp_up", "mlp_down", "skinny16", "skinny64", "skinny128", "unaligned")


def bound_of(M: int, N: int, K: int) -> str:
    """What the shape is priced against: the bf16 MFMA peak, the HBM peak, or neither -- 512^3 is
    0.2 us of either and a few microseconds of launch and pipeline latency (reported as it is)."""
    flops, nbytes = 2.0 * M * N * K, 2.0 * (M * K + N * K + M * N)
    if flops / (PEAK_BF16_TFLOPS * 1e12) < 1e-6 and nbytes / (PEAK_HBM_GBS * 1e9) < 1e-6:
        return "launch"
    return "hbm" if flops / nbytes < PEAK_BF16_TFLOPS * 1e12 / (PEAK_HBM_GBS * 1e9) else "mfma"


def make_inputs(orc, M, N, K, fill, seed=69):
    if fill == "uniform":
        return orc.fill_uniform((M, K), seed, 1), orc.fill_uniform((N, K), seed, 2)
    return orc.fill_normal((M, K), seed, 1, 1.0), orc.fill_normal((N, K), seed, 2, 0.02)


def cpu_baseline(orc, A, B, budget_tiles: int) -> dict:
    """Time the loop-order-faithful oracle on a sample of 64x64 tiles (each tile is the
    full K deep, exactly the reference's arithmetic for those outputs)."""
    M, K = A.shape
    N = B.shape[0]
    tiles = orc.sample_tiles(M, N, budget_tiles)
    t0 = time.perf_counter()
    orc.reference_cpu_gemm(A, B, fast=False, tiles=tiles)
    dt = time.perf_counter() - t0
    flops = 0
    for ti, tj in tiles:
        flops += 2.0 * min(64, M - ti * 64) * min(64, N - tj * 64) * K
    total_tiles = -(-M // 64) * -(-N // 64)
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": orc.num_threads(),
            "kind": "port",
            "sample": f"{len(tiles)} of {total_tiles} 64x64 output tiles, full K={K}, "
                      f"reference loop order, {dt:.1f} s; whole problem extrapolates to "
                      f"{dt * total_tiles / len(tiles):.0f} s"}


def time_workload(mi, orc, name: str, launches: int, check_tiles: int) -> dict:
    """One row of `configs`: the library's own kernel choice on one benchmark shape, a short
    settle, then `launches` back-to-back launches between two HIP events on the launch stream
    (B rotated through three copies where HBM binds, so that the memory-side cache does not
    serve it), and the tolerance check of the last result on a sample of 64x64 tiles."""
    M, N, K, fill = WORKLOADS[name]
    A, B = make_inputs(orc, M, N, K, fill)
    bound = bound_of(M, N, K)
    dA = mi.DeviceBuffer.from_numpy(A)
    dBs = [mi.DeviceBuffer.from_numpy(B) for _ in range(3 if bound == "hbm" else 1)]
    dC = mi.DeviceBuffer(M * N * 2)
    cfg = mi.select_config(M, N, K)
    params = [mi.GemmParams(M, N, K, dA, dB, dC) for dB in dBs]
    t_end = time.perf_counter() + 0.1
    while time.perf_counter() < t_end:
        for i in range(8):
            mi.gpu_gemm(params[i % len(params)], config=cfg)
        mi.synchronize()
    timer = mi.GPUTimer()
    best = None
    for _ in range(2):
        timer.tick()
        for i in range(launches):
            mi.gpu_gemm(params[i % len(params)], config=cfg)
        timer.tick()
        mi.synchronize()
        ms = timer.report_last_ms() / launches
        best = ms if best is None or ms < best else best
    violations = None
    if check_tiles > 0:
        C = dC.to_numpy((M, N), np.uint16)
        tiles = orc.sample_tiles(M, N, check_tiles)
        ref = orc.reference_cpu_gemm(A, B, tiles=tiles)
        violations = orc.check_tolerance(C, ref, K, orc.max_abs(A), orc.max_abs(B), tiles=tiles)["violations"]
    for b in [dA, dC, *dBs]:
        b.free()
    tflops = 2.0 * M * N * K / (best * 1e-3) / 1e12
    gbs = 2.0 * (M * K + N * K + M * N) / (best * 1e-3) / 1e9
    row = {"workload": name, "M": M, "N": N, "K": K, "kernel_config": mi.config_name(cfg),
           "us_per_launch": best * 1e3, "launches": launches, "bound": bound, "tflops": tflops, "gbs_algorithmic": gbs}
    if bound == "mfma":
        row.update(achieved=tflops, unit="TFLOP/s", peak=PEAK_BF16_TFLOPS, frac=tflops / PEAK_BF16_TFLOPS)
    elif bound == "hbm":
        row.update(achieved=gbs, unit="GB/s", peak=PEAK_HBM_GBS, frac=gbs / PEAK_HBM_GBS)
    else:       # launch latency: no roofline fraction is claimed
        row.update(achieved=best * 1e3, unit="us", peak=None, frac=None)
    row["tolerance_violations"] = violations
    return row


def sclk_under_load(launch_batch, sync) -> float | None:
    """Shader clock in MHz as the driver's management interface reports it while the GPU runs
    this workload (the chip is power limited: the sustained clock, not the peak clock, is what
    the measured rate is made of).  None when the tool is missing or prints something else."""
    import re
    import shutil
    import subprocess
    smi = shutil.which("rocm-smi") or "/opt/rocm/bin/rocm-smi"
    if not os.path.exists(smi):
        return None
    # not under a profiler: the child process would inherit its tool library
    if _under_profiler():
        return None
    try:
        proc = subprocess.Popen([smi, "--showclocks", "--json"], stdout=subprocess.PIPE,
                                stderr=subprocess.DEVNULL, text=True)
        t_end = time.perf_counter() + 20.0
        while proc.poll() is None and time.perf_counter() < t_end:
            launch_batch()
            sync()
        if proc.poll() is None:
            proc.kill()
        out = proc.communicate()[0]
        m = re.search(r'"sclk clock speed:"\s*:\s*"\((\d+(?:\.\d+)?)Mhz\)"', out)
        return float(m.group(1)) if m else None
    except (OSError, ValueError):
        return None


def _under_profiler() -> bool:
    return any(k.startswith(("ROCPROF", "ROCP_", "ROCTRACER")) for k in os.environ)


def socket_power_under_load(launch_batch, sync, seconds: float = 0.4) -> float | None:
    """Average socket power in watts (the driver's hwmon power1_input, microwatts) sampled on
    the host while batches of the workload's launches are in flight.  None if no such file."""
    import glob
    files = glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input")
    if not files:
        return None
    samples = []
    t_end = time.perf_counter() + seconds
    try:
        while time.perf_counter() < t_end:
            launch_batch()                    # asynchronous: ~30 ms of work queued
            t_batch = time.perf_counter() + 0.02
            while time.perf_counter() < t_batch:
                with open(files[0]) as f:
                    samples.append(float(f.read()) * 1e-6)
                time.sleep(0.002)
            sync()
    except (OSError, ValueError):
        return None
    tail = samples[len(samples) // 4:]        # the first quarter: the clock is still settling
    return sum(tail) / len(tail) if tail else None


def mfma_ceiling_same_box(fill: str) -> float | None:
    """TFLOP/s of a loop of nothing but v_mfma_f32_16x16x32_bf16 (the kernel's instruction, its
    accumulator tile and operand order, no memory traffic) on operands of the workload's kind,
    run on this box right after the timed region: what the matrix pipes sustain here under
    the chip's power limit.  The harness program h100_gemm_amd/harness/mfma_ceiling does it;
    None when it is not built or under a profiler (the child would inherit its tool library)."""
    import re
    import subprocess
    exe = ROOT / "h100_gemm_amd" / "harness" / "mfma_ceiling"
    if not exe.exists() or _under_profiler():
        return None
    try:
        out = subprocess.run([str(exe), "400", "uniform" if fill == "uniform" else "normal"], capture_output=True,
                             text=True, timeout=60).stdout
    except (OSError, subprocess.SubprocessError):
        return None
    m = re.search(r"clock [\d.]+ GHz, (\d+) TFLOP/s", out)
    return float(m.group(1)) if m else None


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # The first ~100 ms of launches after an idle period run 5-40 % slower while the power
    # management settles (per-launch durations in the kernel trace fall from ~1.1 ms to
    # ~0.7 ms at 8192^3).  The default warmup covers that transient; --settle-ms keeps it
    # covered when a caller passes a small --warmup: the same launches, untimed, for at least
    # that long before the W warmup steps (reported as "settle_ms" in the JSON line).
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=150)
    ap.add_argument("--settle-ms", type=float, default=150.0,
                    help="untimed launches for at least this long before the warmup steps (0 = none)")
    ap.add_argument("--workload", default="square8192", choices=sorted(WORKLOADS))
    ap.add_argument("--config", default=None, help="kernel configuration name or index (default: library's choice)")
    ap.add_argument("--cpu-tiles", type=int, default=2048, help="64x64 tiles in the CPU baseline sample (0 = skip)")
    ap.add_argument("--check-tiles", type=int, default=64, help="64x64 tiles verified against the oracle (0 = skip)")
    ap.add_argument("--no-sclk", dest="sclk", action="store_false",
                    help="do not sample the shader clock under load after the timed region")
    ap.add_argument("--no-ceiling", dest="ceiling", action="store_false",
                    help="do not run the MFMA-only loop (same-box ceiling) and the power sampling after the timed region")
    ap.add_argument("--no-configs", dest="configs", action="store_false",
                    help="headline workload only: do not time the other seven benchmark shapes after it")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain device-to-device copy of 256 MiB (a kernel of known HBM "
                         "traffic, for scaling rocprofv3's FETCH_SIZE / WRITE_SIZE counters)")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus N with N > 1 is not supported "
              "(the GEMM shards by splitting N or M across GPUs with no exchange, each GPU running this kernel on its part)",
              file=sys.stderr)
        return 2
    if int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: launched with WORLD_SIZE > 1; one GPU only", file=sys.stderr)
        return 2

    import __graft_entry__
    __graft_entry__.ensure_built()      # uses what is built; compiles only if nothing is
    import h100_gemm_amd as mi          # raises if libmi_gemm.so is missing
    from oracle import oracle as orc    # checker + CPU baseline only

    M, N, K, fill = WORKLOADS[a.workload]
    props = mi.device_props()
    A, B = make_inputs(orc, M, N, K, fill)
    flops = 2.0 * M * N * K
    algo_bytes = 2.0 * (M * K + N * K + M * N)
    bound = bound_of(M, N, K)
    hbm_bound = bound == "hbm"
    dA = mi.DeviceBuffer.from_numpy(A)
    # HBM-bound shapes: B (128 MiB) would otherwise be served by the 256 MB memory-side
    # cache on every launch after the first; rotate three copies so each launch reads HBM.
    dBs = [mi.DeviceBuffer.from_numpy(B) for _ in range(3 if hbm_bound else 1)]
    dC = mi.DeviceBuffer(M * N * 2)
    if a.config is None:
        cfg = mi.select_config(M, N, K)
    else:
        cfg = int(a.config) if a.config.lstrip("-").isdigit() else mi.find_config(a.config)
        if not 0 <= cfg < mi.num_configs():
            print(f"bench.py: unknown kernel config {a.config!r}", file=sys.stderr)
            return 2
    params = [mi.GemmParams(M, N, K, dA, dB, dC) for dB in dBs]

    if a.calibrate_copy:
        nbytes = 256 << 20
        src, dst = mi.DeviceBuffer(nbytes), mi.DeviceBuffer(nbytes)
        src.fill_bytes(1)
        mi._lib.check(mi._lib.load().mi_memcpy_d2d(dst.ptr, src.ptr, nbytes))
        mi.synchronize()
        src.free()
        dst.free()
    if a.settle_ms > 0:
        t_end = time.perf_counter() + a.settle_ms * 1e-3
        while time.perf_counter() < t_end:
            for i in range(8):
                mi.gpu_gemm(params[i % len(params)], config=cfg)
            mi.synchronize()
    for i in range(a.warmup):
        mi.gpu_gemm(params[i % len(params)], config=cfg)
    mi.synchronize()
    timer = mi.GPUTimer()                 # HIP events on the launch stream (null stream)
    t_host0 = time.perf_counter()
    timer.tick()
    for i in range(a.steps):
        mi.gpu_gemm(params[i % len(params)], config=cfg)
    timer.tick()
    mi.synchronize()
    t_host = time.perf_counter() - t_host0
    ms_total = timer.report_last_ms()
    ms_per_step = ms_total / a.steps

    def launch_batch():      # ~30 ms of the same launches, outside the timed region
        for i in range(max(1, int(30.0 / ms_per_step))):
            mi.gpu_gemm(params[i % len(params)], config=cfg)
    sclk = sclk_under_load(launch_batch, mi.synchronize) if a.sclk else None
    watts = socket_power_under_load(launch_batch, mi.synchronize) if a.ceiling else None

    # correctness of what was just timed, on a sample of tiles
    violations = None
    if a.check_tiles > 0:
        C = dC.to_numpy((M, N), np.uint16)
        tiles = orc.sample_tiles(M, N, a.check_tiles)
        ref = orc.reference_cpu_gemm(A, B, tiles=tiles)
        rep = orc.check_tolerance(C, ref, K, orc.max_abs(A), orc.max_abs(B), tiles=tiles)
        violations = rep["violations"]

    tflops = flops / (ms_per_step * 1e-3) / 1e12
    gbs = algo_bytes / (ms_per_step * 1e-3) / 1e9
    if bound == "mfma":
        roof = {"bound": "mfma", "achieved": tflops, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                "frac": tflops / PEAK_BF16_TFLOPS}
    elif bound == "hbm":
        roof = {"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": gbs / PEAK_HBM_GBS}
    else:       # 512^3: launch and pipeline latency; neither roofline says anything about it
        roof = {"bound": "launch", "achieved": ms_per_step * 1e3, "peak": None, "unit": "us", "frac": None}
    if bound == "mfma" and a.ceiling:
        # the same-box yardstick: a slow box (they differ by +-6 % in the clock they sustain) moves
        # `achieved` and `ceiling_same_box` together, a kernel change moves only the first
        ceiling = mfma_ceiling_same_box(fill)
        roof["ceiling_same_box"] = ceiling
        roof["frac_of_ceiling"] = tflops / ceiling if ceiling else None
    roof["kernel"] = mi.config_name(cfg)
    traffic_kernel, traffic = MEASURED_TRAFFIC_BYTES.get(a.workload, (None, None))
    roof["traffic"] = traffic if traffic_kernel == roof["kernel"] else None
    roof["avg_launch_us"] = ms_per_step * 1e3

    cpu = cpu_baseline(orc, A, B, a.cpu_tiles) if a.cpu_tiles > 0 else None

    # the other benchmark shapes, with the library's own kernel choice, in the same run (not
    # under a profiler, where the run is about one kernel)
    configs = None
    if a.configs and a.workload == "square8192" and a.config is None and not _under_profiler():
        for b in [dA, dC, *dBs]:
            b.free()
        configs = []
        for name in BASELINE_WORKLOADS:
            if name == a.workload:
                row = {"workload": name, "M": M, "N": N, "K": K, "kernel_config": mi.config_name(cfg),
                       "us_per_launch": ms_per_step * 1e3, "launches": a.steps, "bound": bound, "tflops": tflops,
                       "gbs_algorithmic": gbs, "achieved": roof["achieved"], "unit": roof["unit"], "peak": roof["peak"],
                       "frac": roof["frac"], "tolerance_violations": violations}
            else:
                # about 30 ms of launches per timed batch, 20 to 200 of them (estimated at half the peak rate)
                Mw, Nw, Kw, _ = WORKLOADS[name]
                est_us = max(2.0 * Mw * Nw * Kw / 1.25e15, 2.0 * (Mw * Kw + Nw * Kw + Mw * Nw) / 4e12) * 1e6
                launches = int(min(200, max(20, 30000.0 / est_us)))
                row = time_workload(mi, orc, name, launches, min(a.check_tiles, 64 if est_us < 200 else 16))
            configs.append(row)

    out = {
        # the headline metric is quoted on square8192; the other workloads are labelled as what they are
        "metric": ("bf16 GEMM TFLOP/s at M=N=K=8192 on 1 MI355X; % of bf16 MFMA peak" if a.workload == "square8192"
                   else f"bf16 GEMM TFLOP/s at M={M} N={N} K={K} on 1 MI355X"),
        "value": tflops, "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "settle_ms": a.settle_ms, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic" + (", 3 rotating copies of B" if hbm_bound else ""),
        "config": {"workload": f"{a.workload}: M={M} N={N} K={K}, A,B {fill} seeded bf16, fp32 accumulate, bf16 out",
                   "kernel_config": mi.config_name(cfg), "device": props["name"] or props["arch"],
                   "compute_units": props["compute_units"], "peak_clock_mhz": props["clock_khz"] / 1000,
                   "sclk_mhz_under_load": sclk, "socket_power_w_under_load": watts,
                   "joules_per_launch": watts * ms_per_step * 1e-3 if watts else None},
        "pct_of_bf16_mfma_peak": 100.0 * tflops / PEAK_BF16_TFLOPS,
        "achieved_gbs_algorithmic": gbs,
        "tolerance_violations": violations,
        "host_wall_ms_per_step": t_host * 1e3 / a.steps,
        "roofline": roof,
        "cpu_baseline": cpu,
    }
    if configs is not None:
        out["configs"] = configs
    print(json.dumps(out))
    bad = bool(violations) or any(r["tolerance_violations"] for r in (configs or []))
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main())
