"""Check the automatic kernel choice against the candidates it chooses from.

For a seeded set of random shapes this times ``MI_CONFIG_AUTO`` and every candidate tile of
the time model (each at the number of K pieces the model gives it) on the GPU and reports
the shapes where a candidate beats the automatic choice by more than 4 %, the mean loss
against the best candidate and every candidate's time.  A tuning aid for the constants in
``template/kernel_table.hpp.jinja``; the counterpart of the reference's tuner runs
(``gemm_tuner.py:82-133``) for the choice between compiled kernels instead of between
template parameters.

    python -m h100_gemm_amd.selection_check [--seed S] [--cases N] [--mode general|shortk|midm|decode]
                                            [--write-tuned FILE] [MxNxK ...]
"""
from __future__ import annotations

import argparse
import sys

import numpy as np

import h100_gemm_amd as mi
from h100_gemm_amd import kernel_configs as kc


def candidates(decode: bool = False) -> list[int]:
    """indices of the configurations the time model chooses from (those with a measured EFF);
    with `decode` also the decode kernels of the ladder in front of the model"""
    return [i for i, c in enumerate(kc.CONFIGS) if c.get("EFF") or (decode and c["KIND"] in ("stream", "decode"))]


def random_shape(rng: np.random.Generator, it: int, mode: str) -> tuple[int, int, int]:
    kind = it % 3
    if kind == 0:      # multiples of the tile sizes
        M, N, K = 256 * rng.integers(1, 33), 256 * rng.integers(1, 33), 128 * rng.integers(2, 65)
    elif kind == 1:    # arbitrary
        M, N, K = rng.integers(200, 8000), rng.integers(200, 8000), rng.integers(200, 8000)
    else:              # multiples of 64 / 8
        M, N, K = 64 * rng.integers(2, 120), 64 * rng.integers(2, 120), 8 * rng.integers(32, 1000)
    if mode == "shortk":
        K = rng.choice([128 * rng.integers(1, 13), rng.integers(64, 1600), 64 * rng.integers(1, 24)])
    elif mode == "decode":
        M = rng.choice([rng.integers(1, 33), rng.integers(33, 129), 16 * rng.integers(1, 9)])
        N = rng.choice([256 * rng.integers(1, 33), 4 * rng.integers(64, 2048), 1024 * rng.integers(1, 29)])
        K = rng.choice([64 * rng.integers(8, 257), 1024 * rng.integers(1, 29)])
    elif mode == "midm":
        M = rng.choice([rng.integers(129, 1500), 64 * rng.integers(3, 24)])
        N = rng.choice([256 * rng.integers(4, 33), rng.integers(1024, 8192)])
        K = rng.choice([128 * rng.integers(8, 65), rng.integers(1024, 8192)])
        if rng.random() < 0.3:
            M, N = N, M
    M, N, K = int(M), int(N), int(K)
    if M * N * K > 4e11:
        K = max(128, int(4e11 / (M * N)) // 128 * 128)
    return M, N, K


def bf16_pattern(shape, seed: int) -> np.ndarray:
    """bf16 bit patterns with random sign and mantissa and magnitudes below 1 (4M distinct
    values, repeated): the values do not matter for a timing comparison, the switching
    activity of random operands does"""
    rng = np.random.default_rng(seed)
    block = rng.integers(0x3000, 0x3F80, size=1 << 22, dtype=np.uint16) | (rng.integers(0, 2, size=1 << 22, dtype=np.uint16) << 15)
    return np.resize(block, shape)


def time_config(config: int, params: list, launches: int) -> float:
    """best of three batches of back-to-back launches, milliseconds per launch; `params` holds
    one GemmParams per copy of B and the launches go round them"""
    for i in range(max(3, launches // 4)):
        mi.gpu_gemm(params[i % len(params)], config=config)
    mi.synchronize()
    best = float("inf")
    for _ in range(3):
        timer = mi.GPUTimer()
        timer.tick()
        for i in range(launches):
            mi.gpu_gemm(params[i % len(params)], config=config)
        timer.tick()
        best = min(best, timer.report_last_ms() / launches)
    return best


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--cases", type=int, default=30, help="random shapes (0: only the shapes given)")
    ap.add_argument("--mode", default="general", choices=["general", "shortk", "midm", "decode"])
    ap.add_argument("--write-tuned", metavar="FILE", default=None,
                    help="append `M N K config-name` for every shape where a candidate beats the automatic "
                         "choice by more than 2 %% (the format MI_GEMM_TUNED_FILE reads)")
    ap.add_argument("shapes", nargs="*", help="further shapes as MxNxK")
    a = ap.parse_args(argv)
    rng = np.random.default_rng(a.seed)
    shapes = [random_shape(rng, it, a.mode) for it in range(a.cases)]
    shapes += [tuple(int(v) for v in s.split("x")) for s in a.shapes]
    lib = mi._lib.load()
    cands = candidates(decode=a.mode == "decode")
    losses = []
    for M, N, K in shapes:
        A, B = bf16_pattern((M, K), 1), bf16_pattern((N, K), 2)
        # decode shapes stream B from HBM in their real use (many layers of weights): enough
        # copies of B to exceed the 256 MB memory-side cache, visited in turn
        copies = min(8, -(-(600 << 20) // B.nbytes)) if M <= 128 else 1
        dA, dC = mi.DeviceBuffer.from_numpy(A), mi.DeviceBuffer(M * N * 2)
        dBs = [mi.DeviceBuffer.from_numpy(B) for _ in range(copies)]
        params = [mi.GemmParams(M, N, K, dA, dB, dC) for dB in dBs]
        flops = 2.0 * M * N * K
        launches = int(min(200, max(10, 3e-2 / (flops / 1.2e15 + 5e-6))))     # ~30 ms per batch
        auto = mi.select_config(M, N, K)
        t_auto = time_config(mi.MI_CONFIG_AUTO, params, launches)
        times = {c: time_config(c, params, launches) for c in cands if lib.mi_gemm_config_supports(c, 0, M, N, K)}
        t_auto = min(t_auto, time_config(mi.MI_CONFIG_AUTO, params, launches))
        best = min(times, key=times.get)
        loss = max(0.0, t_auto / times[best] - 1.0)
        losses.append(loss)
        every = " ".join(f"{mi.config_name(c).split('_')[0]}={times[c] * 1e3:.0f}" for c in times)
        flag = f"  <-- auto loses {100 * loss:.0f} % to {mi.config_name(best)}" if loss > 0.04 else ""
        print(f"{M}x{N}x{K}: auto {mi.config_name(auto)} {t_auto * 1e3:.1f} us {flops / t_auto / 1e9:.0f} TFLOP/s; "
              f"best candidate {mi.config_name(best)} {times[best] * 1e3:.1f} us [{every}]{flag}", flush=True)
        if a.write_tuned and loss > 0.02:
            with open(a.write_tuned, "a") as f:
                f.write(f"{M} {N} {K} {mi.config_name(best)}\n")
        for b in [dA, dC] + dBs:
            b.free()
    if losses:
        print(f"{len(losses)} shapes: mean loss against the best candidate {100 * float(np.mean(losses)):.2f} %, "
              f"{sum(l > 0.04 for l in losses)} above 4 %, worst {100 * max(losses):.0f} %")
    return 0


if __name__ == "__main__":
    sys.exit(main())
