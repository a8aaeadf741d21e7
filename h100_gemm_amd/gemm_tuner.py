"""Grid-search tuner for the MI355X GEMM kernels.

The counterpart of the reference's ``gemm_tuner.py`` (gemm_tuner.py:11-181), with the same
class, methods, control flow, failure handling and output files, retargeted from Hopper to
CDNA4:

* the search space is MFMA macro tile, wave layout, pipeline kind and LDS stage count (of the
  rings of the decode and small-tile kernels, where the depth is a free parameter), tile-order
  group, occupancy and drain slot instead of cluster shape / block / TMA stages
  (gemm_tuner.py:17-24);
* a configuration is rendered from ``template/matmul_mi355x.hip.jinja``, compiled with
  ``hipcc --offload-arch=gfx950`` (nvcc -arch=sm_90a there, gemm_tuner.py:46) and run as
  ``./test M 5120 N 5120 K 4096`` with a 30 s limit (gemm_tuner.py:55);
* the runtime is parsed from ``Average latency (ms) is X`` (gemm_tuner.py:63); compile
  failure, non-zero exit (the program aborts when its result is wrong), unparsable output
  and timeout each score ``inf`` and the sweep goes on (gemm_tuner.py:49-72);
* after every configuration it rewrites ``tuning_results_<timestamp>.json``
  (``{results:[{params,runtime,success,timestamp}],best_params,best_runtime,timestamp}``)
  and ``tuning_summary.txt``, and keeps the source of the best configuration so far in
  ``best_matmul_mi355x.hip`` (gemm_tuner.py:117-164).

Additions: ``prebuild()`` compiles every valid configuration in parallel into
``<output_dir>/bin`` (hipcc cross-compiles without a GPU, so the slow part can run on a
build host), ``tune(prebuilt=True)`` then only runs the binaries; ``resume_from`` reloads an
earlier results JSON and skips what it already holds; ``--write-tuned FILE MxNxK ...``
(``tune_library_choice``) times the library's compiled candidates for given shapes and writes
the winners in the format ``MI_GEMM_TUNED_FILE`` reads.
"""
from __future__ import annotations

import itertools
import json
import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from datetime import datetime
from pathlib import Path
from typing import Dict, List, Optional, Tuple

from jinja2 import Template

PKG = Path(__file__).resolve().parent
if __package__ in (None, ""):
    sys.path.insert(0, str(PKG.parent))
    from h100_gemm_amd import kernel_configs as kc      # noqa: E402
else:
    from . import kernel_configs as kc

DEFAULT_TEMPLATE = PKG / "template" / "matmul_mi355x.hip.jinja"
LATENCY_RE = re.compile(r"Average latency \(ms\) is ([\d.]+(?:e[-+]?\d+)?)")


def default_compile_command(src: str, exe: str) -> List[str]:
    return [os.environ.get("HIPCC", "/opt/rocm/bin/hipcc"), "--offload-arch=gfx950", "-O3", "-std=c++17",
            "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
            "-Wno-unused-command-line-argument", "-pthread", f"-I{PKG / 'csrc'}", f"-I{PKG / 'harness'}",
            src, "-o", exe, f"-L{PKG / 'lib'}", "-lmi_gemm", f"-Wl,-rpath,{PKG / 'lib'}"]


class GemmTuner:
    def __init__(self, template_file: str = str(DEFAULT_TEMPLATE), output_dir: str = "tuning_results",
                 work_dir: Optional[str] = None, compile_command=default_compile_command,
                 bench_args=("M", "5120", "N", "5120", "K", "4096"), timeout: float = 30.0,
                 resume_from: Optional[str] = None, bin_dir: Optional[str] = None,
                 only: Optional[List[Dict[str, int]]] = None):
        self.output_dir = Path(output_dir)
        self.output_dir.mkdir(parents=True, exist_ok=True)
        self.work_dir = Path(work_dir) if work_dir else self.output_dir
        self.work_dir.mkdir(parents=True, exist_ok=True)
        self.compile_command = compile_command
        self.bench_args = list(bench_args)
        self.timeout = timeout
        # where prebuild() puts the programs and tune(prebuilt=True) looks for them
        self.bin_dir = Path(bin_dir) if bin_dir else self.output_dir / 'bin'
        # an explicit list of configurations instead of the grid below
        self.only = only

        # Define parameter search space: MFMA macro tile, wave layout and LDS stage count (what the
        # reference sweeps as BLOCKM and STAGES, gemm_tuner.py:17-24), plus tile-order group,
        # occupancy and the drain slot of the 16x16x32 kernel.  NS is a real parameter where the
        # LDS ring's depth is one: the decode kinds and the small-tile kind (is_valid_configuration
        # keeps one copy of every configuration it means nothing for, and the ring kinds of the
        # tiled kernels exist with four stages only).
        self.param_space = {
            'KIND': ['mfma16', 'ring', 'ring16', 'tile', 'stream', 'decode', 'wavek'],
            'BM': [16, 32, 64, 96, 128, 192, 256],
            'BN': [32, 64, 96, 128, 192, 256],
            'WM': [2, 4],
            'WN': [2, 4],
            'NS': [4, 1, 2, 3, 5],
            'GROUP': [4, 8],
            'DRAIN': [0, 1, 3],
            'OCC': [1, 2],
            'SHARED': [0, 1],
        }

        # Load template
        with open(template_file, 'r') as f:
            self.template = Template(f.read())

        self.previous: Dict[str, dict] = {}
        if resume_from:
            with open(resume_from, 'r') as f:
                for r in json.load(f).get('results', []):
                    self.previous[self.config_key(r['params'])] = r

    @staticmethod
    def config_key(params: Dict[str, int]) -> str:
        return json.dumps(params, sort_keys=True)

    @staticmethod
    def config_name(params: Dict[str, int]) -> str:
        c = dict({'OCC': 1, 'SWZ': 1, 'DTL': 1, 'EPI': 1}, **params)
        if c['KIND'] == 'stream':
            c['BN'] = 32
        return kc.config_name(c)

    def generate_code(self, params: Dict[str, int]) -> str:
        """Generate code with given parameters"""
        return self.template.render(name=self.config_name(params), **params)

    def _run(self, exe: Path, params) -> Tuple[float, bool]:
        try:
            result = subprocess.run([str(Path(exe).resolve())] + self.bench_args, capture_output=True, text=True,
                                    timeout=self.timeout, cwd=str(self.work_dir))
            if result.returncode != 0:
                print(f"Runtime error for parameters: {params}")
                return float('inf'), False
            # Extract runtime from output
            match = LATENCY_RE.search(result.stdout)
            if match:
                return float(match.group(1)), True
            print(f"Could not parse output for parameters: {params}")
            return float('inf'), False
        except subprocess.TimeoutExpired:
            print(f"Timeout for parameters: {params}")
            return float('inf'), False

    def benchmark_configuration(self, params: Dict[str, int], prebuilt: bool = False) -> Tuple[float, bool]:
        """Benchmark a single configuration. Returns (runtime, success)"""
        if prebuilt:
            exe = self.bin_dir / self.config_name(params)
            if not exe.exists():
                print(f"Compilation failed for parameters: {params}")
                return float('inf'), False
            return self._run(exe, params)

        # Write the generated code to temp.hip
        src = self.work_dir / 'temp.hip'
        with open(src, 'w') as f:
            f.write(self.generate_code(params))

        # If test file exists, remove it
        test_file = self.work_dir / 'test'
        if test_file.exists():
            test_file.unlink()

        # Compile the code
        compile_result = subprocess.run(self.compile_command(str(src), str(test_file)),
                                        stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
        if compile_result.returncode != 0 or not test_file.exists():
            print(f"Compilation failed for parameters: {params}")
            return float('inf'), False

        # Run the benchmark
        return self._run(test_file, params)

    # parameters that mean nothing for a kind: only their first value in the space is kept
    UNUSED = {'tile': ('NS', 'DRAIN', 'SHARED'), 'mfma16': ('NS', 'SHARED'), 'ring': ('DRAIN', 'OCC', 'SHARED'),
              'ring16': ('DRAIN', 'OCC', 'SHARED'), 'stream': ('BN', 'WM', 'WN', 'GROUP', 'DRAIN', 'OCC', 'SHARED'),
              'decode': ('WM', 'WN', 'GROUP', 'DRAIN', 'OCC', 'SHARED'), 'wavek': ('WM', 'WN', 'GROUP', 'DRAIN', 'OCC')}

    def is_valid_configuration(self, params: Dict[str, int]) -> bool:
        """Check if a parameter configuration is valid"""
        c = dict({'OCC': 1, 'SWZ': 1, 'DTL': 1, 'EPI': 1}, **params)
        for key in self.UNUSED.get(c['KIND'], ()):
            if key in params and key in self.param_space and params[key] != self.param_space[key][0]:
                return False        # one copy of the configuration, not one per value of a parameter it ignores
        if c['KIND'] == 'stream':
            c['BN'] = 32            # the single-pass decode kernel owns 32 columns per workgroup
        if c['KIND'] == 'wavek' and not c.get('SHARED'):
            c.pop('SHARED', None)
        try:
            return kc.is_valid_config(c)
        except KeyError:
            return False

    def configurations(self) -> List[Dict[str, int]]:
        if self.only is not None:
            return [p for p in self.only if self.is_valid_configuration(p)]
        combos = [dict(zip(self.param_space.keys(), values))
                  for values in itertools.product(*self.param_space.values())]
        return [p for p in combos if self.is_valid_configuration(p)]

    def prebuild(self, jobs: int = 8) -> Dict[str, bool]:
        """Render and compile every valid configuration into <output_dir>/bin."""
        bindir = self.bin_dir
        srcdir = self.output_dir / 'src'
        bindir.mkdir(parents=True, exist_ok=True)
        srcdir.mkdir(parents=True, exist_ok=True)

        def one(params):
            name = self.config_name(params)
            src = srcdir / f"{name}.hip"
            src.write_text(self.generate_code(params))
            exe = bindir / name
            r = subprocess.run(self.compile_command(str(src), str(exe)), stdout=subprocess.DEVNULL,
                               stderr=subprocess.DEVNULL)
            return name, r.returncode == 0 and exe.exists()

        with ThreadPoolExecutor(max_workers=jobs) as ex:
            return dict(ex.map(one, self.configurations()))

    # ---- the sweep ----------------------------------------------------------------------

    def _measure(self, params: Dict[str, int], prebuilt: bool) -> Tuple[Optional[float], bool]:
        """(runtime in ms or None, success) of one configuration; resumed results are reused."""
        old = self.previous.get(self.config_key(params))
        if old is not None:
            print("(taken from the resumed results)")
            return (old['runtime'] if old['success'] else None), bool(old['success'])
        runtime, ok = self.benchmark_configuration(params, prebuilt=prebuilt)
        return (runtime if ok else None), ok

    def tune(self, prebuilt: bool = False):
        """Time every valid configuration; returns (best_params, best_runtime, results).

        A configuration that fails to compile, exits non-zero, prints no latency line or runs
        out of time is recorded with success = False and the sweep goes on
        (gemm_tuner.py:49-72).  After each one the results JSON and the summary are rewritten
        and, when it is the fastest so far, its rendered source is kept as
        best_matmul_mi355x.hip (gemm_tuner.py:117-133)."""
        todo = self.configurations()
        results: List[Dict] = []
        best: Tuple[float, Optional[Dict[str, int]]] = (float('inf'), None)
        for n, params in enumerate(todo, 1):
            print(f"\nTesting configuration {n}/{len(todo)}:")
            print(params)
            runtime, ok = self._measure(params, prebuilt)
            results.append({'params': params, 'runtime': runtime, 'success': ok,
                            'timestamp': datetime.now().isoformat()})
            if ok:
                print(f"Runtime: {runtime:.4f} ms")
                if runtime < best[0]:
                    best = (runtime, params)
                    print(f"New best runtime: {runtime:.4f} ms")
                    (self.output_dir / 'best_matmul_mi355x.hip').write_text(self.generate_code(params))
            self.save_results(results, best[1], best[0])
        return best[1], best[0], results

    def save_results(self, results: List[Dict], best_params: Optional[Dict[str, int]], best_runtime: float):
        """tuning_results_<timestamp>.json and tuning_summary.txt in the reference's formats
        (gemm_tuner.py:135-164): the JSON holds every result, the summary the best
        configuration followed by all successful ones, fastest first."""
        stamp = datetime.now().strftime('%Y%m%d_%H%M%S')
        doc = {'results': results, 'best_params': best_params, 'best_runtime': best_runtime, 'timestamp': stamp}
        (self.output_dir / f'tuning_results_{stamp}.json').write_text(json.dumps(doc, indent=2))

        def block(params):
            return [f"{k}: {v}" for k, v in params.items()]

        lines = [f"Tuning completed at: {stamp}", f"Best runtime: {best_runtime:.4f} ms"]
        if best_params:
            lines += ["Best parameters:"] + block(best_params)
        lines += ["", "All successful configurations:"]
        for r in sorted((r for r in results if r['success']), key=lambda r: r['runtime']):
            lines += ["", f"Runtime: {r['runtime']:.4f} ms"] + block(r['params'])
        (self.output_dir / 'tuning_summary.txt').write_text("\n".join(lines) + "\n")


def tune_library_choice(shapes, out_file: Optional[str] = None, margin: float = 0.02, all_times: bool = False):
    """The run-time form of the tuner's persisted results: for every (M, N, K) time the
    library's automatic choice and each compiled candidate of its time model on the GPU
    (through the C ABI, best of three batches of ~30 ms of back-to-back launches) and, where a candidate
    beats the automatic choice by more than `margin`, append `M N K config-name` to
    `out_file` -- the format MI_GEMM_TUNED_FILE reads (keyed on all of M, N, K, where the
    reference keys its cached descriptors on M alone, matmul_utils.cuh:49-51).
    Returns [(shape, automatic config, its ms, best config, its ms)]."""
    import numpy as np

    import h100_gemm_amd as mi
    lib = mi._lib.load()
    cands = [i for i, c in enumerate(kc.CONFIGS) if c.get("EFF") or c["KIND"] in ("stream", "decode", "wavek")]

    def time_config(config, params, launches):
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

    rng = np.random.default_rng(1)
    block = rng.integers(0x3000, 0x3F80, size=1 << 22, dtype=np.uint16) | (rng.integers(0, 2, size=1 << 22, dtype=np.uint16) << 15)
    out = []
    for M, N, K in shapes:
        A, B = np.resize(block, (M, K)), np.resize(block[::-1], (N, K))
        # decode shapes stream their weights from HBM in real use: enough copies of B to exceed
        # the 256 MB memory-side cache, visited in turn
        copies = min(8, -(-(600 << 20) // B.nbytes)) if M <= int(os.environ.get('MI_TUNER_ROTATE_B_UP_TO_M', '128')) else 1
        dA, dC = mi.DeviceBuffer.from_numpy(A), mi.DeviceBuffer(M * N * 2)
        dBs = [mi.DeviceBuffer.from_numpy(B) for _ in range(copies)]
        params = [mi.GemmParams(M, N, K, dA, dB, dC) for dB in dBs]
        launches = int(min(200, max(10, 3e-2 / (2.0 * M * N * K / 1.2e15 + 5e-6))))
        auto = mi.select_config(M, N, K)
        t_auto = time_config(mi.MI_CONFIG_AUTO, params, launches)
        times = {c: time_config(c, params, launches) for c in cands if lib.mi_gemm_config_supports(c, 0, M, N, K)}
        t_auto = min(t_auto, time_config(mi.MI_CONFIG_AUTO, params, launches))
        best = min(times, key=times.get)
        print(f"{M}x{N}x{K}: automatic choice {mi.config_name(auto)} {t_auto * 1e3:.1f} us, "
              f"best candidate {mi.config_name(best)} {times[best] * 1e3:.1f} us", flush=True)
        if all_times:
            print("    " + " ".join(f"{mi.config_name(c)}={t * 1e3:.1f}" for c, t in sorted(times.items(), key=lambda ct: ct[1])), flush=True)
        if out_file and t_auto > times[best] * (1.0 + margin):
            with open(out_file, "a") as f:
                f.write(f"{M} {N} {K} {mi.config_name(best)}\n")
        out.append(((M, N, K), mi.config_name(auto), t_auto, mi.config_name(best), times[best]))
        for b in [dA, dC] + dBs:
            b.free()
    if out:
        losses = [max(0.0, t_auto / t_best - 1.0) for _, _, t_auto, _, t_best in out]
        print(f"{len(out)} shapes: the automatic choice loses {100 * sum(losses) / len(losses):.2f} % on average to the "
              f"best candidate, more than 4 % on {sum(l > 0.04 for l in losses)}, at worst {100 * max(losses):.0f} %")
    return out


def main(argv=None):
    import argparse
    ap = argparse.ArgumentParser(description="MI355X GEMM tuner")
    ap.add_argument("--output-dir", default="tuning_results")
    ap.add_argument("--prebuild", action="store_true", help="only render + compile every configuration")
    ap.add_argument("--prebuilt", action="store_true", help="run the binaries a --prebuild left in <output-dir>/bin")
    ap.add_argument("--resume", default=None, help="results JSON of an earlier run to continue from")
    ap.add_argument("--shape", nargs=3, type=int, default=[5120, 5120, 4096], metavar=("M", "N", "K"))
    ap.add_argument("--fill", default=None, choices=["int", "uniform", "normal"])
    ap.add_argument("--iters", type=int, default=None, help="timed launches per configuration (default: the program's 200)")
    ap.add_argument("--no-check", action="store_true",
                    help="skip each program's comparison with the on-device golden (large shapes: the golden "
                         "kernel takes longer than the sweep)")
    ap.add_argument("--kinds", default=None,
                    help="comma-separated kernel kinds to keep of the grid, e.g. stream,decode,wavek (default: all)")
    ap.add_argument("--bin-dir", default=None, help="where --prebuild puts and --prebuilt finds the programs "
                                                    "(default: <output-dir>/bin)")
    ap.add_argument("-j", "--jobs", type=int, default=8)
    ap.add_argument("--write-tuned", metavar="FILE", default=None,
                    help="instead of sweeping the template: time the library's compiled candidates for the shapes "
                         "given as MxNxK arguments and append `M N K config-name` lines (MI_GEMM_TUNED_FILE format) "
                         "where one beats the automatic choice")
    ap.add_argument("--all-times", action="store_true", help="with --write-tuned: print every candidate's time")
    ap.add_argument("shapes", nargs="*", help="shapes as MxNxK (with --write-tuned)")
    a = ap.parse_args(argv)
    if a.write_tuned:
        tune_library_choice([tuple(int(v) for v in s.split("x")) for s in a.shapes], a.write_tuned, all_times=a.all_times)
        return 0
    bench_args = ["M", str(a.shape[0]), "N", str(a.shape[1]), "K", str(a.shape[2])]
    if a.fill:
        bench_args += ["fill", a.fill]
    if a.iters:
        bench_args += ["iters", str(a.iters)]
    if a.no_check:
        bench_args += ["check", "0"]
    tuner = GemmTuner(str(DEFAULT_TEMPLATE), a.output_dir, bench_args=bench_args, resume_from=a.resume,
                      bin_dir=a.bin_dir)
    if a.kinds:
        kinds = a.kinds.split(",")
        unknown = sorted(set(kinds) - set(tuner.param_space['KIND']))
        if unknown:
            ap.error(f"unknown kind(s) {unknown}; the grid has {tuner.param_space['KIND']}")
        tuner.param_space['KIND'] = [k for k in tuner.param_space['KIND'] if k in kinds]
    if a.prebuild:
        built = tuner.prebuild(a.jobs)
        print(f"compiled {sum(built.values())} of {len(built)} configurations into {tuner.bin_dir}")
        return 0 if all(built.values()) else 1
    best_params, best_runtime, results = tuner.tune(prebuilt=a.prebuilt)

    if best_params:
        print("\nTuning completed!")
        print(f"Best runtime: {best_runtime:.4f} ms")
        print("Best parameters:")
        for key, value in best_params.items():
            print(f"{key}: {value}")
        print(f"\nResults saved in {a.output_dir} directory")
    else:
        print("\nNo valid configuration found!")
    return 0


if __name__ == "__main__":
    sys.exit(main())
