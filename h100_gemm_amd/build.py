"""Build libmi_gemm.so: render one HIP translation unit per kernel configuration from the
Jinja templates, compile them for gfx950 in parallel with hipcc, link the C ABI.

    python -m h100_gemm_amd.build [-j JOBS] [--force]

Takes the place of the reference's `nvcc -arch=sm_90a ... -o test` line (Makefile:1-5 and
gemm_tuner.py:46 in the reference tree).  Nothing here needs a GPU.
"""
from __future__ import annotations

import argparse
import hashlib
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

from jinja2 import Template

from . import isa_check
from . import kernel_configs as kc

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
GEN = CSRC / "gen"
LIB = PKG / "lib" / "libmi_gemm.so"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -packed-fp32-ops off: packed fp32 VALU forms are not to be generated on this hardware pool.
HIPFLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature",
            "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
            f"-I{CSRC}", f"-I{GEN}"]


def _write_if_changed(path: Path, text: str) -> None:
    if not path.exists() or path.read_text() != text:
        path.write_text(text)


def _decode_indices(named) -> dict:
    """role -> config index (or None) of the kernels the automatic choice for decode shapes names."""
    names = [c["name"] for c in named]
    return {role: (names.index(n) if n in names else None) for role, n in kc.DECODE_KERNELS.items()}


def render_sources(configs=None) -> list[Path]:
    """Render the per-config units and the kernel table; returns the units' paths."""
    configs = kc.CONFIGS if configs is None else configs
    GEN.mkdir(parents=True, exist_ok=True)
    unit_t = Template((PKG / "template" / "kernel_unit.hip.jinja").read_text())
    table_t = Template((PKG / "template" / "kernel_table.hpp.jinja").read_text())
    named = [dict(c, name=kc.config_name(c), threads=kc.threads(c), lds=kc.lds_bytes(c)) for c in configs]
    units = []
    for c in named:
        p = GEN / f"unit_{c['name']}.hip"
        _write_if_changed(p, unit_t.render(**c))
        units.append(p)
    _write_if_changed(GEN / "kernel_table.hpp",
                      table_t.render(configs=named,
                                     tuned=[(m, n, k, [c["name"] for c in named].index(nm))
                                            for (m, n, k), nm in sorted(getattr(kc, "TUNED_SHAPES", {}).items())
                                            if nm in [c["name"] for c in named]],
                                     decode_idx=_decode_indices(named)))
    # drop units of configs that no longer exist
    keep = {p.name for p in units}
    for old in GEN.glob("unit_*.hip"):
        if old.name not in keep:
            old.unlink()
            for left in GEN.glob(old.stem + ".*"):          # object, stamp
                left.unlink()
            for left in GEN.glob(old.stem + "-hip-*"):      # kept assembly text
                left.unlink()
    return units


def _stamp(src: Path) -> str:
    h = hashlib.sha1()
    # every header of csrc/ (a unit includes a few of them; rebuilding all on any change is cheap)
    for dep in [src, *sorted(CSRC.glob("*.hpp")), GEN / "kernel_table.hpp",
                PKG.parent / "include" / "mi_gemm.h", PKG / "isa_check.py"]:
        h.update(dep.read_bytes())
    h.update(" ".join(HIPFLAGS).encode())
    return h.hexdigest()


def _asm_path(obj: Path) -> Path:
    """where `-save-temps=obj` leaves the device assembly text of a unit"""
    return obj.with_name(obj.stem + "-hip-amdgcn-amd-amdhsa-gfx950.s")


def _check_unit(src: Path, obj: Path) -> None:
    """The invariants of the generated code that the inline asm relies on (isa_check): a unit
    that breaks one fails the build."""
    asm = _asm_path(obj)
    if not asm.exists():
        raise RuntimeError(f"{src.name}: no assembly text at {asm} (needed for the M0 / scratch checks)")
    text = asm.read_text()
    cfg = next((c for c in kc.CONFIGS if src.name == f"unit_{kc.config_name(c)}.hip"), None)
    if cfg is None:
        return                                  # not a kernel unit
    # {bf16, fp16} x {aligned, predicated} x {plain, trace} for the 16x16x32 kernel (and as many again
    # with K cut over workgroups, where the config does not split K over groups of its waves)
    isa_check.check_m0(src.name, text, need_kernels=8 if cfg["KIND"] == "mfma16" else 1)
    if cfg["KIND"] == "mfma16" and cfg.get("EFF"):
        isa_check.check_no_scratch(src.name, text)
    isa_check.check_lds_bytes(src.name, text, kc.lds_bytes(cfg))
    # registers with an asm-issued load in flight are left alone (the decode kernels' ring of A fragments)
    n = isa_check.check_inflight(src.name, text)
    if cfg["KIND"] == "decode" and n == 0:
        raise RuntimeError(f"{src.name}: the decode kernel's asm loads into registers were not found in the assembly text")


def _compile(src: Path, force: bool) -> Path:
    obj = src.with_suffix(".o") if src.parent == GEN else GEN / (src.stem + ".o")
    stamp = obj.with_suffix(".stamp")
    want = _stamp(src)
    if not force and obj.exists() and stamp.exists() and stamp.read_text() == want:
        return obj
    cmd = [HIPCC, *HIPFLAGS, "-save-temps=obj", "-c", str(src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{r.stderr[-4000:]}")
    # of the intermediate files only the device assembly text is kept
    for tmp in list(obj.parent.glob(obj.stem + "-*")) + list(obj.parent.glob(src.name + "-*")):
        if tmp != _asm_path(obj):
            tmp.unlink()
    _check_unit(src, obj)
    stamp.write_text(want)
    return obj


def build(jobs: int | None = None, force: bool = False, verbose: bool = True) -> Path:
    units = render_sources()
    srcs = units + [CSRC / "mi_gemm.hip", CSRC / "reference_gpu_gemm.hip"]
    jobs = jobs or min(8, os.cpu_count() or 1)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), srcs))
    LIB.parent.mkdir(parents=True, exist_ok=True)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *map(str, objs)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr[-4000:]}")
    if verbose:
        print(f"built {LIB} ({LIB.stat().st_size} bytes, {len(units)} kernel configs)")
    return LIB


# Four points of the tuner's search space, rendered from template/matmul_mi355x.hip.jinja and
# compiled as standalone `./test` programs -- the tuner's own flow (render -> hipcc -> run),
# whose programs instantiate the kernels directly instead of going through the library's
# dispatch.  Built here, where hipcc runs without a GPU, so that the GPU tests only run them.
TUNER_SAMPLES = PKG / "harness" / "tuner_samples"
TUNER_SAMPLE_CONFIGS = [
    dict(KIND="mfma16", BM=256, BN=256, WM=2, WN=2, NS=4, SWZ=1, GROUP=4, DTL=1, EPI=1, DRAIN=3, EDRAIN=1, OCC=1),
    dict(KIND="tile", BM=128, BN=128, WM=2, WN=2, NS=4, SWZ=1, GROUP=8, DTL=1, EPI=1, DRAIN=0, OCC=2),
    # kinds whose LDS stage count the tuner sweeps: a split-K decode kernel with a ring of four
    # slabs of B and a small-tile kernel with per-wave rings of three stages (neither depth is
    # among the library's own configurations)
    dict(KIND="decode", BM=128, BN=128, WM=2, WN=2, NS=4, GROUP=4, DRAIN=0, OCC=1, SHARED=0),
    dict(KIND="wavek", BM=32, BN=32, WM=2, WN=2, NS=3, GROUP=4, DRAIN=0, OCC=1, SHARED=0),
]


def build_tuner_samples(jobs: int = 2, verbose: bool = True) -> Path:
    from .gemm_tuner import GemmTuner
    tuner = GemmTuner(output_dir=str(TUNER_SAMPLES), only=TUNER_SAMPLE_CONFIGS)
    built = tuner.prebuild(jobs)
    if len(built) != len(TUNER_SAMPLE_CONFIGS) or not all(built.values()):
        raise RuntimeError(f"tuner sample programs failed to compile: {built}")
    if verbose:
        print(f"built {len(built)} tuner sample programs in {tuner.bin_dir}")
    return tuner.bin_dir


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("-j", "--jobs", type=int, default=None)
    ap.add_argument("--force", action="store_true")
    a = ap.parse_args(argv)
    build(a.jobs, a.force)
    build_tuner_samples()
    return 0


if __name__ == "__main__":
    sys.exit(main())
