"""Invariants of the generated gfx950 code that the kernels' inline assembly relies on and
that no run-time test would catch reliably.  Compiles the default kernel's unit to assembly
text on the CPU (hipcc cross-compiles; no GPU needed) and reads the compiler's own output."""
import re
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
GEN = ROOT / "h100_gemm_amd" / "csrc" / "gen"
def mfma16_units():
    from h100_gemm_amd import kernel_configs as kc
    return [f"unit_{kc.config_name(c)}.hip" for c in kc.CONFIGS if c["KIND"] == "mfma16"]


@pytest.fixture(scope="module")
def asm_text(tmp_path_factory):
    """assembly text of every 16x16x32-kernel unit (all of them keep M0 live across asm statements)"""
    from concurrent.futures import ThreadPoolExecutor
    from h100_gemm_amd import build
    build.render_sources()
    tmp = tmp_path_factory.mktemp("isa")

    def one(unit):
        src = GEN / unit
        assert src.exists(), src
        dst = tmp / (src.stem + ".s")
        cmd = ["/opt/rocm/bin/hipcc", *build.HIPFLAGS, "--cuda-device-only", "-S", f"-I{build.CSRC}", f"-I{GEN}",
               str(src), "-o", str(dst)]
        subprocess.run(cmd, check=True, capture_output=True, timeout=900)
        return unit, dst.read_text()

    with ThreadPoolExecutor(8) as ex:
        return dict(ex.map(one, mfma16_units()))


def kernels(text):
    """name -> body of every kernel function in the assembly text"""
    out = {}
    for m in re.finditer(r"^(_ZN2mi\w+):[^\n]*\n(.*?)^\s*\.amdhsa_kernel \1\s*$", text, flags=re.S | re.M):
        out[m.group(1)] = m.group(2)
    return out


def test_m0_is_only_written_by_the_kernels_own_asm(asm_text):
    """Consecutive direct-to-LDS loads share one M0 value across asm statements, so nothing
    the compiler emits in between may write M0; and every load that follows a write of M0
    directly is preceded by the wait state the hardware needs."""
    for unit, text in asm_text.items():
        ks = kernels(text)
        assert len(ks) >= 8, (unit, list(ks))      # {bf16, fp16} x {aligned, predicated} x {plain, trace, split-K}
        for name, body in ks.items():
            inasm, prev = False, ""
            loads = sets = 0
            for line in body.splitlines():
                t = line.split(";")[0].strip() if not line.strip().startswith(";;#") else line.strip()
                if t.startswith(";;#ASMSTART"):
                    inasm = True
                    continue
                if t.startswith(";;#ASMEND"):
                    inasm = False
                    continue
                if not t:
                    continue
                if not inasm:
                    assert not re.search(r"\bm0\b", t), f"{unit} {name}: compiler touches m0: {t}"
                else:
                    if t.startswith("s_mov_b32 m0"):
                        sets += 1
                    if t.startswith("buffer_load_dwordx4") and t.endswith("lds"):
                        loads += 1
                        assert not prev.startswith("s_mov_b32 m0"), f"{unit} {name}: no wait state before {t}"
                prev = t
            assert loads > 0 and 0 < sets <= loads, (unit, name, loads, sets)


def test_aligned_kernels_do_not_spill(asm_text):
    """The accumulators live in AGPRs and the aligned variants keep everything else in VGPRs:
    no scratch memory (the predicated variants spill in their peeled tail only).  Checked for
    the candidates of the automatic choice (the eight-wave tuner variants have half the
    registers per wave and may spill a few)."""
    from h100_gemm_amd import kernel_configs as kc
    auto = {f"unit_{kc.config_name(c)}.hip" for c in kc.CONFIGS if c["KIND"] == "mfma16" and c.get("EFF")}
    assert len(auto) >= 5
    for unit, text in asm_text.items():
        if unit not in auto:
            continue
        # kernel descriptors: ".amdhsa_kernel NAME ... .amdhsa_private_segment_fixed_size N"
        found = re.findall(r"\.amdhsa_kernel (\S+).*?\.amdhsa_private_segment_fixed_size (\d+)", text, flags=re.S)
        assert found, unit
        # Mfma16Config<..., EDGE, OCC>, TRACE, SPLITK: "...ELb<EDGE>ELi<OCC>EEELb<TRACE>ELb<SPLITK>E..."
        # ...EDGE = false; TRACE = false (the trace variant keeps extra timers alive and may spill a few)
        aligned = [(n, int(sz)) for n, sz in found if re.search(r"Mfma16ConfigI\w*?ELb0ELi\d+EEELb0ELb[01]E", n)]
        assert aligned, (unit, [n for n, _ in found])
        for n, sz in aligned:
            assert sz == 0, f"{unit}: {n} uses {sz} bytes of scratch per lane"
