"""Invariants of the generated gfx950 code that the kernels' inline assembly relies on and
that no run-time test would catch reliably.  Compiles the default kernel's unit to assembly
text on the CPU (hipcc cross-compiles; no GPU needed) and reads the compiler's own output."""
import re
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
GEN = ROOT / "h100_gemm_amd" / "csrc" / "gen"
UNITS = ["unit_m256x256_w2x2_g4_b3.hip", "unit_m256x192_w2x2_g4_b3.hip"]


@pytest.fixture(scope="module")
def asm_text(tmp_path_factory):
    from h100_gemm_amd import build
    build.render_sources()
    out = {}
    for unit in UNITS:
        src = GEN / unit
        assert src.exists(), src
        dst = tmp_path_factory.mktemp("isa") / (src.stem + ".s")
        cmd = ["/opt/rocm/bin/hipcc", *build.HIPFLAGS, "--cuda-device-only", "-S", f"-I{build.CSRC}", f"-I{GEN}",
               str(src), "-o", str(dst)]
        subprocess.run(cmd, check=True, capture_output=True, timeout=600)
        out[unit] = dst.read_text()
    return out


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
        assert len(ks) >= 4, (unit, list(ks))
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
    """The 256 accumulators live in AGPRs and the aligned variants keep everything else in
    VGPRs: no scratch memory (the predicated variants spill in their peeled tail only)."""
    for unit, text in asm_text.items():
        # kernel descriptors: ".amdhsa_kernel NAME ... .amdhsa_private_segment_fixed_size N"
        found = re.findall(r"\.amdhsa_kernel (\S+).*?\.amdhsa_private_segment_fixed_size (\d+)", text, flags=re.S)
        assert found, unit
        # Mfma16Config<..., EDGE, OCC>, TRACE: "...ELb<EDGE>ELi<OCC>EEELb<TRACE>EE..."
        aligned = [(n, int(sz)) for n, sz in found if re.search(r"Mfma16ConfigI\w*?ELb0ELi\d+EEELb[01]ELb[01]E", n)]
        assert aligned, (unit, [n for n, _ in found])
        for n, sz in aligned:
            assert sz == 0, f"{unit}: {n} uses {sz} bytes of scratch per lane"
