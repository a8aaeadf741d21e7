"""Build-time checks of the generated gfx950 assembly that the kernels' inline asm relies on.

The direct-to-LDS loads take their LDS address from M0, which the kernels set in their own
asm statements; in the 16x16x32 kernel up to four consecutive loads share one M0 value across
separate asm statements.  Nothing tells the compiler that M0 is live in between, so a
compiler that put M0 to some use of its own there would silently redirect the loads.  The
library build therefore compiles every unit with its assembly text kept and refuses to link
when the text shows such a use (or a load right behind an M0 write without the wait state the
hardware needs, or scratch memory in an aligned kernel of the automatic choice, whose
accumulators must stay in registers).  `tests/test_isa_invariants.py` runs the same functions
on the build's output and on hand-made counter-examples.
"""
from __future__ import annotations

import re


class IsaCheckError(RuntimeError):
    pass


def kernels(text: str) -> dict[str, str]:
    """name -> body of every kernel function in an assembly text"""
    out = {}
    for m in re.finditer(r"^(_ZN2mi\w+):[^\n]*\n(.*?)^\s*\.amdhsa_kernel \1\s*$", text, flags=re.S | re.M):
        out[m.group(1)] = m.group(2)
    return out


def check_m0(unit: str, text: str, need_kernels: int = 1) -> int:
    """M0 is written only inside the kernels' own asm statements, and no direct-to-LDS load
    follows an M0 write without a wait state.  Returns the number of kernels looked at."""
    ks = kernels(text)
    if len(ks) < need_kernels:
        raise IsaCheckError(f"{unit}: {len(ks)} kernels found in the assembly text, expected at least {need_kernels}")
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
                if re.search(r"\bm0\b", t):
                    raise IsaCheckError(f"{unit} {name}: the compiler touches m0 outside the kernel's asm: {t}")
            else:
                if t.startswith("s_mov_b32 m0"):
                    sets += 1
                if t.startswith("buffer_load_dwordx4") and t.endswith("lds"):
                    loads += 1
                    if prev.startswith("s_mov_b32 m0"):
                        raise IsaCheckError(f"{unit} {name}: no wait state between the m0 write and {t}")
            prev = t
        if loads and not 0 < sets <= loads:
            raise IsaCheckError(f"{unit} {name}: {loads} direct-to-LDS loads but {sets} m0 writes")
    return len(ks)


def check_no_scratch(unit: str, text: str) -> int:
    """The aligned, untraced 16x16x32 kernels of a unit use no scratch memory.  Returns how
    many kernel descriptors were checked."""
    found = re.findall(r"\.amdhsa_kernel (\S+).*?\.amdhsa_private_segment_fixed_size (\d+)", text, flags=re.S)
    # Mfma16Config<..., EDGE, OCC, KG>, TRACE, SPLITK: "...ELb<EDGE>ELi<OCC>ELi<KG>EEELb<TRACE>ELb<SPLITK>..."
    aligned = [(n, int(sz)) for n, sz in found if re.search(r"Mfma16ConfigI\w*?ELb0ELi\d+ELi\d+EEELb0ELb[01]", n)]
    if not aligned:
        raise IsaCheckError(f"{unit}: no aligned 16x16x32 kernel found among {[n for n, _ in found]}")
    for n, sz in aligned:
        if sz != 0:
            raise IsaCheckError(f"{unit}: {n} uses {sz} bytes of scratch per lane")
    return len(aligned)


def check_lds_bytes(unit: str, text: str, expected: int) -> int:
    """The largest LDS allocation among a unit's kernels is what the config table says (the
    table's figure decides how many workgroups the time model lets share a CU and is what
    `mi_gemm_config_lds_bytes` reports).  Returns how many kernel descriptors were read."""
    sizes = [int(v) for v in re.findall(r"\.amdhsa_group_segment_fixed_size (\d+)", text)]
    if not sizes:
        raise IsaCheckError(f"{unit}: no kernel descriptor with an LDS size found")
    if max(sizes) != expected:
        raise IsaCheckError(f"{unit}: kernels allocate up to {max(sizes)} bytes of LDS, the config table says {expected}")
    return len(sizes)
