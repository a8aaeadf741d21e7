"""Build-time checks of the generated gfx950 assembly that the kernels' inline asm relies on.

The direct-to-LDS loads take their LDS address from M0, which the kernels set in their own
asm statements; in the 16x16x32 kernel up to four consecutive loads share one M0 value across
separate asm statements.  Nothing tells the compiler that M0 is live in between, so a
compiler that put M0 to some use of its own there would silently redirect the loads.  The
library build therefore compiles every unit with its assembly text kept and refuses to link
when the text shows such a use (or a load right behind an M0 write without the wait state the
hardware needs, or scratch memory in an aligned kernel of the automatic choice, whose
accumulators must stay in registers).

Some kernels (the decode kernels' ring of A fragments) also load into registers from their own
asm statements and wait for those loads with their own `s_waitcnt vmcnt(n)`.  Between such a
load and the wait that retires it the destination registers belong to the memory system: an
instruction that reads or writes one of them there -- a copy the register allocator inserts, a
spill, a register handed to another value -- gives wrong answers without any error.  The C++
source cannot forbid the compiler to do that, so `check_inflight` follows every kernel's
instruction stream, retires loads at the waits as the hardware does (in order, at most n left
in flight) and refuses the build when anything touches a register with a load still on its way.  `tests/test_isa_invariants.py` runs the same functions
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


_VMEM_LOAD = re.compile(r"^(buffer|global|scratch|flat)_load_(\w+)\s+(.*)$")
_REG = re.compile(r"\b([va])(?:(\d+)\b|\[(\d+):(\d+)\])")
_WIDTH = {"dword": 1, "dwordx2": 2, "dwordx3": 3, "dwordx4": 4, "ubyte": 1, "sbyte": 1, "ushort": 1, "sshort": 1,
          "short_d16": 1, "short_d16_hi": 1, "ubyte_d16": 1, "ubyte_d16_hi": 1, "sbyte_d16": 1, "sbyte_d16_hi": 1}


def _regs(text: str) -> set:
    out = set()
    for m in _REG.finditer(text):
        if m.group(2) is not None:
            out.add((m.group(1), int(m.group(2))))
        else:
            out.update((m.group(1), r) for r in range(int(m.group(3)), int(m.group(4)) + 1))
    return out


def check_inflight(unit: str, text: str) -> int:
    """No instruction reads or writes a vector register between a load into it that one of the
    kernels' own asm statements issued and the `s_waitcnt vmcnt` that retires that load.  (The
    compiler waits for the loads it issues itself; it knows nothing of the asm ones.)  Loads
    return in order, so `vmcnt(n)` retires every load but the n youngest (stores share the
    counter but only ever make a wait stricter); every load counts, whoever issued it.  The scan
    follows the text of each kernel; a loop (a backward branch) is walked a second time with
    the state its end leaves, and a forward branch carries its state to its target, where the
    loads in flight on either path count as in flight.  Returns the number of asm-issued loads
    into registers that were followed."""
    followed = 0
    for name, body in kernels(text).items():
        lines, in_asm, flag = [], [], False
        for raw in body.splitlines():
            st = raw.strip()
            if st.startswith(";;#ASMSTART"):
                flag = True
                continue
            if st.startswith(";;#ASMEND"):
                flag = False
                continue
            t = raw.split(";")[0].strip()
            if t:
                lines.append(t)
                in_asm.append(flag)
        labels = {t[:-1]: i for i, t in enumerate(lines) if re.fullmatch(r"[.\w$]+:", t)}
        pending = {}                       # label -> in-flight list carried by forward branches

        def busy(inflight):
            out = set()
            for dest, _, tracked in inflight:
                if tracked:
                    out |= dest
            return out

        def step(i, inflight, count):
            """effect of line i on the ordered list of loads in flight: [(dest registers, text, asm-issued)]"""
            nonlocal followed
            t = lines[i]
            m = _VMEM_LOAD.match(t)
            if m:
                kind, ops = m.group(2), m.group(3)
                to_lds = kind.startswith("lds_") or (" " + ops + " ").find(" lds ") >= 0
                first = ops.split(",")[0]
                hit = _regs(ops if to_lds else ops[len(first):]) & busy(inflight)
                if hit:
                    raise IsaCheckError(f"{unit} {name}: `{t}` uses {sorted(hit)[:4]} while a load into it is in flight")
                dest = set() if to_lds else _regs(first)
                tracked = in_asm[i] and not to_lds
                if tracked:
                    if _WIDTH.get(kind) != len(dest):
                        raise IsaCheckError(f"{unit} {name}: cannot tell the destination of `{t}`")
                    if count:
                        followed += 1
                if dest & busy(inflight):
                    raise IsaCheckError(f"{unit} {name}: `{t}` loads into a register that still has a load in flight")
                return inflight + [(dest, t, tracked)]
            if t.startswith("s_waitcnt"):
                w = re.search(r"vmcnt\((\d+)\)", t)
                if w:
                    n = int(w.group(1))
                    return inflight[len(inflight) - n:] if n < len(inflight) else inflight
                if re.fullmatch(r"s_waitcnt\s+(0|0x0)", t):
                    return []
                return inflight
            if t.startswith("s_endpgm"):
                return []
            hit = _regs(t) & busy(inflight) if inflight else None
            if hit:
                who = next(l for d, l, tr in inflight if tr and d & hit)
                raise IsaCheckError(f"{unit} {name}: `{t}` touches {sorted(hit)[:4]} while `{who}` is in flight")
            return inflight

        def merge(a, b):
            return a + [e for e in b if e not in a]

        inflight, walked = [], set()
        for i, t in enumerate(lines):
            if t.endswith(":") and t[:-1] in pending:
                inflight = merge(pending.pop(t[:-1]), inflight)
            inflight = step(i, inflight, True)
            br = re.match(r"s_c?branch\w*\s+([.\w$]+)", t)
            if br and br.group(1) in labels:
                tgt = labels[br.group(1)]
                if tgt <= i:
                    if (tgt, i) not in walked:             # the loop once more, with the state its end leaves
                        walked.add((tgt, i))
                        again = list(inflight)
                        for j in range(tgt, i + 1):
                            again = step(j, again, False)
                else:
                    pending[br.group(1)] = merge(pending.get(br.group(1), []), inflight)
                if t.startswith("s_branch"):
                    inflight = []                           # nothing falls through an unconditional branch
    return followed
