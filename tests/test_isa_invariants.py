"""The build gate on the generated gfx950 code (h100_gemm_amd/isa_check.py): the invariants
the kernels' inline assembly relies on and that no run-time test would catch reliably.
`build.py` keeps every unit's assembly text and refuses to link when a check fails; here the
same functions run on what the build left in the tree and on hand-made counter-examples."""
import pytest

from h100_gemm_amd import build, isa_check
from h100_gemm_amd import kernel_configs as kc


def built_units(kinds):
    """(unit file name, config, assembly text) of the built units of the given kinds"""
    build.render_sources()
    out = []
    for c in kc.CONFIGS:
        if c["KIND"] not in kinds:
            continue
        src = build.GEN / f"unit_{kc.config_name(c)}.hip"
        obj = build._compile(src, force=False)       # compiles (and checks) only if stale
        out.append((src.name, c, build._asm_path(obj).read_text()))
    return out


def test_m0_is_only_written_by_the_kernels_own_asm():
    """Consecutive direct-to-LDS loads share one M0 value across asm statements, so nothing
    the compiler emits in between may write M0; and every load that follows a write of M0
    directly is preceded by the wait state the hardware needs."""
    units = built_units(("mfma16", "decode", "stream", "wavek"))
    assert len(units) >= 16
    for name, c, text in units:
        n = isa_check.check_m0(name, text, need_kernels=8 if c["KIND"] == "mfma16" else 1)
        assert n >= (8 if c["KIND"] == "mfma16" else 2), (name, n)


def test_aligned_kernels_do_not_spill():
    """The accumulators live in AGPRs and the aligned variants keep everything else in VGPRs:
    no scratch memory, for the candidates of the automatic choice."""
    auto = [(n, t) for n, c, t in built_units(("mfma16",)) if c.get("EFF")]
    assert len(auto) >= 5
    for name, text in auto:
        assert isa_check.check_no_scratch(name, text) >= 2


def test_lds_sizes_match_the_config_table():
    """What the compiled kernels allocate is what `kernel_configs.lds_bytes` says (the rules
    for workgroups per CU and the C ABI's config query are derived from it)."""
    units = built_units(("tile", "ring", "ring16", "mfma16", "decode", "stream", "wavek"))
    assert len(units) == len(kc.CONFIGS)
    for name, c, text in units:
        assert isa_check.check_lds_bytes(name, text, kc.lds_bytes(c)) >= 1
    with pytest.raises(isa_check.IsaCheckError, match="bytes of LDS"):
        isa_check.check_lds_bytes(units[0][0], units[0][2], kc.lds_bytes(units[0][1]) - 1024)


KERNEL = """_ZN2mi4testE:
	s_load_dwordx2 s[0:1], s[4:5], 0x0
{body}
	s_endpgm
	.amdhsa_kernel _ZN2mi4testE
		.amdhsa_private_segment_fixed_size {scratch}
	.end_amdhsa_kernel
"""
GOOD = """	;;#ASMSTART
	s_mov_b32 m0, s8
	s_nop 0
	buffer_load_dwordx4 v1, s[0:3], s9 offen lds
	;;#ASMEND
	v_mfma_f32_16x16x32_bf16 a[0:3], v[2:5], v[6:9], a[0:3]
	;;#ASMSTART
	buffer_load_dwordx4 v2, s[0:3], s9 offen offset:0x400 lds
	;;#ASMEND"""


def test_the_checks_reject_what_they_are_there_for():
    assert isa_check.check_m0("ok", KERNEL.format(body=GOOD, scratch=0)) == 1
    # the compiler using m0 between two asm statements that share its value
    bad = GOOD.replace("	v_mfma_f32", "	s_mov_b32 m0, -1\n	v_mfma_f32")
    with pytest.raises(isa_check.IsaCheckError, match="touches m0"):
        isa_check.check_m0("bad", KERNEL.format(body=bad, scratch=0))
    # a load right behind the m0 write
    with pytest.raises(isa_check.IsaCheckError, match="wait state"):
        isa_check.check_m0("bad", KERNEL.format(body=GOOD.replace("	s_nop 0\n", ""), scratch=0))
    # loads without any m0 write
    with pytest.raises(isa_check.IsaCheckError, match="m0 writes"):
        isa_check.check_m0("bad", KERNEL.format(body=GOOD.replace("	s_mov_b32 m0, s8\n	s_nop 0\n", ""), scratch=0))
    with pytest.raises(isa_check.IsaCheckError, match="kernels found"):
        isa_check.check_m0("empty", "no kernels here", need_kernels=1)
    spilled = KERNEL.replace("_ZN2mi4testE", "_ZN2mi18gemm_mfma16_kernelINS_12Mfma16ConfigILi256ELi256ELi2ELi2ELi4ELi0ELi3ELb0ELi1ELi1EEELb0ELb0EEEvNS_8GemmArgsE")
    assert isa_check.check_no_scratch("ok", spilled.format(body=GOOD, scratch=0)) == 1
    with pytest.raises(isa_check.IsaCheckError, match="scratch"):
        isa_check.check_no_scratch("bad", spilled.format(body=GOOD, scratch=64))


INFLIGHT = """	;;#ASMSTART
	buffer_load_dwordx4 v[10:13], v1, s[0:3], s9 offen
	;;#ASMEND
	;;#ASMSTART
	s_mov_b32 m0, s8
	s_nop 0
	buffer_load_dwordx4 v2, s[0:3], s9 offen lds
	;;#ASMEND
{between}
	;;#ASMSTART
	s_waitcnt vmcnt({n}) lgkmcnt(0)
	s_barrier
	;;#ASMEND
	v_mfma_f32_16x16x32_bf16 a[0:3], v[10:13], v[6:9], a[0:3]"""


def test_registers_with_an_asm_load_in_flight_are_left_alone():
    """The decode kernels load A fragments into registers from their own asm statements; the
    build follows those loads through the generated code."""
    units = built_units(("decode",))
    assert len(units) == 2
    for name, c, text in units:
        assert isa_check.check_inflight(name, text) >= 16, name
    ok = KERNEL.format(body=INFLIGHT.format(between="	v_mov_b32_e32 v20, v5", n=1), scratch=0)
    assert isa_check.check_inflight("ok", ok) == 1
    # the allocator copying an in-flight register somewhere else
    with pytest.raises(isa_check.IsaCheckError, match="touches"):
        isa_check.check_inflight("bad", KERNEL.format(body=INFLIGHT.format(between="	v_mov_b32_e32 v20, v11", n=1), scratch=0))
    # ... or handing it to another value
    with pytest.raises(isa_check.IsaCheckError, match="touches"):
        isa_check.check_inflight("bad", KERNEL.format(body=INFLIGHT.format(between="	v_add_u32_e32 v12, v1, v1", n=1), scratch=0))
    # ... or spilling it
    with pytest.raises(isa_check.IsaCheckError, match="uses|touches"):
        isa_check.check_inflight("bad", KERNEL.format(body=INFLIGHT.format(between="	scratch_store_dwordx4 off, v[10:13], off offset:16", n=1), scratch=0))
    # a wait that leaves the load in flight (two loads are younger than allowed to be outstanding)
    with pytest.raises(isa_check.IsaCheckError, match="touches"):
        isa_check.check_inflight("bad", KERNEL.format(body=INFLIGHT.format(between="", n=2), scratch=0))
    # a loop whose next trip loads into a register before the wait of this trip has retired the last load
    loop = ".LBB0_1:\n" + INFLIGHT.format(between="", n=2).replace("	v_mfma_f32_16x16x32_bf16 a[0:3], v[10:13]", "	v_mfma_f32_16x16x32_bf16 a[0:3], v[14:17]") + "\n	s_cbranch_scc1 .LBB0_1"
    with pytest.raises(isa_check.IsaCheckError, match="still has a load in flight"):
        isa_check.check_inflight("bad", KERNEL.format(body=loop, scratch=0))
