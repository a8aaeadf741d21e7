"""The kernel configurations compiled into libmi_gemm.so.

Each entry fixes the template constants of ``csrc/gemm_kernel.hpp`` -- the counterpart of the
six constants ``CLUSTER_M, CLUSTER_N, BLOCKM, BLOCKN, BLOCKK, STAGES`` that the reference's
template takes (matmul_h100.cu.jinja:9-14) -- re-cast for CDNA4:

    BM, BN   macro tile of one workgroup (the K step is fixed at 64 = one 128-byte LDS row)
    WM, WN   wave grid: WM*WN waves of 64 lanes, each owning a (BM/WM) x (BN/WN) sub-tile
    SWZ      LDS chunk swizzle (0: row & 7, 1: (row >> 1) & 7)
    GROUP    tile-order group height (L2 locality of the workgroups sharing an XCD)
    OCC      workgroups per CU the register budget is sized for (tile and mfma16 kinds)
    DTL      1: direct-to-LDS global loads in the aligned kernel, 0: register staged
    KIND     "tile" (two-stage kernel above), "ring" (NS-deep LDS ring, K step 32, aligned
             shapes; ragged shapes take the predicated tile kernel of the same tile),
             "mfma16" / "ring16" (the same two pipelines on the 16x16x32 MFMA with eight
             or four waves, csrc/gemm_mfma16_kernel.hpp), "decode" (split-K kernel for decode
             shapes, M <= BM, whose LDS ring holds B only, csrc/gemm_decode_kernel.hpp) or
             "stream" (single-pass decode kernel, csrc/gemm_stream_kernel.hpp), "wavek" (small
             tiles with K split over the waves of a workgroup, or on a ring shared by them, for
             outputs of few tiles: any M, N and K, csrc/gemm_wavek_kernel.hpp)
    EPI      1: C tile transposed through LDS and written 16 bytes per lane, 0: 8-byte stores
    KG       (mfma16, optional) 2: eight waves as two groups that each multiply half of K of the
             same tile and add their accumulators through LDS (K % 256 == 0; tiles alone on a CU)
    DRAIN    (mfma16, optional) d > 0: a second barrier early in each K step (4*d MFMAs after the
             fragment reads) frees the current LDS stage, so the next loads are spread over most
             of the step instead of its second half; EDRAIN (optional): the predicated variant's
             slot where it differs (its loads from unaligned rows arrive later: the earlier slot
             is 2 % ahead at 4095 x 6143 x 3073, the later one on aligned shapes)
    EWM, EWN (optional) wave grid of the predicated twin when it differs from WM, WN (the
             register-staged predicated kernel runs best with eight waves)
    EFF      (optional) per-CU throughput relative to the 256x256 tile, measured at 8192^3;
             configs that carry it are the candidates of the automatic shape -> kernel choice
    SHARED   (wavek, optional) 1: the four waves form a 2 x 2 grid over the tile and share one
             ring of NS stages (a barrier per 64-deep unit, no partial tiles to add) instead of
             each multiplying the whole tile over a quarter of K -- for outputs of up to a few
             tiles per CU with a K too short to split four ways, or tiles too large for that
    WK       (wavek, optional) time model in microseconds, (fixed, per round, per unit, per
             tile): fixed + rounds of co-resident workgroups (tiles / (CUs x OCC), rounded up)
             x per round + tiles per CU (rounded up) x (per tile + K/64 x per unit);
             non-negative least squares on 89-99 shapes (the 96x64 shared-ring config: x 1.035); configs that carry it join the automatic choice
    WK_RAGGED (wavek, optional) what a K unit costs more when K % 64 != 0 (rows that do not start on
             128-byte lines): K % 8 == 0 with K < 2048 / K >= 2048, other even K with K < 2048 /
             K >= 2048 (medians over 160 shapes of four lists); WK_ODD the same for an odd K
    EFF_E    (optional) throughput of the predicated variant relative to the aligned one, from
             7000^3, 6000^3 and 5000^3 (default 0.85); used for shapes the aligned variant cannot run

The index of a config in ``CONFIGS`` is its ``config`` number in the C ABI.
"""
from __future__ import annotations


def config_name(c: dict) -> str:
    if c["KIND"] == "ring":
        return f"r{c['BM']}x{c['BN']}_w{c['WM']}x{c['WN']}_n{c['NS']}_g{c['GROUP']}"
    if c["KIND"] == "mfma16":
        name = f"m{c['BM']}x{c['BN']}_w{c['WM']}x{c['WN']}_g{c['GROUP']}"
        if c.get("DRAIN", 0):
            name += f"_b{c['DRAIN']}"
        if c.get("OCC", 1) != 1:
            name += f"_o{c['OCC']}"
        if c.get("KG", 1) != 1:
            name += f"_k{c['KG']}"
        return name
    if c["KIND"] == "ring16":
        return f"q{c['BM']}x{c['BN']}_w{c['WM']}x{c['WN']}_n{c['NS']}_g{c['GROUP']}"
    if c["KIND"] == "stream":
        return f"s{c['BM']}x{c['BN']}_n{c['NS']}"
    if c["KIND"] == "decode":
        return f"d{c['BM']}x{c['BN']}_n{c['NS']}"
    if c["KIND"] == "wavek":
        return f"k{c['BM']}x{c['BN']}_{'s' if c.get('SHARED') else 'n'}{c['NS']}"
    name = (f"t{c['BM']}x{c['BN']}_w{c['WM']}x{c['WN']}_s{c['SWZ']}_g{c['GROUP']}"
            f"_o{c['OCC']}_d{c['DTL']}_e{c['EPI']}")
    if (c.get("EWM", c["WM"]), c.get("EWN", c["WN"])) != (c["WM"], c["WN"]):
        name += f"_x{c['EWM']}x{c['EWN']}"
    return name


def threads(c: dict) -> int:
    return 256 if c["KIND"] in ("stream", "decode", "wavek") else c["WM"] * c["WN"] * c.get("KG", 1) * 64


def lds_bytes(c: dict) -> int:
    if c["KIND"] in ("ring", "ring16"):
        return c["NS"] * (c["BM"] + c["BN"]) * 64
    if c["KIND"] == "stream":
        return 4 * c["NS"] * (c["BM"] + c["BN"]) * 128
    if c["KIND"] == "decode":
        return c["NS"] * c["BN"] * 128
    if c["KIND"] == "wavek" and c.get("SHARED"):     # one ring for the workgroup, or the padded fp32 C tile
        return max(c["NS"] * (c["BM"] + c["BN"]) * 128, c["BM"] * (c["BN"] + 4) * 4 + (c["BM"] + c["BN"]) * 4)
    if c["KIND"] == "wavek":     # per wave: the ring, or the padded fp32 partial tile (and the last k of an odd K) if that is larger
        return 4 * max(c["NS"] * (c["BM"] + c["BN"]) * 128, c["BM"] * (c["BN"] + 4) * 4 + (c["BM"] + c["BN"]) * 4)
    return c.get("KG", 1) * 2 * (c["BM"] + c["BN"]) * 128


def is_valid_config(c: dict) -> bool:
    """Static rules of the kernels (mirrored as static_asserts in csrc/)."""
    if c["KIND"] in ("ring", "ring16") and not c.get("_twin_checked"):
        # ragged shapes run the predicated two-stage kernel of the same tile and wave grid
        twin = dict(KIND="tile", BM=c["BM"], BN=c["BN"], WM=c.get("EWM", c["WM"]), WN=c.get("EWN", c["WN"]), SWZ=1,
                    GROUP=c["GROUP"], OCC=1, DTL=0, EPI=1)
        return is_valid_config(twin) and is_valid_config(dict(c, _twin_checked=True))
    if c["KIND"] == "tile" and (c.get("EWM", c["WM"]), c.get("EWN", c["WN"])) != (c["WM"], c["WN"]):
        twin = dict(c, WM=c["EWM"], WN=c["EWN"], DTL=0)
        del twin["EWM"], twin["EWN"]
        main = dict(c)
        del main["EWM"], main["EWN"]
        return is_valid_config(twin) and is_valid_config(main)
    if c["KIND"] == "stream":
        return (c["BM"] in (16, 32, 64) and c["BN"] == 32 and c["NS"] >= 2
                and (c["NS"] - 1) * ((c["BM"] + c["BN"]) // 8) <= 63
                and c["NS"] * (c["BM"] + c["BN"]) * 128 >= max(c["BM"], 32) * 128
                and lds_bytes(c) <= 160 * 1024)
    if c["KIND"] == "decode":
        # B-only LDS ring, A fragments in a register ring: per wave and slab BN/32 direct-to-LDS
        # loads and BM/32 fragment loads, NS-1 slabs of them outstanding (6-bit vmcnt)
        return (c["BM"] in (64, 128) and c["BN"] % 32 == 0 and c["NS"] >= 3
                and (c["NS"] - 1) * (c["BM"] // 32 + c["BN"] // 32) <= 63
                and lds_bytes(c) <= 160 * 1024)
    if c["KIND"] == "wavek" and c.get("SHARED"):
        # 2 x 2 waves over the tile, one ring: per wave and stage (BM + BN) / 32 loads, NS - 1 stages outstanding
        return (c["BM"] % 32 == 0 and c["BN"] % 32 == 0 and c["NS"] >= 3
                and (c["NS"] - 1) * ((c["BM"] + c["BN"]) // 32) <= 63
                and c["BM"] * c["BN"] // 4 % 256 == 0 and c["BM"] + c["BN"] <= 256
                and lds_bytes(c) * c.get("OCC", 1) <= 160 * 1024)
    if c["KIND"] == "wavek":
        # per wave and ring stage (BM + BN) / 8 direct-to-LDS loads, NS stages outstanding
        return (c["BM"] % 16 == 0 and c["BN"] % 16 == 0 and c["NS"] >= 1
                and (c["NS"] - 1) * ((c["BM"] + c["BN"]) // 8) <= 63
                and c["BM"] * c["BN"] // 4 % 256 == 0 and c["BM"] + c["BN"] <= 256
                and (c["BM"] // 16) * (c["BN"] // 16) * 4 <= 256
                and lds_bytes(c) * c.get("OCC", 1) <= 160 * 1024)
    kg = c.get("KG", 1)
    if kg not in (1, 2) or (kg == 2 and (c["KIND"] != "mfma16" or c["BM"] * c["BN"] * 4 > lds_bytes(c) // 2)):
        return False            # the second K group's accumulators pass through its LDS stages
    nt = c["WM"] * c["WN"] * kg * 64
    if nt > 1024 or nt < 64:
        return False
    if c["BM"] % (32 * c["WM"]) or c["BN"] % (32 * c["WN"]):
        return False
    mi, ni = c["BM"] // c["WM"] // 32, c["BN"] // c["WN"] // 32
    nmma = mi * ni
    occ = c.get("OCC", 1)
    if lds_bytes(c) * occ > 160 * 1024:
        return False
    waves_per_simd = max(nt // 256, 1) * occ
    if c["KIND"] in ("mfma16", "ring16"):
        # 16x16x32 MFMA kernels: 4 accumulator registers per 16x16 tile; the two-stage kernel
        # runs with four or eight waves, the ring kernel with eight
        if nt not in (256, 512) or c["BM"] * c["BN"] * 2 > lds_bytes(c) // kg:
            return False
        mi16, ni16 = 2 * mi, 2 * ni
        rpp = nt // kg // 8 if c["KIND"] == "mfma16" else nt // 4
        if c["BM"] % rpp or c["BN"] % rpp:
            return False
        l = c["BM"] // rpp + c["BN"] // rpp
        if c["KIND"] == "ring16" and (c["NS"] != 4 or (c["NS"] - 1) * l > 63):
            return False
        tn = c["BN"] // c["WN"]
        if tn < 32 or (c["KIND"] == "ring16" and tn & (tn - 1)):   # ring16: C staging needs a power-of-two row
            return False
        for d in {c.get("DRAIN", 0), c.get("EDRAIN", c.get("DRAIN", 0))} - {0} if c["KIND"] == "mfma16" else ():
            sa = mi16 + ni16 + 4 * d
            if sa + 1 >= mi16 * ni16 or (2 * mi16 * ni16 - 5 - sa) // l < 1:
                return False
        if mi16 + ni16 + l > mi16 * ni16:
            return False
        return mi16 * ni16 * 4 + 2 * (mi16 + ni16) * 4 + 24 <= 512 // waves_per_simd
    if c["KIND"] == "ring":
        rpp = (nt // 64) * 16
        if c["BM"] % rpp or c["BN"] % rpp or c["NS"] != 4:
            return False
        l = c["BM"] // rpp + c["BN"] // rpp
        if l % 2 or l // 2 > nmma - (mi + ni) or (c["NS"] - 2) * l > 63:
            return False
        if c["BM"] * c["BN"] * 2 > lds_bytes(c):
            return False
        return nmma * 16 + 2 * (mi + ni) * 4 + 40 <= 512 // waves_per_simd
    if (c["BM"] * 8) % nt or (c["BN"] * 8) % nt or (nt // 8) % 16:
        return False
    if mi + ni > nmma or c["BM"] * 8 // nt > nmma or c["BN"] * 8 // nt > nmma:
        return False
    # accumulators (16 regs per 32x32 tile) + fragments + staging must fit 512 / waves-per-SIMD
    regs = nmma * 16 + 2 * (mi + ni) * 4 + (c["BM"] + c["BN"]) * 8 // nt * 4 + 40
    return regs <= 512 // waves_per_simd


def _c(BM, BN, WM, WN, SWZ=1, GROUP=8, OCC=1, DTL=0, EPI=0, EFF=None, EW=None):
    c = dict(KIND="tile", BM=BM, BN=BN, WM=WM, WN=WN, SWZ=SWZ, GROUP=GROUP, OCC=OCC, DTL=DTL, EPI=EPI)
    if EW is not None:
        c["EWM"], c["EWN"] = EW
    if EFF is not None:
        c["EFF"] = EFF
    return c


def _r(BM, BN, WM, WN, NS=4, GROUP=8):
    return dict(KIND="ring", BM=BM, BN=BN, WM=WM, WN=WN, NS=NS, GROUP=GROUP)


def _m(BM, BN, WM, WN, GROUP=4, EFF=None, DRAIN=0, OCC=1, EFF_E=None, KG=1, EDRAIN=None):
    c = dict(KIND="mfma16", BM=BM, BN=BN, WM=WM, WN=WN, GROUP=GROUP)
    if EDRAIN is not None:
        c["EDRAIN"] = EDRAIN        # drain slot of the predicated variant, where it differs
    if KG != 1:
        c["KG"] = KG
    if EFF_E is not None:
        c["EFF_E"] = EFF_E
    if OCC != 1:
        c["OCC"] = OCC
    if DRAIN:
        c["DRAIN"] = DRAIN
    if EFF is not None:
        c["EFF"] = EFF
    return c


def _q(BM, BN, WM, WN, NS=4, GROUP=4):
    return dict(KIND="ring16", BM=BM, BN=BN, WM=WM, WN=WN, NS=NS, GROUP=GROUP)


def _s(BM, NS):
    return dict(KIND="stream", BM=BM, BN=32, NS=NS)


def _k(BM, BN, NS, WK=None, OCC=1, SHARED=0, WK_RAGGED=None, WK_ODD=None):
    c = dict(KIND="wavek", BM=BM, BN=BN, NS=NS)
    if WK_ODD is not None:
        c["WK_ODD"] = WK_ODD           # a K unit's cost when K is odd, relative to an aligned pitch (default 2.0)
    if WK_RAGGED is not None:
        # a K unit's cost when K % 64 != 0, relative to an aligned pitch: K % 8 == 0 with K < 2048 /
        # K >= 2048, other even K with K < 2048 / K >= 2048 (default 1.15, 1.45, 1.45, 1.45)
        c["WK_RAGGED"] = WK_RAGGED
    if SHARED:
        c["SHARED"] = 1         # 2 x 2 waves over the tile and one ring, instead of K split over the waves
    if OCC != 1:
        c["OCC"] = OCC          # workgroups that fit a CU together (LDS): rounds of the time model
    if WK is not None:
        c["WK"] = WK
    return c


def _d(BM, NS, BN=128):
    return dict(KIND="decode", BM=BM, BN=BN, NS=NS)


CONFIGS = [
    _c(256, 256, 2, 2, SWZ=1, GROUP=8),
    _c(256, 256, 2, 2, SWZ=1, GROUP=8, DTL=1),
    _c(256, 256, 2, 2, SWZ=1, GROUP=8, DTL=1, EPI=1),
    _c(256, 256, 2, 2, SWZ=1, GROUP=4, DTL=1, EPI=1, EW=(2, 4)),
    _c(256, 256, 2, 4, SWZ=1, GROUP=8, DTL=1, EPI=1),
    _c(256, 192, 2, 2, SWZ=1, GROUP=4, DTL=1, EPI=1),
    _c(256, 192, 2, 2, SWZ=1, GROUP=4, DTL=1, EPI=1, EW=(4, 2)),
    _c(256, 128, 2, 2, SWZ=1, GROUP=8, DTL=1, EPI=1, EW=(4, 2)),
    _c(128, 256, 2, 2, SWZ=1, GROUP=8, DTL=1, EPI=1, EW=(2, 4)),
    _c(256, 128, 2, 2, SWZ=1, GROUP=8, DTL=1, EPI=1),
    _c(128, 256, 2, 2, SWZ=1, GROUP=8, DTL=1, EPI=1),
    _c(128, 128, 2, 2, SWZ=1, GROUP=8, OCC=2, DTL=1, EPI=1),
    _r(256, 256, 2, 2),
    _r(256, 256, 2, 4),
    _m(256, 256, 2, 2),
    _m(256, 256, 2, 2, DRAIN=3, EDRAIN=1, EFF=1.0, EFF_E=0.86),
    _m(256, 192, 2, 2, DRAIN=3, EDRAIN=1, EFF=0.89, EFF_E=0.92),
    _m(128, 256, 2, 2, DRAIN=1, EFF=0.84, EFF_E=0.80),
    _m(256, 128, 2, 2, DRAIN=1, EFF=0.845, EFF_E=0.80),
    _m(128, 128, 2, 2, DRAIN=1, OCC=2, EFF=0.78, EFF_E=0.74),
    _m(256, 256, 4, 2),
    _m(256, 256, 4, 2, DRAIN=3),
    _m(256, 256, 2, 4),
    _q(256, 256, 4, 2),
    _q(256, 256, 2, 2),
    _s(16, 3),
    _s(32, 3),
    _s(64, 3),
    _m(256, 256, 2, 2, GROUP=8, DRAIN=1),
    _m(192, 192, 2, 2, DRAIN=1, EFF=0.80, EFF_E=0.91),
    _m(192, 128, 2, 2, DRAIN=1, EFF=0.74, EFF_E=0.85),
    _m(128, 128, 2, 2, DRAIN=1, KG=2, EFF=0.64, EFF_E=0.93),
    _d(128, NS=3),
    _d(64, NS=4),
    _k(32, 32, NS=1, OCC=5, WK=(2.18, 0.0, 0.0775, 0.314), WK_RAGGED=(1.26, 1.40, 1.46, 1.48), WK_ODD=1.95),
    _k(32, 32, NS=2, OCC=2, WK=(1.71, 0.153, 0.0753, 0.580), WK_RAGGED=(1.19, 1.43, 1.55, 1.49), WK_ODD=1.97),
    _k(64, 32, NS=3, WK=(0.87, 2.10, 0.1188, 0.0), WK_RAGGED=(1.21, 1.49, 1.83, 1.71), WK_ODD=2.05),
    _k(64, 64, NS=1, OCC=2, WK=(1.93, 2.19, 0.1792, 0.0), WK_RAGGED=(1.00, 1.35, 1.34, 1.51), WK_ODD=1.70),
    _k(64, 64, NS=2, WK=(0.88, 2.81, 0.1648, 0.0), WK_RAGGED=(1.11, 1.49, 1.67, 1.69), WK_ODD=1.97),
    _k(96, 64, NS=2, WK=(1.35, 4.06, 0.2306, 0.0), WK_RAGGED=(0.85, 1.27, 1.25, 1.45), WK_ODD=1.73),
    _k(96, 96, NS=4, SHARED=1, WK=(1.03, 3.336, 0.3179, 0.0), WK_RAGGED=(0.98, 1.24, 1.16, 1.37), WK_ODD=1.58),
    _k(64, 64, NS=4, SHARED=1, OCC=2, WK=(1.31, 1.734, 0.1815, 0.0), WK_RAGGED=(1.06, 1.44, 1.31, 1.60), WK_ODD=1.77),
    _k(96, 64, NS=4, SHARED=1, OCC=2, WK=(1.96, 1.90, 0.2313, 0.217), WK_RAGGED=(0.98, 1.32, 1.21, 1.52), WK_ODD=1.72),
    _k(64, 32, NS=4, SHARED=1, OCC=3, WK=(1.54, 1.362, 0.1234, 0.0), WK_RAGGED=(1.20, 1.49, 1.49, 1.64), WK_ODD=1.92),
    _m(192, 256, 2, 2, DRAIN=1, EFF=0.89, EFF_E=0.92),
    # found by the tuner's sweep of the small-tile kinds at 512^3 (256 tiles, one per CU, eight K
    # units: too few to split over the waves); no time model, a tuned shape only
    _k(32, 32, NS=4, SHARED=1, OCC=4),
]

assert all(is_valid_config(c) for c in CONFIGS), [config_name(c) for c in CONFIGS if not is_valid_config(c)]
assert len({config_name(c) for c in CONFIGS}) == len(CONFIGS)

# Exact shapes with a tuned choice (config name), consulted before the model.  From sweeps of
# the 256x256 family (GROUP 4 / 8 x DRAIN 0 / 1 / 3) at the benchmark shapes: at 8192^3 and
# N = 28672 the default is level with or ahead of the others; at K = 28672 groups 8 tiles tall
# with the earlier drain slot are 1.7 % faster (2.426 against 2.468 ms).
# 512^3: the tuner's sweep of the small-tile kinds (32x32 tiles, one per CU: the 2 x 2 wave grid
# on a shared ring of four stages 3.2 us, K split over the waves 3.6).
TUNED_SHAPES = {(8192, 8192, 28672): "m256x256_w2x2_g8_b1", (512, 512, 512): "k32x32_s4"}
assert all(n in {config_name(c) for c in CONFIGS} for n in TUNED_SHAPES.values())

# The kernels the automatic choice for decode shapes names (select_decode_kernel in
# template/kernel_table.hpp.jinja, where the thresholds and the measurements behind them are).
DECODE_KERNELS = {"stream16": "s16x32_n3", "stream32": "s32x32_n3", "stream64": "s64x32_n3",
                  "decode64": "d64x128_n4", "decode128": "d128x128_n3", "tile128x256": "m128x256_w2x2_g4_b1"}
assert all(n in {config_name(c) for c in CONFIGS} for n in DECODE_KERNELS.values())
