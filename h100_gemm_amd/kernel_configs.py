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
             or four waves, csrc/gemm_mfma16_kernel.hpp), or "skinny" (split-K streaming kernel for
             M <= BM, decode shapes)
    EPI      1: C tile transposed through LDS and written 16 bytes per lane, 0: 8-byte stores
    DRAIN    (mfma16, optional) d > 0: a second barrier early in each K step (4*d MFMAs after the
             fragment reads) frees the current LDS stage, so the next loads are spread over most
             of the step instead of its second half
    EWM, EWN (optional) wave grid of the predicated twin when it differs from WM, WN (the
             register-staged predicated kernel runs best with eight waves)
    EFF      (optional) per-CU throughput relative to the 256x256 tile, measured at 8192^3;
             configs that carry it are the candidates of the automatic shape -> kernel choice
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
        return name
    if c["KIND"] == "ring16":
        return f"q{c['BM']}x{c['BN']}_w{c['WM']}x{c['WN']}_n{c['NS']}_g{c['GROUP']}"
    if c["KIND"] == "skinny":
        return f"k{c['BM']}x{c['BN']}_n{c['NS']}"
    if c["KIND"] == "stream":
        return f"s{c['BM']}x{c['BN']}_n{c['NS']}"
    name = (f"t{c['BM']}x{c['BN']}_w{c['WM']}x{c['WN']}_s{c['SWZ']}_g{c['GROUP']}"
            f"_o{c['OCC']}_d{c['DTL']}_e{c['EPI']}")
    if (c.get("EWM", c["WM"]), c.get("EWN", c["WN"])) != (c["WM"], c["WN"]):
        name += f"_x{c['EWM']}x{c['EWN']}"
    return name


def threads(c: dict) -> int:
    return 256 if c["KIND"] in ("skinny", "stream") else c["WM"] * c["WN"] * 64


def lds_bytes(c: dict) -> int:
    if c["KIND"] in ("ring", "ring16"):
        return c["NS"] * (c["BM"] + c["BN"]) * 64
    if c["KIND"] == "skinny":
        return c["NS"] * (c["BM"] + c["BN"]) * 128
    if c["KIND"] == "stream":
        return 4 * c["NS"] * (c["BM"] + c["BN"]) * 128
    return 2 * (c["BM"] + c["BN"]) * 128


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
    if c["KIND"] == "skinny":
        return (c["BM"] % 32 == 0 and c["BN"] % 128 == 0 and c["NS"] >= 3
                and ((c["BM"] + c["BN"]) // 8) % 4 == 0
                and (c["NS"] - 1) * ((c["BM"] + c["BN"]) // 32) <= 63
                and lds_bytes(c) <= 160 * 1024)
    nt = c["WM"] * c["WN"] * 64
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
        if nt not in (256, 512) or c["BM"] * c["BN"] * 2 > lds_bytes(c):
            return False
        mi16, ni16 = 2 * mi, 2 * ni
        rpp = nt // 8 if c["KIND"] == "mfma16" else nt // 4
        if c["BM"] % rpp or c["BN"] % rpp:
            return False
        l = c["BM"] // rpp + c["BN"] // rpp
        if c["KIND"] == "ring16" and (c["NS"] != 4 or (c["NS"] - 1) * l > 63):
            return False
        tn = c["BN"] // c["WN"]
        if tn < 32 or (c["KIND"] == "ring16" and tn & (tn - 1)):   # ring16: C staging needs a power-of-two row
            return False
        if c["KIND"] == "mfma16" and c.get("DRAIN", 0):
            sa = mi16 + ni16 + 4 * c["DRAIN"]
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


def _m(BM, BN, WM, WN, GROUP=4, EFF=None, DRAIN=0, OCC=1, EFF_E=None):
    c = dict(KIND="mfma16", BM=BM, BN=BN, WM=WM, WN=WN, GROUP=GROUP)
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


def _k(BM, BN=128, NS=4):
    return dict(KIND="skinny", BM=BM, BN=BN, NS=NS)


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
    _m(256, 256, 2, 2, DRAIN=3, EFF=1.0, EFF_E=0.82),
    _m(256, 192, 2, 2, DRAIN=3, EFF=0.89, EFF_E=0.90),
    _m(128, 256, 2, 2, DRAIN=1, EFF=0.875, EFF_E=0.80),
    _m(256, 128, 2, 2, DRAIN=1, EFF=0.845, EFF_E=0.80),
    _m(128, 128, 2, 2, DRAIN=1, OCC=2, EFF=0.78, EFF_E=0.74),
    _m(256, 256, 4, 2),
    _m(256, 256, 4, 2, DRAIN=3),
    _m(256, 256, 2, 4),
    _q(256, 256, 4, 2),
    _q(256, 256, 2, 2),
    _s(16, 5),
    _s(32, 4),
    _s(64, 3),
    _k(32, NS=4),
    _k(64, NS=6),
    _k(128, NS=5),
    _m(256, 256, 2, 2, GROUP=8, DRAIN=1),
    _m(192, 192, 2, 2, DRAIN=1, EFF=0.80, EFF_E=0.91),
    _m(192, 128, 2, 2, DRAIN=1, EFF=0.74, EFF_E=0.85),
]

assert all(is_valid_config(c) for c in CONFIGS), [config_name(c) for c in CONFIGS if not is_valid_config(c)]
assert len({config_name(c) for c in CONFIGS}) == len(CONFIGS)

# Exact shapes with a tuned choice (config name), consulted before the model.  From sweeps of
# the 256x256 family (GROUP 4 / 8 x DRAIN 0 / 1 / 3) at the benchmark shapes: at 8192^3 and
# N = 28672 the default is level with or ahead of the others; at K = 28672 groups 8 tiles tall
# with the earlier drain slot are 1.7 % faster (2.426 against 2.468 ms).
TUNED_SHAPES = {(8192, 8192, 28672): "m256x256_w2x2_g8_b1"}
assert all(n in {config_name(c) for c in CONFIGS} for n in TUNED_SHAPES.values())

# Automatic choice for decode shapes (the kernels' preconditions permitting): (largest M,
# config name, further condition on N and K as a C expression), first match wins; shapes that
# match no step go to the tiled kernels (with split-K where the time model wants it).
# Up to M = 32 the single-pass kernel, always (16 x 1024 x 8192: 10.6 us against 13.1 us tiled;
# 16 x 8192 x 28672: 80 against 87).  The split-K decode kernels are ahead for wide B
# (N = 28672: 83 against 120 us at M = 64, 113 against 122 us at M = 128) and level at
# N = 8192 for 8192 <= K <= 16384; the tiled kernels win for narrow B (M = 128, N <= 4096:
# 11-20 against 14-21 us; M = 64, N = 2048: 12.5 against 14.2 us) and for very long K
# (8192 x 28672: 97 against 105 us at M = 64, 106 against 136 us at M = 128).
# Measured with B rotated through enough copies to come from HBM (selection_check, decode mode):
#  * vocabulary-wide B with a short K (N >= 32768, K <= 4096): the split-K kernel's 128-row
#    workgroups beat the single-pass kernel's 32-row ones (32 x 32768 x 4096: 47.5 against
#    54 us; 32 x 65536 x 4096: 93 against 106);
#  * 32 < M <= 64 with a short K: the single-pass kernel, no second launch (64 x 8192 x 2048:
#    10.1 against 12.8 us; 40 x 2048 x 4096: 9.5 against 11.4; level with split-K from K = 8192),
#    but not for wide B (64 x 28672 x 1024: 24.8 against 14.5 us for split-K);
#  * 64 < M <= 128, N = 8192: 128x256 tiles from K = 10240 (12288: 50-53 against 54-62 us;
#    20480: 73-77 against 87-98), except where the row pitch is a power of two (16384: 79-82
#    against 61-68 us: the tiled kernels' rows then start in the same few memory channels).
#  * narrow B with a long K at M <= 32 (N < 4096: fewer 32-row workgroups than CUs, each
#    walking all of K alone) from K = 12288: split-K spreads K over the idle CUs (21 x 1792 x
#    12288: 16.7 against 27.3 us; 32 x 2048 x 28672: 32 against 70; at K = 8192 the single pass
#    is still ahead, 8 x 1024 x 8192: 10.3 against 15.1);
#  * 64 < M <= 128: the split-K decode kernel from N = 12288 (74 x 14336 x 5120: 38 against
#    42 us; 81 x 15360 x 6848: 47 against 55).
#  * the single-pass kernel runs N / 32 workgroups, best when they fill whole rounds of the 256
#    CUs (N = 8192, 16384): at N = 4096, 5120, 9216, 10240, 12288, 18432 (under 80 % of the
#    last round's CUs busy) split-K is 5-30 % ahead once B is large enough to hide its
#    second launch (32 x 5120 x 12288: 28.5 against 35.3 us; 13 x 10240 x 16384: 63 against 70;
#    32 x 12288 x 8192: 40 against 44; but 32 x 4096 x 4096: 14 against 10.6).
_STREAM_ROUNDS_UNDER_80 = "((N + 31) / 32) * 5 < ((((N + 31) / 32) + 255) / 256) * 1024"
DECODE_LADDER = [(32, "k64x128_n6", "(N >= 32768 && K <= 4096) || (N < 4096 && K >= 12288) || "
                                    "(" + _STREAM_ROUNDS_UNDER_80 + " && (long long)N * K >= 50331648LL)"),
                 (16, "s16x32_n5", "true"), (32, "s32x32_n4", "true"),
                 (64, "s64x32_n3", "N <= 12288 && (K <= 4096 || (N >= 4096 && K <= 6144))"),
                 # (also for 32 < M <= 64: 48 x 6584 x 15360 45 against 56 us, 47 x 6144 x 23552 63 against 70)
                 (128, "m128x256_w2x2_g4_b1", "N >= 4096 && N < 12288 && K >= 10240 && K < 24576 && (K & (K - 1)) != 0"),
                 # (narrower B with a long K: 64 x 3328 x 15808 29.4 against 32.4 us tiled, 80 x 2104 x 18432
                 # 27.2 against 29.0, 96 x 3636 x 23552 51 against 55.5)
                 (64, "k64x128_n6", "(N >= 4096 && K < 24576) || (N >= 2048 && N < 4096 && K >= 12288 && K < 24576)"),
                 (128, "k128x128_n5", "N >= 2048 && N < 4096 && K >= 12288"),
                 (128, "k128x128_n5", "N >= 12288 || (N >= 8192 && K >= 8192 && K < 24576)"),
                 # very long K: 128x256 tiles (one row of tiles covers M, B is read once) in split-K
                 # pieces: 97 / 106 us at M = 64 / 128 against 105 / 136 us for the decode kernels
                 # and 115-143 us for the other tiles, between which the time model cannot tell
                 (128, "m128x256_w2x2_g4_b1", "N >= 4096 && K >= 24576")]
assert all(n in {config_name(c) for c in CONFIGS} for _, n, _ in DECODE_LADDER)
