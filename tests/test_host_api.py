"""Host-side checks that need no GPU: the C-ABI library loads and exports every symbol that
include/mi_gemm.h declares, argument validation happens before any device call, the Python
mirror of the reference's host functions behaves like them, the kernel configuration table
is consistent, and the tile-order mapping used by the kernels is a bijection."""
import ctypes
import itertools
import os
import re
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "mi_gemm.h"


def declared_functions():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(mi_[a-z0-9_]+)\s*\(", text)) - {"mi_device_props"})


def test_library_exports_every_declared_symbol(mi):
    from h100_gemm_amd import _lib
    names = declared_functions()
    assert len(names) >= 20
    lib = ctypes.CDLL(str(_lib.LIB_PATH))
    for n in names:
        assert hasattr(lib, n), f"{n} declared in mi_gemm.h but not exported"
    assert set(names) == set(_lib.SYMBOLS), set(names) ^ set(_lib.SYMBOLS)


def test_library_links_no_vendor_blas(mi):
    """The vendor GEMM is a side-by-side program's business (harness/vendor_bench.cpp), never a
    dispatch path of the library: its only run-time dependencies are HIP and the C/C++ runtime."""
    from h100_gemm_amd import _lib
    out = subprocess.run(["readelf", "-d", str(_lib.LIB_PATH)], capture_output=True, text=True, check=True).stdout
    needed = re.findall(r"\(NEEDED\)\s+Shared library: \[([^\]]+)\]", out)
    assert any(n.startswith("libamdhip64") for n in needed)
    assert not [n for n in needed if re.search(r"blas|tensile|miopen|torch", n, re.I)], needed


def test_header_is_plain_c_and_links(mi, tmp_path):
    """include/mi_gemm.h is a C header (what a cgo / JNI / ctypes binding would consume): a C99
    program that takes the address of every declared function compiles with -pedantic -Werror,
    links against the library and runs (no device call is made)."""
    from h100_gemm_amd import _lib
    names = declared_functions()
    src = tmp_path / "abi.c"
    src.write_text('#include "include/mi_gemm.h"\n#include <stdio.h>\ntypedef void (*fn)(void);\n'
                   + "static fn table[] = {" + ", ".join(f"(fn){n}" for n in names) + "};\n"
                   + 'int main(void) {\n    if (sizeof table / sizeof table[0] < 20 || !table[0]) return 1;\n'
                   + '    if (mi_gemm_bf16(0, 1, 1, 0, 0, 0, 0, 0) != MI_ERR_INVALID) return 2;\n'
                   + '    puts(mi_last_error());\n    return mi_gemm_num_configs() > 0 ? 0 : 3;\n}\n')
    exe = tmp_path / "abi"
    libdir = _lib.LIB_PATH.parent
    r = subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Werror", "-Wno-pedantic", f"-I{ROOT}", str(src), "-o", str(exe),
                        f"-L{libdir}", "-lmi_gemm", f"-Wl,-rpath,{libdir}"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    r = subprocess.run([str(exe)], capture_output=True, text=True)
    assert r.returncode == 0 and "positive" in r.stdout, r.stdout + r.stderr


def test_missing_library_fails_loudly(mi, monkeypatch, tmp_path):
    from h100_gemm_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "libmi_gemm.so")
    with pytest.raises(ImportError, match="no fallback"):
        _lib.load()


def test_product_does_not_touch_the_oracle():
    # the oracle is test infrastructure: nothing under the package may import, link or read it
    for p in (ROOT / "h100_gemm_amd").rglob("*"):
        if p.suffix in {".py", ".hpp", ".hip", ".cpp", ".jinja", ".h"} or p.name == "Makefile":
            if "gen" in p.parts:
                continue
            text = p.read_text(errors="ignore")
            assert not re.search(r"\boracle\b", text), f"{p} mentions the oracle"


def test_argument_validation_needs_no_device(mi):
    L = mi._lib.load()
    bf = mi.MI_DTYPE_BF16
    assert L.mi_gemm_bf16(0, 8, 8, 1, 1, 1, None, None) == mi._lib.MI_ERR_INVALID
    assert b"positive" in L.mi_last_error()
    assert L.mi_gemm_bf16(8, 8, 8, None, 1, 1, None, None) == mi._lib.MI_ERR_INVALID
    assert L.mi_gemm_ex(999, bf, 8, 8, 8, 1, 1, 1, None, None) == mi._lib.MI_ERR_INVALID
    assert L.mi_gemm_ex(-1, 7, 8, 8, 8, 1, 1, 1, None, None) == mi._lib.MI_ERR_INVALID
    # size limits: each matrix below 2^31 elements (int indices, as reference.h:30,40), and a
    # 256-row panel of K-long rows within the 32-bit byte offsets of one buffer descriptor
    assert L.mi_gemm_ex(-1, bf, 70000, 70000, 8, 1, 1, 1, None, None) == mi._lib.MI_ERR_INVALID
    assert b"2^31" in L.mi_last_error()
    assert L.mi_gemm_ex(-1, bf, 65536, 8, 32768, 1, 1, 1, None, None) == mi._lib.MI_ERR_INVALID      # M*K = 2^31
    assert L.mi_gemm_ex(-1, bf, 8, 65536, 32768, 1, 1, 1, None, None) == mi._lib.MI_ERR_INVALID      # N*K = 2^31
    assert L.mi_gemm_ex(-1, bf, 1, 1, 4194304, 1, 1, 1, None, None) == mi._lib.MI_ERR_INVALID        # K*512 = 2^31
    assert b"K too large" in L.mi_last_error()
    assert L.mi_reference_gpu_gemm(bf, 8, -1, 8, 1, 1, 1, 1.0, 0.0, None) == mi._lib.MI_ERR_INVALID
    assert L.mi_gemm_epilogue(-1, bf, 8, 8, 8, 1, 1, 1, 1.0, 0.0, 2, None) == mi._lib.MI_ERR_INVALID
    assert b"layout" in L.mi_last_error()
    assert L.mi_gemm_epilogue(-1, bf, 8, 8, 8, 1, 1, 1, float("nan"), 0.0, 0, None) == mi._lib.MI_ERR_INVALID
    assert L.mi_gemm_epilogue(-1, bf, 8, 0, 8, 1, 1, 1, 1.0, 0.0, mi.MI_C_COL_MAJOR, None) == mi._lib.MI_ERR_INVALID
    assert L.mi_gemm_epilogue(-1, bf, 8, 8, 8, 1, None, 1, 1.0, 0.0, mi.MI_C_COL_MAJOR, None) == mi._lib.MI_ERR_INVALID
    # the shape queries apply the same limits instead of computing with extents a launch refuses
    big = 2**31 - 1
    for M, N, K in [(big, big, big), (0, 8, 8), (8, -1, 8), (70000, 70000, 8), (1, 1, 4194304)]:
        assert L.mi_gemm_select_config(bf, M, N, K) == -1
        assert L.mi_gemm_config_supports(0, bf, M, N, K) == 0
        assert L.mi_gemm_config_grid(0, M, N, K) == 0
        assert L.mi_gemm_workspace_bytes(-1, bf, M, N, K, 0) == 0
        assert L.mi_gemm_trace_words(M, N, K) == 1
    with pytest.raises(mi.MiGemmError):
        mi.runKernel(8, 8, 0, 1, 1, 1)
    with pytest.raises(ValueError):
        mi.run_kernel(0, 8, 8, 8, 1, 1, 1)          # 0 = vendor BLAS in the reference
    with pytest.raises(ValueError):
        mi.gpu_gemm(mi.GemmParams(8, 8, 8, 1, 1, 1, alpha=2.0))
    with pytest.raises(ValueError):
        mi.gpu_gemm(mi.GemmParams(8, 8, 8, 1, 1, 1), config="no_such_config")
    with pytest.raises(TypeError):
        mi.runKernel(8, 8, 8, "x", 1, 1)


def test_config_table(mi):
    from h100_gemm_amd import kernel_configs as kc
    n = mi.num_configs()
    assert n == len(kc.CONFIGS) >= 4
    names = [mi.config_name(i) for i in range(n)]
    assert names == [kc.config_name(c) for c in kc.CONFIGS]
    assert mi.config_name(n) is None and mi.config_name(-1) is None
    for i, nm in enumerate(names):
        assert mi.find_config(nm) == i
    assert mi.find_config("nope") == -1
    L = mi._lib.load()
    for i, c in enumerate(kc.CONFIGS):
        assert L.mi_gemm_config_lds_bytes(i) == kc.lds_bytes(c) <= 160 * 1024
        assert kc.is_valid_config(c)
        if c["KIND"] in ("stream", "decode"):
            # decode kernels: M <= BM, whole 64-deep K slabs, N a multiple of 4; no ragged twin
            assert L.mi_gemm_config_supports(i, 0, c["BM"], 8192, 8192) == 1
            assert L.mi_gemm_config_supports(i, 0, c["BM"] + 1, 8192, 8192) == 0
            assert L.mi_gemm_config_supports(i, 0, 16, 8192, 8200) == 0
            assert L.mi_gemm_config_supports(i, 0, 16, 8190, 8192) == 0
            assert mi.config_grid(i, 16, 8192, 8192) >= 64
            assert mi.config_grid(i, c["BM"] + 1, 8192, 8192) == 0
        elif c["KIND"] == "wavek":
            # any M, N and K (operands on 4-byte boundaries, which a shape does not tell); no ragged twin
            assert mi.config_grid(i, 1000, 780, 64) == -(-1000 // c["BM"]) * -(-780 // c["BN"])
            assert L.mi_gemm_config_supports(i, 0, 1000, 780, 4096) == 1
            assert L.mi_gemm_config_supports(i, 0, 1000, 777, 4098) == 1
            assert L.mi_gemm_config_supports(i, 0, 1, 1, 1) == 1
            # a long K may be cut into pieces (one workgroup per tile and piece) where N % 4 == 0
            tiles = mi.config_grid(i, 1000, 780, 64)
            grid = mi.config_grid(i, 1000, 780, 4097)
            assert grid % tiles == 0 and 1 <= grid // tiles <= 4
            assert mi.config_grid(i, 1000, 777, 4097) == -(-1000 // c["BM"]) * -(-777 // c["BN"])
            # (the number of pieces comes from the config's time model: one without a model runs whole)
            if c.get("WK"):
                assert mi.config_grid(i, 128, 384, 13376) > -(-128 // c["BM"]) * -(-384 // c["BN"])
        elif c.get("KG", 1) > 1:
            # K split over groups of waves inside the workgroup: any M, N; K in equal halves of whole double steps
            assert L.mi_gemm_config_supports(i, 0, 4095, 6143, 3072) == 1
            assert L.mi_gemm_config_supports(i, 0, 4095, 6143, 3073) == 0
            assert L.mi_gemm_config_supports(i, 0, 512, 512, 384) == 0
            assert mi.config_grid(i, 1000, 777, 256) == -(-1000 // c["BM"]) * -(-777 // c["BN"])
        else:
            tiles = -(-1000 // c["BM"]) * -(-777 // c["BN"])
            assert mi.config_grid(i, 1000, 777, 64) == tiles
            assert L.mi_gemm_config_supports(i, 0, 4095, 6143, 3073) == 1
    assert mi.config_grid(0, 0, 8, 8) == 0
    # the automatic choice is a valid index for every benchmark shape
    for M, N, K in [(512, 512, 512), (8192, 8192, 8192), (8192, 28672, 8192), (8192, 8192, 28672),
                    (16, 8192, 8192), (64, 8192, 8192), (128, 8192, 8192), (4095, 6143, 3073)]:
        assert 0 <= mi.select_config(M, N, K) < n
        assert L.mi_gemm_trace_words(M, N, K) >= 7
    kinds = {kc.CONFIGS[mi.select_config(M, 8192, 8192)]["KIND"] for M in (16, 64, 128)}
    assert kinds <= {"stream", "decode"}
    assert kc.CONFIGS[mi.select_config(16, 8192, 8200)]["KIND"] not in ("stream", "decode")     # K % 64 != 0
    assert kc.CONFIGS[mi.select_config(8192, 8192, 8192)]["KIND"] in ("tile", "ring", "mfma16")
    # exact shapes with a tuned entry take it; everything else goes through the cost model
    for (M, N, K), name in kc.TUNED_SHAPES.items():
        assert mi.config_name(mi.select_config(M, N, K)) == name
    assert kc.CONFIGS[mi.select_config(8192, 8192, 8192)]["KIND"] == "mfma16"
    assert kc.CONFIGS[mi.select_config(4096, 4096, 4096)]["KIND"] == "mfma16"
    # few tiles and a long K: small tiles with K split over the waves, when the kernel can run the shape
    assert kc.CONFIGS[mi.select_config(512, 512, 4096)]["KIND"] == "wavek"
    assert kc.CONFIGS[mi.select_config(1024, 1024, 4096)]["KIND"] == "wavek"
    assert kc.CONFIGS[mi.select_config(512, 512, 4100)]["KIND"] == "wavek"     # any K and any N will do
    assert kc.CONFIGS[mi.select_config(512, 510, 4096)]["KIND"] == "wavek"
    assert kc.CONFIGS[mi.select_config(512, 511, 4101)]["KIND"] == "wavek"
    # a mid-sized output with a K of moderate length: small tiles on a shared ring (K is not split
    # over the waves), also with a short K and many tiles, where the K-splitting ones are shut out
    assert not kc.CONFIGS[mi.select_config(512, 512, 4096)].get("SHARED")
    for M, N, K in [(1440, 1440, 1472), (1344, 1344, 1344), (1536, 1472, 320)]:
        c = kc.CONFIGS[mi.select_config(M, N, K)]
        assert c["KIND"] == "wavek" and c.get("SHARED") == 1, (M, N, K, c)
    assert mi.config_name(mi.select_config(1536, 1536, 1536)) == "k96x96_s4"               # 256 tiles of 96x96, one per CU
    assert mi.config_name(mi.select_config(2048, 2048, 2048)) == "m128x128_w2x2_g4_b1_k2"  # 256 tiles of 128x128, two K groups each
    # wave quantisation: 256 CUs; 8192^2 fills four rounds of 256x256 tiles, 4095x6143 fills
    # two rounds of 256x192 tiles exactly (256x256 would leave half of the second round
    # idle), and 512^2 is a single partial round whatever the tiled kernel: the small-tile
    # kernel gives every CU a 32x32 tile
    def picked(M, N, K):
        c = kc.CONFIGS[mi.select_config(M, N, K)]
        return c["BM"], c["BN"]
    assert picked(8192, 8192, 8192) == (256, 256)
    assert picked(8192, 28672, 8192) == (256, 256)
    assert picked(4095, 6143, 3073) == (256, 192)
    assert picked(512, 512, 512) == (32, 32)
    assert kc.CONFIGS[mi.select_config(512, 512, 512)]['KIND'] == 'wavek'
    assert kc.CONFIGS[mi.select_config(512, 512, 521)]['KIND'] == 'wavek'      # a ragged K too
    assert all("EFF" in kc.CONFIGS[mi.select_config(M, N, 4101)] for M in (3000, 5000) for N in (3000, 6001))   # large: tiled
    # a large ragged shape whose last row of tiles is nearly empty runs as two GEMMs: the rows up to
    # the last full row of tiles, then the rest; shapes that fill their rounds, small ones and
    # tuned ones run whole
    assert mi.row_cut(7000, 7000, 7000) == 6912 and mi.row_cut(7000, 7000, 4096) == 6912
    for M, N, K in [(8192, 8192, 8192), (6000, 6000, 6000), (5000, 8192, 4096), (4095, 6143, 3073), (1000, 1000, 1000),
                    (8192, 8192, 28672), (0, 8, 8)]:
        assert mi.row_cut(M, N, K) == 0, (M, N, K)
    assert mi.workspace_bytes(7000, 7000, 7000) >= mi.workspace_bytes(88, 7000, 7000, config=mi.select_config(88, 7000, 7000))
    # a few small tiles and a very long K: the small-tile kernels cut K over workgroups too, and
    # the workspace query covers their pieces' sums; an odd N cannot be reduced and runs whole
    c = mi.select_config(128, 384, 13376)
    assert kc.CONFIGS[c]["KIND"] == "wavek"
    pieces = mi.config_grid(c, 128, 384, 13376) // mi.config_grid(c, 128, 384, 64)
    assert 2 <= pieces <= 16 and mi.workspace_bytes(128, 384, 13376) >= pieces * 128 * 384 * 4
    assert mi.workspace_bytes(128, 383, 13376) == 0
    assert kc.CONFIGS[mi.select_config(4828, 413, 13248)]["KIND"] == "wavek"    # narrow output, very long K: beyond 48 MB of operands
    assert kc.CONFIGS[mi.select_config(448, 4864, 8192)]["KIND"] == "mfma16"
    # few tiles and a long K: split-K pieces of a tiled kernel fill the CUs
    c = mi.select_config(256, 8192, 8192)
    assert kc.CONFIGS[c]["KIND"] == "mfma16" and (kc.CONFIGS[c]["BM"], kc.CONFIGS[c]["BN"]) == (256, 128)
    assert 128 < mi.config_grid(c, 256, 8192, 8192) <= 256          # 64 tiles x 3 or 4 pieces
    c = mi.find_config("m128x128_w2x2_g4_b1_o2")                    # (the automatic choice is the small-tile kernel)
    assert mi.config_grid(c, 512, 512, 4096) == 16 * 8              # 128x128 tiles x 8 pieces of 512
    assert mi.config_grid(mi.select_config(8192, 8192, 8192), 8192, 8192, 8192) == 1024   # no split-K when the tiles fill the chip
    c = mi.find_config("m128x128_w2x2_g4_b1_o2")
    assert mi.config_grid(c, 512, 512, 521) == 16                                         # nor for a short K
    assert mi.config_grid(mi.select_config(512, 512, 512), 512, 512, 512) == 256          # 32x32 tiles, one per CU
    c = mi.select_config(512, 510, 4097)
    assert mi.config_grid(c, 512, 510, 4097) == -(-512 // kc.CONFIGS[c]["BM"]) * -(-510 // kc.CONFIGS[c]["BN"])   # N % 4 != 0: no split-K
    assert "EFF" in kc.CONFIGS[mi.select_config(200, 8190, 8192)]        # N % 4 != 0: tiled
    assert not kc.is_valid_config(dict(KIND="tile", BM=256, BN=256, WM=2, WN=2, SWZ=1, GROUP=8, OCC=2, DTL=0, EPI=0))
    assert not kc.is_valid_config(dict(KIND="tile", BM=96, BN=256, WM=2, WN=2, SWZ=1, GROUP=8, OCC=1, DTL=0, EPI=0))
    assert not kc.is_valid_config(dict(KIND="ring", BM=256, BN=256, WM=2, WN=2, NS=5, GROUP=8))
    assert not kc.is_valid_config(dict(KIND="decode", BM=48, BN=128, NS=4))
    assert not kc.is_valid_config(dict(KIND="decode", BM=128, BN=128, NS=9))     # vmcnt is 6 bits


def tile_of_block(pid, nwg, tiles_m, tiles_n, group):
    """Python model of mi::tile_of_block (gemm_kernel.hpp)."""
    q, r = nwg >> 3, nwg & 7
    x, loc = pid & 7, pid >> 3
    logical = x * q + min(x, r) + loc
    gw = group * tiles_n
    gid = logical // gw
    first = gid * group
    gsz = min(tiles_m - first, group)
    inn = logical - gid * gw
    return first + inn % gsz, inn // gsz


def test_tile_order_is_a_bijection():
    for tm, tn, g in itertools.product([1, 2, 3, 7, 16, 24, 32, 33], [1, 2, 5, 24, 32, 112], [1, 4, 8, 16]):
        nwg = tm * tn
        seen = {tile_of_block(p, nwg, tm, tn, g) for p in range(nwg)}
        assert len(seen) == nwg and all(0 <= a < tm and 0 <= b < tn for a, b in seen)
    # XCD locality: the 128 workgroups that land on XCD 0 of an 8192^2 launch (ids 0, 8, 16, ..)
    # own a compact 8 x 16 block of tiles
    tiles = {tile_of_block(p, 1024, 32, 32, 8) for p in range(0, 1024, 8)}
    rows = {t[0] for t in tiles}
    cols = {t[1] for t in tiles}
    assert len(rows) == 8 and len(cols) == 16


def test_harness_header_is_plain_host_cxx(tmp_path):
    # gemm_host.hpp must compile with a host compiler alone (no HIP headers) and keep the
    # reference's names and signatures usable
    src = tmp_path / "t.cpp"
    src.write_text(r'''
#include "h100_gemm_amd/harness/gemm_host.hpp"
int main() {
    std::vector<int> s = {2, 3};
    bf16* a = alloc_cpu_tensor<bf16>(s);
    random_fill(a, s); arange_fill(a, s); constant_fill(a, s, bf16(1.5f));
    GemmParams<bf16, bf16, bf16, float> p(2, 2, 3, a, a, a, 1.0f, 0.0f);
    void (*f1)(int, int, int, bf16*, bf16*, bf16*, int*) = runKernel;
    void (*f2)(int, int, int, int, bf16*, bf16*, bf16*, int*) = run_kernel;
    (void)f1; (void)f2; (void)p;
    CPUTimer t; t.tick(); t.tick(); (void)t.report_last_ms();
    float x = (float)bf16(1.00390625f);      // tie -> even
    float y = (float)half_t(65520.0f);       // overflow -> inf
    const bool filled = (float)a[0] == 1.5f;  // constant_fill was the last fill
    free_cpu_tensor(a);
    return (x == 1.0f && std::isinf(y) && filled) ? 0 : 1;
}
''')
    exe = tmp_path / "t"
    r = subprocess.run(["g++", "-std=c++17", "-O1", f"-I{ROOT}", str(src), "-o", str(exe),
                        f"-L{ROOT}/h100_gemm_amd/lib", "-lmi_gemm",
                        f"-Wl,-rpath,{ROOT}/h100_gemm_amd/lib"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    assert subprocess.run([str(exe)]).returncode == 0


def test_harness_fills_match_the_oracle(orc, tmp_path):
    # the harness' seeded fills (product side, C++) and the oracle's (C) are two
    # implementations of the same generators: same bits
    src = tmp_path / "f.cpp"
    src.write_text(r'''
#include <cstdio>
#include "h100_gemm_amd/harness/gemm_host.hpp"
int main() {
    std::vector<int> s = {4096};
    std::vector<bf16> u(4096), n(4096);
    uniform_fill(u.data(), s, 69, 1); normal_fill(n.data(), s, 69, 2, 0.02f);
    fwrite(u.data(), 2, 4096, stdout); fwrite(n.data(), 2, 4096, stdout);
    return 0;
}
''')
    exe = tmp_path / "f"
    r = subprocess.run(["g++", "-std=c++17", "-O1", f"-I{ROOT}", str(src), "-o", str(exe),
                        f"-L{ROOT}/h100_gemm_amd/lib", "-lmi_gemm",
                        f"-Wl,-rpath,{ROOT}/h100_gemm_amd/lib"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    raw = subprocess.run([str(exe)], capture_output=True).stdout
    got = np.frombuffer(raw, dtype=np.uint16)
    assert (got[:4096] == orc.fill_uniform((4096,), 69, 1)).all()
    assert (got[4096:] == orc.fill_normal((4096,), 69, 2, 0.02)).all()


def test_tuner_write_tuned_mode_without_shapes_writes_nothing(mi, tmp_path):
    """`gemm_tuner --write-tuned FILE MxNxK ...` times the library's compiled candidates on the
    GPU (tune_library_choice); with no shapes it touches neither the GPU nor the file"""
    from h100_gemm_amd import gemm_tuner
    out = tmp_path / "tuned.txt"
    assert gemm_tuner.main(["--write-tuned", str(out)]) == 0
    assert not out.exists()
    assert gemm_tuner.tune_library_choice([], str(out)) == []


def test_tuned_shapes_file_overrides_the_model(mi, tmp_path):
    """MI_GEMM_TUNED_FILE: `M N K config-name` lines, read once per process, consulted before
    the time model; malformed lines, unknown names and decode configurations whose
    preconditions the shape violates are ignored."""
    tuned = tmp_path / "tuned.txt"
    tuned.write_text("# shapes tuned on this machine\n"
                     "8192 8192 8192 m256x256_w2x2_g8_b1   # not the model's choice\n"
                     "1000 1000 1000 m256x192_w2x2_g4_b3\n"
                     "512 512 512 no_such_config\n"
                     "this line does not parse\n"
                     "4096 4096 4096 d128x128_n3            # decode kernel: M too large, ignored at use\n"
                     "64 8192 8192 s64x32_n3\n")
    code = ("import h100_gemm_amd as mi\n"
            "L = mi._lib.load()\n"
            "print(L.mi_gemm_tuned_entries())\n"
            "for s in [(8192, 8192, 8192), (1000, 1000, 1000), (512, 512, 512), (4096, 4096, 4096), (64, 8192, 8192), (8192, 8192, 4096)]:\n"
            "    print(mi.config_name(mi.select_config(*s)))\n")
    env = dict(os.environ, MI_GEMM_TUNED_FILE=str(tuned), PYTHONPATH=str(ROOT))
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=env, cwd=ROOT)
    assert out.returncode == 0, out.stderr
    lines = out.stdout.split()
    assert lines[0] == "4"                                   # four lines name a compiled configuration
    assert lines[3] == "k32x32_s4"                           # no_such_config is ignored: the library's own choice for the shape
    assert lines[1:3] + lines[4:] == ["m256x256_w2x2_g8_b1", "m256x192_w2x2_g4_b3",
                                      "m256x256_w2x2_g4_b3", "s64x32_n3", "m256x256_w2x2_g4_b3"], lines
    assert mi._lib.load().mi_gemm_tuned_entries() == 0       # this process has no such file



def test_bench_tables_are_well_formed(mi):
    """bench.py's workload table names shapes and fills; its profile constants name a compiled
    configuration each and only workloads that exist; more than one GPU is refused."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench_module", ROOT / "bench.py")
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    for name, w in bench.WORKLOADS.items():
        M, N, K, fill = w
        assert all(isinstance(v, int) and v > 0 for v in (M, N, K)) and fill in ("uniform", "normal", "int"), name
        assert 0 <= mi.select_config(M, N, K) < mi.num_configs()
    for name in ("square512", "square8192", "mlp_up", "mlp_down", "skinny16", "skinny64", "skinny128", "unaligned"):
        assert name in bench.WORKLOADS                   # the BASELINE configurations
    for name, (config, nbytes) in bench.MEASURED_TRAFFIC_BYTES.items():
        assert name in bench.WORKLOADS and mi.find_config(config) >= 0 and nbytes > 0, name
    # every traffic figure is the one the profile it cites shows (thousands separated by a space there)
    for name, (config, profile, fetch, write) in bench.MEASURED_TRAFFIC_KIB.items():
        text = (ROOT / "profiles" / profile).read_text()
        for kib in (*fetch, *write):
            assert f"{kib:,}".replace(",", " ") in text or str(kib) in text, f"{name}: {kib} KiB is not in profiles/{profile}"
        assert f"`{config}`" in text or config in text, f"{name}: profiles/{profile} is not about {config}"
    assert set(bench.BASELINE_WORKLOADS) <= set(bench.WORKLOADS) and len(bench.BASELINE_WORKLOADS) == 8
    assert bench.bound_of(512, 512, 512) == "launch" and bench.bound_of(8192, 8192, 8192) == "mfma"
    assert bench.bound_of(16, 8192, 8192) == "hbm" and bench.bound_of(128, 8192, 8192) == "hbm"
    assert bench.bound_of(4095, 6143, 3073) == "mfma" and bench.bound_of(8192, 8192, 28672) == "mfma"
    out = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, cwd=ROOT)
    assert out.returncode == 2 and "ONE GPU" in out.stderr


def test_automatic_choice_always_names_a_kernel_that_can_run_the_shape(mi):
    """For any shape the automatic choice is a configuration that supports it (the decode and
    small-tile kernels have preconditions on M, N % 4 and K % 64; everything else has a
    predicated variant) with a non-empty grid -- seeded random shapes over every regime of the
    choice, and the same answer when asked twice."""
    import numpy as np
    from h100_gemm_amd import kernel_configs as kc
    L = mi._lib.load()
    rng = np.random.default_rng(20)
    picks = set()
    for it in range(4000):
        kind = it % 5
        if kind == 0:       # decode
            M, N, K = rng.integers(1, 129), 4 * rng.integers(1, 8000), 64 * rng.integers(1, 400)
        elif kind == 1:     # few tiles
            M, N, K = rng.integers(1, 2049), 4 * rng.integers(1, 513), 64 * rng.integers(1, 257)
        elif kind == 2:     # arbitrary
            M, N, K = rng.integers(1, 9000), rng.integers(1, 9000), rng.integers(1, 9000)
        elif kind == 3:     # large, aligned
            M, N, K = 256 * rng.integers(1, 40), 256 * rng.integers(1, 120), 128 * rng.integers(1, 230)
        else:               # extreme aspect ratios
            M, N, K = rng.choice([1, 3, 100000]), rng.choice([1, 4, 8, 200000]), rng.choice([1, 64, 4096, 100000])
        M, N, K = int(M), int(N), int(K)
        c = mi.select_config(M, N, K)
        if max(M * K, N * K, M * N) > 2**31 - 1:          # a shape no launch accepts
            assert c == -1, (M, N, K, c)
            continue
        assert 0 <= c < mi.num_configs(), (M, N, K, c)
        assert L.mi_gemm_config_supports(c, 0, M, N, K) == 1, (M, N, K, mi.config_name(c))
        assert mi.config_grid(c, M, N, K) > 0, (M, N, K, mi.config_name(c))
        assert mi.select_config(M, N, K) == c
        picks.add(kc.CONFIGS[c]["KIND"])
    assert picks >= {"mfma16", "stream", "decode", "wavek"}
