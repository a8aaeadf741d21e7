"""Parity of the gfx950 kernels with the CPU oracle, through the C ABI (libmi_gemm.so).

Tolerance (floating point, stated by the benchmark definition): per element
    |out - ref| <= 2^-7 * |ref| + 1e-3 * sqrt(K) * max|a| * max|b|
with `ref` the oracle's restatement of reference_cpu_gemm on the same seeded inputs.  With
the reference's integer random_fill every partial sum is an exact integer, so there the
bar is bit-exact.  Full-size shapes are compared on a fixed sample of 64x64 tiles (every
tile of reference.h is independent, so a sampled tile holds exactly the full run's values)
plus size-independent properties (row/column permutation equivariance, identity, run-to-run
determinism).
"""
import os
import re
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent


class Dev:
    """Device copies of A, B and an output buffer; frees on exit."""

    def __init__(self, mi, A, B, M, N, pad=0):
        self.mi, self.M, self.N, self.pad = mi, M, N, pad
        self.dA = mi.DeviceBuffer.from_numpy(A)
        self.dB = mi.DeviceBuffer.from_numpy(B)
        self.dC = mi.DeviceBuffer(M * N * 2 + 64)
        self.dC.fill_bytes(0xFF)

    def run(self, K, config=-1, dtype=0, DB=None):
        p = self.mi.GemmParams(self.M, self.N, K, self.dA, self.dB, self.dC)
        self.mi.gpu_gemm(p, config=config, dtype=dtype, DB=DB)
        self.mi.synchronize()
        return self.dC.to_numpy((self.M, self.N), np.uint16)

    def run_epilogue(self, K, alpha, beta, c_layout=0, config=-1, dtype=0):
        p = self.mi.GemmParams(self.M, self.N, K, self.dA, self.dB, self.dC, alpha, beta)
        self.mi.gemm_epilogue(p, config=config, dtype=dtype, c_layout=c_layout)
        self.mi.synchronize()
        shape = (self.N, self.M) if c_layout == self.mi.MI_C_COL_MAJOR else (self.M, self.N)
        return self.dC.to_numpy(shape, np.uint16)


def make_inputs(orc, M, N, K, fill, dtype=0, seed=69):
    if fill == "uniform":
        return orc.fill_uniform((M, K), seed, 1, dtype), orc.fill_uniform((N, K), seed, 2, dtype)
    if fill == "normal":      # activations N(0,1), weights N(0, 0.02^2)
        return orc.fill_normal((M, K), seed, 1, 1.0, dtype), orc.fill_normal((N, K), seed, 2, 0.02, dtype)
    if fill == "int":
        return orc.fill_randint((M, K), seed, 1, dtype), orc.fill_randint((N, K), seed, 2, dtype)
    raise ValueError(fill)


def check(mi, orc, M, N, K, fill, config=-1, dtype=0, tiles=None, exact=False):
    print(f"case M={M} N={N} K={K} fill={fill} config={config} dtype={dtype}", flush=True)
    A, B = make_inputs(orc, M, N, K, fill, dtype)
    C = Dev(mi, A, B, M, N).run(K, config, dtype)
    ref = orc.reference_cpu_gemm(A, B, dtype=dtype, tiles=tiles)
    rep = orc.check_tolerance(C, ref, K, orc.max_abs(A, dtype), orc.max_abs(B, dtype), dtype, tiles=tiles)
    assert rep["violations"] == 0, rep
    assert rep["compared"] > 0
    if exact:
        assert tiles is None
        assert (C == ref).all(), f"{int((C != ref).sum())} elements differ"
    return C, ref, rep


# ---------------------------------------------------------------- benchmark configs ----

def test_c1_square_512(mi, orc):
    check(mi, orc, 512, 512, 512, "uniform")


def test_c2_square_8192_sampled_tiles(mi, orc):
    tiles = orc.sample_tiles(8192, 8192, 256)
    check(mi, orc, 8192, 8192, 8192, "uniform", tiles=tiles)


@pytest.mark.parametrize("M,N,K", [(8192, 28672, 8192), (8192, 8192, 28672)])
def test_c3_mlp_shapes_sampled_tiles(mi, orc, M, N, K):
    tiles = orc.sample_tiles(M, N, 256)
    check(mi, orc, M, N, K, "normal", tiles=tiles)


@pytest.mark.parametrize("M,N,K,fill", [(8192, 8192, 8192, "uniform"), (8192, 28672, 8192, "normal"),
                                        (8192, 8192, 28672, "normal")])
def test_c2_c3_full_matrix_against_the_gpu_golden(mi, orc, M, N, K, fill):
    """Every element of the large benchmark shapes, the way the reference's own harness checks
    them (matmul_h100.cu.jinja:1043-1058: whole matrix against reference_gpu_gemm): the
    on-device golden (ascending-k fp32 sums, bit-identical to the CPU oracle, which 256
    sampled tiles re-confirm here at full size) and the kernel's result are copied back and
    compared element by element with the benchmark tolerance."""
    print(f"case full matrix M={M} N={N} K={K} fill={fill}", flush=True)
    A, B = make_inputs(orc, M, N, K, fill)
    d = Dev(mi, A, B, M, N)
    C = d.run(K)
    dG = mi.DeviceBuffer(M * N * 2)
    dG.fill_bytes(0xFF)
    mi.reference_gpu_gemm(mi.GemmParams(M, N, K, d.dA, d.dB, dG, 1.0, 0.0))
    mi.synchronize()
    G = dG.to_numpy((M, N), np.uint16)
    rep = orc.check_tolerance(C, G, K, orc.max_abs(A), orc.max_abs(B))
    assert rep["violations"] == 0 and rep["compared"] == M * N, rep
    tiles = orc.sample_tiles(M, N, 256)
    ref = orc.reference_cpu_gemm(A, B, tiles=tiles)
    for tm, tn in np.asarray(tiles).reshape(-1, 2):
        blk = (slice(tm * 64, tm * 64 + 64), slice(tn * 64, tn * 64 + 64))
        assert (G[blk] == ref[blk]).all(), f"golden differs from the oracle in tile ({tm}, {tn})"


def test_c3_mlp_up_permutation_equivariance_and_determinism(mi, orc):
    """Size-independent properties at a full MLP shape: run-to-run bit identity and
    equivariance under row permutations of A and of B (an element's value does not depend on
    which tile, workgroup or XCD computes it)."""
    M, N, K = 8192, 28672, 8192
    A, B = make_inputs(orc, M, N, K, "normal")
    d = Dev(mi, A, B, M, N)
    C0 = d.run(K).copy()
    assert (d.run(K) == C0).all()
    rng = np.random.default_rng(5)
    pm, pn = rng.permutation(M), rng.permutation(N)
    C1 = Dev(mi, A[pm], B[pn], M, N).run(K)
    assert (C1 == C0[pm][:, pn]).all()


@pytest.mark.parametrize("M", [16, 64, 128])
def test_c4_skinny_full(mi, orc, M):
    check(mi, orc, M, 8192, 8192, "normal")


def test_c5_unaligned_full(mi, orc):
    check(mi, orc, 4095, 6143, 3073, "uniform")


# ------------------------------------------------------ every kernel configuration ----

def all_configs(kinds=("tile", "ring", "mfma16", "ring16"), k_groups=True):
    from h100_gemm_amd import kernel_configs as kc
    return [i for i, c in enumerate(kc.CONFIGS) if c["KIND"] in kinds and (k_groups or c.get("KG", 1) == 1)]


def k_for(config, K):
    """K as the configuration can take it: a kernel that splits K over two groups of waves needs
    equal halves of whole 128-deep double steps, so K is rounded up to a multiple of 256 for it"""
    from h100_gemm_amd import kernel_configs as kc
    kg = kc.CONFIGS[config].get("KG", 1) if config >= 0 else 1
    return K if kg == 1 else -(-K // (128 * kg)) * 128 * kg


@pytest.mark.parametrize("config", all_configs())
def test_every_config_bit_exact_on_integer_fill(mi, orc, config):
    # aligned (512^3: the aligned kernel), and ragged M, N, odd K (the predicated kernel)
    for M, N, K in [(512, 512, 512), (768, 1536, 1152), (257, 515, 77), (300, 200, 136), (65, 70, 33),
                    (256, 384, 191), (1, 1, 1)]:
        check(mi, orc, M, N, k_for(config, K), "int", config=config, exact=True)


@pytest.mark.parametrize("config", all_configs())
def test_every_config_uniform_within_tolerance(mi, orc, config):
    for M, N, K in [(1024, 768, 256), (255, 511, 129), (513, 391, 320)]:
        check(mi, orc, M, N, k_for(config, K), "uniform", config=config)


# ------------------------------------------------ decode (split-K streaming) kernels ----

@pytest.mark.parametrize("config", all_configs(("stream", "decode")))
def test_decode_kernels(mi, orc, config):
    from h100_gemm_amd import kernel_configs as kc
    bm = kc.CONFIGS[config]["BM"]
    for M in sorted({1, bm // 2 + 1, bm - 1, bm}):
        for N, K in [(128, 64), (8192, 4096), (1028, 8192), (260, 192), (4, 1024)]:
            check(mi, orc, M, N, K, "int", config=config, exact=True)     # split-K sums of exact ints
    check(mi, orc, bm, 8192, 8192, "normal", config=config)
    check(mi, orc, bm, 2048, 512, "uniform", config=config, dtype=orc.FP16)
    # shapes the kernel cannot run are refused, not mis-computed
    A, B = make_inputs(orc, bm + 1, 256, 128, "int")
    d = Dev(mi, A, B, bm + 1, 256)
    with pytest.raises(mi.MiGemmError) as ei:
        d.run(128, config=config)
    assert ei.value.code == mi._lib.MI_ERR_UNSUPPORTED
    A, B = make_inputs(orc, 8, 256, 100, "int")
    with pytest.raises(mi.MiGemmError):
        Dev(mi, A, B, 8, 256).run(100, config=config)


# ------------------------- small tiles, K split over the waves of a workgroup (few tiles, long K) ----

@pytest.mark.parametrize("config", all_configs(("wavek",)))
def test_wave_split_k_kernels(mi, orc, config):
    from h100_gemm_amd import kernel_configs as kc
    bm, bn = kc.CONFIGS[config]["BM"], kc.CONFIGS[config]["BN"]
    # whole tiles, ragged M and N (rows past M / N are never fetched nor stored), one tile, a
    # single K unit (three of the four waves have nothing to add), K units that do not divide
    # over the waves, several rounds of workgroups
    for M, N, K in [(512, 512, 4096), (bm, bn, 64), (bm + 1, bn + 4, 128), (1, 4, 64), (100, 36, 192),
                    (777, 1000, 320), (1536, 1536, 1536), (33, 8, 448), (2 * bm - 1, 5 * bn - 4, 2112)]:
        check(mi, orc, M, N, K, "int", config=config, exact=True)     # sums of exact ints: any order gives the oracle's bits
    check(mi, orc, 1024, 1024, 4096, "uniform", config=config)
    check(mi, orc, 512, 768, 2048, "normal", config=config, dtype=orc.FP16)
    # hundreds of thousands of tile rows / columns (64-bit row offsets), the longest K the library takes
    check(mi, orc, 600000, 8, 128, "int", config=config, exact=True)
    check(mi, orc, 8, 600000, 128, "int", config=config, exact=True)
    check(mi, orc, 40, 36, 4194240, "uniform", config=config)
    check_epilogue(mi, orc, 300, 260, 1024, "int", -0.5, 2.75, config=config, exact=True)
    check_epilogue(mi, orc, 512, 512, 4096, "uniform", 0.37, 1.25, config=config)
    check_epilogue(mi, orc, 200, 132, 1024, "int", 2.0, -1.0, config=config, c_layout=mi.MI_C_COL_MAJOR, exact=True)
    # shapes the kernel cannot run are refused, not mis-computed
    # any even K: the partial last unit is filled with zeros (what lies at k >= K in memory is
    # the next row) -- whole 16-byte chunks by fetching nothing, the chunk that K ends in by
    # zeroing its tail in LDS -- down to a single chunk and a single unit, the partial unit with
    # each of the four waves; any N (C stored element by element where rows of C do not start on
    # 8-byte boundaries)
    for M, N, K in [(bm, bn, 8), (97, 100, 72), (300, 260, 200), (1000, 1000, 1000), (1440, 1440, 1480),
                    (33, 8, 456), (2 * bm - 1, 5 * bn - 4, 2168), (130, 132, 136), (130, 132, 248),
                    (bm, bn, 2), (bm + 3, bn + 1, 6), (97, 101, 66), (300, 259, 100), (500, 500, 500),
                    (1500, 1500, 1500), (255, 1001, 1030), (130, 130, 190), (7, 3, 254), (640, 77, 4100)]:
        check(mi, orc, M, N, K, "int", config=config, exact=True)
    check(mi, orc, 1000, 1000, 1000, "uniform", config=config)
    check(mi, orc, 1500, 1002, 1500, "uniform", config=config)
    check(mi, orc, 300, 201, 500, "normal", config=config, dtype=orc.FP16)
    check_epilogue(mi, orc, 300, 260, 1000, "int", -0.5, 2.75, config=config, exact=True)
    check_epilogue(mi, orc, 300, 261, 1002, "int", -0.5, 2.75, config=config, exact=True)
    check_epilogue(mi, orc, 200, 131, 1026, "int", 2.0, -1.0, config=config, c_layout=mi.MI_C_COL_MAJOR, exact=True)
    # an odd K: the loops take the even part, the last k is added in the epilogue
    for M, N, K in [(bm, bn, 1), (bm + 3, bn + 1, 3), (97, 101, 65), (300, 259, 101), (500, 500, 501),
                    (257, 515, 77), (1001, 1001, 1001), (130, 130, 191), (7, 3, 255), (640, 77, 4101)]:
        check(mi, orc, M, N, K, "int", config=config, exact=True)
    check(mi, orc, 999, 1001, 1003, "uniform", config=config)
    check(mi, orc, 300, 201, 501, "normal", config=config, dtype=orc.FP16)
    check_epilogue(mi, orc, 300, 261, 1003, "int", -0.5, 2.75, config=config, exact=True)
    # few tiles with a very long K: K cut into pieces over workgroups, fp32 sums of the pieces
    # in the workspace, a second launch adds them -- whole units, a partial last unit, an odd
    # K (all in the last piece), a last piece of a single unit; N % 4 != 0 does not split
    # (the number of pieces comes from the config's time model; one without a model runs these whole)
    from h100_gemm_amd import kernel_configs as kc
    if kc.CONFIGS[config].get("WK"):
        assert mi.config_grid(config, 128, 384, 13376) > -(-128 // bm) * -(-384 // bn)
    for M, N, K in [(128, 384, 13376), (bm, bn, 4096), (100, 36, 8200), (33, 8, 16390), (200, 132, 9001),
                    (150, 100, 6002), (97, 101, 8193), (64, 64, 2112), (2 * bm + 1, bn + 4, 12352)]:
        check(mi, orc, M, N, K, "int", config=config, exact=True)
    check(mi, orc, 256, 256, 16384, "uniform", config=config)
    check(mi, orc, 96, 200, 10001, "normal", config=config, dtype=orc.FP16)
    check_epilogue(mi, orc, 200, 132, 9001, "int", -0.5, 2.75, config=config, exact=True)
    check_epilogue(mi, orc, 132, 200, 8200, "int", 2.0, -1.0, config=config, c_layout=mi.MI_C_COL_MAJOR, exact=True)
    # operands that do not start on 4-byte boundaries are refused, not mis-computed
    for offA, offB in [(2, 0), (0, 6)]:
        with pytest.raises(mi.MiGemmError) as ei:
            _run_offset(mi, orc, config, 100, 100, 128, offA, offB, 0)
        assert ei.value.code == mi._lib.MI_ERR_UNSUPPORTED


@pytest.mark.parametrize("config", [i for i in all_configs(("mfma16",)) if i not in all_configs(("mfma16",), k_groups=False)])
def test_k_groups_inside_the_workgroup(mi, orc, config):
    """Eight waves as two groups that each multiply half of K of the same tile and add their
    accumulators through LDS: aligned and ragged M and N (the predicated variant), the shortest
    K (one double step per group), fp16, epilogue, trace records; K that does not divide into
    equal halves of whole double steps is refused."""
    for M, N, K in [(512, 512, 256), (1536, 1536, 1536), (257, 515, 768), (1, 1, 256), (129, 127, 1280), (2048, 2048, 2048)]:
        check(mi, orc, M, N, K, "int", config=config, exact=True)
    check(mi, orc, 1024, 768, 2048, "uniform", config=config)
    check(mi, orc, 300, 200, 512, "normal", config=config, dtype=orc.FP16)
    check_epilogue(mi, orc, 384, 260, 1024, "int", -0.5, 2.75, config=config, exact=True)
    check_epilogue(mi, orc, 200, 132, 512, "int", 2.0, -1.0, config=config, c_layout=mi.MI_C_COL_MAJOR, exact=True)
    for K in (128, 384, 1000):
        A, B = make_inputs(orc, 256, 256, K, "int")
        with pytest.raises(mi.MiGemmError) as ei:
            Dev(mi, A, B, 256, 256).run(K, config=config)
        assert ei.value.code == mi._lib.MI_ERR_UNSUPPORTED
    A, B = make_inputs(orc, 1536, 1536, 1536, "uniform")
    d = Dev(mi, A, B, 1536, 1536)
    C0 = d.run(1536, config=config)
    for _ in range(3):
        assert (d.run(1536, config=config) == C0).all()          # fixed summation order: bit-reproducible
    # seeded sweep: ragged M and N, base pointers at arbitrary even byte offsets (the predicated variant)
    rng = np.random.default_rng(20241126)
    for it in range(12):
        M, N, K = int(rng.integers(1, 600)), int(rng.integers(1, 600)), 256 * int(rng.integers(1, 6))
        offA, offB, offC = (int(2 * rng.integers(0, 16)) for _ in range(3))
        print(f"case {it}: M={M} N={N} K={K} offsets {offA},{offB},{offC}", flush=True)
        C, ref, guard = _run_offset(mi, orc, config, M, N, K, offA, offB, offC)
        assert (C == ref).all(), f"{int((C != ref).sum())} elements differ"
        assert (guard == 0xEEEE).all(), "bytes outside C were written"


def test_wave_split_k_dispatch_and_determinism(mi, orc):
    from h100_gemm_amd import kernel_configs as kc
    # the automatic choice for few-tile shapes; the same answers as the tiled kernels where
    # its preconditions fail (K % 64, N % 4)
    for M, N, K in [(512, 512, 4096), (1024, 1024, 4096), (512, 512, 4100), (512, 510, 4096), (640, 384, 3328)]:
        check(mi, orc, M, N, K, "int", exact=True)
    assert kc.CONFIGS[mi.select_config(512, 512, 4096)]["KIND"] == "wavek"
    # the shared-ring kernels through the automatic choice (also a K that is no multiple of 64:
    # the tiled kernels give the same answers)
    for M, N, K in [(1440, 1440, 1472), (1344, 1344, 1344), (1536, 1472, 320), (1440, 1440, 1480)]:
        check(mi, orc, M, N, K, "int", exact=True)
    assert kc.CONFIGS[mi.select_config(1440, 1440, 1472)].get("SHARED") == 1
    A, B = make_inputs(orc, 1440, 1440, 1472, "uniform")
    d = Dev(mi, A, B, 1440, 1440)
    C0 = d.run(1472)
    for _ in range(3):
        assert (d.run(1472) == C0).all()
    A, B = make_inputs(orc, 1024, 1024, 4096, "uniform")
    d = Dev(mi, A, B, 1024, 1024)
    C0 = d.run(4096)
    for _ in range(3):
        assert (d.run(4096) == C0).all()          # fixed summation order: bit-reproducible


def test_decode_dispatch_and_determinism(mi, orc):
    # automatic choice: decode kernel when its preconditions hold, the predicated tile kernel
    # otherwise -- same answers either way
    for M, N, K in [(16, 8192, 8192), (100, 4100, 2112), (128, 8190, 1024), (5, 256, 8200), (128, 8192, 8192)]:
        check(mi, orc, M, N, K, "int", exact=True)
    for M in (16, 64):                            # single-pass kernel, split-K kernel
        A, B = make_inputs(orc, M, 8192, 8192, "normal")
        d = Dev(mi, A, B, M, 8192)
        C0 = d.run(8192)
        for _ in range(3):
            assert (d.run(8192) == C0).all()      # fixed summation order: bit-reproducible


# --------------------------------------------------------------------- edge cases ----

@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (1, 1, 64), (1, 300, 7), (300, 1, 9), (2, 3, 1),
                                   (64, 64, 63), (65, 63, 65), (129, 127, 128), (256, 256, 127),
                                   (256, 256, 2048), (31, 33, 4097), (1000, 1000, 8)])
def test_ragged_and_tiny_shapes(mi, orc, M, N, K):
    check(mi, orc, M, N, K, "int", exact=True)
    check(mi, orc, M, N, K, "uniform")


@pytest.mark.parametrize("M,N,K", [(1, 1, 4194303), (3, 130, 1048577), (1 << 22, 8, 8), (8, 1 << 22, 8),
                                   (1, 1 << 23, 16), (1 << 21, 1, 64), (20000, 20000, 1), (600000, 8, 2048), (8, 600000, 2048)])
def test_extreme_aspect_ratios(mi, orc, M, N, K):
    # the largest K the library accepts (K * 512 < 2^31), millions of tile rows / columns
    # (64-bit row offsets, 32-bit offsets inside a tile's panel), a single column, K = 1,
    # operands of 2.4 GB (byte offsets past 2^31)
    fill = "uniform" if K > 100000 else "int"
    check(mi, orc, M, N, K, fill, exact=fill == "int")


def test_k_tail_with_page_aligned_matrix_end(mi, orc):
    # odd K with M a multiple of 2048: the last element of A sits right below a 4 KiB
    # boundary of the allocation; the kernel must fetch it without reading past the matrix
    check(mi, orc, 2048, 96, 77, "int", exact=True)
    check(mi, orc, 96, 2048, 65, "int", exact=True)


def test_misaligned_base_pointers(mi, orc):
    # sub-matrices that start 2 bytes into an allocation: nothing is 16-byte aligned
    M, N, K = 200, 264, 160
    A, B = make_inputs(orc, M, N, K, "int")
    ref = orc.reference_cpu_gemm(A, B)
    dA = mi.DeviceBuffer(A.nbytes + 16)
    dB = mi.DeviceBuffer(B.nbytes + 16)
    dC = mi.DeviceBuffer(M * N * 2 + 16)
    L = mi._lib.load()
    mi._lib.check(L.mi_memcpy_h2d(dA.ptr + 2, A.ctypes.data, A.nbytes))
    mi._lib.check(L.mi_memcpy_h2d(dB.ptr + 6, B.ctypes.data, B.nbytes))
    dC.fill_bytes(0xEE)
    mi.runKernel(M, N, K, dA.ptr + 2, dB.ptr + 6, dC.ptr + 2)
    mi.synchronize()
    raw = dC.to_numpy((M * N + 8,), np.uint16)
    assert (raw[1:1 + M * N].reshape(M, N) == ref).all()
    assert raw[0] == 0xEEEE and (raw[1 + M * N:] == 0xEEEE).all()      # nothing written outside C


def _run_offset(mi, orc, config, M, N, K, offA, offB, offC, dtype=0):
    """GEMM on sub-buffers that start offA/offB/offC bytes into their allocations; returns
    (C, ref, guard words before and after C)."""
    A, B = make_inputs(orc, M, N, K, "int", dtype)
    ref = orc.reference_cpu_gemm(A, B, dtype=dtype)
    dA = mi.DeviceBuffer(A.nbytes + 64)
    dB = mi.DeviceBuffer(B.nbytes + 64)
    dC = mi.DeviceBuffer(M * N * 2 + 128)
    L = mi._lib.load()
    mi._lib.check(L.mi_memcpy_h2d(dA.ptr + offA, A.ctypes.data, A.nbytes))
    mi._lib.check(L.mi_memcpy_h2d(dB.ptr + offB, B.ctypes.data, B.nbytes))
    dC.fill_bytes(0xEE)
    mi._lib.check(L.mi_gemm_ex(config, dtype, M, N, K, dA.ptr + offA, dB.ptr + offB, dC.ptr + offC, None, None))
    mi.synchronize()
    raw = dC.to_numpy((M * N + 64,), np.uint16)
    lo = offC // 2
    C = raw[lo:lo + M * N].reshape(M, N)
    guard = np.concatenate([raw[:lo], raw[lo + M * N:]])
    for b in (dA, dB, dC):
        b.free()
    return C, ref, guard


def test_random_shapes_and_alignments_every_tiled_kind(mi, orc):
    # seeded sweep: ragged M, N, K (K tails of every length class, K < 64, K just above a
    # multiple of 128), base pointers at arbitrary even byte offsets, through the automatic
    # choice and through one configuration of every tiled kernel kind
    from h100_gemm_amd import kernel_configs as kc
    rng = np.random.default_rng(20240607)
    picks = {}
    for i, c in enumerate(kc.CONFIGS):
        if c["KIND"] in ("tile", "ring", "mfma16", "ring16"):
            picks.setdefault((c["KIND"], c.get("DRAIN", 0) > 0, c["BN"] == 192), i)
    configs = [-1] + sorted(picks.values())
    # MI_GEMM_RANDOM_CASES=<n> turns this into a longer sweep (36 cases by default)
    for it in range(int(os.environ.get("MI_GEMM_RANDOM_CASES", "36"))):
        M = int(rng.integers(1, 700))
        N = int(rng.integers(1, 700))
        K = int(rng.choice([rng.integers(1, 64), rng.integers(64, 400), 128 * rng.integers(1, 5) + rng.integers(0, 9)]))
        offA, offB, offC = (int(2 * rng.integers(0, 16)) for _ in range(3))
        config = configs[it % len(configs)]
        print(f"case {it}: M={M} N={N} K={K} offsets {offA},{offB},{offC} config={config}", flush=True)
        C, ref, guard = _run_offset(mi, orc, config, M, N, K, offA, offB, offC)
        assert (C == ref).all(), f"{int((C != ref).sum())} elements differ"
        assert (guard == 0xEEEE).all(), "bytes outside C were written"


def test_random_shapes_small_tile_and_decode_kinds(mi, orc):
    # seeded sweep for the kernels that need whole 64-deep K units, N % 4 == 0 and 16-byte aligned
    # operands: ragged M and N, one to many K units, base pointers at multiples of 16 (A, B) and
    # 8 (C) bytes, through the automatic choice and through every such configuration that can
    # run the shape; an odd operand offset must send the automatic choice to a predicated kernel
    from h100_gemm_amd import kernel_configs as kc
    rng = np.random.default_rng(20241125)
    special = [i for i, c in enumerate(kc.CONFIGS) if c["KIND"] in ("wavek", "stream", "decode")]
    small = [i for i, c in enumerate(kc.CONFIGS) if c["KIND"] == "wavek"]
    # MI_GEMM_RANDOM_CASES=<n> turns this into a longer sweep (36 cases by default)
    for it in range(int(os.environ.get("MI_GEMM_RANDOM_CASES", "36"))):
        M = int(rng.choice([rng.integers(1, 130), rng.integers(1, 700)]))
        N = 4 * int(rng.integers(1, 180))
        K = 64 * int(rng.choice([1, 2, 3, rng.integers(4, 40)]))
        offA, offB, offC = 16 * int(rng.integers(0, 4)), 16 * int(rng.integers(0, 4)), 8 * int(rng.integers(0, 8))
        pool = special
        if it % 2 == 1:
            # what only the small-tile kernels take: any K, any N, operands on 4-byte and C on
            # 2-byte boundaries
            # (a K beyond 2048 may be cut into pieces over workgroups where N % 4 == 0 and C is 8-byte aligned)
            K = int(rng.choice([rng.integers(1, 80), rng.integers(80, 2600), rng.integers(2048, 9000)]))
            N = int(rng.choice([rng.integers(1, 720), 4 * rng.integers(1, 180)]))
            offA, offB, offC = 4 * int(rng.integers(0, 16)), 4 * int(rng.integers(0, 16)), int(rng.choice([2, 8])) * int(rng.integers(0, 8))
            pool = small
        able = [i for i in pool if mi._lib.load().mi_gemm_config_supports(i, 0, M, N, K)]
        config = -1 if it % 3 == 0 or not able else able[int(rng.integers(0, len(able)))]
        if it % 7 == 3:
            config, offA = -1, offA + 2          # not 4-byte aligned: none of these kernels may be chosen
        print(f"case {it}: M={M} N={N} K={K} offsets {offA},{offB},{offC} config={config}", flush=True)
        C, ref, guard = _run_offset(mi, orc, config, M, N, K, offA, offB, offC)
        assert (C == ref).all(), f"{int((C != ref).sum())} elements differ"
        assert (guard == 0xEEEE).all(), "bytes outside C were written"


def test_large_ragged_shape_cut_into_two_gemms(mi, orc):
    """7000 x 7000 x 4096 runs as 6912 rows and then 88 (the last row of 256x256 tiles would be a
    third full and cost a whole round): every element against the on-device golden, bit for bit
    on an integer fill, with alpha / beta and a column-major C as well."""
    M, N, K = 7000, 7000, 4096
    assert mi.row_cut(M, N, K) == 6912
    A, B = make_inputs(orc, M, N, K, "int")
    dA, dB = mi.DeviceBuffer.from_numpy(A), mi.DeviceBuffer.from_numpy(B)
    dC, dR = mi.DeviceBuffer(M * N * 2), mi.DeviceBuffer(M * N * 2)
    for alpha, beta, layout in [(1.0, 0.0, mi.MI_C_ROW_MAJOR), (-0.5, 2.75, mi.MI_C_ROW_MAJOR), (1.0, 0.0, mi.MI_C_COL_MAJOR)]:
        dC.fill_bytes(0xEE)
        mi.gemm_epilogue(mi.GemmParams(M, N, K, dA, dB, dC, alpha=alpha, beta=beta), c_layout=layout)
        mi.reference_gpu_gemm(mi.GemmParams(M, N, K, dA, dB, dR, alpha=alpha, beta=beta))
        mi.synchronize()
        C, R = dC.to_numpy((M * N,), np.uint16), dR.to_numpy((M, N), np.uint16)
        C = C.reshape(N, M).T if layout == mi.MI_C_COL_MAJOR else C.reshape(M, N)
        assert (C == R).all(), f"alpha {alpha} beta {beta} layout {layout}: {int((C != R).sum())} elements differ"
    for b in (dA, dB, dC, dR):
        b.free()


def test_non_default_streams_and_host_threads(mi, orc):
    """The ABI's stream argument: two host threads, each launching on a stream of its own
    (created with default priority) and waiting with mi_stream_sync.  The shapes include
    split-K ones (decode 128 x 8192 x 8192, few tiles 384 x 512 x 4096): the library keeps one
    workspace per stream, so the two threads' partial sums never meet."""
    import ctypes
    import threading
    hip = ctypes.CDLL("libamdhip64.so")
    L = mi._lib.load()
    shapes = [(512, 512, 512), (384, 512, 4096), (16, 2048, 1024), (257, 515, 77), (128, 8192, 8192),
              (768, 1280, 384)]
    assert mi.workspace_bytes(384, 512, 4096) > 0 and mi.workspace_bytes(128, 8192, 8192) > 0
    cases = []
    for seed in range(2):
        for M, N, K in shapes:
            A, B = make_inputs(orc, M, N, K, "int", seed=69 + seed)
            cases.append((seed, M, N, K, A, B, orc.reference_cpu_gemm(A, B)))
    errors = []

    def worker(seed):
        try:
            stream = ctypes.c_void_p()
            assert hip.hipStreamCreate(ctypes.byref(stream)) == 0
            for rep in range(2):
                for s, M, N, K, A, B, ref in cases:
                    if s != seed:
                        continue
                    dA, dB = mi.DeviceBuffer.from_numpy(A), mi.DeviceBuffer.from_numpy(B)
                    dC = mi.DeviceBuffer(M * N * 2)
                    dC.fill_bytes(0xFF)
                    for _ in range(4):      # back to back, so that the two streams' launches overlap
                        mi._lib.check(L.mi_gemm_ex(-1, 0, M, N, K, dA.ptr, dB.ptr, dC.ptr, None, stream))
                    mi._lib.check(L.mi_stream_sync(stream))
                    C = dC.to_numpy((M, N), np.uint16)
                    if not (C == ref).all():
                        errors.append(f"thread {seed} rep {rep} {M}x{N}x{K}: {int((C != ref).sum())} elements differ")
                    for b in (dA, dB, dC):
                        b.free()
            assert hip.hipStreamDestroy(stream) == 0
        except Exception as e:      # surfaced in the main thread
            errors.append(f"thread {seed}: {type(e).__name__}: {e}")

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors


def test_split_k_workspace_growth_keeps_enqueued_launches_valid(mi, orc):
    """A split-K launch that needs a larger library workspace than the stream has must not
    free the one that launches already enqueued on that stream still use: a small split-K
    GEMM and a large one go out back to back without a wait in between, twice, on a stream
    that has never run split-K before."""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    L = mi._lib.load()
    stream = ctypes.c_void_p()
    assert hip.hipStreamCreate(ctypes.byref(stream)) == 0
    runs = []
    for M, N, K in [(384, 512, 4096), (128, 8192, 8192), (256, 8192, 8192)]:
        assert mi.workspace_bytes(M, N, K) > 0
        A, B = make_inputs(orc, M, N, K, "int")
        runs.append((Dev(mi, A, B, M, N), M, N, K, orc.reference_cpu_gemm(A, B)))
    need = [mi.workspace_bytes(M, N, K) for _, M, N, K, _ in runs]
    assert need[0] < need[1] < need[2], need             # each launch outgrows the buffer before it
    for rep in range(2):
        for d, M, N, K, ref in runs:
            mi._lib.check(L.mi_gemm_ex(-1, 0, M, N, K, d.dA.ptr, d.dB.ptr, d.dC.ptr, None, stream))
        mi._lib.check(L.mi_stream_sync(stream))
        for d, M, N, K, ref in runs:
            C = d.dC.to_numpy((M, N), np.uint16)
            assert (C == ref).all(), f"rep {rep} {M}x{N}x{K}: {int((C != ref).sum())} elements differ"
            d.dC.fill_bytes(0xFF)
    assert hip.hipStreamDestroy(stream) == 0


def test_library_workspace_is_released_and_its_table_capped(mi, orc):
    """A server that creates and destroys streams: 64 streams in turn run the split-K decode
    shape 128 x 8192 x 8192 through the library's own workspace.  The first half give their
    buffer back before the stream is destroyed (mi_gemm_release_workspace), the second half
    never do: the library then holds buffers for at most 16 streams.  After a release of
    everything the device's free memory is back to within one buffer of where it started, and
    every result is bit-exact."""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    L = mi._lib.load()
    M, N, K = 128, 8192, 8192
    need = mi.workspace_bytes(M, N, K)
    assert need > 0
    buf = 4 << 20
    while buf < need:
        buf <<= 1
    A, B = make_inputs(orc, M, N, K, "int")
    ref = orc.reference_cpu_gemm(A, B)
    d = Dev(mi, A, B, M, N)
    mi._lib.check(L.mi_gemm_release_workspace(None))           # whatever earlier tests left
    assert L.mi_gemm_library_workspace_bytes() == 0

    def free_bytes():
        f, t = ctypes.c_size_t(), ctypes.c_size_t()
        assert hip.hipMemGetInfo(ctypes.byref(f), ctypes.byref(t)) == 0
        return f.value

    start = free_bytes()

    def run_on(stream, tag):
        d.dC.fill_bytes(0xFF)
        mi._lib.check(L.mi_gemm_ex(-1, 0, M, N, K, d.dA.ptr, d.dB.ptr, d.dC.ptr, None, stream))
        mi._lib.check(L.mi_stream_sync(stream))
        C = d.dC.to_numpy((M, N), np.uint16)
        assert (C == ref).all(), f"{tag}: {int((C != ref).sum())} elements differ"

    for i in range(64):
        stream = ctypes.c_void_p()
        assert hip.hipStreamCreate(ctypes.byref(stream)) == 0
        run_on(stream, f"stream {i}")
        held = L.mi_gemm_library_workspace_bytes()
        if i < 32:
            assert held == buf, (i, held, buf)
            mi._lib.check(L.mi_gemm_release_workspace(stream))
            assert L.mi_gemm_library_workspace_bytes() == 0
        else:
            # never released: a later stream may get the destroyed one's handle value and with it
            # its buffer; either way no more than the table's 16 entries
            assert buf <= held <= 16 * buf, (i, held, buf)
        assert hip.hipStreamDestroy(stream) == 0
    # 24 streams alive at once: the table stops at 16 buffers, the others take one over
    alive = []
    for i in range(24):
        stream = ctypes.c_void_p()
        assert hip.hipStreamCreate(ctypes.byref(stream)) == 0
        alive.append(stream)
        run_on(stream, f"live stream {i}")
        assert L.mi_gemm_library_workspace_bytes() <= 16 * buf
    assert L.mi_gemm_library_workspace_bytes() == 16 * buf
    for i, stream in enumerate(alive):                         # and again, every stream taking turns
        run_on(stream, f"live stream {i}, second round")
    assert L.mi_gemm_library_workspace_bytes() == 16 * buf
    for stream in alive:
        assert hip.hipStreamDestroy(stream) == 0
    mi._lib.check(L.mi_gemm_release_workspace(None))
    assert L.mi_gemm_library_workspace_bytes() == 0
    assert abs(free_bytes() - start) <= buf, (free_bytes(), start, buf)
    # a reservation made ahead of the first GEMM is what that GEMM then uses
    mi._lib.check(L.mi_gemm_reserve_workspace(None, need))
    assert L.mi_gemm_library_workspace_bytes() == buf
    d.dC.fill_bytes(0xFF)
    mi._lib.check(L.mi_gemm_ex(-1, 0, M, N, K, d.dA.ptr, d.dB.ptr, d.dC.ptr, None, None))
    mi.synchronize()
    assert (d.dC.to_numpy((M, N), np.uint16) == ref).all()
    assert L.mi_gemm_library_workspace_bytes() == buf
    mi._lib.check(L.mi_gemm_release_workspace(None))


def test_caller_workspace_launches_on_two_streams(mi, orc):
    """mi_gemm_epilogue_ws: split-K partial sums in buffers the caller owns, one per stream;
    interleaved launches on two streams, bit-exact on the integer fill and bit-identical to
    the library-workspace entry point; a NULL or short workspace runs the launch unsplit (same
    integers), a misaligned one is refused."""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    L = mi._lib.load()
    streams = [ctypes.c_void_p(), ctypes.c_void_p()]
    for s in streams:
        assert hip.hipStreamCreate(ctypes.byref(s)) == 0
    shapes = [(128, 8192, 8192), (384, 512, 4096), (64, 4096, 8192), (512, 512, 512)]
    per_stream = []
    for i, s in enumerate(streams):
        runs = []
        for M, N, K in shapes:
            A, B = make_inputs(orc, M, N, K, "int", seed=69 + i)
            need = mi.workspace_bytes(M, N, K)
            assert (need > 0) == ((M, N, K) != (512, 512, 512)), (M, N, K, need)
            ws = mi.DeviceBuffer(max(need, 16))
            ws.fill_bytes(0xFF)                          # NaN partials: every one must be overwritten
            runs.append((Dev(mi, A, B, M, N), M, N, K, orc.reference_cpu_gemm(A, B), ws, need))
        per_stream.append(runs)
    for rep in range(3):
        for k in range(len(shapes)):
            for i, s in enumerate(streams):
                d, M, N, K, ref, ws, need = per_stream[i][k]
                mi._lib.check(L.mi_gemm_epilogue_ws(-1, 0, M, N, K, d.dA.ptr, d.dB.ptr, d.dC.ptr, 1.0, 0.0, 0,
                                                    ws.ptr, need, s))
    for i, s in enumerate(streams):
        mi._lib.check(L.mi_stream_sync(s))
        for d, M, N, K, ref, ws, need in per_stream[i]:
            C = d.dC.to_numpy((M, N), np.uint16)
            assert (C == ref).all(), f"stream {i} {M}x{N}x{K}: {int((C != ref).sum())} elements differ"
    # against the library-workspace entry point on random data (same kernel, same order of sums)
    M, N, K = 128, 8192, 8192
    A, B = make_inputs(orc, M, N, K, "normal")
    d = Dev(mi, A, B, M, N)
    want = d.run(K).copy()
    ws = mi.DeviceBuffer(mi.workspace_bytes(M, N, K))
    for ws_ptr, ws_bytes, same in [(ws.ptr, ws.nbytes, True), (None, 0, False), (ws.ptr, 4096, False)]:
        d.dC.fill_bytes(0xFF)
        mi._lib.check(L.mi_gemm_epilogue_ws(-1, 0, M, N, K, d.dA.ptr, d.dB.ptr, d.dC.ptr, 1.0, 0.0, 0,
                                            ws_ptr, ws_bytes, streams[0]))
        mi._lib.check(L.mi_stream_sync(streams[0]))
        C = d.dC.to_numpy((M, N), np.uint16)
        if same:
            assert (C == want).all()
        else:           # unsplit: another order of sums, inside the tolerance
            ref = orc.reference_cpu_gemm(A, B)
            rep = orc.check_tolerance(C, ref, K, orc.max_abs(A), orc.max_abs(B))
            assert rep["violations"] == 0, rep
    assert L.mi_gemm_epilogue_ws(-1, 0, M, N, K, d.dA.ptr, d.dB.ptr, d.dC.ptr, 1.0, 0.0, 0, ws.ptr + 4, 1 << 20,
                                 None) == mi._lib.MI_ERR_INVALID
    for s in streams:
        assert hip.hipStreamDestroy(s) == 0


def test_hip_graph_replay_of_gemm_launches(mi, orc):
    """A launch is kernel launches only and can be captured into a HIP graph: a tiled, a decode
    and two split-K GEMMs (caller workspaces) recorded on a capturing stream, plus one split-K
    shape through the library-workspace entry point on a stream that has no buffer yet (the
    library must not allocate under capture: it records the unsplit launch).  Replayed three
    times with eager work and synchronisation in between, every replay compared."""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    L = mi._lib.load()
    cases = [(512, 512, 512), (16, 2048, 1024), (300, 200, 100), (384, 512, 4096), (96, 4096, 8192)]
    bufs, want = [], []
    for M, N, K in cases:
        A, B = make_inputs(orc, M, N, K, "int")
        d = Dev(mi, A, B, M, N)
        want.append(d.run(K).copy())                       # eager result (also loads the kernels)
        assert (want[-1] == orc.reference_cpu_gemm(A, B)).all()
        ws = mi.DeviceBuffer(max(mi.workspace_bytes(M, N, K), 16))
        bufs.append((d, M, N, K, ws))
    assert sum(mi.workspace_bytes(M, N, K) > 0 for M, N, K in cases) >= 2
    M2, N2, K2 = 320, 512, 4096                             # split-K shape, library workspace, fresh stream
    assert mi.workspace_bytes(M2, N2, K2) > 0
    A2, B2 = make_inputs(orc, M2, N2, K2, "int")
    d2 = Dev(mi, A2, B2, M2, N2)
    want2 = orc.reference_cpu_gemm(A2, B2)
    stream, graph, gexec = ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_void_p()
    assert hip.hipStreamCreate(ctypes.byref(stream)) == 0
    assert hip.hipStreamBeginCapture(stream, 0) == 0       # hipStreamCaptureModeGlobal
    rcs = [L.mi_gemm_epilogue_ws(-1, 0, M, N, K, d.dA.ptr, d.dB.ptr, d.dC.ptr, 1.0, 0.0, 0, ws.ptr, ws.nbytes, stream)
           for d, M, N, K, ws in bufs]
    rcs.append(L.mi_gemm_ex(-1, 0, M2, N2, K2, d2.dA.ptr, d2.dB.ptr, d2.dC.ptr, None, stream))
    assert hip.hipStreamEndCapture(stream, ctypes.byref(graph)) == 0
    assert rcs == [0] * (len(cases) + 1), (rcs, L.mi_last_error())
    assert hip.hipGraphInstantiate(ctypes.byref(gexec), graph, None, None, ctypes.c_size_t(0)) == 0
    for replay in range(3):
        for d, M, N, K, ws in bufs:
            d.dC.fill_bytes(0xFF)                          # eager work between the replays
            ws.fill_bytes(0xFF)
        d2.dC.fill_bytes(0xFF)
        mi.synchronize()
        assert hip.hipGraphLaunch(gexec, stream) == 0
        mi._lib.check(L.mi_stream_sync(stream))
        for (d, M, N, K, ws), ref in zip(bufs, want):
            C = d.dC.to_numpy((M, N), np.uint16)
            assert (C == ref).all(), f"replay {replay} {M}x{N}x{K}: {int((C != ref).sum())} elements differ"
        assert (d2.dC.to_numpy((M2, N2), np.uint16) == want2).all(), f"replay {replay} {M2}x{N2}x{K2}"
    assert hip.hipGraphExecDestroy(gexec) == 0
    assert hip.hipGraphDestroy(graph) == 0
    assert hip.hipStreamDestroy(stream) == 0


SPECIAL_SHAPES = [(256, 256, 128), (130, 70, 72), (16, 2048, 1024), (64, 4096, 8192), (256, 256, 4096)]


@pytest.mark.parametrize("M,N,K", SPECIAL_SHAPES)
def test_overflow_underflow_and_nan_follow_ieee(mi, orc, M, N, K):
    """Every epilogue (direct, predicated, in-LDS reduction, split-K reduction) rounds like the
    oracle at the ends of the range: fp16 overflow to +-inf, fp32 accumulator overflow to inf
    in bf16, fp16 results in the subnormal range (round to nearest even there too), subnormal
    inputs and sums kept (nothing is flushed to zero), and a NaN in one row of A makes exactly
    that row of C NaN."""
    FP16, BF16 = orc.FP16, orc.BF16
    # fp16: +-(64 * 64 * K) is far above 65504
    A = orc.fill_constant((M, K), 64.0, FP16)
    B = orc.fill_constant((N, K), 64.0, FP16)
    B[1::2] = orc.fill_constant((N, K), -64.0, FP16)[1::2]
    C = Dev(mi, A, B, M, N).run(K, dtype=FP16)
    ref = orc.reference_cpu_gemm(A, B, dtype=FP16)
    assert set(np.unique(ref)) <= {0x7C00, 0xFC00} and (C == ref).all()
    # bf16: 1e19 * 1e19 * K overflows the fp32 accumulator
    A = orc.fill_constant((M, K), 1e19, BF16)
    B = orc.fill_constant((N, K), 1e19, BF16)
    C = Dev(mi, A, B, M, N).run(K)
    ref = orc.reference_cpu_gemm(A, B)
    assert (ref == 0x7F80).all() and (C == ref).all()
    # fp16 subnormal results: products 2^-13 * 2^-12 * {1, 0, 1, ...} sum to small multiples of 2^-25
    A = orc.fill_constant((M, K), 2.0 ** -13, FP16)
    B = np.zeros((N, K), np.uint16)
    for j in range(N):
        B[j, :(j % 7) + 1] = orc.fill_constant((1,), 2.0 ** -12, FP16)[0]     # (j % 7 + 1) * 2^-25
    C = Dev(mi, A, B, M, N).run(K, dtype=FP16)
    ref = orc.reference_cpu_gemm(A, B, dtype=FP16)
    assert len(np.unique(ref)) >= 4 and (ref < 0x0400).all()                    # subnormal halves, several values
    assert (C == ref).all(), f"{int((C != ref).sum())} elements differ"
    # subnormal inputs (bf16 2^-127, fp16 2^-15) are not flushed, nor are sums in the
    # subnormal range of fp32 / of the storage type
    for dtype, tiny, big, pa, pb in ((BF16, 0x0040, 2.0 ** 100, 2.0 ** -70, 2.0 ** -65),
                                    (FP16, 0x0200, 2.0 ** 10, 2.0 ** -14, 2.0 ** -14)):
        A = np.full((M, K), tiny, np.uint16)
        B = orc.fill_constant((N, K), big, dtype)
        ref = orc.reference_cpu_gemm(A, B, dtype=dtype)
        assert (ref != 0).all() and (Dev(mi, A, B, M, N).run(K, dtype=dtype) == ref).all()
        A = orc.fill_constant((M, K), pa, dtype)
        B = orc.fill_constant((N, K), pb, dtype)
        ref = orc.reference_cpu_gemm(A, B, dtype=dtype)
        assert (ref != 0).all() and (Dev(mi, A, B, M, N).run(K, dtype=dtype) == ref).all()
    # NaN in row 3 of A (if there is one)
    A, B = make_inputs(orc, M, N, K, "int")
    row = min(3, M - 1)
    A[row, K // 2] = 0x7FC0
    C = orc.to_f32(Dev(mi, A, B, M, N).run(K))
    assert np.isnan(C[row]).all() and not np.isnan(np.delete(C, row, axis=0)).any()


def test_tuned_shapes_file_is_used_by_the_launch(mi, orc, tmp_path):
    """A shape listed in MI_GEMM_TUNED_FILE runs the listed configuration: in a process of its
    own (the file is read once), the automatic launch leaves the trace records of that
    configuration's grid and the oracle's bits."""
    tuned = tmp_path / "tuned.txt"
    tuned.write_text("768 1024 512 m128x128_w2x2_g4_b1_o2\n")
    code = (
        "import numpy as np, h100_gemm_amd as mi\n"
        "from oracle import oracle as orc\n"
        "M, N, K = 768, 1024, 512\n"
        "A, B = orc.fill_randint((M, K), 69, 1), orc.fill_randint((N, K), 69, 2)\n"
        "dA, dB, dC = mi.DeviceBuffer.from_numpy(A), mi.DeviceBuffer.from_numpy(B), mi.DeviceBuffer(M * N * 2)\n"
        "words = mi._lib.load().mi_gemm_trace_words(M, N, K)\n"
        "dDB = mi.DeviceBuffer(words * 4); dDB.fill_bytes(0xFF)\n"
        "mi.runKernel(M, N, K, dA, dB, dC, dDB); mi.synchronize()\n"
        "db = dDB.to_numpy((words,), np.int32)\n"
        "print(mi.config_name(mi.select_config(M, N, K)), int((db[5::6] == 1).sum()),\n"
        "      bool((dC.to_numpy((M, N), np.uint16) == orc.reference_cpu_gemm(A, B)).all()))\n")
    env = dict(os.environ, MI_GEMM_TUNED_FILE=str(tuned), PYTHONPATH=str(ROOT))
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=env, cwd=ROOT, timeout=100)
    assert out.returncode == 0, out.stdout + out.stderr
    assert out.stdout.split() == ["m128x128_w2x2_g4_b1_o2", "48", "True"], out.stdout     # 6 x 8 tiles of 128 x 128


def test_output_buffer_is_not_overrun(mi, orc):
    M, N, K = 257, 515, 77
    A, B = make_inputs(orc, M, N, K, "int")
    d = Dev(mi, A, B, M, N)
    d.run(K)
    tail = d.dC.to_numpy((M * N + 32,), np.uint16)[M * N:]
    assert (tail == 0xFFFF).all()


def test_fp16_storage(mi, orc):
    for M, N, K in [(512, 512, 512), (130, 70, 200)]:
        check(mi, orc, M, N, K, "int", dtype=orc.FP16, exact=True)
        check(mi, orc, M, N, K, "uniform", dtype=orc.FP16)


def test_known_answer_fills(mi, orc):
    # constant_fill / arange_fill closed forms (common.h:292-307)
    M, N, K = 256, 256, 256
    A = orc.fill_constant((M, K), 0.5)
    B = orc.fill_constant((N, K), 2.0)
    C = Dev(mi, A, B, M, N).run(K)
    assert (orc.to_f32(C) == 256.0).all()
    A = orc.fill_arange((M, K), bound=16)
    want = np.array([sum((i * K + k) % 16 for k in range(K)) for i in range(M)], dtype=np.float32)
    C = Dev(mi, A, orc.fill_constant((N, K), 1.0), M, N).run(K)
    assert (C == orc.from_f32(np.repeat(want[:, None], N, 1))).all()
    # identity: I . B^T = B^T exactly
    eye = orc.from_f32(np.eye(256, dtype=np.float32))
    Bu = orc.fill_uniform((384, 256), 5, 2)
    assert (Dev(mi, eye, Bu, 256, 384).run(256) == Bu.T).all()


# ------------------------------------------------------- properties at full size ------

def test_full_size_permutation_equivariance_and_determinism(mi, orc):
    M = N = K = 8192
    A, B = make_inputs(orc, M, N, K, "uniform")
    d = Dev(mi, A, B, M, N)
    C0 = d.run(K)
    assert (d.run(K) == C0).all()                         # run-to-run bit identical
    rng = np.random.default_rng(3)
    pm, pn = rng.permutation(M), rng.permutation(N)
    C1 = Dev(mi, A[pm], B[pn], M, N).run(K)
    assert (C1 == C0[pm][:, pn]).all()                    # element values do not depend on tile
    # zero K tail: K columns of zeros appended change nothing
    Ah = np.concatenate([A[:, :4096], np.zeros((M, 64), np.uint16)], axis=1)
    Bh = np.concatenate([B[:, :4096], np.zeros((N, 64), np.uint16)], axis=1)
    Ca = Dev(mi, np.ascontiguousarray(A[:, :4096]), np.ascontiguousarray(B[:, :4096]), M, N).run(4096)
    Cb = Dev(mi, Ah, Bh, M, N).run(4160)
    assert (Ca == Cb).all()


# ----------------------------------------------------- the harness's GPU golden -------

def test_reference_gpu_gemm_is_bit_identical_to_the_oracle(mi, orc):
    # same ascending-k fp32 accumulation, so not merely close: identical
    for M, N, K, fill in [(300, 200, 517, "uniform"), (64, 64, 64, "normal"), (1, 5, 3, "uniform")]:
        A, B = make_inputs(orc, M, N, K, fill)
        dA, dB = mi.DeviceBuffer.from_numpy(A), mi.DeviceBuffer.from_numpy(B)
        dC = mi.DeviceBuffer(M * N * 2)
        mi.reference_gpu_gemm(mi.GemmParams(M, N, K, dA, dB, dC, 1.0, 0.0))
        mi.synchronize()
        assert (dC.to_numpy((M, N), np.uint16) == orc.reference_cpu_gemm(A, B)).all()
        mi.reference_gpu_gemm(mi.GemmParams(M, N, K, dA, dB, dC, 0.5, 0.25))   # scalar beta
        mi.synchronize()
        assert (dC.to_numpy((M, N), np.uint16) == orc.reference_cpu_gemm(A, B, alpha=0.5, beta=0.25)).all()


# ------------------------------------------------------------------ trace buffer ------

def test_db_trace_records(mi, orc):
    """The DB buffer of runKernel's signature (matmul_h100_optimal.cu:32,132-139,182-198): every
    kernel family writes one record {sumLoad, cntLoad, sumCompute, cntCompute, sumStore,
    cntStore} per workgroup, a trace buffer never changes which kernel the automatic choice
    runs, and results are the same with and without it."""
    from h100_gemm_amd import kernel_configs as kc
    L = mi._lib.load()

    def records(M, N, K, config, fill="int"):
        A, B = make_inputs(orc, M, N, K, fill)
        d = Dev(mi, A, B, M, N)
        plain = d.run(K, config).copy()
        words = L.mi_gemm_trace_words(M, N, K)
        dDB = mi.DeviceBuffer(words * 4)
        dDB.fill_bytes(0xFF)
        d.dC.fill_bytes(0xFF)
        C = d.run(K, config, DB=dDB)
        assert (C == plain).all(), f"{M}x{N}x{K}: tracing changed {int((C != plain).sum())} elements"
        if fill == "int":
            assert (C == orc.reference_cpu_gemm(A, B)).all()
        db = dDB.to_numpy((words,), np.int32)
        n = 0
        while n + 5 < words and db[n] != -1:
            n += 6
        assert db[n] == -1 and (db[n:] == -1).all()         # the records are contiguous, the sentinel untouched
        for b in (d.dA, d.dB, d.dC, dDB):
            b.free()
        rec = db[:n].reshape(-1, 6)
        assert (rec[:, 5] == 1).all() and (rec[:, 2] > 0).all() and (rec[:, 4] > 0).all()
        assert (rec[:, 0] >= 0).all() and (rec[:, 0] < rec[:, 2]).all() and (rec[:, 1] > 0).all()
        return rec

    # a tiled kernel by name: one record per tile, K / 64 steps each
    cfg = mi.find_config("m128x128_w2x2_g4_b1_o2")
    rec = records(1024, 1024, 1024, cfg)
    assert len(rec) == mi.config_grid(cfg, 1024, 1024, 1024) == 64 and (rec[:, 3] == 16).all()
    # the automatic choice on the shapes of the benchmark's other kernel families: 512^3 (small
    # tiles on a shared ring: every unit of K), 512 x 512 x 4096 (small tiles, K split over the
    # waves: wave 0's units), 16 x 8192 x 8192 (single-pass decode: wave 0's slabs), 128 x 8192 x
    # 8192 (split-K decode: a record per column tile and piece), and a mid-sized output on the
    # shared-ring kernel
    for (M, N, K), kind, units in [((512, 512, 512), "wavek", lambda c: 512 // 64),
                                   ((512, 512, 4096), "wavek", lambda c: 4096 // 64 // 4),
                                   ((16, 8192, 8192), "stream", lambda c: 8192 // 64 // 4),
                                   ((128, 8192, 8192), "decode", lambda c: 8192 // 64 // 4),
                                   ((1440, 1440, 1472), "wavek", lambda c: 1472 // 64)]:
        auto = mi.select_config(M, N, K)
        assert kc.CONFIGS[auto]["KIND"] == kind, (M, N, K, mi.config_name(auto))
        rec = records(M, N, K, mi.MI_CONFIG_AUTO)
        assert len(rec) == mi.config_grid(auto, M, N, K), (M, N, K, len(rec))
        assert (rec[:, 3] == units(auto)).all(), (M, N, K, rec[:4])
    # K cut over workgroups: the tiled split-K (256 x 8192 x 8192) and the small-tile kernels' (128 x 384 x 13376)
    for M, N, K in [(256, 8192, 8192), (128, 384, 13376)]:
        auto = mi.select_config(M, N, K)
        grid = mi.config_grid(auto, M, N, K)
        tiles = -(-M // kc.CONFIGS[auto]["BM"]) * -(-N // kc.CONFIGS[auto]["BN"])
        assert grid > tiles and grid % tiles == 0                       # more than one piece per tile
        rec = records(M, N, K, mi.MI_CONFIG_AUTO)
        assert len(rec) == grid, (M, N, K, len(rec), grid)
    # a shape that runs as two GEMMs: the first part's records, then the second part's
    M, N, K = 7000, 7000, 4096
    m1 = mi.row_cut(M, N, K)
    assert m1 > 0
    rec = records(M, N, K, mi.MI_CONFIG_AUTO, fill="uniform")
    first, second = mi.select_config(m1, N, K), mi.select_config(M - m1, N, K)
    assert len(rec) == mi.config_grid(first, m1, N, K) + mi.config_grid(second, M - m1, N, K)


# --------------------------------------------------------------- C++ harness ----------

def test_harness_programs(mi):
    h = ROOT / "h100_gemm_amd" / "harness"
    if not (h / "test").exists():
        pytest.fail("harness programs are not built (make -C h100_gemm_amd/harness)")
    r = subprocess.run([str(h / "test"), "M", "640", "N", "384", "K", "512", "iters", "5"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "Shape M=640, N=384, K=512" in r.stdout and "Correct!" in r.stdout
    assert re.search(r"Average latency \(ms\) is ([\d.]+)", r.stdout)        # the tuner's regex
    # an HBM-bound shape whose operands would fit the memory-side cache is timed over several
    # copies of A and B by default (64 x 4096 x 4096: 32.5 MiB a set -> 8 copies), `rotate` overrides
    r = subprocess.run([str(h / "test"), "M", "64", "N", "4096", "K", "4096", "iters", "20"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "Correct!" in r.stdout and "Timing over 8 copies of A and B in turn" in r.stdout, r.stdout + r.stderr
    r = subprocess.run([str(h / "test"), "M", "64", "N", "4096", "K", "4096", "iters", "20", "rotate", "3"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "Timing over 3 copies of A and B in turn" in r.stdout, r.stdout + r.stderr
    assert "Timing over" not in subprocess.run([str(h / "test"), "M", "640", "N", "384", "K", "512", "iters", "5", "rotate", "1"],
                                               capture_output=True, text=True, timeout=120).stdout
    r = subprocess.run([str(h / "test"), "M", "333", "N", "129", "K", "77", "iters", "2",
                        "dtype", "fp16"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "Correct!" in r.stdout, r.stdout + r.stderr
    for extra in (["alpha", "0.5", "beta", "2"], ["cmajor", "1"], ["alpha", "-2", "beta", "0.25", "cmajor", "1", "fill", "uniform"]):
        r = subprocess.run([str(h / "test"), "M", "333", "N", "129", "K", "77", "iters", "2", *extra],
                           capture_output=True, text=True, timeout=120)
        assert r.returncode == 0 and "Correct!" in r.stdout, r.stdout + r.stderr
    r = subprocess.run([str(h / "bf16_bench"), "1024", "4"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "KERNEL 1" in r.stdout
    assert re.search(r"Average elapsed time: \(\s*[\d.]+\) s, performance: \(\s*[\d.]+\) TFLOPS\. size: \(1024\)\.", r.stdout)


def test_tuner_rendered_programs_run_and_feed_the_tuner(mi, tmp_path):
    """The tuner's own flow on the GPU (gemm_tuner.py:34-72 of the reference: render -> compile
    -> run `./test M m N n K k` -> parse the latency line).  The sample configurations the
    build rendered from template/matmul_mi355x.hip.jinja -- a 16x16x32 kernel with the drain
    barrier, a 32x32x16 two-per-CU kernel, and two points of the LDS-stage sweep that the
    library itself does not compile: a split-K decode kernel with a ring of four slabs and a
    small-tile kernel with per-wave rings of three stages -- instantiate their kernels directly,
    without the library's dispatch.  Each runs aligned and ragged shapes against the on-device
    golden; then GemmTuner.tune(prebuilt=True) sweeps them and its outputs are checked."""
    import json
    from h100_gemm_amd import build as lib_build
    from h100_gemm_amd.gemm_tuner import DEFAULT_TEMPLATE, GemmTuner, LATENCY_RE
    bindir = lib_build.TUNER_SAMPLES / "bin"
    tuner = GemmTuner(str(DEFAULT_TEMPLATE), str(tmp_path / "out"), bin_dir=str(bindir),
                      only=lib_build.TUNER_SAMPLE_CONFIGS, bench_args=("M", "128", "N", "768", "K", "512", "iters", "20"))
    configs = tuner.configurations()
    names = [tuner.config_name(p) for p in configs]
    assert len(names) == 4 and {p["KIND"] for p in configs} == {"mfma16", "tile", "decode", "wavek"}
    shapes = {"decode": (("128", "1024", "1024"), ("100", "516", "1088"), ("37", "8192", "4096")),      # M <= 128, N % 4 == 0, K % 64 == 0
              None: (("512", "512", "512"), ("257", "515", "77"), ("1000", "300", "1032"))}
    for p, name in zip(configs, names):
        exe = bindir / name
        assert exe.exists(), f"{exe} is not built (python -m h100_gemm_amd.build)"
        for shape in shapes.get(p["KIND"], shapes[None]):
            for extra in ([], ["dtype", "fp16"], ["fill", "uniform"]):
                print(f"case tuner program {name} M N K = {shape} {extra}", flush=True)
                r = subprocess.run([str(exe), "M", shape[0], "N", shape[1], "K", shape[2], "iters", "3", *extra],
                                   capture_output=True, text=True, timeout=120)
                assert r.returncode == 0, r.stdout + r.stderr
                assert f"Shape M={shape[0]}, N={shape[1]}, K={shape[2]}" in r.stdout and "Correct!" in r.stdout
                assert LATENCY_RE.search(r.stdout) and name in r.stdout, r.stdout
    # a shape a decode configuration cannot run ends its program with an error, which the tuner scores as a failure
    decode_exe = bindir / names[[p["KIND"] for p in configs].index("decode")]
    r = subprocess.run([str(decode_exe), "M", "512", "N", "512", "K", "512", "iters", "3"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "needs M <= 128" in r.stderr
    best_params, best_runtime, results = tuner.tune(prebuilt=True)
    assert len(results) == 4 and all(r["success"] and 0 < r["runtime"] < 5 for r in results), results
    assert best_params in lib_build.TUNER_SAMPLE_CONFIGS and best_runtime == min(r["runtime"] for r in results)
    doc = json.loads(sorted((tmp_path / "out").glob("tuning_results_*.json"))[-1].read_text())
    assert set(doc) == {"results", "best_params", "best_runtime", "timestamp"}
    assert set(doc["results"][0]) == {"params", "runtime", "success", "timestamp"}
    assert doc["best_params"] == best_params
    assert f"Best runtime: {best_runtime:.4f} ms" in (tmp_path / "out" / "tuning_summary.txt").read_text()
    assert f"STAGES = {best_params['NS']};" in (tmp_path / "out" / "best_matmul_mi355x.hip").read_text()
    # a configuration that was not compiled scores as a failure and the sweep goes on
    tuner2 = GemmTuner(str(DEFAULT_TEMPLATE), str(tmp_path / "out2"), bin_dir=str(bindir),
                       only=[dict(lib_build.TUNER_SAMPLE_CONFIGS[0], GROUP=8)] + lib_build.TUNER_SAMPLE_CONFIGS[1:2],
                       bench_args=("M", "512", "N", "512", "K", "512", "iters", "5"))
    bp, br, res = tuner2.tune(prebuilt=True)
    assert [r["success"] for r in res] == [False, True] and bp == lib_build.TUNER_SAMPLE_CONFIGS[1]


def test_mfma_ceiling_program(mi):
    """The MFMA-only yardstick program: same issue rate for every data set (a 16x16x32 MFMA is
    16 cycles), and zeros must not be slower than random operands (the chip is power limited)."""
    exe = ROOT / "h100_gemm_amd" / "harness" / "mfma_ceiling"
    assert exe.exists(), f"{exe} is not built (make -C h100_gemm_amd/harness)"
    out = subprocess.run([str(exe), "60"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    rows = re.findall(r"^(.+?)\s+([\d.]+) cycles per MFMA, clock ([\d.]+) GHz, (\d+) TFLOP/s$", out.stdout, re.M)
    assert [r[0].strip() for r in rows] == ["zeros", "uniform [-1,1) bf16", "normal(0,1) bf16"], out.stdout
    for name, cyc, clock, tf in rows:
        assert 16.0 <= float(cyc) <= 17.5, (name, cyc)
        assert 0.5 <= float(clock) <= 2.6, (name, clock)
    assert int(rows[0][3]) >= int(rows[1][3]) * 0.98, rows


def test_vendor_side_by_side_program(mi):
    """kernel 0 (vendor BLAS, linked into this program only) and kernel 1 on the same buffers:
    the loop of matmul_h100_optimal.cu:157-217 with the comparison of :177-180 switched on."""
    exe = ROOT / "h100_gemm_amd" / "harness" / "vendor_bench"
    if not exe.exists():
        pytest.fail("vendor_bench is not built (make -C h100_gemm_amd/harness)")
    for shape in (("512", "512", "512"), ("333", "257", "130"), ("16", "1024", "512")):
        r = subprocess.run([str(exe), *shape, "3", "0"], capture_output=True, text=True, timeout=120)
        assert r.returncode == 0, r.stdout + r.stderr
        assert r.stdout.index("KERNEL 0") < r.stdout.index("KERNEL 1")
        assert "Matches the vendor BLAS within tolerance." in r.stdout
        assert len(re.findall(r"Average elapsed time: \(\s*[\d.]+\) s, performance: \(\s*[\d.]+\) TFLOPS\.", r.stdout)) == 2


# ------------------------------- alpha / beta epilogue and column-major C (mi_gemm_epilogue) ----

def check_epilogue(mi, orc, M, N, K, fill, alpha, beta, c_layout=0, config=-1, dtype=0, exact=False):
    """C = storage(acc * alpha + beta), beta a plain scalar (reference.h:40); column-major C is
    C[n*M + m] (matmul_utils.cuh:545), i.e. the transpose of the oracle's row-major result.
    Tolerance: the benchmark bound with its absolute term scaled by |alpha|."""
    print(f"case epilogue M={M} N={N} K={K} fill={fill} alpha={alpha} beta={beta} layout={c_layout} "
          f"config={config} dtype={dtype}", flush=True)
    A, B = make_inputs(orc, M, N, K, fill, dtype)
    C = Dev(mi, A, B, M, N).run_epilogue(K, alpha, beta, c_layout, config, dtype)
    ref = orc.reference_cpu_gemm(A, B, alpha=alpha, beta=beta, dtype=dtype)
    if c_layout == mi.MI_C_COL_MAJOR:
        C = np.ascontiguousarray(C.T)
    if exact:
        assert (C == ref).all(), f"{int((C != ref).sum())} elements differ"
    rep = orc.check_tolerance(C, ref, K, orc.max_abs(A, dtype) * abs(alpha), orc.max_abs(B, dtype), dtype)
    assert rep["violations"] == 0 and rep["compared"] == M * N, rep


@pytest.mark.parametrize("config", all_configs(("tile", "ring", "mfma16", "ring16")))
def test_alpha_beta_every_tiled_config_bit_exact_on_integer_fill(mi, orc, config):
    # integer inputs, alpha a small integer or a power of two, beta a multiple of 1/4: acc * alpha
    # and + beta are exact in fp32, so every summation order must give the oracle's bits
    for (M, N, K), (alpha, beta) in [((512, 512, 512), (0.5, 3.0)), ((257, 515, 77), (-2.0, 0.25)),
                                     ((300, 200, 136), (3.0, -1.5)), ((256, 384, 191), (1.0, 7.0)),
                                     ((512, 768, 256), (0.25, 0.0))]:
        check_epilogue(mi, orc, M, N, k_for(config, K), "int", alpha, beta, config=config, exact=True)


@pytest.mark.parametrize("config", all_configs(("stream", "decode")))
def test_alpha_beta_decode_kernels(mi, orc, config):
    from h100_gemm_amd import kernel_configs as kc
    bm = kc.CONFIGS[config]["BM"]
    for N, K in [(8192, 4096), (260, 192), (128, 64)]:      # several splits / one split
        check_epilogue(mi, orc, bm - 1, N, K, "int", -0.5, 2.75, config=config, exact=True)
    check_epilogue(mi, orc, bm, 2048, 8192, "normal", 0.37, 1.25, config=config)


@pytest.mark.parametrize("M,N,K", [(512, 512, 512), (1024, 768, 256), (255, 511, 129), (16, 2048, 1024),
                                   (64, 4096, 4096), (4095, 6143, 3073)])
def test_alpha_beta_uniform_within_tolerance_auto_config(mi, orc, M, N, K):
    check_epilogue(mi, orc, M, N, K, "uniform", 0.37, 1.25)
    check_epilogue(mi, orc, M, N, K, "uniform", -1.5, 0.0)


def test_alpha_one_beta_zero_is_the_plain_gemm(mi, orc):
    for M, N, K in [(512, 512, 512), (257, 515, 77), (16, 2048, 1024), (100, 4096, 2048)]:
        A, B = make_inputs(orc, M, N, K, "uniform")
        d = Dev(mi, A, B, M, N)
        plain = d.run(K)
        assert (d.run_epilogue(K, 1.0, 0.0) == plain).all()


@pytest.mark.parametrize("M,N,K", [(512, 512, 512), (257, 515, 77), (768, 256, 384), (16, 2048, 1024),
                                   (2048, 16, 1024), (1, 7, 3)])
def test_column_major_c_bit_exact_on_integer_fill(mi, orc, M, N, K):
    check_epilogue(mi, orc, M, N, K, "int", 1.0, 0.0, c_layout=mi.MI_C_COL_MAJOR, exact=True)
    check_epilogue(mi, orc, M, N, K, "int", 0.5, -3.0, c_layout=mi.MI_C_COL_MAJOR, exact=True)


@pytest.mark.parametrize("M,N,K", [(1024, 768, 256), (4095, 6143, 3073), (128, 8192, 8192)])
def test_column_major_c_uniform_within_tolerance(mi, orc, M, N, K):
    check_epilogue(mi, orc, M, N, K, "uniform", 1.0, 0.0, c_layout=mi.MI_C_COL_MAJOR)


def test_epilogue_fp16_and_argument_errors(mi, orc):
    check_epilogue(mi, orc, 300, 200, 136, "int", 0.5, 1.0, dtype=1, exact=True)
    check_epilogue(mi, orc, 300, 200, 136, "int", 0.5, 1.0, c_layout=mi.MI_C_COL_MAJOR, dtype=1, exact=True)
    A, B = make_inputs(orc, 64, 64, 64, "int")
    d = Dev(mi, A, B, 64, 64)
    with pytest.raises(mi.MiGemmError, match="layout"):
        d.run_epilogue(64, 1.0, 0.0, c_layout=2)
    with pytest.raises(mi.MiGemmError, match="NaN"):
        d.run_epilogue(64, float("nan"), 0.0)


# ------------------------------------------- split-K of the tiled 16x16x32 kernel ----------

@pytest.mark.parametrize("config", all_configs(("mfma16",), k_groups=False))
def test_tiled_split_k_bit_exact_on_integer_fill(mi, orc, config):
    """Few tiles and a long K: the K range is cut into pieces, fp32 partials are added in order.
    Integer fills keep every partial sum exact, so the result must match the oracle's bits."""
    from h100_gemm_amd import kernel_configs as kc
    c = kc.CONFIGS[config]
    for M, N, K in [(512, 768, 4096), (300, 260, 5000), (256, 256, 8192 + 64), (130, 512, 2048)]:
        tiles = -(-M // c["BM"]) * -(-N // c["BN"])
        assert mi.config_grid(config, M, N, K) >= 2 * tiles, "shape chosen so that split-K is in effect"
        check(mi, orc, M, N, K, "int", config=config, exact=True)


def test_tiled_split_k_auto_config_uniform_fp16_and_epilogue(mi, orc):
    for M, N, K in [(512, 512, 4096), (512, 512, 8192), (1000, 500, 3000)]:
        cfg = mi.select_config(M, N, K)
        assert mi.config_grid(cfg, M, N, K) > -(-M // 128) * -(-N // 128) or "mfma16" not in str(cfg)
        check(mi, orc, M, N, K, "uniform")
    check(mi, orc, 512, 512, 4096, "int", dtype=1, exact=True)
    check_epilogue(mi, orc, 512, 512, 4096, "int", 0.5, -3.0, exact=True)
    check_epilogue(mi, orc, 300, 260, 5000, "uniform", 0.37, 1.25)
    check_epilogue(mi, orc, 4096, 256, 4096, "int", 2.0, 1.0, c_layout=mi.MI_C_COL_MAJOR, exact=True)
    # odd N: no split-K (the reduction needs N % 4 == 0), same answer
    check(mi, orc, 512, 511, 4096, "int", exact=True)


def test_tiled_split_k_is_deterministic(mi, orc):
    A, B = make_inputs(orc, 512, 512, 8192, "uniform")
    d = Dev(mi, A, B, 512, 512)
    first = d.run(8192)
    for _ in range(3):
        assert (d.run(8192) == first).all()


def test_tiled_split_k_random_shapes_and_alignments(mi, orc):
    # seeded sweep over few-tile shapes with a long, ragged K (split-K pieces with a K tail in
    # the last one), operands at arbitrary even byte offsets; C at 8-byte offsets (split-K) and at
    # 2-byte offsets (the reduction cannot be used: one piece); automatic choice and every
    # candidate tile of it
    from h100_gemm_amd import kernel_configs as kc
    rng = np.random.default_rng(20241125)
    configs = [-1] + [i for i, c in enumerate(kc.CONFIGS) if c["KIND"] == "mfma16" and c.get("EFF") and c.get("KG", 1) == 1]
    for it in range(32):
        M = int(rng.integers(1, 420))
        N = int(rng.integers(1, 110)) * 4
        K = int(rng.choice([rng.integers(2048, 6000), 128 * rng.integers(16, 40), 128 * rng.integers(16, 40) + rng.integers(1, 9)]))
        offA, offB = (int(2 * rng.integers(0, 16)) for _ in range(2))
        offC = int(rng.choice([0, 8, 16, 2, 6]))
        config = configs[it % len(configs)]
        print(f"case {it}: M={M} N={N} K={K} offsets {offA},{offB},{offC} config={config}", flush=True)
        C, ref, guard = _run_offset(mi, orc, config, M, N, K, offA, offB, offC)
        assert (C == ref).all(), f"{int((C != ref).sum())} elements differ"
        assert (guard == 0xEEEE).all(), "bytes outside C were written"


# (alpha, beta, acc) for which bf16(fl(fl(acc*alpha) + beta)) != bf16(fma(acc, alpha, beta)): found by
# search; acc = a*b with small integers, so the accumulator is exact in every kernel
UNFUSED_CASES = [(2.1086061000823975, 6.344648361206055, 936), (3.681880235671997, -1.8010832071304321, -276),
                 (1.982526421546936, -5.732435703277588, 187), (1.0196295976638794, -5.7203168869018555, 6),
                 (0.6559985280036926, 5.435117244720459, -3240), (1.5280640125274658, -5.5986127853393555, 2480),
                 (0.19303591549396515, 2.4593822956085205, -35)]


def _bf16_bits(x):
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


@pytest.mark.parametrize("alpha,beta,acc", UNFUSED_CASES)
def test_alpha_beta_are_two_roundings_not_an_fma(mi, orc, alpha, beta, acc):
    """reference.h:40 computes acc * alpha + beta as a product rounded to fp32 and then a sum
    rounded to fp32.  These inputs give a different bf16 result when the two are fused into one
    fma, in every kernel family: tiled aligned / predicated, split-K pieces, both decode kernels,
    the GPU golden."""
    a = next(d for d in range(1, 65) if acc % d == 0 and abs(acc // d) <= 64)
    b = acc // a
    un = (np.float32(np.float32(acc) * np.float32(alpha)) + np.float32(beta)).astype(np.float32)
    fu = np.float32(np.float64(acc) * np.float64(np.float32(alpha)) + np.float64(np.float32(beta)))
    assert _bf16_bits(un) != _bf16_bits(fu), "the case no longer tells one fma from two roundings"
    for M, N, K in [(64, 64, 1), (256, 256, 128), (300, 260, 200), (512, 512, 4096), (16, 256, 128), (64, 256, 256),
                    (128, 512, 2048)]:
        A = np.zeros((M, K), np.float32)
        B = np.zeros((N, K), np.float32)
        A[:, K // 2] = a
        B[:, K // 2] = b
        A, B = orc.from_f32(A, 0), orc.from_f32(B, 0)
        ref = orc.reference_cpu_gemm(A, B, alpha=alpha, beta=beta)
        assert (ref == _bf16_bits(un)).all()
        d = Dev(mi, A, B, M, N)
        assert (d.run_epilogue(K, alpha, beta) == ref).all(), (M, N, K)
        p = mi.GemmParams(M, N, K, d.dA, d.dB, d.dC, alpha, beta)
        mi.reference_gpu_gemm(p)
        mi.synchronize()
        assert (d.dC.to_numpy((M, N), np.uint16) == ref).all(), ("golden", M, N, K)


def test_automatic_choice_across_regimes_bit_exact(mi, orc):
    """The shape -> kernel choice has many branches (decode rules with their N / K conditions,
    tuned shapes, tile model, split-K pieces, aligned / predicated twins).  Shapes on both sides
    of each boundary, integer fill, automatic choice: every result must match the oracle's bits,
    whichever kernel ran."""
    shapes = []
    for M in (1, 16, 17, 32, 33, 64, 65, 128, 129, 256, 257):
        shapes += [(M, 4096, 4096), (M, 1024, 8192), (M, 8192, 512), (M, 4100, 1088)]
    shapes += [(64, 4096, 24576), (128, 4096, 24576), (96, 16384, 1024), (128, 8192, 8192), (48, 8192, 2048),
               (130, 4096, 24640), (512, 512, 4096), (3000, 3000, 264), (384, 384, 6016), (192, 8192, 2048),
               (64, 8192, 8192), (24, 32768, 2048), (96, 8192, 12288), (96, 8192, 16384), (40, 8192, 6144)]
    seen = set()
    for M, N, K in shapes:
        cfg = mi.select_config(M, N, K)
        seen.add(mi.config_name(cfg))
        print(f"case M={M} N={N} K={K} -> {mi.config_name(cfg)} grid {mi.config_grid(cfg, M, N, K)}", flush=True)
        check(mi, orc, M, N, K, "int", exact=True)
    # the sweep is only worth its time if it reaches the different kernel families
    assert {"s16x32_n3", "s32x32_n3", "s64x32_n3", "d64x128_n4", "d128x128_n3"} <= seen, seen
    assert any(n.startswith("m128x256") for n in seen) and any(n.startswith("m128x128") for n in seen), seen
