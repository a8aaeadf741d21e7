"""Pins the CPU oracle (oracle/ref_gemm.c) -- CPU only, no GPU.

The reference tree holds no golden vectors, known-answer tests or fixtures for this path
(its programs self-check against a GPU kernel or a vendor BLAS at run time), and its header
cannot be compiled in this image, so every function of the oracle is pinned by what the
mathematics fixes:

  reference_cpu_gemm   exact-integer fills (any summation order must agree bit for bit),
                       closed forms (constant, arange), brute-force Python loops on tiny
                       ragged shapes, a float64 BLAS product within the fp32-sum bound,
                       identity / permutation invariants, the scalar-beta quirk, poisoned
                       out-of-range rows, loop-order-faithful == vectorised, tile subsets
  bf16 / fp16 rounding exhaustive round trip + an independent implementation (torch, numpy)
  fills                committed known answers produced by a pure-Python restatement
  checkers             hand-worked cases
"""
import json
import math
from pathlib import Path

import numpy as np
import pytest

GOLD = json.loads((Path(__file__).parent / "golden" / "rng_fixture.json").read_text())


def f32_of(orc, bits, dtype=0):
    return orc.to_f32(np.asarray(bits, dtype=np.uint16), dtype)


# --------------------------------------------------------------------- conversions ----

def test_bf16_round_trip_exhaustive(orc):
    allbits = np.arange(65536, dtype=np.uint16)
    f = orc.to_f32(allbits)
    back = orc.from_f32(f)
    nan = np.isnan(f)
    assert (back[~nan] == allbits[~nan]).all()
    assert np.isnan(orc.to_f32(back[nan])).all()          # NaN stays NaN
    # exact widening: bf16 bits are the top half of the float32 pattern
    assert (f.view(np.uint32) == allbits.astype(np.uint32) << 16).all()


def test_bf16_rounding_matches_independent_implementation(orc):
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(0)
    bits = rng.integers(0, 2**32, size=400000, dtype=np.uint64).astype(np.uint32)
    f = bits.view(np.float32)
    f = f[~np.isnan(f)]
    want = torch.from_numpy(f.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert (orc.from_f32(f) == want).all()


def test_bf16_ties_and_specials_known_answers(orc):
    for fbits, want in GOLD["bf16_cases"]:
        f = np.array([fbits], dtype=np.uint32).view(np.float32)
        got = int(orc.from_f32(f)[0])
        assert got == want, (hex(fbits), hex(got), hex(want))
    # 1 + 2^-8 is a tie -> 1.0 (even); 1 + 3*2^-8 is a tie -> 1 + 2^-6
    assert orc.to_f32(orc.from_f32(np.float32([1 + 2**-8])))[0] == 1.0
    assert orc.to_f32(orc.from_f32(np.float32([1 + 3 * 2**-8])))[0] == 1 + 2**-6


def test_fp16_matches_numpy_exhaustive(orc):
    allbits = np.arange(65536, dtype=np.uint16)
    want = allbits.view(np.float16).astype(np.float32)
    got = orc.to_f32(allbits, orc.FP16)
    nan = np.isnan(want)
    assert (got[~nan] == want[~nan]).all() and np.isnan(got[nan]).all()
    rng = np.random.default_rng(1)
    f = (rng.standard_normal(300000) * np.exp(rng.uniform(-20, 12, 300000))).astype(np.float32)
    f = np.concatenate([f, np.float32([0, -0.0, 65504, 65519.9, 65520, 1e-8, 5.96e-8, 2.98e-8,
                                       2.9802322e-08, 6.1035156e-05, np.inf, -np.inf])])
    with np.errstate(over="ignore"):
        want_bits = f.astype(np.float16).view(np.uint16)
    assert (orc.from_f32(f, orc.FP16) == want_bits).all()


# --------------------------------------------------------------------------- fills ----

def test_rng_known_answers(orc):
    for s, i, v in GOLD["u64"]:
        assert orc.lib().orc_rng_u64(GOLD["seed"], s, i) == v
    assert (orc.fill_uniform((64,), 69, 1) == np.array(GOLD["uniform_stream1"])).all()
    assert (orc.fill_uniform((64,), 69, 2) == np.array(GOLD["uniform_stream2"])).all()
    assert (orc.fill_normal((64,), 69, 1, 1.0) == np.array(GOLD["normal_stream1_sigma1"])).all()
    assert (orc.fill_normal((64,), 69, 2, 0.02) == np.array(GOLD["normal_stream2_sigma002"])).all()
    assert (orc.fill_randint((64,), 69, 1) == np.array(GOLD["randint_stream1"])).all()


def test_fill_statistics_and_ranges(orc):
    u = orc.to_f32(orc.fill_uniform((1 << 18,), 69, 1))
    assert u.min() >= -1.0 and u.max() <= 1.0 and abs(u.mean()) < 0.01
    assert abs(u.var() - 1 / 3) < 0.01
    z = orc.to_f32(orc.fill_normal((1 << 18,), 69, 1, 1.0))
    assert abs(z.mean()) < 0.01 and abs(z.std() - 1.0) < 0.01
    w = orc.to_f32(orc.fill_normal((1 << 18,), 69, 2, 0.02))
    assert abs(w.std() - 0.02) < 3e-4
    r = orc.to_f32(orc.fill_randint((1 << 16,), 69, 1))
    assert set(np.unique(r)) == set(range(-5, 5))            # common.h:287 -> [-5, 4]
    # counter based: a slice regenerates identically, streams differ
    full = orc.fill_uniform((1000,), 69, 1)
    assert (orc.fill_uniform((10,), 69, 1) == full[:10]).all()
    assert (orc.fill_uniform((1000,), 69, 2) != full).any()


def test_arange_and_constant_fill(orc):
    a = orc.to_f32(orc.fill_arange((3, 100), bound=128))          # common.h:292-299
    assert (a.reshape(-1) == np.arange(300) % 128).all()
    c = orc.to_f32(orc.fill_constant((5, 7), 0.5))
    assert (c == 0.5).all()


# ---------------------------------------------------------------------------- GEMM ----

def brute_force(orc, A, B, alpha=1.0, beta=0.0, dtype=0):
    """Pure-Python triple loop: ascending-k float32 running sum, one rounding per add."""
    a = orc.to_f32(A, dtype)
    b = orc.to_f32(B, dtype)
    M, K = a.shape
    N = b.shape[0]
    out = np.zeros((M, N), dtype=np.float32)
    for i in range(M):
        for j in range(N):
            acc = np.float32(0)
            for k in range(K):
                acc = np.float32(acc + np.float32(a[i, k] * b[j, k]))
            out[i, j] = np.float32(np.float32(acc * np.float32(alpha)) + np.float32(beta))
    return orc.from_f32(out, dtype)


@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (3, 5, 7), (65, 66, 33), (64, 64, 32), (70, 3, 95),
                                   (2, 130, 31)])
@pytest.mark.parametrize("fast", [False, True])
def test_gemm_equals_brute_force_on_ragged_shapes(orc, M, N, K, fast):
    # exercises the k-block break (reference.h:25), modulo-wrapped reads (:30) and the
    # predicated store (:39) with M, N not multiples of 64 and K not a multiple of 32
    A = orc.fill_uniform((M, K), 7, 1)
    B = orc.fill_uniform((N, K), 7, 2)
    want = brute_force(orc, A, B)
    assert (orc.reference_cpu_gemm(A, B, fast=fast) == want).all()
    assert (orc.naive_gemm(A, B) == want).all()


def test_faithful_and_fast_agree_bitwise(orc):
    for (M, N, K, seed) in [(200, 130, 517, 1), (64, 64, 64, 2), (129, 257, 100, 3)]:
        A = orc.fill_normal((M, K), seed, 1, 1.0)
        B = orc.fill_normal((N, K), seed, 2, 0.02)
        c0, a0 = orc.reference_cpu_gemm(A, B, fast=False, want_acc=True)
        c1, a1 = orc.reference_cpu_gemm(A, B, fast=True, want_acc=True)
        assert (c0 == c1).all() and (a0.view(np.uint32) == a1.view(np.uint32)).all()


def test_integer_fill_is_exact_in_any_order(orc):
    # random_fill values are integers in [-5, 4]; with K*25 < 2^24 every partial sum is an
    # exact integer in fp32, so the GEMM must equal the int64 product rounded once to bf16
    M, N, K = 150, 140, 1000
    A = orc.fill_randint((M, K), 69, 1)
    B = orc.fill_randint((N, K), 69, 2)
    exact = orc.to_f32(A).astype(np.int64) @ orc.to_f32(B).astype(np.int64).T
    C, acc = orc.reference_cpu_gemm(A, B, want_acc=True)
    assert (acc == exact.astype(np.float32)).all()
    assert (C == orc.from_f32(exact.astype(np.float32))).all()


def test_constant_fill_closed_form(orc):
    # constant_fill(a), constant_fill(b) -> every C element is bf16(K*a*b) while K*a*b stays
    # exactly representable through the running sum
    for a, b, K in [(0.5, 2.0, 300), (1.0, 1.0, 256), (-0.25, 4.0, 1000), (3.0, 0.125, 77)]:
        A = orc.fill_constant((10, K), a)
        B = orc.fill_constant((9, K), b)
        C = orc.to_f32(orc.reference_cpu_gemm(A, B))
        want = orc.to_f32(orc.from_f32(np.float32([K * a * b])))[0]
        assert (C == want).all()


def test_arange_fill_closed_form(orc):
    # A[i,k] = (i*K+k) % 16, B = ones  ->  C[i,j] = sum_k ((i*K+k) % 16), exact small ints
    M, N, K = 20, 6, 48
    A = orc.fill_arange((M, K), bound=16)
    B = orc.fill_constant((N, K), 1.0)
    want = np.array([sum((i * K + k) % 16 for k in range(K)) for i in range(M)], dtype=np.float32)
    C, acc = orc.reference_cpu_gemm(A, B, want_acc=True)
    assert (acc == want[:, None]).all()


def test_against_float64_blas_within_fp32_sum_bound(orc):
    M, N, K = 130, 190, 2048
    A = orc.fill_uniform((M, K), 5, 1)
    B = orc.fill_uniform((N, K), 5, 2)
    _, acc = orc.reference_cpu_gemm(A, B, want_acc=True)
    a64 = orc.to_f32(A).astype(np.float64)
    b64 = orc.to_f32(B).astype(np.float64)
    exact = a64 @ b64.T
    # recursive fp32 summation: |err| <= (K-1) * 2^-24 * sum|a_k b_k| (first order)
    bound = (K - 1) * 2.0**-24 * (np.abs(a64) @ np.abs(b64).T) * 1.01
    assert (np.abs(acc.astype(np.float64) - exact) <= bound).all()
    # and a transposed operand or dropped term would be far outside it
    assert (np.abs((a64 @ b64.T) - (a64[:, ::-1] @ b64.T)) > bound).mean() > 0.9


def test_identity_and_permutation_invariants(orc):
    n = 96
    eye = orc.from_f32(np.eye(n, dtype=np.float32))
    B = orc.fill_uniform((70, n), 11, 2)
    C = orc.reference_cpu_gemm(eye, B)                 # I . B^T = B^T, already bf16-exact
    assert (C == B.T).all()
    A = orc.fill_uniform((50, n), 11, 1)
    perm_m = np.random.default_rng(0).permutation(50)
    perm_n = np.random.default_rng(1).permutation(70)
    C0 = orc.reference_cpu_gemm(A, B)
    assert (orc.reference_cpu_gemm(A[perm_m], B[perm_n]) == C0[perm_m][:, perm_n]).all()
    # zero K tail: appending zero columns to both operands changes nothing
    Az = np.concatenate([A, np.zeros((50, 37), np.uint16)], axis=1)
    Bz = np.concatenate([B, np.zeros((70, 37), np.uint16)], axis=1)
    assert (orc.reference_cpu_gemm(Az, Bz) == C0).all()


def test_alpha_beta_is_scale_then_scalar_add(orc):
    # reference.h:40 -- (CType)(acc * alpha + beta): beta is added to every element, it does
    # not multiply C; acc*alpha is rounded to fp32 before the add.
    A = orc.from_f32(np.float32([[1.0, 2.0]]))
    B = orc.from_f32(np.float32([[3.0, 4.0], [0.0, 0.0]]))
    C = orc.to_f32(orc.reference_cpu_gemm(A, B, alpha=0.5, beta=0.25))
    assert C[0, 0] == 0.5 * 11.0 + 0.25 and C[0, 1] == 0.25
    # previous content of C is irrelevant, and -0 * 1 + 0 = +0
    out = np.full((1, 2), 0xFFFF, dtype=np.uint16)
    An = orc.from_f32(np.float32([[-0.0, 0.0]]))
    Cb = orc.reference_cpu_gemm(An, B, out=out)
    assert (Cb == 0).all()
    assert (orc.naive_gemm(A, B, 0.5, 0.25) == orc.reference_cpu_gemm(A, B, alpha=0.5, beta=0.25)).all()


def test_wrapped_reads_never_reach_the_result(orc):
    # tiles past M/N read rows modulo M/N (reference.h:30) but store nothing for them (:39):
    # the rows that get wrapped onto must not leak into other elements
    M, N, K = 70, 67, 40
    A = orc.fill_uniform((M, K), 3, 1)
    B = orc.fill_uniform((N, K), 3, 2)
    C0 = orc.reference_cpu_gemm(A, B)
    A2, B2 = A.copy(), B.copy()
    A2[:58] = orc.from_f32(np.full((58, K), 1e30, np.float32))   # rows 0..57 are what 70..127 wrap to
    keep = orc.reference_cpu_gemm(A2, B2)
    assert (keep[58:] == C0[58:]).all()


def test_tile_subset_equals_full_run(orc):
    M, N, K = 300, 260, 96
    A = orc.fill_uniform((M, K), 9, 1)
    B = orc.fill_uniform((N, K), 9, 2)
    full = orc.reference_cpu_gemm(A, B)
    tiles = np.array([[0, 0], [4, 4], [2, 1], [4, 0]], dtype=np.int32)
    part = orc.reference_cpu_gemm(A, B, tiles=tiles)
    for ti, tj in tiles:
        sl = (slice(ti * 64, ti * 64 + 64), slice(tj * 64, tj * 64 + 64))
        assert (part[sl] == full[sl]).all()
    mask = np.ones((M, N), bool)
    for ti, tj in tiles:
        mask[ti * 64:ti * 64 + 64, tj * 64:tj * 64 + 64] = False
    assert (part[mask] == 0).all()
    st = orc.sample_tiles(8192, 8192, 64)
    assert len(st) == 64 and len({tuple(t) for t in st}) == 64
    assert {(0, 0), (0, 127), (127, 0), (127, 127)} <= {tuple(t) for t in st}
    assert len(orc.sample_tiles(100, 100, 64)) == 4


def test_fp16_gemm(orc):
    A = orc.fill_randint((40, 50), 1, 1, orc.FP16)
    B = orc.fill_randint((30, 50), 1, 2, orc.FP16)
    exact = orc.to_f32(A, orc.FP16).astype(np.int64) @ orc.to_f32(B, orc.FP16).astype(np.int64).T
    C = orc.reference_cpu_gemm(A, B, dtype=orc.FP16)
    assert (orc.to_f32(C, orc.FP16) == exact.astype(np.float16).astype(np.float32)).all()
    Au = orc.fill_uniform((5, 9), 1, 1, orc.FP16)
    Bu = orc.fill_uniform((4, 9), 1, 2, orc.FP16)
    assert (orc.reference_cpu_gemm(Au, Bu, dtype=orc.FP16) == brute_force(orc, Au, Bu, dtype=orc.FP16)).all()


# ------------------------------------------------------------------------ checkers ----

def test_allclose_semantics(orc):
    # common.h:367-397: error iff |r-g| > rtol*|g|  (g == 0 tolerates nothing)
    g = orc.from_f32(np.float32([1.0, 0.0, 100.0, -2.0]))
    r = orc.from_f32(np.float32([1.0, 0.0, 100.0, -2.0]))
    assert orc.allclose_count(r, g, 1e-3) == (0, 0.0, 0)
    r2 = orc.from_f32(np.float32([1.0078125, 0.0078125, 100.0, -2.0]))   # bf16-exact values
    e, avg, ninf = orc.allclose_count(r2, g, 1e-3)
    assert e == 2 and abs(avg - 0.0078125) < 1e-9 and ninf == 0
    assert orc.allclose_count(r2, g, 1e-2)[0] == 1            # only the g == 0 element left
    rinf = orc.from_f32(np.float32([np.inf, 0, 100, -2]))
    assert orc.allclose_count(rinf, g, 1e-3)[2] == 1


def test_absdiff_verify(orc):
    # matmul_h100_optimal.cu:94-108: first index with |bf16(ref - out)| > 0.1, or -1
    ref = orc.from_f32(np.float32([1.0, 2.0, 3.0, 19.125]))
    assert orc.absdiff_first_fail(ref, ref) == -1
    out = orc.from_f32(np.float32([1.0, 2.0, 3.0, 19.0]))
    assert orc.absdiff_first_fail(ref, out) == 3
    out2 = orc.from_f32(np.float32([1.0625, 2.0, 3.0, 19.125]))
    assert orc.absdiff_first_fail(ref, out2) == -1


def test_tolerance_checker(orc):
    K = 1024
    ref = orc.from_f32(np.float32([[100.0, 0.0], [-50.0, 8.0]]))
    # bound = 2^-7*|ref| + 1e-3*sqrt(K)*max_a*max_b = |ref|/128 + 0.032
    ok = orc.from_f32(np.float32([[100.5, 0.03125], [-50.25, 8.0625]]))
    rep = orc.check_tolerance(ok, ref, K, 1.0, 1.0)
    assert rep["violations"] == 0 and rep["compared"] == 4
    assert abs(rep["abs_term"] - 1e-3 * math.sqrt(K)) < 1e-12
    bad = orc.from_f32(np.float32([[101.0, 0.0], [-50.0, 8.0]]))        # err 1.0 > 0.813
    assert orc.check_tolerance(bad, ref, K, 1.0, 1.0)["violations"] == 1
    nan = ok.copy()
    nan[1, 1] = 0x7FC0
    assert orc.check_tolerance(nan, ref, K, 1.0, 1.0)["violations"] == 1
    # tile-restricted compare looks only at the listed tiles
    big_ref = np.zeros((128, 128), np.uint16)
    big_out = big_ref.copy()
    big_out[100, 100] = orc.from_f32(np.float32([5.0]))[0]
    assert orc.check_tolerance(big_out, big_ref, K, 1.0, 1.0, tiles=[[0, 0]])["violations"] == 0
    assert orc.check_tolerance(big_out, big_ref, K, 1.0, 1.0, tiles=[[1, 1]])["violations"] == 1
    assert orc.max_abs(orc.from_f32(np.float32([-3.0, 2.0]))) == 3.0
