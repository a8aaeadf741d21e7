"""ctypes front end of the CPU oracle (``oracle/ref_gemm.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` -- as the checker, never as the thing measured or
shipped.  The product package must not import this module.

All matrices are numpy ``uint16`` arrays holding bf16 (dtype code 0) or fp16 (code 1) bit
patterns, row-major: A is (M, K), B is (N, K) "K-major", C is (M, N) -- the layouts of
``reference_cpu_gemm`` (reference.h:5-46 in the reference tree).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from pathlib import Path

import numpy as np

BF16, FP16 = 0, 1
_HERE = Path(__file__).resolve().parent
_LIB_PATH = _HERE / "liboracle.so"
_lib = None

_u16p = np.ctypeslib.ndpointer(dtype=np.uint16, flags="C_CONTIGUOUS")
_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")


def build(force: bool = False) -> Path:
    """Compile liboracle.so with the Makefile beside this file."""
    if force or not _LIB_PATH.exists():
        subprocess.run(["make", "-C", str(_HERE), "-B" if force else "-s", "liboracle.so"],
                       check=True, stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    build()
    L = C.CDLL(str(_LIB_PATH))
    vp = C.c_void_p
    L.orc_bf16_to_f32.restype = C.c_float
    L.orc_bf16_to_f32.argtypes = [C.c_uint16]
    L.orc_f32_to_bf16.restype = C.c_uint16
    L.orc_f32_to_bf16.argtypes = [C.c_float]
    L.orc_fp16_to_f32.restype = C.c_float
    L.orc_fp16_to_f32.argtypes = [C.c_uint16]
    L.orc_f32_to_fp16.restype = C.c_uint16
    L.orc_f32_to_fp16.argtypes = [C.c_float]
    L.orc_to_f32_array.argtypes = [_u16p, _f32p, C.c_size_t, C.c_int]
    L.orc_from_f32_array.argtypes = [_f32p, _u16p, C.c_size_t, C.c_int]
    L.orc_rng_u64.restype = C.c_uint64
    L.orc_rng_u64.argtypes = [C.c_uint64, C.c_uint64, C.c_uint64]
    L.orc_fill_uniform.argtypes = [_u16p, C.c_size_t, C.c_uint64, C.c_uint64, C.c_int]
    L.orc_fill_normal.argtypes = [_u16p, C.c_size_t, C.c_uint64, C.c_uint64, C.c_float, C.c_int]
    L.orc_fill_randint.argtypes = [_u16p, C.c_size_t, C.c_uint64, C.c_uint64, C.c_int]
    L.orc_fill_arange.argtypes = [_u16p, C.c_size_t, C.c_int, C.c_int]
    L.orc_fill_constant.argtypes = [_u16p, C.c_size_t, C.c_float, C.c_int]
    L.orc_reference_cpu_gemm.argtypes = [C.c_int, C.c_int, C.c_int, _u16p, _u16p, vp, vp,
                                         C.c_float, C.c_float, C.c_int, C.c_int]
    L.orc_reference_cpu_gemm_tiles.argtypes = [C.c_int, C.c_int, C.c_int, _u16p, _u16p, vp, vp,
                                               C.c_float, C.c_float, C.c_int, C.c_int, vp, C.c_int]
    L.orc_naive_gemm.argtypes = [C.c_int, C.c_int, C.c_int, _u16p, _u16p, _u16p,
                                 C.c_float, C.c_float, C.c_int]
    L.orc_allclose_count.restype = C.c_longlong
    L.orc_allclose_count.argtypes = [_u16p, _u16p, C.c_size_t, C.c_float, C.c_int,
                                     C.POINTER(C.c_double), C.POINTER(C.c_longlong)]
    L.orc_absdiff_first_fail.restype = C.c_longlong
    L.orc_absdiff_first_fail.argtypes = [_u16p, _u16p, C.c_size_t, C.c_float, C.c_int]
    L.orc_max_abs.restype = C.c_double
    L.orc_max_abs.argtypes = [_u16p, C.c_size_t, C.c_int]
    L.orc_check_tolerance.restype = C.c_longlong
    L.orc_check_tolerance.argtypes = [C.c_int, C.c_int, C.c_int, _u16p, _u16p, C.c_double,
                                      C.c_double, C.c_double, C.c_double, C.c_int, vp, C.c_int,
                                      C.POINTER(C.c_double)]
    L.orc_num_threads.restype = C.c_int
    _lib = L
    return L


# ------------------------------------------------------------------ conversions ------

def to_f32(x: np.ndarray, dtype: int = BF16) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.uint16)
    out = np.empty(x.shape, dtype=np.float32)
    lib().orc_to_f32_array(x.reshape(-1), out.reshape(-1), x.size, dtype)
    return out


def from_f32(x: np.ndarray, dtype: int = BF16) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().orc_from_f32_array(x.reshape(-1), out.reshape(-1), x.size, dtype)
    return out


# ------------------------------------------------------------------------ fills ------

def fill_uniform(shape, seed: int, stream: int, dtype: int = BF16) -> np.ndarray:
    """U[-1, 1) on a 2^-23 grid, rounded to the storage type."""
    out = np.empty(shape, dtype=np.uint16)
    lib().orc_fill_uniform(out.reshape(-1), out.size, seed, stream, dtype)
    return out


def fill_normal(shape, seed: int, stream: int, sigma: float = 1.0, dtype: int = BF16) -> np.ndarray:
    out = np.empty(shape, dtype=np.uint16)
    lib().orc_fill_normal(out.reshape(-1), out.size, seed, stream, sigma, dtype)
    return out


def fill_randint(shape, seed: int, stream: int, dtype: int = BF16) -> np.ndarray:
    """The reference's random_fill values (integers in [-5, 4]), seeded."""
    out = np.empty(shape, dtype=np.uint16)
    lib().orc_fill_randint(out.reshape(-1), out.size, seed, stream, dtype)
    return out


def fill_arange(shape, bound: int = 1024, dtype: int = BF16) -> np.ndarray:
    out = np.empty(shape, dtype=np.uint16)
    lib().orc_fill_arange(out.reshape(-1), out.size, bound, dtype)
    return out


def fill_constant(shape, value: float, dtype: int = BF16) -> np.ndarray:
    out = np.empty(shape, dtype=np.uint16)
    lib().orc_fill_constant(out.reshape(-1), out.size, value, dtype)
    return out


# ------------------------------------------------------------------------- GEMM ------

def _check_abc(A, B):
    assert A.dtype == np.uint16 and B.dtype == np.uint16
    assert A.ndim == 2 and B.ndim == 2 and A.shape[1] == B.shape[1], (A.shape, B.shape)
    return A.shape[0], B.shape[0], A.shape[1]


def reference_cpu_gemm(A, B, alpha: float = 1.0, beta: float = 0.0, dtype: int = BF16,
                       fast: bool = True, want_acc: bool = False, tiles=None, out=None):
    """C = storage_round(acc * alpha + beta), acc = ascending-k fp32 sum of A[i,k]*B[j,k].

    ``tiles`` -- optional int array of shape (T, 2) of 64x64 tile coordinates; only those
    tiles are computed (the rest of the returned C keeps the content of ``out``, or zeros).
    ``fast=False`` runs the reference's loop nest order verbatim.
    """
    M, N, K = _check_abc(A, B)
    A = np.ascontiguousarray(A)
    B = np.ascontiguousarray(B)
    Cm = out if out is not None else np.zeros((M, N), dtype=np.uint16)
    acc = np.zeros((M, N), dtype=np.float32) if want_acc else None
    accp = acc.ctypes.data if acc is not None else None
    if tiles is None:
        lib().orc_reference_cpu_gemm(M, N, K, A, B, Cm.ctypes.data, accp, alpha, beta, dtype,
                                     int(fast))
    else:
        t = np.ascontiguousarray(tiles, dtype=np.int32).reshape(-1, 2)
        lib().orc_reference_cpu_gemm_tiles(M, N, K, A, B, Cm.ctypes.data, accp, alpha, beta,
                                           dtype, int(fast), t.ctypes.data, t.shape[0])
    return (Cm, acc) if want_acc else Cm


def naive_gemm(A, B, alpha: float = 1.0, beta: float = 0.0, dtype: int = BF16) -> np.ndarray:
    M, N, K = _check_abc(A, B)
    Cm = np.empty((M, N), dtype=np.uint16)
    lib().orc_naive_gemm(M, N, K, np.ascontiguousarray(A), np.ascontiguousarray(B), Cm,
                         alpha, beta, dtype)
    return Cm


# --------------------------------------------------------------------- checkers ------

def allclose_count(res, golden, rtol: float = 1e-5, dtype: int = BF16):
    """(errors, avg_diff_of_errors, n_inf) with the reference's pure-relative rule."""
    res = np.ascontiguousarray(res).reshape(-1)
    golden = np.ascontiguousarray(golden).reshape(-1)
    avg = C.c_double(0.0)
    ninf = C.c_longlong(0)
    e = lib().orc_allclose_count(res, golden, res.size, rtol, dtype, C.byref(avg), C.byref(ninf))
    return int(e), float(avg.value), int(ninf.value)


def absdiff_first_fail(ref, out, thresh: float = 0.1, dtype: int = BF16) -> int:
    ref = np.ascontiguousarray(ref).reshape(-1)
    out = np.ascontiguousarray(out).reshape(-1)
    return int(lib().orc_absdiff_first_fail(ref, out, ref.size, thresh, dtype))


def max_abs(x, dtype: int = BF16) -> float:
    x = np.ascontiguousarray(x).reshape(-1)
    return float(lib().orc_max_abs(x, x.size, dtype))


REL_TOL = 2.0 ** -7
ABS_COEF = 1e-3


def check_tolerance(out, ref, K: int, max_a: float, max_b: float, dtype: int = BF16,
                    tiles=None, rel: float = REL_TOL, abs_coef: float = ABS_COEF) -> dict:
    """|out-ref| <= rel*|ref| + abs_coef*sqrt(K)*max|a|*max|b| per element."""
    M, N = ref.shape
    rep = (C.c_double * 5)()
    tp, nt = None, 0
    if tiles is not None:
        t = np.ascontiguousarray(tiles, dtype=np.int32).reshape(-1, 2)
        tp, nt = t.ctypes.data, t.shape[0]
    bad = lib().orc_check_tolerance(M, N, K, np.ascontiguousarray(out), np.ascontiguousarray(ref),
                                    max_a, max_b, rel, abs_coef, dtype, tp, nt, rep)
    return {"violations": int(bad), "max_err": rep[1], "max_err_over_bound": rep[2],
            "compared": int(rep[3]), "abs_term": rep[4]}


def sample_tiles(M: int, N: int, count: int, seed: int = 69) -> np.ndarray:
    """A fixed, seeded sample of 64x64 tile coordinates that always holds the four corner
    tiles and tiles on each edge; all tiles when the matrix has no more than ``count``."""
    tm, tn = (M + 63) // 64, (N + 63) // 64
    if tm * tn <= count:
        return np.array([(i, j) for i in range(tm) for j in range(tn)], dtype=np.int32)
    chosen = {(0, 0), (0, tn - 1), (tm - 1, 0), (tm - 1, tn - 1),
              (0, tn // 2), (tm - 1, tn // 2), (tm // 2, 0), (tm // 2, tn - 1)}
    i = 0
    while len(chosen) < count:
        r = lib().orc_rng_u64(seed, 0x7113, i)
        chosen.add((int(r % tm), int((r >> 32) % tn)))
        i += 1
    return np.array(sorted(chosen), dtype=np.int32)


def num_threads() -> int:
    return int(lib().orc_num_threads())
