"""mi_gemm_bf16_noalloc: the entry point that allocates nothing (split-K partial sums in a
__device__ array inside the library), checked through the C ABI against mi_gemm_bf16.

Bar: bit-identical to the existing entry point (same kernels, same order of sums), and
bit-exact against the CPU oracle on the integer fill.  Two calls in a row share the array, the
second with a smaller input; a shape whose partial sums exceed the array is refused.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _inputs(orc, M, N, K, fill, seed):
    if fill == "int":
        return orc.fill_randint((M, K), seed, 1), orc.fill_randint((N, K), seed, 2)
    return orc.fill_normal((M, K), seed, 1, 1.0), orc.fill_normal((N, K), seed, 2, 0.02)


def test_noalloc_entry_point_matches_mi_gemm_bf16(mi, orc):
    L = mi._lib.load()
    limit = 32 << 20
    # decode split-K, then a smaller decode split-K, a few-tiles split-K of the tiled kernel,
    # a shape that uses no scratch at all, and the first one again
    shapes = [(128, 8192, 8192), (64, 4096, 8192), (384, 512, 4096), (512, 512, 512), (16, 2048, 1024),
              (128, 8192, 8192)]
    assert mi.workspace_bytes(*shapes[0]) > mi.workspace_bytes(*shapes[1]) > 0
    for fill in ("int", "normal"):
        held = []
        for i, (M, N, K) in enumerate(shapes):
            print(f"noalloc case {fill} {M}x{N}x{K}", flush=True)
            assert mi.workspace_bytes(M, N, K) <= limit
            A, B = _inputs(orc, M, N, K, fill, 69 + i)
            dA, dB = mi.DeviceBuffer.from_numpy(A), mi.DeviceBuffer.from_numpy(B)
            dC, dW = mi.DeviceBuffer(M * N * 2), mi.DeviceBuffer(M * N * 2)
            dC.fill_bytes(0xFF)
            dW.fill_bytes(0xFF)
            held.append((M, N, K, A, B, dA, dB, dC, dW))
        # all launches back to back on the null stream (ordered: they share the scratch array)
        for M, N, K, A, B, dA, dB, dC, dW in held:
            mi._lib.check(L.mi_gemm_bf16_noalloc(M, N, K, dA.ptr, dB.ptr, dC.ptr, None))
        mi.synchronize()
        for M, N, K, A, B, dA, dB, dC, dW in held:
            mi._lib.check(L.mi_gemm_bf16(M, N, K, dA.ptr, dB.ptr, dW.ptr, None, None))
        mi.synchronize()
        for M, N, K, A, B, dA, dB, dC, dW in held:
            got = dC.to_numpy((M, N), np.uint16)
            want = dW.to_numpy((M, N), np.uint16)
            assert (got == want).all(), f"{fill} {M}x{N}x{K}: {int((got != want).sum())} elements differ"
            if fill == "int":
                assert (got == orc.reference_cpu_gemm(A, B)).all(), f"{M}x{N}x{K} against the oracle"
            for b in (dA, dB, dC, dW):
                b.free()


def test_noalloc_entry_point_refuses_what_does_not_fit(mi, orc):
    L = mi._lib.load()
    M, N, K = 1024, 4096, 16384          # 4 pieces of 1024 x 4096 floats: twice the 32 MiB array
    need = mi.workspace_bytes(M, N, K)
    assert need > (32 << 20), need
    dA, dB, dC = mi.DeviceBuffer(M * K * 2), mi.DeviceBuffer(N * K * 2), mi.DeviceBuffer(M * N * 2)
    rc = L.mi_gemm_bf16_noalloc(M, N, K, dA.ptr, dB.ptr, dC.ptr, None)
    assert rc == mi._lib.MI_ERR_UNSUPPORTED
    assert b"static scratch array" in L.mi_last_error()
    assert L.mi_gemm_bf16_noalloc(0, N, K, dA.ptr, dB.ptr, dC.ptr, None) == mi._lib.MI_ERR_INVALID
    mi.synchronize()


def test_noalloc_entry_point_refuses_a_cut_shape_before_it_writes_anything(mi, orc):
    """A large ragged shape that the automatic choice runs as two GEMMs (the first 4096 rows,
    then the 200 left) and whose second part would need more partial sums than the array holds
    (four pieces of 200 x 12288 fp32: 37.5 MiB): the call is refused before the first part is
    launched, so C is untouched."""
    L = mi._lib.load()
    M, N, K = 4296, 12288, 16384
    assert mi.row_cut(M, N, K) == 4096 and mi.workspace_bytes(M, N, K) > 32 << 20
    dA, dB, dC = mi.DeviceBuffer(M * K * 2), mi.DeviceBuffer(N * K * 2), mi.DeviceBuffer(M * N * 2)
    dA.fill_bytes(0)
    dB.fill_bytes(0)
    dC.fill_bytes(0xFF)
    rc = L.mi_gemm_bf16_noalloc(M, N, K, dA.ptr, dB.ptr, dC.ptr, None)
    mi.synchronize()
    assert rc == mi._lib.MI_ERR_UNSUPPORTED, rc
    assert b"static scratch array" in L.mi_last_error()
    C = dC.to_numpy((M, N), np.uint16)
    assert (C == 0xFFFF).all(), f"{int((C != 0xFFFF).sum())} elements of C were written by a refused call"
    for b in (dA, dB, dC):
        b.free()
