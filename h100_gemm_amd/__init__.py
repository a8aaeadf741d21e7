"""h100_gemm_amd -- MI355X-native dense GEMM behind the host surface of Faraz9877/H100_GEMM.

    C[M,N] = A[M,K] . B[N,K]^T     bf16 / fp16 storage, fp32 accumulate, row-major A, B, C

The product is the C-ABI library ``lib/libmi_gemm.so`` (hand-written gfx950 kernels; see
``include/mi_gemm.h``).  This module is the Python mirror of the reference's host entry
points, used by the tests, the tuner and ``bench.py``:

    runKernel(M, N, K, A, B, C, DB)          matmul_h100_optimal.cu:32-59
    run_kernel(kernel_num, M, N, K, A, B, C) matmul_h100_optimal.cu:75-84
    GemmParams / gpu_gemm(params, ...)       common.h:206-221, matmul_h100.cu.jinja:927-985

Pointers are device pointers: pass an ``int`` address, a ``DeviceBuffer`` or anything with
``data_ptr()`` (a torch tensor on the GPU).  Launches are asynchronous on the null stream
unless a stream is given; the caller synchronises, as with the reference launchers.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Optional

from . import _lib
from ._lib import (MI_C_COL_MAJOR, MI_C_ROW_MAJOR, MI_CONFIG_AUTO, MI_DTYPE_BF16, MI_DTYPE_FP16, DeviceProps,
                   MiGemmError)

__all__ = ["runKernel", "run_kernel", "gpu_gemm", "gemm_epilogue", "workspace_bytes", "MI_C_ROW_MAJOR", "MI_C_COL_MAJOR", "reference_gpu_gemm", "GemmParams", "DeviceBuffer", "GPUTimer",
           "device_props", "num_configs", "config_name", "find_config", "select_config",
           "config_grid", "synchronize", "MiGemmError", "MI_CONFIG_AUTO", "MI_DTYPE_BF16",
           "MI_DTYPE_FP16"]


def _ptr(x: Any) -> Optional[int]:
    if x is None:
        return None
    if isinstance(x, int):
        return x
    if isinstance(x, DeviceBuffer):
        return x.ptr
    if hasattr(x, "data_ptr"):
        return int(x.data_ptr())
    raise TypeError(f"not a device pointer: {type(x).__name__}")


def _stream(s: Any) -> Optional[int]:
    if s is None or isinstance(s, int):
        return s
    if hasattr(s, "cuda_stream"):          # torch.cuda.Stream
        return int(s.cuda_stream)
    raise TypeError(f"not a stream: {type(s).__name__}")


@dataclass
class GemmParams:
    """The reference's GemmParams (common.h:206-221).  alpha/beta are carried for parity of
    the signature; like the reference kernels (matmul_h100.cu.jinja:696) ``gpu_gemm``
    computes alpha = 1, beta = 0 and rejects anything else; ``gemm_epilogue`` honours both."""
    M: int
    N: int
    K: int
    A: Any
    B: Any
    C: Any
    alpha: float = 1.0
    beta: float = 0.0


def runKernel(M: int, N: int, K: int, A, B, C, DB=None, stream=None) -> None:
    """bf16 GEMM with the library's choice of kernel (matmul_h100_optimal.cu:32-59)."""
    L = _lib.load()
    _lib.check(L.mi_gemm_bf16(M, N, K, _ptr(A), _ptr(B), _ptr(C), _ptr(DB), _stream(stream)))


def run_kernel(kernel_num: int, M: int, N: int, K: int, A, B, C, DB=None, stream=None) -> None:
    """Dispatcher of matmul_h100_optimal.cu:75-84: 1 = this library's kernel.  0 is the
    vendor BLAS in the reference; no vendor library is linked here, so 0 is an error, and
    (unlike the reference's silent switch fall-through) so is any other number."""
    if kernel_num == 1:
        return runKernel(M, N, K, A, B, C, DB, stream)
    raise ValueError(f"kernel_num {kernel_num}: only 1 (the gfx950 kernel) is built in")


def gpu_gemm(params: GemmParams, config: int | str = MI_CONFIG_AUTO, dtype: int = MI_DTYPE_BF16,
             DB=None, stream=None) -> None:
    """gpu_gemm<...>(GemmParams) of matmul_h100.cu.jinja:927-985; the template arguments
    become ``config`` (index or name of a compiled kernel configuration) and ``dtype``."""
    if params.alpha != 1.0 or params.beta != 0.0:
        raise ValueError("gpu_gemm computes alpha = 1, beta = 0 only (as the reference's kernels do); "
                         "gemm_epilogue applies alpha and beta")
    L = _lib.load()
    config = _config_index(L, config)
    _lib.check(L.mi_gemm_ex(config, dtype, params.M, params.N, params.K, _ptr(params.A),
                            _ptr(params.B), _ptr(params.C), _ptr(DB), _stream(stream)))


def _config_index(L, config) -> int:
    if isinstance(config, str):
        idx = L.mi_gemm_find_config(config.encode())
        if idx < 0:
            raise ValueError(f"unknown kernel config {config!r}")
        return idx
    return config


def gemm_epilogue(params: GemmParams, config: int | str = MI_CONFIG_AUTO, dtype: int = MI_DTYPE_BF16,
                  c_layout: int = MI_C_ROW_MAJOR, stream=None, workspace: "DeviceBuffer | None" = None) -> None:
    """The GEMM with the golden's epilogue, C = (CType)(acc * alpha + beta) with beta a plain
    scalar (reference.h:40), and C row-major or column-major (C[n*M + m], the layout the
    reference's bf16 kernel writes, matmul_utils.cuh:529,545).  With ``workspace`` (a
    DeviceBuffer of at least ``workspace_bytes(...)`` bytes) split-K partial sums go there and
    the call allocates nothing, like the reference's launcher (matmul_h100_optimal.cu:32-59)."""
    L = _lib.load()
    if workspace is not None:
        _lib.check(L.mi_gemm_epilogue_ws(_config_index(L, config), dtype, params.M, params.N, params.K,
                                         _ptr(params.A), _ptr(params.B), _ptr(params.C), params.alpha,
                                         params.beta, c_layout, workspace.ptr, workspace.nbytes,
                                         _stream(stream)))
        return
    _lib.check(L.mi_gemm_epilogue(_config_index(L, config), dtype, params.M, params.N, params.K,
                                  _ptr(params.A), _ptr(params.B), _ptr(params.C), params.alpha,
                                  params.beta, c_layout, _stream(stream)))


def workspace_bytes(M: int, N: int, K: int, config: int | str = MI_CONFIG_AUTO, dtype: int = MI_DTYPE_BF16,
                    c_layout: int = MI_C_ROW_MAJOR) -> int:
    """Bytes of split-K workspace the library's kernel choice wants for this shape (0: none)."""
    L = _lib.load()
    return int(L.mi_gemm_workspace_bytes(_config_index(L, config), dtype, M, N, K, c_layout))


def reference_gpu_gemm(params: GemmParams, dtype: int = MI_DTYPE_BF16, stream=None) -> None:
    """reference_gpu_gemm(GemmParams) of reference.h:78-90: the plain ascending-k GPU GEMM
    the harness uses as golden; honours alpha and beta (beta is a scalar added to every
    element, as in reference.h:40,72)."""
    L = _lib.load()
    _lib.check(L.mi_reference_gpu_gemm(dtype, params.M, params.N, params.K, _ptr(params.A),
                                       _ptr(params.B), _ptr(params.C), params.alpha, params.beta,
                                       _stream(stream)))


# ---- config table --------------------------------------------------------------------

def num_configs() -> int:
    return _lib.load().mi_gemm_num_configs()


def config_name(i: int) -> Optional[str]:
    s = _lib.load().mi_gemm_config_name(i)
    return s.decode() if s else None


def find_config(name: str) -> int:
    return _lib.load().mi_gemm_find_config(name.encode())


def select_config(M: int, N: int, K: int, dtype: int = MI_DTYPE_BF16) -> int:
    return _lib.load().mi_gemm_select_config(dtype, M, N, K)


def row_cut(M: int, N: int, K: int, dtype: int = MI_DTYPE_BF16) -> int:
    """Rows the automatic choice runs as a GEMM of their own ahead of the rest (0: one GEMM)."""
    return _lib.load().mi_gemm_row_cut(dtype, M, N, K)


def config_grid(config: int, M: int, N: int, K: int) -> int:
    return _lib.load().mi_gemm_config_grid(config, M, N, K)


# ---- thin HIP layer (alloc_gpu_tensor / copy_to_gpu / copy_to_cpu / GPUTimer) ----------

class DeviceBuffer:
    """Device allocation through the C ABI (alloc_gpu_tensor / free_gpu_tensor,
    common.h:309-329)."""

    def __init__(self, nbytes: int):
        import ctypes as C
        L = _lib.load()
        p = C.c_void_p()
        _lib.check(L.mi_malloc(C.byref(p), max(int(nbytes), 1)))
        self.ptr = int(p.value)
        self.nbytes = int(nbytes)

    @classmethod
    def from_numpy(cls, arr) -> "DeviceBuffer":
        import numpy as np
        arr = np.ascontiguousarray(arr)
        buf = cls(arr.nbytes)
        buf.copy_from(arr)
        return buf

    def copy_from(self, arr) -> None:       # copy_to_gpu, common.h:331-339
        import numpy as np
        arr = np.ascontiguousarray(arr)
        assert arr.nbytes <= self.nbytes
        _lib.check(_lib.load().mi_memcpy_h2d(self.ptr, arr.ctypes.data, arr.nbytes))

    def to_numpy(self, shape, dtype):       # copy_to_cpu, common.h:351-358
        import numpy as np
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes
        _lib.check(_lib.load().mi_memcpy_d2h(out.ctypes.data, self.ptr, out.nbytes))
        return out

    def fill_bytes(self, value: int) -> None:
        _lib.check(_lib.load().mi_memset(self.ptr, value, self.nbytes))

    def free(self) -> None:
        if self.ptr:
            _lib.check(_lib.load().mi_free(self.ptr))
            self.ptr = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class GPUTimer:
    """tick()/report_last_ms() on HIP events (GPUTimer, common.h:246-273)."""

    def __init__(self, stream=None):
        import ctypes as C
        L = _lib.load()
        self._ev = []
        for _ in range(2):
            e = C.c_void_p()
            _lib.check(L.mi_event_create(C.byref(e)))
            self._ev.append(e)
        self._cur = 0
        self._stream = _stream(stream)

    def tick(self) -> None:
        _lib.check(_lib.load().mi_event_record(self._ev[self._cur], self._stream))
        self._cur = 1 - self._cur

    def report_last_ms(self) -> float:
        import ctypes as C
        L = _lib.load()
        _lib.check(L.mi_event_sync(self._ev[1 - self._cur]))
        ms = C.c_float()
        _lib.check(L.mi_event_elapsed_ms(C.byref(ms), self._ev[self._cur], self._ev[1 - self._cur]))
        return float(ms.value)

    def sync_all(self) -> None:
        synchronize()

    def __del__(self):
        try:
            L = _lib.load()
            for e in self._ev:
                L.mi_event_destroy(e)
        except Exception:
            pass


def synchronize() -> None:
    _lib.check(_lib.load().mi_device_sync())


def device_props() -> dict:
    p = DeviceProps()
    _lib.check(_lib.load().mi_get_device_props(p))
    return {"name": p.name.decode(), "arch": p.arch.decode(), "compute_units": p.compute_units,
            "clock_khz": p.clock_khz, "mem_clock_khz": p.mem_clock_khz,
            "mem_bus_bits": p.mem_bus_bits, "lds_bytes_per_block": p.lds_bytes_per_block,
            "l2_bytes": p.l2_bytes, "wavefront": p.wavefront, "hbm_bytes": p.hbm_bytes}
