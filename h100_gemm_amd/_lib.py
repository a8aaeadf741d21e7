"""ctypes binding of libmi_gemm.so (the C ABI declared in include/mi_gemm.h).

There is no fallback: if the shared library has not been built, loading raises.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

PKG = Path(__file__).resolve().parent
LIB_PATH = PKG / "lib" / "libmi_gemm.so"

MI_OK = 0
MI_ERR_INVALID = -1
MI_ERR_HIP = -2
MI_ERR_UNSUPPORTED = -3
MI_DTYPE_BF16 = 0
MI_DTYPE_FP16 = 1
MI_CONFIG_AUTO = -1
MI_C_ROW_MAJOR = 0
MI_C_COL_MAJOR = 1


class MiGemmError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"mi_gemm error {code}: {message}")
        self.code = code


class DeviceProps(C.Structure):
    _fields_ = [("name", C.c_char * 256), ("arch", C.c_char * 64), ("compute_units", C.c_int),
                ("clock_khz", C.c_int), ("mem_clock_khz", C.c_int), ("mem_bus_bits", C.c_int),
                ("lds_bytes_per_block", C.c_int), ("l2_bytes", C.c_int), ("wavefront", C.c_int),
                ("hbm_bytes", C.c_size_t)]


# name -> (restype, argtypes): every symbol include/mi_gemm.h declares
SYMBOLS = {
    "mi_gemm_bf16": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p,
                               C.c_void_p, C.c_void_p]),
    "mi_gemm_ex": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p,
                             C.c_void_p, C.c_void_p, C.c_void_p]),
    "mi_gemm_epilogue": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p,
                                   C.c_void_p, C.c_float, C.c_float, C.c_int, C.c_void_p]),
    "mi_gemm_workspace_bytes": (C.c_size_t, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]),
    "mi_gemm_epilogue_ws": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p,
                                      C.c_void_p, C.c_float, C.c_float, C.c_int, C.c_void_p, C.c_size_t,
                                      C.c_void_p]),
    "mi_gemm_reserve_workspace": (C.c_int, [C.c_void_p, C.c_size_t]),
    "mi_gemm_release_workspace": (C.c_int, [C.c_void_p]),
    "mi_gemm_library_workspace_bytes": (C.c_size_t, []),
    "mi_gemm_bf16_noalloc": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "mi_reference_gpu_gemm": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p,
                                        C.c_void_p, C.c_float, C.c_float, C.c_void_p]),
    "mi_gemm_num_configs": (C.c_int, []),
    "mi_gemm_config_name": (C.c_char_p, [C.c_int]),
    "mi_gemm_find_config": (C.c_int, [C.c_char_p]),
    "mi_gemm_select_config": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int]),
    "mi_gemm_tuned_entries": (C.c_int, []),
    "mi_gemm_row_cut": (C.c_int, [C.c_int] * 4),
    "mi_gemm_config_supports": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]),
    "mi_gemm_config_grid": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int]),
    "mi_gemm_config_lds_bytes": (C.c_int, [C.c_int]),
    "mi_gemm_trace_words": (C.c_size_t, [C.c_int, C.c_int, C.c_int]),
    "mi_malloc": (C.c_int, [C.POINTER(C.c_void_p), C.c_size_t]),
    "mi_free": (C.c_int, [C.c_void_p]),
    "mi_memcpy_h2d": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "mi_memcpy_d2h": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "mi_memcpy_d2d": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "mi_memset": (C.c_int, [C.c_void_p, C.c_int, C.c_size_t]),
    "mi_device_sync": (C.c_int, []),
    "mi_stream_sync": (C.c_int, [C.c_void_p]),
    "mi_event_create": (C.c_int, [C.POINTER(C.c_void_p)]),
    "mi_event_destroy": (C.c_int, [C.c_void_p]),
    "mi_event_record": (C.c_int, [C.c_void_p, C.c_void_p]),
    "mi_event_sync": (C.c_int, [C.c_void_p]),
    "mi_event_elapsed_ms": (C.c_int, [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]),
    "mi_get_device_props": (C.c_int, [C.POINTER(DeviceProps)]),
    "mi_last_error": (C.c_char_p, []),
}

_lib = None


def load() -> C.CDLL:
    """Load the in-tree library; raises if it is not built (no CPU path exists)."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m h100_gemm_amd.build` "
            "(hipcc cross-compiles gfx950 without a GPU). There is no fallback path.")
    L = C.CDLL(str(LIB_PATH))
    for name, (res, args) in SYMBOLS.items():
        fn = getattr(L, name)      # AttributeError if the library lacks a declared symbol
        fn.restype = res
        fn.argtypes = args
    _lib = L
    return L


def check(rc: int) -> None:
    if rc != MI_OK:
        raise MiGemmError(rc, load().mi_last_error().decode(errors="replace"))
