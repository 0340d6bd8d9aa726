"""ctypes binding of include/mi_gemm_vendor.h: the hipBLASLt comparator behind the same argument bundle.  Lives in its
own shared library so that libmi_gemm.so never depends on a BLAS library; used by the benchmark and tests to time the
vendor GEMM on exactly the same operand buffers (role of the cuBLAS / CUTLASS rows, gemm/gemm_test.cu:249-261)."""
from __future__ import annotations

import ctypes as C
import os
import re

from .capi import GpuTensors, MiGemmError, status_string

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "csrc", "libmi_gemm_vendor.so")
_HEADER = os.path.join(os.path.dirname(_HERE), "include", "mi_gemm_vendor.h")

_lib = None


def lib_path() -> str:
    return _LIB_PATH


def exported_symbols() -> list[str]:
    text = re.sub(r"/\*.*?\*/", "", open(_HEADER).read(), flags=re.S)
    return sorted(set(re.findall(r"\b(mi_vendor_[a-z0-9_]+)\s*\(", text)))


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise MiGemmError(-1, f"{_LIB_PATH} is missing: run `python -c 'import __graft_entry__ as g; g.build()'`")
        L = C.CDLL(_LIB_PATH)
        L.mi_vendor_enabled.restype = C.c_int
        L.mi_vendor_enabled.argtypes = []
        L.mi_vendor_last_status.restype = C.c_int
        L.mi_vendor_last_status.argtypes = []
        L.mi_vendor_matmul.restype = C.c_int
        L.mi_vendor_matmul.argtypes = [C.POINTER(GpuTensors), C.c_void_p, C.c_size_t, C.c_void_p]
        L.mi_vendor_accepts_algorithm.restype = C.c_int
        L.mi_vendor_accepts_algorithm.argtypes = [C.c_int, C.c_size_t, C.c_size_t]
        L.mi_vendor_library.restype = C.c_int
        L.mi_vendor_library.argtypes = [C.c_char_p, C.c_size_t]
        L.mi_vendor_version.restype = C.c_int
        L.mi_vendor_version.argtypes = []
        _lib = L
    return _lib


def enabled() -> bool:
    return bool(lib().mi_vendor_enabled())


def library() -> str:
    """File the process resolved hipBLASLt from (after `import torch` that is the copy inside the torch wheel)."""
    buf = C.create_string_buffer(4096)
    st = lib().mi_vendor_library(buf, len(buf))
    if st != 0:
        raise MiGemmError(st, f"mi_vendor_library: {status_string(st)}")
    return buf.value.decode()


def version() -> int:
    return int(lib().mi_vendor_version())


def matmul(t: GpuTensors, workspace_ptr: int = 0, workspace_bytes: int = 0, stream: int = 0) -> None:
    st = lib().mi_vendor_matmul(C.byref(t), workspace_ptr, workspace_bytes, stream)
    if st != 0:
        raise MiGemmError(st, f"mi_vendor_matmul: {status_string(st)} (hipblasStatus {lib().mi_vendor_last_status()})")
