"""ctypes binding of include/mi_gemm.h.  Fails loudly if the HIP library has not been built: there is no fallback."""
from __future__ import annotations

import ctypes as C
import os
import re
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
_CSRC = os.path.join(_HERE, "csrc")
_LIB_PATH = os.path.join(_CSRC, "libmi_gemm.so")
_HEADER = os.path.join(os.path.dirname(_HERE), "include", "mi_gemm.h")

F16, BF16, F32 = 0, 1, 2
F32_BF16X1, F32_BF16X3 = 0, 1
K_OUTPUT_STATIONARY, K_SPLIT, K_AUTO, K_SPLIT_REDUCE, K_STREAM = 0, 1, 2, 3, 4
STATIC_SCRATCH_BYTES = 64 << 20  # MI_STATIC_SCRATCH_BYTES


def _tile_codes() -> dict:
    """TILE_AUTO, TILE_256x256, ...: the MI_TILE_* enumerators as the header lists them (the header is the one place
    that names the tiles of the ABI; their shapes come from the library, see tile_shape)."""
    text = re.sub(r"/\*.*?\*/", "", open(_HEADER).read(), flags=re.S)
    codes = {f"TILE_{m.group(1)}": int(m.group(2)) for m in re.finditer(r"\bMI_TILE_(AUTO|\d+x\d+)\s*=\s*(\d+)", text)}
    assert codes.get("TILE_AUTO") == 0 and sorted(codes.values()) == list(range(len(codes))), codes
    return codes


TILE_CODES = _tile_codes()
globals().update(TILE_CODES)
DATA_RANDOM, DATA_IDENTITY, DATA_TILED_NUMBERS, DATA_UNIFORM, DATA_NORMAL = 0, 1, 2, 3, 4


class MiGemmError(RuntimeError):
    def __init__(self, status: int, what: str):
        self.status = status
        super().__init__(what)


class GpuTensors(C.Structure):
    """Mirror of ``mi_gemm_tensors`` (itself the 16-bit counterpart of GPU_Tensors, gemm/gpu_tensor.h:9-21)."""

    _fields_ = [
        ("M", C.c_uint32),
        ("N", C.c_uint32),
        ("K", C.c_uint32),
        ("a", C.c_void_p),
        ("b", C.c_void_p),
        ("c", C.c_void_p),
        ("a_col_major", C.c_uint8),
        ("b_col_major", C.c_uint8),
        ("c_col_major", C.c_uint8),
        ("ab_dtype", C.c_uint8),
    ]

    @classmethod
    def make(cls, M, N, K, a_ptr, b_ptr, c_ptr, dtype, a_col_major=0, b_col_major=1, c_col_major=0):
        return cls(M, N, K, a_ptr, b_ptr, c_ptr, a_col_major, b_col_major, c_col_major, dtype)


def lib_path() -> str:
    return _LIB_PATH


def build(clean: bool = True) -> str:
    """Compile libmi_gemm.so and the host driver for gfx950 with hipcc (cross-compiles without a GPU)."""
    if clean:
        subprocess.run(["make", "-C", _CSRC, "clean"], check=True, capture_output=True)
    r = subprocess.run(["make", "-C", _CSRC, "-j8", "all"], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("building libmi_gemm.so failed:\n" + r.stdout[-4000:] + r.stderr[-4000:])
    return _LIB_PATH


def exported_symbols() -> list[str]:
    """Function names declared in include/mi_gemm.h."""
    text = open(_HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi_[a-z0-9_]+)\s*\(", text)))


class XgemmContext(C.Structure):
    """Mirror of ``mi_xgemm_context``: what the `ctxt` argument of the xgemm entry points brings."""

    _fields_ = [
        ("d_workspace", C.c_void_p),
        ("workspace_bytes", C.c_size_t),
        ("hip_stream", C.c_void_p),
        ("precision", C.c_int),
        ("tile", C.c_int),
    ]


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise MiGemmError(-1, f"{_LIB_PATH} is missing: run `python -c 'import __graft_entry__ as g; g.build()'` "
                              "(there is no CPU or PyTorch fallback)")
    L = C.CDLL(_LIB_PATH)
    vp, u32, i32, sz = C.c_void_p, C.c_uint32, C.c_int, C.c_size_t
    tp = C.POINTER(GpuTensors)
    ip = C.POINTER(C.c_int)

    def sig(name, res, args):
        f = getattr(L, name)
        f.restype = res
        f.argtypes = args

    sig("mi_status_string", C.c_char_p, [i32])
    sig("mi_last_hip_error", i32, [])
    sig("mi_last_hip_error_string", C.c_char_p, [])
    sig("mi_matmul_baseline", i32, [tp, vp])
    sig("mi_matmul_mfma_direct", i32, [tp, vp])
    sig("mi_matmul_mfma_supports", i32, [tp, i32, i32])
    sig("mi_matmul_mfma", i32, [tp, i32, i32, vp])
    sig("mi_matmul_mfma_plan", i32, [tp, i32, i32, ip, ip, ip])
    sig("mi_matmul_mfma_describe", i32, [tp, i32, i32, sz, C.c_char_p, sz])
    sig("mi_matmul_mfma_estimate_us", i32, [tp, i32, i32, sz, C.POINTER(C.c_double)])
    sig("mi_matmul_mfma_workspace_bytes", i32, [tp, C.POINTER(sz)])
    sig("mi_matmul_mfma_workspace_bytes_for", i32, [tp, i32, i32, C.POINTER(sz), C.POINTER(sz)])
    sig("mi_matmul_mfma_ws", i32, [tp, i32, i32, vp, sz, vp])
    sig("mi_matmul_mfma_static", i32, [tp, i32, i32, vp])
    sig("mi_matmul_mfma_timeline", i32, [tp, i32, i32, vp, u32, u32, C.POINTER(u32), vp])
    sig("mi_matmul_mfma_batched", i32, [tp, u32, C.c_uint64, C.c_uint64, C.c_uint64, i32, i32, vp])
    sig("mi_mfma_ceiling", i32, [vp, sz, i32, i32, u32, vp, vp, C.POINTER(u32), C.POINTER(C.c_double), vp])
    sig("mi_hbm_stream_ceiling", i32, [vp, vp, sz, i32, u32, vp, vp])
    sig("mi_hbm_stream_rows_ceiling", i32, [vp, u32, u32, u32, vp])
    sig("mi_matmul_f32_workspace_bytes", i32, [tp, i32, C.POINTER(sz)])
    sig("mi_matmul_f32_ws", i32, [tp, i32, i32, i32, vp, sz, vp])
    xp = C.POINTER(XgemmContext)
    sig("mi_xgemm_workspace_bytes", i32, [i32, i32, i32, i32, i32, C.POINTER(sz)])
    sig("mi_xgemm_Sm80", i32, [xp, i32, i32, i32, vp, vp, vp])
    sig("mi_xgemm_Sm90_wgmma", i32, [xp, i32, i32, i32, i32, i32, vp, vp, vp])
    sig("mi_widen_to_f32", i32, [vp, i32, vp, sz, vp])
    sig("mi_tile_name", C.c_char_p, [i32])
    sig("mi_tile_count", i32, [])
    sig("mi_tile_shape", i32, [i32, C.POINTER(u32), C.POINTER(u32), ip, ip])
    sig("mi_tile_planner_constants", i32, [i32, C.POINTER(C.c_double), C.POINTER(C.c_double)])
    sig("mi_tile_set_planner_constants", i32, [i32, C.c_double, C.c_double])
    sig("mi_matmul_mfma_prepare", i32, [tp, i32, i32, sz])
    sig("mi_matmul_mfma_sum_in_launch", i32, [i32, C.POINTER(C.c_uint64)])
    sig("mi_k_mode_name", C.c_char_p, [i32])
    sig("mi_init_test_data", i32, [vp, u32, u32, i32, i32, i32, C.c_double, u32, vp])
    sig("mi_compare_tensors", i32, [vp, vp, u32, u32, vp, vp])
    sig("mi_rt_device_count", i32, [ip])
    sig("mi_rt_set_device", i32, [i32])
    sig("mi_rt_device_info", i32, [i32, C.c_char_p, C.c_char_p, ip, ip, C.POINTER(sz), C.POINTER(sz)])
    sig("mi_rt_malloc", i32, [C.POINTER(vp), sz])
    sig("mi_rt_free", i32, [vp])
    sig("mi_rt_memset_async", i32, [vp, i32, sz, vp])
    sig("mi_rt_memcpy_h2d", i32, [vp, vp, sz])
    sig("mi_rt_memcpy_d2h", i32, [vp, vp, sz])
    sig("mi_rt_stream_create", i32, [C.POINTER(vp)])
    sig("mi_rt_stream_destroy", i32, [vp])
    sig("mi_rt_stream_synchronize", i32, [vp])
    sig("mi_rt_device_synchronize", i32, [])
    sig("mi_rt_event_create", i32, [C.POINTER(vp)])
    sig("mi_rt_event_record", i32, [vp, vp])
    sig("mi_rt_event_synchronize", i32, [vp])
    sig("mi_rt_event_elapsed_ms", i32, [C.POINTER(C.c_float), vp, vp])
    sig("mi_rt_event_destroy", i32, [vp])
    _lib = L
    return L


def status_string(status: int) -> str:
    return lib().mi_status_string(status).decode()


def check(status: int, what: str) -> None:
    if status != 0:
        msg = f"{what}: {status_string(status)}"
        if status == 4:
            msg += f" ({lib().mi_last_hip_error_string().decode()})"
        raise MiGemmError(status, msg)


def matmul_baseline(t: GpuTensors, stream: int = 0) -> None:
    check(lib().mi_matmul_baseline(C.byref(t), stream), "mi_matmul_baseline")


def matmul_mfma_direct(t: GpuTensors, stream: int = 0) -> None:
    check(lib().mi_matmul_mfma_direct(C.byref(t), stream), "mi_matmul_mfma_direct")


def matmul_mfma_supports(t: GpuTensors, k_mode: int = K_AUTO, tile: int = TILE_AUTO) -> bool:
    return bool(lib().mi_matmul_mfma_supports(C.byref(t), k_mode, tile))


def matmul_mfma(t: GpuTensors, k_mode: int = K_AUTO, tile: int = TILE_AUTO, stream: int = 0) -> None:
    check(lib().mi_matmul_mfma(C.byref(t), k_mode, tile, stream), "mi_matmul_mfma")


def matmul_mfma_workspace_bytes(t: GpuTensors) -> int:
    n = C.c_size_t()
    check(lib().mi_matmul_mfma_workspace_bytes(C.byref(t), C.byref(n)), "mi_matmul_mfma_workspace_bytes")
    return n.value


def matmul_mfma_workspace_bytes_for(t: GpuTensors, k_mode: int = K_AUTO, tile: int = TILE_AUTO) -> tuple:
    """(required, preferred) workspace bytes: below `required` matmul_mfma_ws fails; from `preferred` on, K partitions
    may keep private copies of C there and be summed without atomics (K_SPLIT_REDUCE)."""
    req, pref = C.c_size_t(0), C.c_size_t(0)
    check(lib().mi_matmul_mfma_workspace_bytes_for(C.byref(t), k_mode, tile, C.byref(req), C.byref(pref)),
          "mi_matmul_mfma_workspace_bytes_for")
    return req.value, pref.value


def matmul_mfma_ws(t: GpuTensors, workspace_ptr: int, workspace_bytes: int, k_mode: int = K_AUTO, tile: int = TILE_AUTO,
                   stream: int = 0) -> None:
    """Any layout / any K: operands the kernel cannot read in place are re-packed into the caller's workspace."""
    check(lib().mi_matmul_mfma_ws(C.byref(t), k_mode, tile, workspace_ptr, workspace_bytes, stream), "mi_matmul_mfma_ws")


def tile_count() -> int:
    """Tile codes run from 1 to tile_count() - 1 (0 is TILE_AUTO)."""
    return int(lib().mi_tile_count())


def tile_shape(tile: int) -> dict:
    bm, bn, per_cu, twin = C.c_uint32(), C.c_uint32(), C.c_int(), C.c_int()
    check(lib().mi_tile_shape(tile, C.byref(bm), C.byref(bn), C.byref(per_cu), C.byref(twin)), "mi_tile_shape")
    return {"code": tile, "name": lib().mi_tile_name(tile).decode(), "bm": bm.value, "bn": bn.value,
            "workgroups_per_cu": per_cu.value, "has_32_deep_twin": bool(twin.value)}


def tile_planner_constants(tile: int) -> tuple:
    """(microseconds per 64-deep K step of a round, microseconds per workgroup besides its K loop) the planner prices `tile` with."""
    k64, fixed = C.c_double(), C.c_double()
    check(lib().mi_tile_planner_constants(tile, C.byref(k64), C.byref(fixed)), "mi_tile_planner_constants")
    return k64.value, fixed.value


def tile_set_planner_constants(tile: int, us_per_k64: float, fixed_us: float) -> None:
    """Replaces the pair for the rest of the process (what `gemm --calibrate` measures on the machine at hand)."""
    check(lib().mi_tile_set_planner_constants(tile, us_per_k64, fixed_us), "mi_tile_set_planner_constants")


def tiles() -> list:
    """Every tile of the family, as the library reports it."""
    return [tile_shape(i) for i in range(1, tile_count())]


def matmul_mfma_prepare(t: GpuTensors, k_mode: int = K_AUTO, tile: int = TILE_AUTO, workspace_bytes: int = 0) -> None:
    """Sets the attributes of every kernel the call would launch (needed before a first call inside a graph capture)."""
    check(lib().mi_matmul_mfma_prepare(C.byref(t), k_mode, tile, workspace_bytes), "mi_matmul_mfma_prepare")


def matmul_mfma_static(t: GpuTensors, k_mode: int = K_AUTO, tile: int = TILE_AUTO, stream: int = 0) -> None:
    """matmul_mfma_ws on the library's own scratch array (STATIC_SCRATCH_BYTES): the call allocates nothing."""
    check(lib().mi_matmul_mfma_static(C.byref(t), k_mode, tile, stream), "mi_matmul_mfma_static")


def matmul_mfma_batched(t: GpuTensors, batches: int, a_batch_stride: int = 0, b_batch_stride: int = 0,
                        c_batch_stride: int = 0, k_mode: int = K_AUTO, tile: int = TILE_AUTO, stream: int = 0) -> None:
    """`batches` problems of one shape in one launch; strides in elements, 0 = densely packed."""
    check(lib().mi_matmul_mfma_batched(C.byref(t), batches, a_batch_stride, b_batch_stride, c_batch_stride, k_mode, tile,
                                       stream), "mi_matmul_mfma_batched")


def matmul_f32_workspace_bytes(t: GpuTensors, precision: int = F32_BF16X3) -> int:
    n = C.c_size_t()
    check(lib().mi_matmul_f32_workspace_bytes(C.byref(t), precision, C.byref(n)), "mi_matmul_f32_workspace_bytes")
    return n.value


def matmul_f32_ws(t: GpuTensors, workspace_ptr: int, workspace_bytes: int, precision: int = F32_BF16X3,
                  k_mode: int = K_AUTO, tile: int = TILE_AUTO, stream: int = 0) -> None:
    """fp32 A and B (ab_dtype = F32), converted on the device to one or three bf16 terms in the caller's workspace."""
    check(lib().mi_matmul_f32_ws(C.byref(t), precision, k_mode, tile, workspace_ptr, workspace_bytes, stream),
          "mi_matmul_f32_ws")


def xgemm_workspace_bytes(L: int, M: int, N: int, K: int, precision: int = F32_BF16X3) -> int:
    n = C.c_size_t()
    check(lib().mi_xgemm_workspace_bytes(L, M, N, K, precision, C.byref(n)), "mi_xgemm_workspace_bytes")
    return n.value


def xgemm_Sm80(ctxt: XgemmContext | None, M: int, N: int, K: int, a_ptr: int, b_ptr: int, c_ptr: int) -> None:
    """Argument list of xgemm_Sm80_fence / _mbarrier (xgemm_Sm80.py:18-21): A f32[M,K], B f32[K,N], C f32[M,N]."""
    check(lib().mi_xgemm_Sm80(C.byref(ctxt) if ctxt is not None else None, M, N, K, a_ptr, b_ptr, c_ptr), "mi_xgemm_Sm80")


def xgemm_Sm90_wgmma(ctxt: XgemmContext | None, L: int, M: int, N: int, K_splits: int, cluster_k: int, a_ptr: int,
                     b_ptr: int, c_ptr: int) -> None:
    """Argument list of xgemm_Sm90_wgmma_* (xgemm_Sm90.py:43-48): A f32[L,M,K], B f32[L,N,K], C f32[L,N,M] with
    K = K_splits * cluster_k."""
    check(lib().mi_xgemm_Sm90_wgmma(C.byref(ctxt) if ctxt is not None else None, L, M, N, K_splits, cluster_k, a_ptr, b_ptr,
                                    c_ptr), "mi_xgemm_Sm90_wgmma")


STREAM_READ, STREAM_DMA, STREAM_COPY = 0, 1, 2


def hbm_stream_ceiling(src_ptr: int, dst_ptr: int, nbytes: int, mode: int, workgroups_per_cu: int, sink_ptr: int,
                       stream: int = 0) -> None:
    """One launch of the streaming probe (see mi_hbm_stream_ceiling); time it with events."""
    check(lib().mi_hbm_stream_ceiling(src_ptr, dst_ptr, nbytes, mode, workgroups_per_cu, sink_ptr, stream),
          "mi_hbm_stream_ceiling")


def hbm_stream_rows_ceiling(src_ptr: int, rows: int, row_bytes: int, rows_per_workgroup: int, stream: int = 0) -> None:
    """One launch of the LDS DMA probe with a GEMM operand panel's access pattern (see mi_hbm_stream_rows_ceiling)."""
    check(lib().mi_hbm_stream_rows_ceiling(src_ptr, rows, row_bytes, rows_per_workgroup, stream), "mi_hbm_stream_rows_ceiling")


def matmul_mfma_sum_in_launch(enable: int = -1) -> tuple[bool, int]:
    """Where K partitions' copies and stream-K parts are summed: inside the GEMM launch (True, the default) or by a second
    kernel.  A negative `enable` only asks.  Returns (the setting as it was, calls so far that summed inside their launch)."""
    calls = C.c_uint64()
    was = lib().mi_matmul_mfma_sum_in_launch(int(enable), C.byref(calls))
    return bool(was), calls.value


def widen_to_f32(src_ptr: int, dtype: int, dst_ptr: int, count: int, stream: int = 0) -> None:
    check(lib().mi_widen_to_f32(src_ptr, dtype, dst_ptr, count, stream), "mi_widen_to_f32")


def matmul_mfma_timeline(t: GpuTensors, stamps_ptr: int, slots_per_workgroup: int, max_workgroups: int,
                         k_mode: int = K_AUTO, tile: int = TILE_AUTO, stream: int = 0) -> int:
    """The launch matmul_mfma would make, recording (100 MHz clock, core clock) stamp pairs per workgroup into the
    caller's zero-filled uint64 buffer; returns the number of workgroups launched."""
    n = C.c_uint32()
    check(lib().mi_matmul_mfma_timeline(C.byref(t), k_mode, tile, stamps_ptr, slots_per_workgroup, max_workgroups,
                                        C.byref(n), stream), "mi_matmul_mfma_timeline")
    return n.value


def matmul_mfma_plan(t: GpuTensors, k_mode: int = K_AUTO, tile: int = TILE_AUTO) -> dict:
    tl, km, ks = C.c_int(), C.c_int(), C.c_int()
    check(lib().mi_matmul_mfma_plan(C.byref(t), k_mode, tile, C.byref(tl), C.byref(km), C.byref(ks)), "mi_matmul_mfma_plan")
    return {"tile": lib().mi_tile_name(tl.value).decode(), "k_mode": lib().mi_k_mode_name(km.value).decode(),
            "k_splits": ks.value, "tile_code": tl.value, "k_mode_code": km.value}


def matmul_mfma_describe(t: GpuTensors, k_mode: int = K_AUTO, tile: int = TILE_AUTO, workspace_bytes: int = 0) -> str:
    """Every launch matmul_mfma (workspace_bytes = 0) or matmul_mfma_ws would make for this problem, as text."""
    buf = C.create_string_buffer(512)
    check(lib().mi_matmul_mfma_describe(C.byref(t), k_mode, tile, workspace_bytes, buf, len(buf)), "mi_matmul_mfma_describe")
    return buf.value.decode()


def matmul_mfma_estimate_us(t: GpuTensors, k_mode: int = K_AUTO, tile: int = TILE_AUTO, workspace_bytes: int = 0) -> float:
    """The planner's estimate (microseconds) for the launches matmul_mfma_describe names."""
    us = C.c_double()
    check(lib().mi_matmul_mfma_estimate_us(C.byref(t), k_mode, tile, workspace_bytes, C.byref(us)), "mi_matmul_mfma_estimate_us")
    return us.value


def init_test_data(d_ptr: int, rows: int, cols: int, code: int, transpose_rule: bool, dtype: int, param: float = 1.0,
                   seed: int = 0, stream: int = 0) -> None:
    check(lib().mi_init_test_data(d_ptr, rows, cols, code, int(transpose_rule), dtype, float(param), seed, stream),
          "mi_init_test_data")


def compare_tensors(d_a: int, d_b: int, rows: int, cols: int, d_result: int, stream: int = 0) -> None:
    check(lib().mi_compare_tensors(d_a, d_b, rows, cols, d_result, stream), "mi_compare_tensors")
