"""spork_amd — MI355X (gfx950) dense GEMM behind the GEMM entry points of the akeley98/spork testbed.

The product is the HIP library ``csrc/libmi_gemm.so`` (C ABI in ``include/mi_gemm.h``) and the C++ host driver
``csrc/gemm``.  This package is the Python mirror of that ABI (ctypes, no torch types in any signature) used by the
tests and the benchmark; PyTorch only provides device memory and streams.
"""
from .capi import (  # noqa: F401
    BF16,
    F16,
    DATA_IDENTITY,
    DATA_NORMAL,
    DATA_RANDOM,
    DATA_TILED_NUMBERS,
    DATA_UNIFORM,
    K_AUTO,
    K_OUTPUT_STATIONARY,
    K_SPLIT,
    K_SPLIT_REDUCE,
    K_STREAM,
    TILE_CODES,
    GpuTensors,
    MiGemmError,
    build,
    compare_tensors,
    exported_symbols,
    init_test_data,
    lib,
    lib_path,
    matmul_baseline,
    matmul_mfma,
    matmul_mfma_direct,
    matmul_mfma_plan,
    matmul_mfma_describe,
    matmul_mfma_estimate_us,
    matmul_mfma_supports,
    matmul_mfma_workspace_bytes,
    matmul_mfma_workspace_bytes_for,
    matmul_mfma_ws,
    matmul_mfma_static,
    matmul_mfma_prepare,
    tile_count,
    tile_shape,
    tiles,
    STATIC_SCRATCH_BYTES,
    matmul_mfma_timeline,
    matmul_mfma_batched,
    matmul_f32_workspace_bytes,
    matmul_f32_ws,
    F32,
    F32_BF16X1,
    F32_BF16X3,
    status_string,
)

# TILE_AUTO, TILE_256x256, ...: one name per MI_TILE_* enumerator of include/mi_gemm.h
globals().update(TILE_CODES)
