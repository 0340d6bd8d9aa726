// Internal helpers shared by the translation units of libmi_gemm.so (not part of the C ABI).
#pragma once

#include <hip/hip_runtime.h>

#include "mi_gemm.h"

namespace mi_gemm {

// hipError_t of the last failing runtime call on this thread (read back through mi_last_hip_error()).
void record_hip_error(hipError_t err);

// Evaluate a HIP runtime call; on failure remember the error and return MI_ERR_HIP from the enclosing function.
#define MI_HIP_TRY(expr)                             \
    do {                                             \
        const hipError_t mi_hip_err_ = (expr);       \
        if (mi_hip_err_ != hipSuccess) {             \
            ::mi_gemm::record_hip_error(mi_hip_err_); \
            return MI_ERR_HIP;                       \
        }                                            \
    } while (0)

// Launch errors (bad configuration, missing code object) surface through hipGetLastError.
#define MI_CHECK_LAUNCH() MI_HIP_TRY(hipGetLastError())

inline hipStream_t as_stream(void* s)
{
    return reinterpret_cast<hipStream_t>(s);
}

// Number of compute units of the current device (cached per device).
int device_compute_units();

// Address, on the current device, of the scratch array behind mi_matmul_mfma_static (looked up on the first call per
// device; `out` may be null).  Allocates nothing.
int resolve_static_scratch(void** out);

// Looks up, on the current device, the address of the arrival counters behind the launches that sum their K partitions
// themselves (the first such call on a device does it otherwise).  Allocates nothing.
int resolve_tile_counters();

// Basic validation shared by every GEMM entry point: non-null, non-zero, known dtype, flags are 0/1.
int validate_tensors(const mi_gemm_tensors* t);

// 16-bit storage -> fp32, exact
__device__ __forceinline__ float widen16(uint16_t bits, int dtype)
{
    if (dtype == MI_BF16) {
        return __builtin_bit_cast(float, (uint32_t)bits << 16);
    }
    return (float)__builtin_bit_cast(_Float16, bits);
}

}  // namespace mi_gemm
