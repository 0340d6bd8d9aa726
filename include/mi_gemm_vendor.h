/* Vendor comparator (hipBLASLt) behind the same argument bundle, in a shared library of its own
 * (libmi_gemm_vendor.so) so that libmi_gemm.so never depends on a BLAS library.
 *
 * Takes the place of the comparator rows of the reference harness: `matmul_cutlass(GPU_Tensors, StreamWorkspace&)`
 * / `cutlass_enabled()` (gemm/cutlass_gemm.h:5-6, gemm/cutlass_gemm.cu:97-127) and the cuBLAS call
 * (gemm/gemm_test.cu:249-261).  Not part of the product path: it exists so that the host driver and the benchmark
 * can time the vendor library on exactly the same operand buffers. */
#ifndef MI_GEMM_VENDOR_H
#define MI_GEMM_VENDOR_H

#include "mi_gemm.h"

#ifdef __cplusplus
extern "C" {
#endif

/* 1 if a hipBLASLt handle could be created on the current device (cutlass_enabled(), gemm/cutlass_gemm.h:6). */
int mi_vendor_enabled(void);

/* C = A * B through hipblasLtMatmul, fp16/bf16 inputs, fp32 accumulate and fp32 output, every GPU_Tensors layout.
 * d_workspace: at least MI_VENDOR_MIN_WORKSPACE bytes of device memory (the harness gives it 128 MiB, as it gives
 * CUTLASS its workspace, gemm/cutlass_gemm.cu:124-125); without one the call returns MI_ERR_WORKSPACE: running
 * hipBLASLt with no workspace was never validated here.  Asynchronous on hip_stream.
 * Returns MI_OK, MI_ERR_BAD_ARGUMENT, MI_ERR_WORKSPACE, MI_ERR_UNSUPPORTED (no algorithm for this problem) or
 * MI_ERR_HIP (any hipBLASLt failure; mi_vendor_last_status() holds its hipblasStatus_t). */
#define MI_VENDOR_MIN_WORKSPACE ((size_t)32 << 20)
int mi_vendor_matmul(const mi_gemm_tensors* t, void* d_workspace, size_t workspace_bytes, void* hip_stream);

int mi_vendor_last_status(void);

/* The rule mi_vendor_matmul applies to what hipblasLtMatmulAlgoGetHeuristic returns before it keeps an algorithm: the
 * result's own state must be success (MI_ERR_UNSUPPORTED otherwise) and the workspace the algorithm asks for must fit
 * the bytes the caller gave (MI_ERR_WORKSPACE otherwise), since every later call runs the kept algorithm with the
 * caller's pointer and size.  Pure host arithmetic; exported so that the rule can be checked without a device. */
int mi_vendor_accepts_algorithm(int heuristic_state, size_t algorithm_workspace_bytes, size_t given_workspace_bytes);

/* Which hipBLASLt this process is bound to: the file the dynamic linker resolved `hipblasLtMatmul` from, copied
 * into out (NUL-terminated, truncated to out_size).  A process that has loaded another copy of the library first
 * (PyTorch's wheel bundles its own, under the same soname) is bound to that copy, not to the one under /opt/rocm, and
 * the two differ in speed on deep-K problems: every figure quoted for the comparator should name this path.
 * Touches no device.  Returns MI_OK, MI_ERR_BAD_ARGUMENT or MI_ERR_UNSUPPORTED (the linker cannot tell). */
int mi_vendor_library(char* out, size_t out_size);

/* hipblasLtGetVersion() of that library (for example 100200 for 1.2.0), or -1 without a device. */
int mi_vendor_version(void);

#ifdef __cplusplus
}
#endif
#endif
