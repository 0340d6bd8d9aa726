// Host-side tensor bundle of the GEMM testbed, the 16-bit counterpart of gemm/gpu_tensor.h:9-21.
// Plain C++: the host driver never includes HIP headers; everything goes through the C ABI in mi_gemm.h.
#pragma once

#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include <new>

#include "mi_gemm.h"
#include "mi_gemm_vendor.h"

typedef void* gpu_stream_t;  // a hipStream_t, opaque on the host side

// Same fields and meaning as the reference's GPU_Tensors; A and B hold 16-bit elements of type `ab_dtype`.
struct GPU_Tensors
{
    uint32_t M;
    uint32_t N;
    uint32_t K;
    const void* a; /* pointer to GPU memory */
    const void* b; /* pointer to GPU memory */
    float* c;      /* pointer to GPU memory */

    bool a_col_major;
    bool b_col_major;
    bool c_col_major;

    int ab_dtype; /* MI_F16 | MI_BF16 */

    mi_gemm_tensors abi() const
    {
        mi_gemm_tensors t{};
        t.M = M;
        t.N = N;
        t.K = K;
        t.a = a;
        t.b = b;
        t.c = c;
        t.a_col_major = a_col_major;
        t.b_col_major = b_col_major;
        t.c_col_major = c_col_major;
        t.ab_dtype = static_cast<uint8_t>(ab_dtype);
        return t;
    }
};

// Reports a failed library call the way the reference reports CUDA errors (gemm/gemm_test.cu:228-232,474-477).
inline void gpu_check(int status, const char* what)
{
    if (status != MI_OK) {
        fprintf(stderr, "%s: %s", what, mi_status_string(status));
        if (status == MI_ERR_HIP) {
            fprintf(stderr, " (%i: %s)", mi_last_hip_error(), mi_last_hip_error_string());
        }
        fprintf(stderr, "\n");
        exit(1);
    }
}

// Entry points with the reference's names and shapes (gemm/gemm_baseline.h:5, gemm_sm80.h:5-6, gemm_sm90.h:14).
inline void matmul_baseline(GPU_Tensors t, gpu_stream_t stream)
{
    const mi_gemm_tensors abi = t.abi();
    gpu_check(mi_matmul_baseline(&abi, stream), "matmul_baseline");
}

inline void matmul_mfma_direct(GPU_Tensors t, gpu_stream_t stream)
{
    const mi_gemm_tensors abi = t.abi();
    gpu_check(mi_matmul_mfma_direct(&abi, stream), "matmul_mfma_direct");
}

inline bool matmul_mi355_supports(GPU_Tensors t, int k_mode, int tile)
{
    const mi_gemm_tensors abi = t.abi();
    return mi_matmul_mfma_supports(&abi, k_mode, tile) != 0;
}

inline void matmul_mi355(GPU_Tensors t, int k_mode, int tile, gpu_stream_t stream)
{
    const mi_gemm_tensors abi = t.abi();
    gpu_check(mi_matmul_mfma(&abi, k_mode, tile, stream), "matmul_mi355");
}

// Stream-ordered scratch allocator with the interface of the reference's StreamWorkspace (gemm/gpu_tensor.h:23-68).
// matmul_mi355_any_layout (below) uses it the way matmul_cutlass does in the reference (gemm/cutlass_gemm.cu:124-125).
class StreamWorkspace
{
  public:
    gpu_stream_t stream = {};

  private:
    void* d_workspace = nullptr;
    size_t current_workspace_bytes = 0;

  public:
    explicit StreamWorkspace(gpu_stream_t _stream) : stream(_stream)
    {
    }

    StreamWorkspace(StreamWorkspace&&) = delete;

    ~StreamWorkspace()
    {
        if (d_workspace) {
            mi_rt_stream_synchronize(stream);
            mi_rt_free(d_workspace);
        }
    }

    operator gpu_stream_t() const
    {
        return stream;
    }

    void* alloc_at_least(size_t bytes)
    {
        if (!d_workspace || bytes > current_workspace_bytes) {
            if (d_workspace) {
                mi_rt_stream_synchronize(stream);
                mi_rt_free(d_workspace);
                d_workspace = nullptr;
            }
            if (mi_rt_malloc(&d_workspace, bytes) != MI_OK) {
                fprintf(stderr, "Error allocating workspace: %s\n", mi_last_hip_error_string());
                throw std::bad_alloc{};
            }
            current_workspace_bytes = bytes;
        }
        return d_workspace;
    }
};

// Every GPU_Tensors layout and any K: operands the MFMA kernel cannot read in place are re-packed into the workspace.
// The workspace is sized to what the library prefers, so K partitions may be summed from private copies of C there
// instead of meeting in C through atomics.
inline void matmul_mi355_any_layout(GPU_Tensors t, StreamWorkspace& stream_ws, int k_mode = MI_K_AUTO, int tile = MI_TILE_AUTO)
{
    const mi_gemm_tensors abi = t.abi();
    size_t required = 0, preferred = 0;
    gpu_check(mi_matmul_mfma_workspace_bytes_for(&abi, k_mode, tile, &required, &preferred),
              "matmul_mi355_any_layout (workspace size)");
    void* d_ws = preferred ? stream_ws.alloc_at_least(preferred) : nullptr;
    gpu_check(mi_matmul_mfma_ws(&abi, k_mode, tile, d_ws, preferred, stream_ws.stream), "matmul_mi355_any_layout");
}

// The entry points that the reference's Exo procs compile to, by their names and argument lists (proc signatures
// xgemm_Sm80.py:18-21 and xgemm_Sm90.py:43-48, instances xgemm_Sm90_n{64,128,256}.py:3 and
// xgemm_Sm90_n256_tma_to_gmem.py:3-4; called at gemm/gemm_test.cu:288-294,326-362).  The reference passes ctxt = nullptr,
// which is accepted here too and means stream 0 and the library's own 64 MiB scratch array for the converted fp32
// operands (problems whose converted operands do not fit it end in MI_ERR_WORKSPACE).  Otherwise ctxt points to a
// mi_xgemm_context, which names the stream and the scratch memory (xgemm_context below fills one from a StreamWorkspace).  The n64 / n128 / n256 instances differ in
// their tile; here each stands for the tile of this chip's family nearest to it, unless ctxt->tile names one.  The
// fence and mbarrier builds of the Sm80 proc, and the plain and tma_to_gmem builds of the Sm90 one, differ in how the
// kernel synchronises and stores, not in what is computed: they are one call each here.
inline mi_xgemm_context xgemm_context(StreamWorkspace& stream_ws, int L, int M, int N, int K, int precision = MI_F32_BF16X3,
                                      int tile = MI_TILE_AUTO)
{
    size_t bytes = 0;
    gpu_check(mi_xgemm_workspace_bytes(L, M, N, K, precision, &bytes), "xgemm_context (workspace size)");
    return mi_xgemm_context{stream_ws.alloc_at_least(bytes), bytes, stream_ws.stream, precision, tile};
}

inline void xgemm_Sm80_fence(void* ctxt, int M, int N, int K, const float* A, const float* B, float* C)
{
    gpu_check(mi_xgemm_Sm80(static_cast<const mi_xgemm_context*>(ctxt), M, N, K, A, B, C), "xgemm_Sm80_fence");
}

inline void xgemm_Sm80_mbarrier(void* ctxt, int M, int N, int K, const float* A, const float* B, float* C)
{
    gpu_check(mi_xgemm_Sm80(static_cast<const mi_xgemm_context*>(ctxt), M, N, K, A, B, C), "xgemm_Sm80_mbarrier");
}

inline void xgemm_Sm90_wgmma_variant(const char* what, int namesake_tile, void* ctxt, int L, int M, int N, int K_splits,
                                     int cluster_k, const float* A, const float* B, float* C)
{
    if (!ctxt) {
        // the reference's own call form (gemm/gemm_test.cu:335): stream 0, the library's resident scratch, bf16x3, any tile
        gpu_check(mi_xgemm_Sm90_wgmma(nullptr, L, M, N, K_splits, cluster_k, A, B, C), what);
        return;
    }
    mi_xgemm_context with_tile = *static_cast<const mi_xgemm_context*>(ctxt);
    if (with_tile.tile == MI_TILE_AUTO) {
        with_tile.tile = namesake_tile;
    }
    gpu_check(mi_xgemm_Sm90_wgmma(&with_tile, L, M, N, K_splits, cluster_k, A, B, C), what);
}

#define MI_XGEMM_SM90_INSTANCE(name, namesake_tile)                                                                          \
    inline void name(void* ctxt, int L, int M, int N, int K_splits, int cluster_k, const float* A, const float* B, float* C) \
    {                                                                                                                        \
        xgemm_Sm90_wgmma_variant(#name, namesake_tile, ctxt, L, M, N, K_splits, cluster_k, A, B, C);                         \
    }
MI_XGEMM_SM90_INSTANCE(xgemm_Sm90_wgmma_n256, MI_TILE_256x256)
MI_XGEMM_SM90_INSTANCE(xgemm_Sm90_wgmma_n256_tma_to_gmem, MI_TILE_256x256)
MI_XGEMM_SM90_INSTANCE(xgemm_Sm90_wgmma_n256_split_k, MI_TILE_256x256)
MI_XGEMM_SM90_INSTANCE(xgemm_Sm90_wgmma_n128, MI_TILE_256x128)
MI_XGEMM_SM90_INSTANCE(xgemm_Sm90_wgmma_n64, MI_TILE_64x128)
#undef MI_XGEMM_SM90_INSTANCE

// Vendor comparator, shaped like matmul_cutlass / cutlass_enabled (gemm/cutlass_gemm.h:5-6).
inline bool hipblaslt_enabled()
{
    return mi_vendor_enabled() != 0;
}

inline void matmul_hipblaslt(GPU_Tensors t, StreamWorkspace& stream_ws)
{
    const mi_gemm_tensors abi = t.abi();
    const size_t bytes = size_t(128) << 20;
    void* d_ws = stream_ws.alloc_at_least(bytes);
    gpu_check(mi_vendor_matmul(&abi, d_ws, bytes, stream_ws.stream), "matmul_hipblaslt");
}
