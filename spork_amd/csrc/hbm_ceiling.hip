// What the chip sustains when a kernel does nothing but stream an operand in: the yardstick for the GEMM shapes that are
// bound by memory, as mfma_ceiling.hip is for the ones bound by the matrix cores.  A measurement tool, not a GEMM.  No
// counterpart in the reference, whose harness only times whole launches (gemm/gemm_test.cu:392-404).
//
// Three ways of moving the same bytes, each with every CU busy:
//   MI_STREAM_READ       16-byte non-temporal vector loads into registers (what a reduction would do);
//   MI_STREAM_DMA        `buffer_load_dwordx4 ... lds`, the GEMM kernel's own producer: 1 KB per wave instruction
//                        straight into a ring in LDS, nothing ever read back, as many in flight as the GEMM's ring keeps;
//   MI_STREAM_COPY       read and write back (half of the bytes each way), the usual "copy bandwidth" figure.
// And the DMA again with the access pattern of a GEMM operand panel (mi_hbm_stream_rows_ceiling): 128-byte pieces of many
// rows instead of contiguous kilobytes.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mi_gemm.h"
#include "mi_internal.hpp"

namespace mi_gemm {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) char lds_char;

// READ / COPY: a grid-stride walk over 16-byte chunks, eight loads of a lane in flight.
template <bool COPY>
__global__ __launch_bounds__(256) void stream_vector_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, size_t chunks,
                                                            uint32_t* sink)
{
    const size_t stride = (size_t)gridDim.x * 256;
    u32x4 seen = {0u, 0u, 0u, 0u};
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    for (; i + 7 * stride < chunks; i += 8 * stride) {
        u32x4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            v[u] = __builtin_nontemporal_load(src + i + u * stride);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            if constexpr (COPY) {
                __builtin_nontemporal_store(v[u], dst + i + u * stride);
            }
            else {
                seen ^= v[u];
            }
        }
    }
    for (; i < chunks; i += stride) {
        const u32x4 v = __builtin_nontemporal_load(src + i);
        if constexpr (COPY) {
            __builtin_nontemporal_store(v, dst + i);
        }
        else {
            seen ^= v;
        }
    }
    // (keeps the loads alive: one lane per workgroup leaves a word that depends on everything the lane has read)
    if (!COPY && threadIdx.x == 0) {
        *sink = seen.x ^ seen.y ^ seen.z ^ seen.w;
    }
}

// DMA: every wave keeps `IN_FLIGHT` 1 KB DMA instructions outstanding into its own part of a ring in LDS and never reads
// the ring.  A workgroup of four waves with IN_FLIGHT = 18 has 72 KB in flight, what the 64x128 GEMM tile's four-slot
// ring has (three slots of 24 KB ahead of the one being read).  Wave w of workgroup g walks the 1 KB pieces
// g * 4 + w, + grid * 4, ... of the buffer.
template <int IN_FLIGHT>
__global__ __launch_bounds__(256) void stream_dma_kernel(const void* src, uint32_t pieces)
{
    extern __shared__ __attribute__((aligned(1024))) char ring[];
    const uint32_t w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63u;
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(src), 0, pieces * 1024u, 0x00020000);
    lds_char* const mine = (lds_char*)ring + w * (IN_FLIGHT * 1024);
    const uint32_t step = gridDim.x * 4u;
    uint32_t piece = blockIdx.x * 4u + w;
    // fill the ring, then one wait and one new DMA per piece
#pragma unroll
    for (int s = 0; s < IN_FLIGHT; ++s) {
        if (piece < pieces) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, mine + s * 1024, 16, lane * 16u, piece * 1024u, 0, 2);
        }
        piece += step;
    }
    while (piece < pieces) {
#pragma unroll
        for (int s = 0; s < IN_FLIGHT; ++s) {
            if (piece < pieces) {
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"(IN_FLIGHT - 1) : "memory");
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, mine + s * 1024, 16, lane * 16u, piece * 1024u, 0, 2);
            }
            piece += step;
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// DMA_ROWS: the same ring, fed the way the GEMM's tall-skinny tile reads its A panel: workgroup g owns `rows_per_wg`
// consecutive rows of a row-major matrix with `row_bytes` per row and walks them 128 bytes (one 64-deep K tile of 16-bit
// elements) at a time, every DMA instruction fetching 128 bytes from each of eight rows (lane i: row i / 8 of the eight,
// chunk i % 8).  Same bytes as DMA, same number in flight, but 128-byte pieces a whole row apart instead of contiguous 1 KB.
// byte offset of piece p = (K tile p / groups, group of eight rows p % groups) within a workgroup's rows
__device__ __forceinline__ uint32_t rows_piece_offset(uint32_t p, uint32_t groups, uint32_t row_bytes)
{
    return (p % groups) * 8u * row_bytes + (p / groups) * 128u;
}

template <int IN_FLIGHT>
__global__ __launch_bounds__(256) void stream_dma_rows_kernel(const void* src, uint32_t rows, uint32_t row_bytes, uint32_t rows_per_wg)
{
    extern __shared__ __attribute__((aligned(1024))) char ring[];
    const uint32_t w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63u;
    lds_char* const mine = (lds_char*)ring + w * (IN_FLIGHT * 1024);
    const uint32_t first_row = blockIdx.x * rows_per_wg;
    if (first_row + rows_per_wg > rows) {
        return;
    }
    // descriptor over this workgroup's rows; the lane's part of the address never changes
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char*>((const char*)src + (size_t)first_row * row_bytes), 0, rows_per_wg * row_bytes, 0x00020000);
    const uint32_t voff = (lane / 8u) * row_bytes + (lane % 8u) * 16u;
    // one K tile = rows_per_wg / 8 instructions, dealt round-robin to the four waves; piece p = (K tile, group of 8 rows)
    const uint32_t groups = rows_per_wg / 8u, pieces = (row_bytes / 128u) * groups;
    uint32_t piece = w;
#pragma unroll
    for (int s = 0; s < IN_FLIGHT; ++s) {
        if (piece < pieces) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, mine + s * 1024, 16, voff, rows_piece_offset(piece, groups, row_bytes), 0, 0);
        }
        piece += 4u;
    }
    while (piece < pieces) {
#pragma unroll
        for (int s = 0; s < IN_FLIGHT; ++s) {
            if (piece < pieces) {
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"(IN_FLIGHT - 1) : "memory");
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, mine + s * 1024, 16, voff, rows_piece_offset(piece, groups, row_bytes), 0, 0);
            }
            piece += 4u;
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

}  // namespace mi_gemm

using namespace mi_gemm;

extern "C" int mi_hbm_stream_rows_ceiling(const void* d_src, uint32_t rows, uint32_t row_bytes, uint32_t rows_per_workgroup,
                                          void* hip_stream)
{
    if (!d_src || (uintptr_t)d_src % 16 || rows == 0 || row_bytes == 0 || row_bytes % 128 || rows_per_workgroup == 0 ||
        rows_per_workgroup % 8 || rows_per_workgroup > rows) {
        return MI_ERR_BAD_ARGUMENT;
    }
    if ((uint64_t)rows_per_workgroup * row_bytes >= ((uint64_t)1 << 31)) {
        return MI_ERR_UNSUPPORTED;  // a workgroup's rows must stay within the reach of one buffer descriptor
    }
    constexpr int lds = 4 * 18 * 1024;
    MI_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(&stream_dma_rows_kernel<18>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    hipLaunchKernelGGL(stream_dma_rows_kernel<18>, dim3(rows / rows_per_workgroup), dim3(256), lds, as_stream(hip_stream), d_src, rows,
                       row_bytes, rows_per_workgroup);
    MI_CHECK_LAUNCH();
    return MI_OK;
}

extern "C" int mi_hbm_stream_ceiling(const void* d_src, void* d_dst, size_t bytes, int mode, uint32_t workgroups_per_cu,
                                     uint32_t* d_sink, void* hip_stream)
{
    if (!d_src || bytes < 1024 || (uintptr_t)d_src % 16 || workgroups_per_cu == 0 || workgroups_per_cu > 8 ||
        mode < MI_STREAM_READ || mode > MI_STREAM_COPY) {
        return MI_ERR_BAD_ARGUMENT;
    }
    if ((mode == MI_STREAM_COPY && (!d_dst || (uintptr_t)d_dst % 16)) || (mode == MI_STREAM_READ && !d_sink)) {
        return MI_ERR_BAD_ARGUMENT;
    }
    const int cus = device_compute_units();
    if (cus <= 0) {
        return MI_ERR_NO_DEVICE;
    }
    hipStream_t stream = as_stream(hip_stream);
    const uint32_t grid = (uint32_t)cus * workgroups_per_cu;
    if (mode == MI_STREAM_DMA) {
        // (a buffer descriptor reaches 4 GB; a workgroup has the 64x128 GEMM tile's 72 KB in flight, and two of them fit a CU's LDS)
        if (bytes >= ((size_t)1 << 32) || workgroups_per_cu > 2) {
            return MI_ERR_UNSUPPORTED;
        }
        const uint32_t pieces = (uint32_t)(bytes / 1024);
        constexpr int lds = 4 * 18 * 1024;
        MI_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(&stream_dma_kernel<18>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        hipLaunchKernelGGL(stream_dma_kernel<18>, dim3(grid), dim3(256), lds, stream, d_src, pieces);
        MI_CHECK_LAUNCH();
        return MI_OK;
    }
    const size_t chunks = bytes / 16;
    if (mode == MI_STREAM_COPY) {
        hipLaunchKernelGGL(stream_vector_kernel<true>, dim3(grid), dim3(256), 0, stream, (const u32x4*)d_src, (u32x4*)d_dst,
                           chunks, d_sink);
    }
    else {
        hipLaunchKernelGGL(stream_vector_kernel<false>, dim3(grid), dim3(256), 0, stream, (const u32x4*)d_src, (u32x4*)nullptr,
                           chunks, d_sink);
    }
    MI_CHECK_LAUNCH();
    return MI_OK;
}
