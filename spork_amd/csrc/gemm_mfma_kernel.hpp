// LDS-tiled MFMA GEMM kernel for gfx950 (CDNA4), C[M,N] (fp32) = A[M,K] * B[N,K]^T with A and B K-contiguous.
//
// This is the kernel that takes the place of the reference's hand-written tensor-core kernels
// (gemm/gemm_sm80.cu:417-465, gemm/gemm_sm90.cu:806-990) and of the Exo tile family (xgemm_Sm90.py:11-204).  It is
// derived for the CDNA4 execution model, not translated:
//
//  * producer: `buffer_load_dwordx4 ... lds` (direct global->LDS DMA, 16 B per lane, 1 KiB per wave instruction)
//    fills a ring of K tiles; there is no register staging.  The DMA writes LDS in lane order, so the
//    bank-conflict-avoiding XOR swizzle is applied on the *source* side: lane i of an instruction fetches the
//    global 16 B chunk whose swizzled position is i.  With BK = 64 one LDS row is a whole 128 B cache line, so the
//    8 lanes of a row form one full-line L2 request (64 B requests halve the L2 request throughput).
//    (Role of cp.async / TMA + 128 B hardware swizzle, gemm_sm80.cu:285-308, gemm_sm90.cu:730-753.)
//  * ring hand-off: one workgroup `s_barrier` per K tile, placed *before the MFMAs of the tile's last k-step*.  At
//    that point a wave has every fragment of tile kt in registers (lgkmcnt(0)) and has seen its own DMA of tile
//    kt+1 land (vmcnt), so after the barrier (a) the LDS regions of tile kt are free and are refilled, and (b) tile
//    kt+1 is visible to everyone.  The last k-step's MFMAs then run while the first fragments of tile kt+1 are read,
//    so no wave waits on LDS latency after a barrier.  (Role of the RAW/WAR mbarrier pairs, gemm_sm80.cu:161-218.)
//    The 256x256 tile cannot fit a third 64 KB slot in 160 KB and runs a ring of five half-slot units instead
//    (see "ring organisation" in the kernel).
//  * consumer: every wave both loads and computes (no dedicated producer wave: CDNA4 cannot re-balance registers
//    between waves).  Fragments are `ds_read_b128` (8 K-contiguous 16-bit values per lane) feeding
//    v_mfma_f32_16x16x32_{f16,bf16} (or 32x32x16 in the short-K twins); the reads for k-step s+1 are issued in the
//    shadow of the MFMAs of k-step s and waited for one fragment at a time (lgkmcnt counts down in order).
//  * the LDS reads are inline asm on purpose: the compiler cannot prove that a DS read does not alias an in-flight
//    LDS DMA and would put `s_waitcnt vmcnt(0)` in front of every one of them, serialising the ring.
//  * epilogue: accumulators go straight to global memory with buffer stores; with 16x16x32 tiles the rows of B are
//    permuted on their way into LDS so that a lane owns four consecutive columns of C and stores 16 B at a time.
//    Split-K partials use fp32 atomic adds onto a zero-filled C.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mi_gemm.h"

namespace mi_gemm {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

typedef __attribute__((address_space(3))) char lds_char;
typedef __attribute__((address_space(3))) uint32_t lds_u32;
typedef const __attribute__((address_space(1))) char global_char;

struct GemmArgs {
    const void* a;  // M x K, K contiguous
    const void* b;  // N x K, K contiguous
    float* c;       // M x N, N contiguous
    uint32_t M, N, K;
    uint32_t lda, ldb, ldc;      // leading dimensions in elements
    uint32_t tiles_m, tiles_n;   // output tile grid
    uint32_t k_splits;           // number of K partitions (1 = output stationary)
    uint32_t k_tiles_per_split;  // BK-tiles per partition (last one may be shorter)
    uint32_t group_m;            // tile-rows per raster group
    // K rotation (0 = none; whole-tile builds only): the workgroups on XCD x walk their K range starting k_rotate * x
    // K tiles in (modulo the range's length) and wrap around to its start, so that the XCDs are not all at the same
    // K offset of their rows at the same time.
    uint32_t k_rotate;
    uint32_t batches;            // independent problems of the same shape (>= 1)
    uint64_t a_batch_bytes, b_batch_bytes, c_batch_bytes;  // distance between consecutive problems
    // 0: every K partition adds into the one C (the ATOMIC build).  Otherwise partition s stores its partial tile at
    // c + s * c_split_bytes with plain stores and a later pass sums the partitions.
    uint64_t c_split_bytes;
    // Stream-K launches (the STREAM build) only, see StreamKShape: the tail tiles are raster tiles sk.first_tile ...
    // sk.first_tile + sk.tiles - 1 of the tile grid above; `c` is then the parts buffer.
    struct StreamKShape {
        uint32_t first_tile;  // raster index of the first tile this launch works on
        uint32_t tiles;       // r: how many tiles (fewer than workgroups)
        uint32_t splits;      // S = workgroups / tiles: main partitions per tile, all tiles' partition s walked in step
        uint32_t main_k;      // Km: K tiles of every tile that the main partitions cover ([s*Km/S, (s+1)*Km/S) each)
    } sk;
    // K partitions summed inside the launch (null: not).  Otherwise the launch stores parts of output tiles (the K
    // partitions' copies of C, c_split_bytes != 0, or the parts of a stream-K launch) and the workgroup that stores the
    // last part of a tile adds that tile's parts, in their fixed order, and writes the tile of `c_final` (row pitch
    // `ldc_final` floats, problem l at c_final + l * c_final_batch_bytes).  tile_counters[l * tiles + tile] counts the
    // parts of a tile that have been stored; it is zero before the launch and the workgroup that finds it complete sets
    // it back to zero.  (Role of the reduce-adding epilogue of gemm/gemm_sm90.cu:944-963.)
    uint32_t* tile_counters;
    float* c_final;
    uint32_t ldc_final;
    uint64_t c_final_batch_bytes;
    // Diagnostic timeline (null in normal use): workgroup g writes stamp i to timeline[(g * timeline_slots + i) * 2]
    // (the 100 MHz constant clock) and [.. + 1] (the core clock counter): kernel entry, then per work item the point where
    // K tile 0 has landed, the end of its K loop and the end of its epilogue issue, then the point where all of the
    // workgroup's stores have landed.  The last slot is not a stamp: it names the CU the workgroup ran on.
    unsigned long long* timeline;
    uint32_t timeline_slots;
};

constexpr uint32_t NUM_XCD = 8;

// compile-time loop: f(std::integral_constant<int, I>) for I in [0, N)
template <int I>
struct IntC {
    static constexpr int value = I;
};
template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f)
{
    if constexpr (I < N) {
        f(IntC<I>{});
        static_for<I + 1, N>(f);
    }
}

// The two dense 16-bit MFMA shapes of gfx950, both 8 K-contiguous values per lane and operand:
//   32x32x16: lane l feeds row (column) l%32, k group l/32 (2 groups of 8); 16 result registers per lane,
//             register r = C[8*(r/4) + 4*(l/32) + r%4][l%32]; 32 cycles.
//   16x16x32: lane l feeds row (column) l%16, k group l/16 (4 groups of 8); 4 result registers per lane,
//             register r = C[4*(l/16) + r][l%16]; 16 cycles.
// Same arithmetic rate; the 16x16x32 form runs a 32-deep dot product per accumulator update and draws less power per
// flop, which on this power-limited part is a higher sustained clock.
template <int MT>
struct AccOf;
template <>
struct AccOf<32> {
    using type = f32x16;
};
template <>
struct AccOf<16> {
    using type = f32x4;
};

template <int DTYPE>
__device__ __forceinline__ f32x16 mfma_tile(u32x4 a, u32x4 b, f32x16 c)
{
    if constexpr (DTYPE == MI_F16) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    else {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
}
template <int DTYPE>
__device__ __forceinline__ f32x4 mfma_tile(u32x4 a, u32x4 b, f32x4 c)
{
    if constexpr (DTYPE == MI_F16) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    else {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
}

template <int IMM>
__device__ __forceinline__ void lds_read_b128(u32x4& dst, uint32_t addr)
{
    static_assert(IMM >= 0 && IMM < 65536, "ds_read offset field is 16 bits");
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(IMM));
}

// Empty volatile asm that reads and "writes" x: a definition point the compiler cannot move or see through.
__device__ __forceinline__ void touch(u32x4& x)
{
    asm volatile("" : "+v"(x));
}

// A scalar move / a scalar-plus-vector add that stays where it is written (the compiler would otherwise gather such
// bookkeeping at the top of the loop, where it delays the first MFMAs of a K tile).
__device__ __forceinline__ uint32_t pinned_move(uint32_t x)
{
    uint32_t r;
    asm volatile("s_mov_b32 %0, %1" : "=s"(r) : "s"(x));
    return r;
}
__device__ __forceinline__ uint32_t pinned_add(uint32_t s, uint32_t v)
{
    uint32_t r;
    asm volatile("v_add_u32 %0, %1, %2" : "=v"(r) : "s"(s), "v"(v));
    return r;
}

// The DMA in two hand-placed halves, for loops that give every instruction an MFMA gap of its own: the LDS base goes
// into M0 one gap ahead (base + a constant in one scalar add; the write needs a wait state before a DMA may use it,
// which the MFMA in between provides), the
// DMA itself names a descriptor held in four scalar registers.  The compiler does not know that M0 is live between the
// two: the code between them contains no other writer of M0 (checked in every tile's listing by the code generation test,
// which finds the two halves by the comments they carry: every `dma-issue` must find, as the last write of M0 before it
// in the listing, a `dma-base`, with an MFMA or a wait state in between).
// (M0 is on the clobber list so that the compiler re-initialises it before any LDS DMA of its own that follows, e.g.
// the ring fill of a stream-K workgroup's next part; clang remarks that M0 is a reserved register, which is the point.)
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
template <int IMM>
__device__ __forceinline__ void dma_set_lds_base(uint32_t lds_addr)
{
    if constexpr (IMM == 0) {
        asm volatile("s_mov_b32 m0, %0 ; dma-base" ::"s"(lds_addr) : "memory", "m0");
    }
    else {
        asm volatile("s_add_i32 m0, %0, %1 ; dma-base" ::"s"(lds_addr), "n"(IMM) : "memory", "m0", "scc");
    }
}
#pragma clang diagnostic pop
template <bool NONTEMPORAL>
__device__ __forceinline__ void dma_issue_16B(u32x4 rsrc, uint32_t voffset, uint32_t soffset)
{
    if constexpr (NONTEMPORAL) {
        asm volatile("buffer_load_dwordx4 %0, %1, %2 offen nt lds ; dma-issue" ::"v"(voffset), "s"(rsrc), "s"(soffset) : "memory");
    }
    else {
        asm volatile("buffer_load_dwordx4 %0, %1, %2 offen lds ; dma-issue" ::"v"(voffset), "s"(rsrc), "s"(soffset) : "memory");
    }
}
// Descriptor words for [base, base + bytes), as make_rsrc builds them
__device__ __forceinline__ u32x4 make_rsrc_words(const void* base, uint32_t bytes)
{
    const uint64_t b = (uint64_t)(uintptr_t)base & 0xffffffffffffull;
    return u32x4{(uint32_t)b, (uint32_t)(b >> 32), bytes, 0x00020000u};
}

// No instruction may be scheduled across this point.  (Device-only builtins are kept out of lambda bodies: the host
// pass silently drops the kernel stub of a __global__ template whose lambdas name them.)
__device__ __forceinline__ void sched_fence()
{
    __builtin_amdgcn_sched_barrier(0);
}

// One wave-level DMA (`buffer_load_dwordx4 ... lds`): lane i copies 16 B from buffer byte (voffset_i + soffset) to
// LDS byte (lds_dst + 16*i).  lds_dst is wave-uniform (it travels in M0), soffset is wave-uniform (an SGPR), so a
// K-tile advance is scalar work on the descriptor's base and no vector ALU work; the per-lane offset is a single
// 32-bit VGPR.  Bytes
// past the descriptor's num_records read as zero.  Completion is tracked by vmcnt.  NONTEMPORAL sets the
// instruction's `nt` bit: the line is marked for early eviction in the L2 and the memory-side cache.
template <bool NONTEMPORAL = false>
__device__ __forceinline__ void dma_buffer_to_lds_16B(__amdgpu_buffer_rsrc_t rsrc, uint32_t voffset, uint32_t soffset,
                                                      lds_char* lds_dst)
{
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, lds_dst, 16, voffset, soffset, 0, NONTEMPORAL ? 2 : 0);
}

// After a store of more than 8 bytes per lane the hardware needs two more instruction slots before the registers that
// held its data may be written again.  The compiler knows the rule for ordinary vector instructions but not for the
// moves between accumulation registers that it builds the next store's data with (seen in the ISA: the first register
// of a store's quad overwritten by the very next instruction; on the GPU: one dword of a 16-byte store wrong, rarely,
// when the store sat in the queue behind another workgroup's).  So every 16-byte store is followed by the two slots,
// fenced so that nothing is scheduled into them.
__device__ __forceinline__ void after_wide_store()
{
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_nop 1");
    __builtin_amdgcn_sched_barrier(0);
}

// Buffer descriptor over [base, base + bytes): raw (stride 0) addressing, 32-bit data format (dword 3 = 0x00020000).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}

template <int N>
__device__ __forceinline__ void wait_vmcnt_then_barrier()
{
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(N) : "memory");
}

// LDS reads return in order: wait until at most N are outstanding.
template <int N>
__device__ __forceinline__ void wait_lgkmcnt()
{
    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(N));
}

// Cache policy of a buffer access (the instruction's aux operand on gfx950): bit 1 `nt`, streaming; bit 4 `sc1`, coherent
// at device scope - the access is performed where every XCD sees it (a store is written through its XCD's private L2, a
// load does not take that L2's word for it).  Parts of an output tile that another workgroup, possibly on another XCD,
// is going to add up inside the same launch are stored and loaded with `sc1`: that is what makes them visible to it
// without a write-back or an invalidation of a whole L2, which cost about 15 us per launch and hit every workgroup that is
// still running.
constexpr int AUX_NT = 2, AUX_NT_SC1 = 2 | 16, AUX_SC1 = 16;

// (Device-only builtins are kept out of lambda bodies, see sched_fence.)
template <int AUX>
__device__ __forceinline__ void buffer_store_16B(u32x4 bits, __amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t soff)
{
    __builtin_amdgcn_raw_buffer_store_b128(bits, rsrc, voff, soff, AUX);
}
template <int AUX>
__device__ __forceinline__ void buffer_store_4B(uint32_t bits, __amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t soff)
{
    __builtin_amdgcn_raw_buffer_store_b32(bits, rsrc, voff, soff, AUX);
}
__device__ __forceinline__ f32x4 load_part(__amdgpu_buffer_rsrc_t rsrc, uint32_t byte_offset, f32x4)
{
    return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte_offset, 0, AUX_SC1));
}
__device__ __forceinline__ float load_part(__amdgpu_buffer_rsrc_t rsrc, uint32_t byte_offset, float)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, byte_offset, 0, AUX_SC1));
}

// A wave's whole tile of 16-wide MFMA tiles with permuted B rows (see TileCfg::perm_row) to global memory: a lane's
// accumulators of four neighbouring MFMA tiles are four consecutive columns, 16 bytes per store, 256 contiguous bytes per
// row and instruction.  `voff`: the lane's fixed byte offset; the rest of an address is a scalar.
template <int AUX, typename Cfg, typename AccT>
__device__ __forceinline__ void store_wave_tile_16B(const AccT (&acc)[Cfg::MI][Cfg::NI], __amdgpu_buffer_rsrc_t rsrc_c, uint32_t voff,
                                                    uint32_t ldc)
{
#pragma unroll
    for (int mi = 0; mi < Cfg::MI; ++mi) {
#pragma unroll
        for (int nq = 0; nq < Cfg::NI / 4; ++nq) {
#pragma unroll
            for (int r = 0; r < Cfg::NACC; ++r) {
                const uint32_t soff = ((mi * Cfg::MT + r) * ldc + nq * 64) * 4u;  // (register r of a 16-wide tile is its row r)
                const float v0 = acc[mi][4 * nq + 0][r], v1 = acc[mi][4 * nq + 1][r];
                const float v2 = acc[mi][4 * nq + 2][r], v3 = acc[mi][4 * nq + 3][r];
                const u32x4 bits = {__builtin_bit_cast(uint32_t, v0), __builtin_bit_cast(uint32_t, v1),
                                    __builtin_bit_cast(uint32_t, v2), __builtin_bit_cast(uint32_t, v3)};
                buffer_store_16B<AUX>(bits, rsrc_c, voff, soff);
                after_wide_store();
            }
        }
    }
}

// Stream-K: the leftover workgroups [j_lo, j_hi) whose runs overlap tail tile t.  Leftover workgroup j owns the
// leftover (tile, K tile) pairs [j * units / lefts, (j + 1) * units / lefts), units = tiles * kr; tile t's pairs are
// [t * kr, (t + 1) * kr).  (A run may be empty when there are more leftover workgroups than pairs: see leftover_run_empty.)
__device__ __forceinline__ void leftover_runs_of_tile(uint32_t tiles, uint32_t kr, uint32_t lefts, uint32_t t, uint32_t& j_lo,
                                                      uint32_t& j_hi)
{
    j_lo = j_hi = 0;
    if (lefts == 0) {
        return;
    }
    const uint64_t units = (uint64_t)tiles * kr, first = (uint64_t)t * kr, last = first + kr;
    j_lo = (uint32_t)(first * lefts / units);
    j_lo = j_lo ? j_lo - 1 : 0;
    while (j_lo < lefts && (j_lo + 1) * units / lefts <= first) {
        ++j_lo;
    }
    j_hi = j_lo;
    while (j_hi < lefts && j_hi * units / lefts < last) {
        ++j_hi;
    }
}
__device__ __forceinline__ bool leftover_run_empty(uint32_t tiles, uint32_t kr, uint32_t lefts, uint32_t j)
{
    const uint64_t units = (uint64_t)tiles * kr;
    return (uint64_t)j * units / lefts == (uint64_t)(j + 1) * units / lefts;
}

// A workgroup has stored one part of an output tile (with device-coherent stores, AUX_NT_SC1): count it, and tell every
// thread of the workgroup whether it was the tile's last part (the counter is then set back to zero, for the next launch:
// nobody else touches it any more in this one).  Nobody waits for anybody.  `lds_flag`: a dword of LDS that no one is
// using.  Every wave waits until its own stores have been performed (vmcnt counts a store until the level that holds it
// coherently has it), the barrier gathers the waves, and only then is the arrival counted, by a device-scope atomic;
// whoever reads the count as complete reads the parts with device-coherent loads (load_part), which go past the L2.
__device__ __forceinline__ bool part_stored_is_it_the_last(uint32_t* counter, uint32_t expected, volatile lds_u32* lds_flag)
{
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t before = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const bool last = before + 1 == expected;
        if (last) {
            __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        *lds_flag = last ? 1u : 0u;
    }
    __syncthreads();
    return *lds_flag != 0u;
}

// C tile = part(0) + part(1) + ... + part(n_parts - 1), added in that order (so the result does not depend on which
// workgroup does the adding, or when).  part(i) is where element (0, 0) of the tile lies in part i; every part has row
// pitch `ld_part` (the tile's last element less than 2 GiB from its first).  T = f32x4: every pointer and pitch is a
// multiple of 16 bytes and columns come four at a time; T = float otherwise.  Rows from `m_rem` and columns from `n_rem` on
// do not exist.  The parts of U places of a thread, G parts at a time, are requested before the first is awaited: a lone
// workgroup has only its own loads in flight to cover the memory latency with (these loads go past the L2).  U * (G + 1)
// values of T are live at once.
template <int BM, int BN, int NTHREADS, typename T, uint32_t U, uint32_t G, typename PartFn>
__device__ __forceinline__ void sum_tile_parts(PartFn part, uint32_t n_parts, uint32_t ld_part, float* c_tile, uint32_t ldc,
                                               int32_t m_rem, int32_t n_rem)
{
    constexpr uint32_t W = sizeof(T) / 4, Q = BN / W, TOTAL = BM * Q;
    constexpr uint32_t REACH = 0x80000000u;  // bytes a part's descriptor covers (offsets beyond it would read as zero)
    for (uint32_t first = threadIdx.x; first < TOTAL; first += NTHREADS * U) {
        uint32_t at_part[U], at_c[U];
        bool exists[U];
#pragma unroll
        for (uint32_t u = 0; u < U; ++u) {
            const uint32_t idx = first + u * NTHREADS, row = idx / Q, col = (idx % Q) * W;
            exists[u] = idx < TOTAL && (int32_t)row < m_rem && (int32_t)col < n_rem;
            // (a place that does not exist reads element (0, 0), which does, and stores nothing)
            at_part[u] = exists[u] ? (row * ld_part + col) * 4u : 0u;
            at_c[u] = row * ldc + col;
        }
        T acc[U];
        {
            const __amdgpu_buffer_rsrc_t r0 = make_rsrc(part(0), REACH);
#pragma unroll
            for (uint32_t u = 0; u < U; ++u) {
                acc[u] = load_part(r0, at_part[u], T{});
            }
        }
        for (uint32_t i = 1; i < n_parts; i += G) {
            // up to G parts at once; a part beyond the last is not loaded and not added (the adds stay in part order)
            T v[G][U];
#pragma unroll
            for (uint32_t k = 0; k < G; ++k) {
                if (i + k < n_parts) {
                    const __amdgpu_buffer_rsrc_t rk = make_rsrc(part(i + k), REACH);
#pragma unroll
                    for (uint32_t u = 0; u < U; ++u) {
                        v[k][u] = load_part(rk, at_part[u], T{});
                    }
                }
            }
#pragma unroll
            for (uint32_t k = 0; k < G; ++k) {
                if (i + k < n_parts) {
#pragma unroll
                    for (uint32_t u = 0; u < U; ++u) {
                        acc[u] += v[k][u];
                    }
                }
            }
        }
#pragma unroll
        for (uint32_t u = 0; u < U; ++u) {
            if (exists[u]) {
                __builtin_nontemporal_store(acc[u], reinterpret_cast<T*>(c_tile + at_c[u]));
            }
        }
    }
}

// Tile configuration.  BK is the K depth of one ring slot; WM x WN waves tile the BM x BN block.
// SWZ: 0 none; 1 chunk ^= (row / rows_per_256B) % chunks_per_row (conflict-free for 64 banks x 4 B);
//      2 chunk ^= row % chunks_per_row (the 32-bank form).
// SPREAD: number of consecutive k-steps (starting with the one right after the barrier) over which a wave spreads
//      the DMA instructions of one slot refill.  The texture-address unit takes ~16 cycles per 1 KiB DMA
//      instruction; issuing a whole refill in one k-step from all waves at once backs up the vector-memory queue
//      and stalls the MFMA stream behind it.
// MT: edge of the MFMA tile, 32 (v_mfma_f32_32x32x16) or 16 (v_mfma_f32_16x16x32).
// SPLIT: the ring is made of 5 half-slot units instead of NSTAGE (= 2) whole slots; see "ring organisation" at the
//      kernel.
template <int BM_, int BN_, int BK_, int WM_, int WN_, int NSTAGE_, int SWZ_, int SPREAD_ = 1, int MT_ = 32, bool SPLIT_ = false>
struct TileCfg {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_, NSTAGE = NSTAGE_, SWZ = SWZ_;
    static constexpr int SPREAD = SPREAD_, MT = MT_;
    static constexpr bool SPLIT = SPLIT_;
    static constexpr int KSTEP = 512 / MT;            // K depth of one MFMA
    static constexpr int NACC = MT * MT / 64;         // accumulator registers per lane and MFMA tile
    static constexpr int CPS = KSTEP / 8;             // 16 B chunks (lane groups) per k-step
    static constexpr int NWAVES = WM * WN;
    static constexpr int NTHREADS = NWAVES * 64;
    static constexpr int TM = BM / WM, TN = BN / WN;  // wave tile
    static constexpr int MI = TM / MT, NI = TN / MT;  // MFMA tiles per wave tile
    static constexpr int KS = BK / KSTEP;             // MFMA k-steps per ring slot
    static constexpr int ROWB = BK * 2;               // bytes per LDS row
    static constexpr int CPR = BK / 8;                // 16 B chunks per row
    static constexpr int RW = 256 / ROWB;             // rows per 256 B (64 banks x 4 B)
    static constexpr int A_BYTES = BM * ROWB, B_BYTES = BN * ROWB;
    static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr int UNITS = 5;                                            // split ring: units of UNIT bytes
    static constexpr int UNIT = A_BYTES > B_BYTES ? A_BYTES : B_BYTES;         // each holds an A or a B tile
    static constexpr int LDS_BYTES = SPLIT ? UNIT * UNITS : STAGE_BYTES * NSTAGE;
    // prefetch distances in K tiles: tile kt+DIST_A of A and kt+DIST_B of B are requested while tile kt is computed
    static constexpr int DIST_A = SPLIT ? 3 : NSTAGE, DIST_B = SPLIT ? 2 : NSTAGE;
    static constexpr int PF = DIST_A;                                          // the larger of the two
    static constexpr int DMA_PER_STAGE = STAGE_BYTES / 1024;  // wave-level DMA instructions per slot
    static constexpr int LPW = DMA_PER_STAGE / NWAVES;        // ... per wave
    static constexpr int RPI = 1024 / ROWB;                   // LDS rows filled by one DMA instruction
    static constexpr int A_DMA = A_BYTES / 1024 / NWAVES;     // per wave: DMA instructions [0, A_DMA) fetch A
    static constexpr int NR = MI + NI;                        // fragment reads per k-step
    static constexpr int NMFMA = MI * NI;
    static_assert(MT == 32 || NI % 4 == 0, "16-wide MFMA tiles are stored four at a time");
    // a fragment read of the next k-step follows every RS-th MFMA of the current one
    static constexpr int RS = NMFMA / (2 * NR) > 1 ? NMFMA / (2 * NR) : 1;
    static constexpr int LOOP_READS = (NMFMA + RS - 1) / RS < NR ? (NMFMA + RS - 1) / RS : NR;
    static_assert(BK == 32 || BK == 64, "BK");
    static_assert(MT == 16 || MT == 32, "MFMA tile");
    static_assert(TM % MT == 0 && TN % MT == 0, "wave tile must be a multiple of the MFMA tile");
    static_assert(BK % KSTEP == 0, "ring slot must hold whole k-steps");
    static_assert(A_BYTES % 1024 == 0 && B_BYTES % 1024 == 0, "DMA instruction must not straddle A/B");
    static_assert((A_BYTES / 1024) % NWAVES == 0 && (B_BYTES / 1024) % NWAVES == 0,
                  "each wave issues the same number of A and of B DMA instructions");
    static_assert((NWAVES * RPI) % 16 == 0, "swizzle phase must not depend on the DMA instruction index");
    static_assert(NSTAGE >= 2, "ring needs a slot in use and a slot being filled");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
    static_assert(KS % 2 == 0, "fragment double buffer indexes by k-step parity");
    static_assert((NSTAGE - 1) * LPW <= 63, "vmcnt is 6 bits");
    static_assert(!SPLIT || NSTAGE == 2, "the split ring stands in for two whole slots");
    static_assert(SPREAD >= 1 && SPREAD <= KS, "a refill must be fully issued before the next barrier");
    static constexpr int DMA_PER_STEP = (LPW + SPREAD - 1) / SPREAD;

    // PERM (MT = 16, not for atomics): B rows are placed in LDS permuted within blocks of 64, LDS row p of a block holding the block's
    // row 4*(p%16) + p/16.  MFMA tile j of a wave then covers columns 64*(j/4) + 4*c + j%4 (c = 0..15) of the wave tile,
    // so a lane's accumulators of four neighbouring MFMA tiles are four consecutive columns of C: one 16 B store per
    // lane, 256 contiguous bytes per row and instruction, instead of four 64 B row segments.  The permutation costs
    // nothing: it only changes which global row each DMA lane asks for.
    static_assert(MT == 32 || (TN % 64 == 0 && NWAVES * RPI <= 64 && 64 % (NWAVES * RPI) == 0 && NWAVES * RPI % 16 == 0),
                  "row permutation splits into a per-lane and a per-instruction part only for these shapes");
    template <bool PERM>
    __device__ __host__ static constexpr uint32_t perm_row(uint32_t p)
    {
        return PERM ? 64u * (p / 64u) + 4u * (p % 16u) + (p / 16u) % 4u : p;
    }
    // tile row of B fetched by lane row 0 of DMA instruction jj of wave 0 (the per-instruction part)
    template <bool PERM>
    __device__ __host__ static constexpr uint32_t b_row(int jj)
    {
        return perm_row<PERM>((uint32_t)jj * NWAVES * RPI);
    }
    // column of the wave tile held by accumulator ni of a lane feeding MFMA column c
    template <bool PERM>
    __device__ __host__ static constexpr uint32_t acc_col(int ni, uint32_t c)
    {
        return PERM ? 64u * (ni / 4) + 4u * c + (ni % 4) : (uint32_t)ni * MT + c;
    }

    // DMA instruction issued d-th in a refill: the split ring fetches the B half first (it is needed a tile sooner)
    __device__ __host__ static constexpr int dma_index(int d)
    {
        return SPLIT ? (d + A_DMA) % LPW : d;
    }

    __device__ __host__ static constexpr uint32_t swz(uint32_t row)
    {
        return SWZ == 1 ? (row / RW) % CPR : SWZ == 2 ? row % CPR : 0u;
    }
};

// Map the hardware workgroup id to a logical work id so that consecutive logical ids run on the same XCD
// (workgroups are dealt round-robin to the 8 XCDs, each with a private L2), then rasterise logical ids in groups
// of `group_m` tile-rows so that the ~32 workgroups resident on one XCD share A row-panels and B column-panels.
// (Role of the super-block rasterisation, gemm_sm80.cu:425-451, gemm_sm90.cu:318-345.)
__device__ __forceinline__ uint32_t logical_workgroup(uint32_t pid, uint32_t nwg)
{
    const uint32_t xcd = pid % NUM_XCD, j = pid / NUM_XCD;
    const uint32_t q = nwg / NUM_XCD, r = nwg % NUM_XCD;
    return xcd * q + (xcd < r ? xcd : r) + j;
}

// Tile t of a problem in raster order -> tile coordinates.
__device__ __forceinline__ void raster_tile(const GemmArgs& p, uint32_t t, uint32_t& tm, uint32_t& tn)
{
    const uint32_t group_sz = p.group_m * p.tiles_n;
    const uint32_t g = t / group_sz;
    const uint32_t first_m = g * p.group_m;
    const uint32_t gm = p.tiles_m - first_m < p.group_m ? p.tiles_m - first_m : p.group_m;
    const uint32_t in_group = t % group_sz;
    tm = first_m + in_group % gm;
    tn = in_group / gm;
}

__device__ __forceinline__ void map_work(const GemmArgs& p, uint32_t pid, uint32_t nwg, uint32_t& tm, uint32_t& tn,
                                         uint32_t& split, uint32_t& batch)
{
    const uint32_t logical = logical_workgroup(pid, nwg);
    // logical ids run over the tiles of one K partition of one problem, then its next partition, then the next problem
    const uint32_t tiles = p.tiles_m * p.tiles_n;
    const uint32_t per_batch = tiles * p.k_splits;
    batch = logical / per_batch;
    const uint32_t in_batch = logical % per_batch;
    split = in_batch / tiles;
    raster_tile(p, in_batch % tiles, tm, tn);
}

// One workgroup per work item (an output tile and a K range).  A persistent workgroup per CU walking several tiles
// with the ring running across them (the scheme of gemm_sm80.cu:434, gemm_sm90.cu:1121) was built and measured slower
// here: gfx950 counts loads and stores in the one vmcnt counter, so the next tile's first ring hand-off waits for
// the previous tile's C stores to drain, whereas a fresh workgroup starts with a clean counter while the old
// workgroup's stores complete in the background.
// EDGE: M and N need not be multiples of the tile and K only a multiple of 8 (one 16 B chunk).  Rows of A/B beyond
// M/N and chunks beyond K are fetched through an out-of-range buffer offset, which the DMA turns into zeros in LDS;
// stores outside C are dropped the same way.  Costs a few vector ALU operations per DMA and per store instruction, so
// shapes that divide evenly use the EDGE = false build.  (Role of the predicated loads/stores of
// gemm_baseline.cu:46,62,93 and of TMA out-of-bounds fill plus the bounds-checked store gemm_sm90.cu:654-668.)
// STREAM (stream-K, the role of gemm_sm90.cu's stream_k modes, gemm/gemm_sm90.cu:1004-1095): a launch of g workgroups
// (one per CU) over r < g output tiles - the tiles that do not fill a round of CUs; full rounds run the plain build, as
// the reference keeps them output stationary - with every workgroup given the same number of K tiles, r * KT / g.  A
// contiguous run per workgroup over the (tile, K tile) pairs (the reference's dealing) puts workgroups that run side
// by side at unrelated K offsets: on a chip with eight private L2s no two of them then read the same panel at the
// same time and every byte of A and B is fetched once per workgroup.  So the dealing here keeps what makes split K
// fast: S = g / r main partitions per tile, each Km / S K tiles long, and all r workgroups of partition s walk the
// same K range in step (neighbouring tiles share their A and B panels through the L2); the K tiles [Km, KT) that are
// left of every tile, r * (KT - Km) pairs, go in equal contiguous runs to the g - r * S workgroups that are left, each
// of which then works on the leftovers of one or more tiles, one part after the other.  Every part is stored as a dense
// BM x BN tile (ldc = BN) in the parts buffer: main partition s of tile t in slot t * S + s, the part of leftover
// workgroup j on tile t in slot r * S + j + t (a run's parts and a tile's parts are consecutive in j and t, so j + t
// names each once); a second kernel sums each tile's parts, in slot order, into C.  Whole tiles only (no EDGE), plain
// stores (no ATOMIC), one problem.
//
// ONCE (whole tiles only): 1 = every byte of A, 2 = every byte of B is read by exactly one workgroup of
// the launch (the problem is one tile wide in the other dimension) and the operand is larger than the memory-side
// cache: its DMA is issued non-temporal, so that the stream does not push the other operand's panels, which every
// workgroup re-reads, out of the L2.  Measured on 256 x 28672 x 8192 (B is 470 MB): 159 -> 124 us.  On an operand that
// is re-read (or that fits the 256 MB memory-side cache, where a benchmark loop finds it again) the same bit costs
// 8 to 40 %, hence a build of its own that the host picks per launch.
template <int DTYPE, typename Cfg, bool ATOMIC, bool EDGE, bool STREAM = false, int ONCE = 0>
__global__ __launch_bounds__(Cfg::NTHREADS) void gemm_tn_kernel(const GemmArgs p)
{
    static_assert(!STREAM || (!ATOMIC && !EDGE), "stream-K parts are whole tiles stored with plain stores");
    static_assert(ONCE == 0 || (!EDGE && !STREAM), "the non-temporal builds exist for whole tiles");
    constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, WN = Cfg::WN, NSTAGE = Cfg::NSTAGE, NWAVES = Cfg::NWAVES;
    constexpr int MI = Cfg::MI, NI = Cfg::NI, KS = Cfg::KS, ROWB = Cfg::ROWB, CPR = Cfg::CPR, RPI = Cfg::RPI;
    constexpr int LPW = Cfg::LPW, A_DMA = Cfg::A_DMA, NR = Cfg::NR, NMFMA = Cfg::NMFMA, STAGE_BYTES = Cfg::STAGE_BYTES;
    constexpr int MT = Cfg::MT, NACC = Cfg::NACC, RS = Cfg::RS;
    using AccT = typename AccOf<MT>::type;
    // B rows permuted in LDS so that 16-wide MFMA tiles store 16 B per lane (see TileCfg::perm_row); atomics have no
    // 16 B form and keep the plain placement, whose dword accesses are contiguous across lanes
    constexpr bool PERM = MT == 16 && !ATOMIC;

    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_char*)smem;

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t wm = w / WN, wn = w % WN;
    const uint32_t n_items = gridDim.x;  // (all items of the problem, or its first whole rounds of tiles: see launch_cfg)
    const uint32_t kt_total = (p.K + BK - 1) / BK;
    constexpr uint32_t OOB = 0x80000000u;  // buffer offset that no descriptor below covers: loads give 0, stores drop

    // ---- producer addressing.  DMA instruction j of wave w fills slot bytes [q*1024, q*1024+1024) with
    // q = j*NWAVES + w (A region) or A_BYTES/1024 + (j-A_DMA)*NWAVES + w (B region): RPI consecutive rows each.
    // A and B are each addressed through a buffer descriptor based at the tile's first row and first K element;
    // the address splits into a per-lane 32-bit offset that never changes (the swizzle phase of a row repeats every
    // 16 rows, so it does not depend on j) and a wave-uniform scalar offset advanced by j and by the K tile.
    const uint32_t lrow = w * RPI + lane / CPR;             // row (mod NWAVES*RPI) this lane fetches
    const uint32_t lchunk = (lane % CPR) ^ Cfg::swz(lrow);  // global chunk that lands at LDS position lane%CPR
    const uint32_t voff_a = lrow * p.lda * 2u + lchunk * 16u;
    const uint32_t lrow_b = Cfg::template perm_row<PERM>(lrow);            // tile row of B behind LDS row lrow (the per-lane part)
    const uint32_t voff_b = lrow_b * p.ldb * 2u + lchunk * 16u;
    const uint32_t a_jstride = NWAVES * RPI * p.lda * 2u, ldb2 = p.ldb * 2u;
    lds_char* const lds_w = (lds_char*)smem + w * 1024u;

    // one work item: an output tile and a K range
    struct Item {
        uint32_t tm, tn, KT;
        uint32_t rot;        // K tile of the range that the walk starts at (it wraps around to tile 0)
        const char* a_base;  // first row of the A panel, first K element of the range
        const char* b_base;
        float* c_tile;                // where element (0, 0) of this item's output tile goes
        int32_t m_rem, n_rem, k_rem;  // rows of A, rows of B and K elements that exist from this item's origin on
        // parts summed inside the launch (p.tile_counters != null): the tile's arrival counter, how many parts it has,
        // this part's place in their order, and where the tile's sum goes
        uint32_t counter, parts, part_index;
        float* final_tile;
    };
    auto make_item = [&](uint32_t id) {
        Item it;
        uint32_t split, batch;
        map_work(p, id, n_items, it.tm, it.tn, split, batch);
        const uint32_t kt_begin = split * p.k_tiles_per_split;
        it.KT = kt_total - kt_begin < p.k_tiles_per_split ? kt_total - kt_begin : p.k_tiles_per_split;
        it.a_base = (const char*)p.a + batch * p.a_batch_bytes + ((size_t)it.tm * BM * p.lda + (size_t)kt_begin * BK) * 2;
        it.b_base = (const char*)p.b + batch * p.b_batch_bytes + ((size_t)it.tn * BN * p.ldb + (size_t)kt_begin * BK) * 2;
        it.c_tile = (float*)((char*)p.c + batch * p.c_batch_bytes + split * p.c_split_bytes) +
                    ((size_t)it.tm * BM * p.ldc + (size_t)it.tn * BN);
        it.m_rem = (int32_t)(p.M - it.tm * BM);
        it.n_rem = (int32_t)(p.N - it.tn * BN);
        it.k_rem = (int32_t)(p.K - kt_begin * BK);
        it.counter = batch * (p.tiles_m * p.tiles_n) + it.tm * p.tiles_n + it.tn;
        it.parts = p.k_splits;
        it.part_index = split;
        it.final_tile = (float*)((char*)p.c_final + batch * p.c_final_batch_bytes) +
                        ((size_t)it.tm * BM * p.ldc_final + (size_t)it.tn * BN);
        // (short ranges are not rotated: the walk's look-ahead must stay inside one lap)
        it.rot = EDGE || it.KT < 16 ? 0u : ((blockIdx.x % NUM_XCD) * p.k_rotate) % it.KT;
        return it;
    };
    // Stream-K: this workgroup is main partition sk_split of tail tile sk_tile, or leftover workgroup sk_left with the
    // run [sk_cur, sk_end) of the leftover (tile, K tile) pairs, walked one part (one tile's share) at a time.
    uint32_t sk_tile = 0, sk_split = 0, sk_left = 0, sk_kr = 0;
    uint64_t sk_cur = 0, sk_end = 0;
    bool sk_main = false;
    if constexpr (STREAM) {
        const uint32_t l = logical_workgroup(blockIdx.x, gridDim.x);
        const uint32_t mains = p.sk.tiles * p.sk.splits;
        sk_kr = kt_total - p.sk.main_k;
        if (l < mains) {
            // partition-major: the tiles of one partition are consecutive workgroups (and share panels in one L2)
            sk_main = true;
            sk_split = l / p.sk.tiles;
            sk_tile = l % p.sk.tiles;
            sk_cur = 0;
            sk_end = 1;  // one part
        }
        else {
            sk_left = l - mains;
            const uint64_t units = (uint64_t)p.sk.tiles * sk_kr, lefts = gridDim.x - mains;
            sk_cur = sk_left * units / lefts;
            sk_end = (sk_left + 1) * units / lefts;
        }
    }
    auto make_part = [&]() {
        Item it;
        uint32_t tile, kt_begin, kt_end, slot;
        if (sk_main) {
            tile = sk_tile;
            kt_begin = (uint32_t)((uint64_t)sk_split * p.sk.main_k / p.sk.splits);
            kt_end = (uint32_t)((uint64_t)(sk_split + 1) * p.sk.main_k / p.sk.splits);
            slot = sk_tile * p.sk.splits + sk_split;
            sk_cur = sk_end;
        }
        else {
            tile = (uint32_t)(sk_cur / sk_kr);
            const uint32_t in_tile = (uint32_t)(sk_cur % sk_kr);
            const uint64_t left_in_run = sk_end - sk_cur;
            const uint32_t len = left_in_run < sk_kr - in_tile ? (uint32_t)left_in_run : sk_kr - in_tile;
            kt_begin = p.sk.main_k + in_tile;
            kt_end = kt_begin + len;
            slot = p.sk.tiles * p.sk.splits + sk_left + tile;
            sk_cur += len;
        }
        raster_tile(p, p.sk.first_tile + tile, it.tm, it.tn);
        it.KT = kt_end - kt_begin;
        it.a_base = (const char*)p.a + ((size_t)it.tm * BM * p.lda + (size_t)kt_begin * BK) * 2;
        it.b_base = (const char*)p.b + ((size_t)it.tn * BN * p.ldb + (size_t)kt_begin * BK) * 2;
        it.c_tile = p.c + (size_t)slot * (BM * BN);
        it.m_rem = BM;
        it.n_rem = BN;
        it.k_rem = (int32_t)(p.K - kt_begin * BK);
        it.rot = 0;
        it.counter = tile;
        it.part_index = tile;  // (stream-K: the tail tile; the parts' order is their slots')
        it.parts = 0;          // (counted when the part has been stored)
        it.final_tile = p.c_final + ((size_t)it.tm * BM * p.ldc_final + (size_t)it.tn * BN);
        return it;
    };
    Item cur;
    if constexpr (!STREAM) {
        cur = make_item(blockIdx.x);
    }
    // K tile of the item's range that step `step` of the walk works on (steps beyond the range are never fetched)
    auto walk_tile = [](const Item& it, uint32_t step) {
        const uint32_t at = it.rot + step;
        return at >= it.KT ? at - it.KT : at;
    };

    // ---- consumer addressing (LDS byte addresses inside slot 0)
    const uint32_t g = lane / MT;      // which 8-wide k group of the MFMA's K depth this lane feeds
    const uint32_t lrc = lane % MT;    // row of A / column of B (row of the N x K operand) this lane feeds
    uint32_t a_off[KS], b_off[KS];
    {
        const uint32_t row_a = wm * Cfg::TM + lrc;
        const uint32_t row_b = wn * Cfg::TN + lrc;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const uint32_t c = (uint32_t)Cfg::CPS * ks + g;
            a_off[ks] = lds_base + row_a * ROWB + ((c ^ Cfg::swz(row_a)) * 16u);
            b_off[ks] = lds_base + row_b * ROWB + ((c ^ Cfg::swz(row_b)) * 16u);
        }
    }

    AccT acc[MI][NI];
    u32x4 fa[2][MI], fb[2][NI];

    // Scalar byte offsets of the rows that DMA instruction jj of wave 0 fetches (the per-instruction part of the
    // address): loop invariant, one SGPR each.
    uint32_t soff_a[A_DMA > 0 ? A_DMA : 1], soff_b[LPW - A_DMA > 0 ? LPW - A_DMA : 1];
#pragma unroll
    for (int jj = 0; jj < A_DMA; ++jj) {
        soff_a[jj] = jj * a_jstride;
    }
#pragma unroll
    for (int jj = 0; jj < LPW - A_DMA; ++jj) {
        soff_b[jj] = Cfg::template b_row<PERM>(jj) * ldb2;
    }
    // DMA instruction j of this wave: for j < A_DMA rows of A into the LDS region at byte `dst_a`, else rows of B into
    // the region at `dst_b`.  The K tile is the one the buffer descriptors `ka` / `kb` are based at (the first K
    // element of some K tile of this item's panels): the descriptors move on by one K tile per iteration, at the
    // hand-off barrier (a few scalar operations), and the DMA itself needs no address arithmetic.
    // `kla` / `klb` (range-checked build only): K elements that exist from the descriptor's K tile on.
    auto issue_dma = [&](auto jc, const char* ka, const char* kb, int32_t kla, int32_t klb, uint32_t dst_a,
                         uint32_t dst_b) {
        constexpr int j = jc.value;
        constexpr bool is_a = j < A_DMA;
        constexpr int jj = is_a ? j : j - A_DMA;
        const Item& it = cur;  // (captured by reference: the item lives for the whole kernel)
        lds_char* const dst = lds_w + (is_a ? dst_a : dst_b) + jj * (NWAVES * 1024);
        if constexpr (!EDGE) {
            if constexpr (is_a) {
                dma_buffer_to_lds_16B<ONCE == 1>(make_rsrc(ka, BM * p.lda * 2u), voff_a, soff_a[jj], dst);
            }
            else {
                dma_buffer_to_lds_16B<ONCE == 2>(make_rsrc(kb, BN * p.ldb * 2u), voff_b, soff_b[jj], dst);
            }
        }
        else {
            // the row part moves into the (range-checked) vector offset; a lane whose row or K chunk does not exist
            // asks for offset OOB instead
            const int32_t rows_left = is_a ? it.m_rem - jj * (NWAVES * RPI) : it.n_rem - (int32_t)Cfg::template b_row<PERM>(jj);
            const int32_t k_left = is_a ? kla : klb;
            const bool exists = (int32_t)(is_a ? lrow : lrow_b) < rows_left && (int32_t)(lchunk * 8u) < k_left;
            const uint32_t voff = (is_a ? voff_a + jj * a_jstride : voff_b + Cfg::template b_row<PERM>(jj) * ldb2);
            dma_buffer_to_lds_16B(make_rsrc(is_a ? ka : kb, OOB), exists ? voff : OOB, 0, dst);
        }
    };
    // fragment read i of a k-step: B fragments first, then A fragments (the order the MFMA rows need them)
    auto issue_read = [&](auto ic, auto bufc, uint32_t a_addr, uint32_t b_addr) {
        constexpr int i = ic.value, buf = bufc.value;
        if constexpr (i < NI) {
            lds_read_b128<i * MT * ROWB>(fb[buf][i], b_addr);
        }
        else {
            lds_read_b128<(i - NI) * MT * ROWB>(fa[buf][i - NI], a_addr);
        }
    };


    uint32_t n_stamps = 0;
    auto stamp = [&]() {
        if (p.timeline != nullptr) {
            if (threadIdx.x == 0 && n_stamps + 1 < p.timeline_slots) {
                unsigned long long* const dst = p.timeline + ((size_t)blockIdx.x * p.timeline_slots + n_stamps) * 2;
                dst[0] = wall_clock64();
                dst[1] = clock64();
            }
            ++n_stamps;
        }
    };
    stamp();

    // ---- ring organisation.  A ring position names where K tile kt lives in LDS.
    // Slot ring (SPLIT = false): NSTAGE slots of one K tile each (A rows, then B rows); position = slot index.  The
    // slot of tile kt is refilled with tile kt+NSTAGE.
    // Split ring (SPLIT = true): 5 units, each large enough for an A or a B tile; the stream A(0) B(0) A(1) B(1) ... occupies units 0 1 2 3 4 0 ...
    // so A(kt) is unit 2kt mod 5 (the position) and B(kt) the unit after it.  When tile kt retires, its A unit takes
    // B(kt+2) and its B unit takes A(kt+3): two and a half tiles are resident or in flight instead of two, and at the
    // hand-off barrier only the older half of the outstanding DMA has to have landed.  This is what lets a 256x256x64
    // tile (64 KB per K tile, 160 KB of LDS) hide the L2-to-LDS latency.
    constexpr bool SPLIT = Cfg::SPLIT;
    constexpr int DIST_A = Cfg::DIST_A, DIST_B = Cfg::DIST_B, PF = Cfg::PF;
    constexpr uint32_t UNIT = Cfg::UNIT;
    auto ring_a = [](uint32_t pos) { return SPLIT ? pos * UNIT : pos * (uint32_t)STAGE_BYTES; };
    auto ring_b = [](uint32_t pos) {
        return SPLIT ? (pos + 1 == (uint32_t)Cfg::UNITS ? 0u : pos + 1) * UNIT
                     : pos * (uint32_t)STAGE_BYTES + (uint32_t)Cfg::A_BYTES;
    };
    auto ring_next = [](uint32_t pos) {
        if constexpr (SPLIT) {
            return pos + 2 >= (uint32_t)Cfg::UNITS ? pos + 2 - (uint32_t)Cfg::UNITS : pos + 2;
        }
        else {
            return pos + 1 == (uint32_t)NSTAGE ? 0u : pos + 1;
        }
    };

    for (bool first_part = true; first_part || (STREAM && sk_cur < sk_end); first_part = false) {
    if constexpr (STREAM) {
        if (sk_cur >= sk_end) {
            break;  // (a leftover workgroup whose run is empty)
        }
        if (!first_part) {
            // every wave has drained its fragment reads of the previous part (lgkmcnt(0) below): the ring may be refilled.
            // (The full wait: the K loop counts its fragment reads with partial waits, and no scalar load that the code
            // behind the previous part's K loop may have issued can be allowed to still be in flight then.)
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        }
        cur = make_part();
    }
    // ---- prologue: start filling the ring, wait for tile 0, fetch its first fragments
    {
        uint32_t pos = 0;
#pragma unroll
        for (int t = 0; t < PF; ++t) {
            if ((uint32_t)t < cur.KT) {
                const uint32_t kt_of_t = walk_tile(cur, t);
                const char* const ka = cur.a_base + (size_t)kt_of_t * (BK * 2);
                const char* const kb = cur.b_base + (size_t)kt_of_t * (BK * 2);
                const int32_t kl = cur.k_rem - t * BK;  // (range-checked build: never rotated)
                static_for<0, A_DMA>([&](auto jc) { issue_dma(jc, ka, kb, kl, kl, ring_a(pos), ring_b(pos)); });
                if (t < DIST_B) {
                    static_for<A_DMA, LPW>([&](auto jc) { issue_dma(jc, ka, kb, kl, kl, ring_a(pos), ring_b(pos)); });
                }
            }
            pos = ring_next(pos);
        }
    }
    // everything after tile 0 may still be in flight
    constexpr int PROLOGUE_AFTER_TILE0 = SPLIT ? (PF - 1) * A_DMA + (DIST_B - 1) * (LPW - A_DMA) : (NSTAGE - 1) * LPW;
    if (cur.KT >= (uint32_t)PF) {
        wait_vmcnt_then_barrier<PROLOGUE_AFTER_TILE0>();
    }
    else {
        wait_vmcnt_then_barrier<0>();
    }
    stamp();
    static_for<0, NR>([&](auto ic) { issue_read(ic, IntC<0>{}, a_off[0], b_off[0] + ring_b(0)); });

    {
        const uint32_t KT = cur.KT;
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) {
#pragma unroll
            for (int ni = 0; ni < NI; ++ni) {
#pragma unroll
                for (int r = 0; r < NACC; ++r) {
                    acc[mi][ni][r] = 0.0f;
                }
            }
        }

        // Ring offsets in rotated order: u[k] is the LDS byte offset of ring position (position of tile kt) + k.  Moving
        // on to the next K tile renames these scalars; no ring position is ever computed inside the loop.
        constexpr int PERIOD = SPLIT ? Cfg::UNITS : NSTAGE;
        constexpr int STEP = SPLIT ? 2 : 1;
        uint32_t u[PERIOD];
#pragma unroll
        for (int k = 0; k < PERIOD; ++k) {
            u[k] = (uint32_t)k * (SPLIT ? UNIT : (uint32_t)STAGE_BYTES);
        }
        // Step kt + DIST - 1 of the walk over this item's panels: the rest of the refill begun in iteration kt-1 fetches
        // it.  At the hand-off barrier of iteration kt the descriptors move on to the next step (wrapping around at the
        // end of the range when the walk is rotated), which the refill begun there fetches.
        const char* const a_begin = cur.a_base, * const b_begin = cur.b_base;
        const char* ka = a_begin + (size_t)walk_tile(cur, DIST_A - 1) * (BK * 2);
        const char* kb = b_begin + (size_t)walk_tile(cur, DIST_B - 1) * (BK * 2);
        const char* const a_end = a_begin + (size_t)cur.KT * (BK * 2);
        const char* const b_end = b_begin + (size_t)cur.KT * (BK * 2);
        int32_t kla = cur.k_rem - (DIST_A - 1) * BK, klb = cur.k_rem - (DIST_B - 1) * BK;  // K elements from there on
        // LDS addresses (per lane) that the fragment reads issued during the coming k-step start from: computed one
        // k-step ahead, in MFMA gaps of their own, so that no k-step begins with a clump of address arithmetic
        uint32_t rd_a = a_off[1 % KS] + u[0], rd_b = b_off[1 % KS] + u[SPLIT ? 1 : 0] + (SPLIT ? 0u : (uint32_t)Cfg::A_BYTES);
        // The ring offsets are turned in place, one scalar move per MFMA gap at the end of a K tile's last k-step (after
        // the last DMA that names an old offset), when a k-step has the gaps to spare (LATE: all tiles but the three
        // smallest 64-deep ones and the 32-deep twins).
        constexpr int ROT_MOVES = PERIOD + 1;
        constexpr int RD_I = (NR - 1) * RS + 2;  // first gap after the k-step's last fragment read
        // DMA d of a k-step sits in gap d * DMA_STRIDE + 1: evenly over the k-step if that leaves the last gaps free for
        // the moves below, else over the part of the k-step ahead of them
        constexpr int DPS = Cfg::DMA_PER_STEP;
        constexpr int TAIL_GAPS = ROT_MOVES > 5 ? ROT_MOVES : 5;  // ring moves (last k-step) / descriptor advance (the one before)
        constexpr int EVEN_STRIDE = NMFMA / DPS;
        constexpr int DMA_STRIDE = (DPS - 1) * EVEN_STRIDE + 1 < NMFMA - TAIL_GAPS ? EVEN_STRIDE : (NMFMA - TAIL_GAPS - 1) / DPS;
        constexpr int LAST_DMA_I = (DPS - 1) * DMA_STRIDE + 1;
        constexpr bool LATE = Cfg::LOOP_READS == NR && KS >= 2 && DMA_STRIDE >= 2 && RD_I + 3 <= NMFMA - ROT_MOVES &&
                              LAST_DMA_I < NMFMA - TAIL_GAPS;
        uint32_t u_tmp = 0;
        // Loops with gaps to spare also place their DMAs by hand (dma_set_lds_base / dma_issue_16B) and carry the two
        // descriptors themselves (words 0 and 1 are the 48-bit base) instead of the pointers `ka` / `kb`.
        // (every DMA sits at least two gaps after the one before it and not in gap 0, so that the gap ahead of it exists and
        // lies behind the previous DMA)
        constexpr bool ASM_DMA = LATE && !EDGE;
        u32x4 qa = make_rsrc_words(ka, BM * p.lda * 2u), qb = make_rsrc_words(kb, BN * p.ldb * 2u);
        const uint64_t a_begin48 = (uint64_t)(uintptr_t)a_begin & 0xffffffffffffull, a_end48 = a_begin48 + (uint64_t)cur.KT * (BK * 2);
        const uint64_t b_begin48 = (uint64_t)(uintptr_t)b_begin & 0xffffffffffffull, b_end48 = b_begin48 + (uint64_t)cur.KT * (BK * 2);
        auto quad_step = [](u32x4& q) {
            const uint64_t b = (((uint64_t)q.y << 32) | q.x) + BK * 2;
            q.x = (uint32_t)b;
            q.y = (uint32_t)(b >> 32);
        };
        auto quad_wrap = [](u32x4& q, uint64_t begin, uint64_t end) {
            uint64_t b = ((uint64_t)q.y << 32) | q.x;
            b = b == end ? begin : b;
            q.x = (uint32_t)b;
            q.y = (uint32_t)(b >> 32);
        };
        // ... and the descriptors move on in the last gaps of the k-step before the hand-off barrier (their old
        // position is last named by that k-step's last DMA), not in the gap right behind the barrier.
        constexpr bool EARLY_ADV = LATE;
        // One K tile.  `steady` (compile time): every refill certainly happens, so the hot loop carries no branches;
        // otherwise (first and last PF iterations) they are decided at run time.
        auto k_tile = [&](auto steady, uint32_t kt) __attribute__((always_inline)) {
            constexpr bool STEADY = steady.value != 0;
            // (split ring: the B tile sits in the unit after its A tile; slot ring: behind the A rows of the same slot)
            constexpr int B_UNIT = SPLIT ? 1 : 0;
            constexpr uint32_t B_BYTE = SPLIT ? 0u : (uint32_t)Cfg::A_BYTES;
            const uint32_t a_cur = u[0], b_cur = u[B_UNIT] + B_BYTE;
            const uint32_t a_nxt = u[STEP], b_nxt = u[STEP + B_UNIT] + B_BYTE;
            // Refill begun in this iteration, once tile kt has retired: A of tile kt+DIST_A and B of tile kt+DIST_B
            // into the regions tile kt occupied.
            const bool ra_on = STEADY || kt + DIST_A < KT, rb_on = STEADY || kt + DIST_B < KT;
            const uint32_t ra_dst = SPLIT ? b_cur : a_cur, rb_dst = SPLIT ? a_cur : b_cur;
            // Rest of the refill begun in iteration kt-1 (its first part went out right after that tile's barrier).
            const bool pa_on = STEADY || (kt > 0 && kt + DIST_A < KT + 1);
            const bool pb_on = STEADY || (kt > 0 && kt + DIST_B < KT + 1);
            const uint32_t pv_a = u[PERIOD - STEP], pv_b = u[PERIOD - STEP + B_UNIT] + B_BYTE;
            const uint32_t pa_dst = SPLIT ? pv_b : pv_a;
            const uint32_t pb_dst = SPLIT ? pv_a : pv_b;
            static_for<0, KS>([&](auto ksc) {
                constexpr int ks = ksc.value, cu = ks & 1, nx = cu ^ 1;
                constexpr bool last = ks == KS - 1;
                // which part of a refill this k-step issues: step 0 of a refill is the k-step right after the barrier
                constexpr int rstep = last ? 0 : ks + 1;
                constexpr int dma_lo = rstep < Cfg::SPREAD ? rstep * Cfg::DMA_PER_STEP : LPW;
                constexpr int dma_hi = dma_lo + Cfg::DMA_PER_STEP < LPW ? dma_lo + Cfg::DMA_PER_STEP : LPW;
                constexpr int dma_n = dma_hi - dma_lo;
                // source of the next k-step's fragments: same tile, or k-step 0 of the next tile
                uint32_t a_nx, b_nx, a_nn = 0, b_nn = 0;
                if constexpr (LATE) {
                    a_nx = rd_a;
                    b_nx = rd_b;
                }
                else {
                    a_nx = last ? a_off[0] + a_nxt : a_off[(ks + 1) % KS] + a_cur;
                    b_nx = last ? b_off[0] + b_nxt : b_off[(ks + 1) % KS] + b_cur;
                }
                if constexpr (last) {
                    // Every fragment of tile kt is now in registers and this wave's share of tile kt+1 has landed:
                    // after the barrier the regions of tile kt may be refilled and tile kt+1 may be read.  DMAs land
                    // in issue order, so the wait may leave the most recently issued ones outstanding: a whole tile
                    // per extra slot of the slot ring, the A half issued last in the split ring.
                    wait_lgkmcnt<0>();
                    constexpr int ALLOWED = SPLIT ? A_DMA : (NSTAGE - 2) * LPW;
                    const bool all_issued = kt + PF - 1 < KT;  // the newest refill was complete
                    if (STEADY || all_issued) {
                        wait_vmcnt_then_barrier<ALLOWED>();
                    }
                    else {
                        wait_vmcnt_then_barrier<0>();
                    }
                    if constexpr (!EARLY_ADV) {
                        ka += BK * 2;
                        kb += BK * 2;
                        if constexpr (EDGE) {
                            kla -= BK;
                            klb -= BK;
                        }
                        else {
                            ka = ka == a_end ? a_begin : ka;
                            kb = kb == b_end ? b_begin : kb;
                        }
                    }
                }
                else {
                    // B fragments and the first A fragment of this k-step; the other A fragments may still be in flight
                    wait_lgkmcnt<(MI - 1 < 15 ? MI - 1 : 15)>();
                }
                static_for<0, NI>([&](auto ni) { touch(fb[cu][ni.value]); });
                touch(fa[cu][0]);
                static_for<0, NMFMA>([&](auto ic) {
                    // rows of MFMA tiles are walked boustrophedon: at a row change only the A operand changes (the
                    // chip is power-limited and the operand buses toggle less: measured +0.5 % on 8192^3)
                    constexpr int i = ic.value, mi = i / NI, ni_seq = i % NI, ni = (mi & 1) ? NI - 1 - ni_seq : ni_seq;
                    if constexpr (ni_seq == 0 && mi > 0) {
                        if constexpr (!last) {
                            // outstanding: A fragments mi+1.. of this k-step, plus the reads issued so far for the next
                            // (the counter is 4 bits wide: a clamped wait is merely stricter)
                            constexpr int issued = (mi * NI + RS - 1) / RS < NR ? (mi * NI + RS - 1) / RS : NR;
                            constexpr int allowed = (MI - 1 - mi) + issued;
                            wait_lgkmcnt<(allowed < 15 ? allowed : 15)>();
                        }
                        touch(fa[cu][mi]);
                    }
                    acc[mi][ni] = mfma_tile<DTYPE>(fa[cu][mi], fb[cu][ni], acc[mi][ni]);
                    sched_fence();
                    if constexpr (LATE && (i == RD_I || i == RD_I + 2)) {
                        // read bases of the next k-step: fragments of k-step ks+2 of this tile, of k-step 0 of the next
                        // tile (next k-step is this tile's last) or of k-step 1 of the next tile (this one is)
                        constexpr int of = ks + 2 < KS ? ks + 2 : ks + 2 == KS ? 0 : 1;
                        const uint32_t su = i == RD_I ? (ks + 2 < KS ? a_cur : a_nxt) : (ks + 2 < KS ? b_cur : b_nxt);
                        if constexpr (i == RD_I) {
                            a_nn = pinned_add(su, a_off[of]);
                        }
                        else {
                            b_nn = pinned_add(su, b_off[of]);
                        }
                    }
                    if constexpr (EARLY_ADV && ks == KS - 2 && i >= NMFMA - 5 && i < NMFMA - 1) {
                        constexpr int m = i - (NMFMA - 5);
                        if constexpr (ASM_DMA) {
                            if constexpr (m == 0) {
                                quad_step(qa);
                            }
                            else if constexpr (m == 1) {
                                quad_wrap(qa, a_begin48, a_end48);
                            }
                            else if constexpr (m == 2) {
                                quad_step(qb);
                            }
                            else {
                                quad_wrap(qb, b_begin48, b_end48);
                            }
                        }
                        else if constexpr (m == 0) {
                            ka += BK * 2;
                            if constexpr (EDGE) {
                                kla -= BK;
                            }
                        }
                        else if constexpr (m == 1) {
                            if constexpr (!EDGE) {
                                ka = ka == a_end ? a_begin : ka;
                            }
                        }
                        else if constexpr (m == 2) {
                            kb += BK * 2;
                            if constexpr (EDGE) {
                                klb -= BK;
                            }
                        }
                        else {
                            if constexpr (!EDGE) {
                                kb = kb == b_end ? b_begin : kb;
                            }
                        }
                    }
                    if constexpr (LATE && last && i >= NMFMA - ROT_MOVES) {
                        // move m of the rotation u[k] <- u[(k + STEP) % PERIOD], walked as one cycle from position 0
                        constexpr int m = i - (NMFMA - ROT_MOVES);
                        if constexpr (m == 0) {
                            u_tmp = pinned_move(u[0]);
                        }
                        else if constexpr (m == PERIOD) {
                            u[((PERIOD - 1) * STEP) % PERIOD] = pinned_move(u_tmp);
                        }
                        else {
                            u[((m - 1) * STEP) % PERIOD] = pinned_move(u[(m * STEP) % PERIOD]);
                        }
                    }
                    if constexpr (i % RS == 0 && i / RS < NR) {
                        issue_read(IntC<i / RS>{}, IntC<nx>{}, a_nx, b_nx);
                    }
                    // DMA d of this k-step goes after MFMA d * DMA_STRIDE + 1 (hand-scheduled loops), else after MFMA
                    // d*NMFMA/dma_n (evenly spaced; one further on when the fragment reads sit in the even gaps)
                    static_for<0, dma_n>([&](auto dc) {
                        constexpr int slot = LATE ? dc.value * DMA_STRIDE + 1
                                                  : (dc.value * NMFMA) / dma_n + ((NMFMA / dma_n) >= 2 && RS % 2 == 0 ? 1 : 0);
                        constexpr int j = Cfg::dma_index(dma_lo + dc.value);
                        if constexpr (ASM_DMA) {
                            constexpr bool is_a = j < A_DMA;
                            constexpr int jj = is_a ? j : j - A_DMA;
                            const uint32_t region = last ? (is_a ? ra_dst : rb_dst) : (is_a ? pa_dst : pb_dst);
                            if constexpr (slot - 1 == i) {
                                // LDS base of the DMA, a gap ahead of it
                                dma_set_lds_base<jj * (NWAVES * 1024)>((uint32_t)(uintptr_t)(lds_w + region));
                            }
                            if constexpr (slot == i) {
                                if (last ? (is_a ? ra_on : rb_on) : (is_a ? pa_on : pb_on)) {
                                    if constexpr (is_a) {
                                        dma_issue_16B<ONCE == 1>(qa, voff_a, soff_a[jj]);
                                    }
                                    else {
                                        dma_issue_16B<ONCE == 2>(qb, voff_b, soff_b[jj]);
                                    }
                                }
                            }
                        }
                        else if constexpr (slot == i) {
                            if constexpr (last) {
                                if (j < A_DMA ? ra_on : rb_on) {
                                    issue_dma(IntC<j>{}, ka, kb, kla, klb, ra_dst, rb_dst);
                                }
                            }
                            else {
                                if (j < A_DMA ? pa_on : pb_on) {
                                    issue_dma(IntC<j>{}, ka, kb, kla, klb, pa_dst, pb_dst);
                                }
                            }
                        }
                    });
                    sched_fence();
                });
                static_for<Cfg::LOOP_READS, NR>([&](auto ic) { issue_read(ic, IntC<nx>{}, a_nx, b_nx); });
                if constexpr (LATE) {
                    rd_a = a_nn;
                    rd_b = b_nn;
                }
            });
            // on to the next K tile: the ring turns by STEP positions
            if constexpr (!LATE) {
                uint32_t turned[PERIOD];
#pragma unroll
                for (int k = 0; k < PERIOD; ++k) {
                    turned[k] = u[(k + STEP) % PERIOD];
                }
#pragma unroll
                for (int k = 0; k < PERIOD; ++k) {
                    u[k] = turned[k];
                }
            }
        };
        {
            uint32_t kt = 0;
            // the first PF-1 iterations run the general code: the refill bookkeeping of kt == 0 lives there
            for (; kt < KT && kt + 1 < (uint32_t)PF; ++kt) {
                k_tile(IntC<0>{}, kt);
            }
            {
                // (the steady iterations do not look at kt: a plain countdown)
                const uint32_t n_steady = __builtin_amdgcn_readfirstlane(KT > kt + (uint32_t)PF ? KT - kt - (uint32_t)PF : 0u);
                for (uint32_t n = n_steady; n != 0; --n) {
                    k_tile(IntC<1>{}, 0u);
                }
                kt += n_steady;
            }
            for (; kt < KT; ++kt) {
                k_tile(IntC<0>{}, kt);
            }
        }
        // drain the fragment prefetch of the (non-existent) tile KT so no LDS return is outstanding
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");

        stamp();

        // ---- epilogue.  Register r of lane l of an accumulator tile is C[row_of(r) + 4*(l/MT)][l%MT] of that tile.
        auto row_of = [](int r) { return MT == 32 ? 8 * (r / 4) + (r % 4) : r; };
        float* const c_wave = cur.c_tile + ((size_t)(wm * Cfg::TM) * p.ldc + wn * Cfg::TN);  // this wave's corner of C
        const int32_t m_left = cur.m_rem - (int32_t)(wm * Cfg::TM) - (int32_t)(4u * g);  // rows from this lane's first row
        const int32_t n_left = cur.n_rem - (int32_t)(wn * Cfg::TN);  // columns from this wave's first column
        if constexpr (ATOMIC) {
            // Buffer atomics addressed like the plain stores below: a fixed per-lane 32-bit offset, the register-dependent
            // rest a scalar offset, so the epilogue computes no per-element addresses.  One dword per lane, two full
            // 128 B (MT = 32) or four 64 B (MT = 16) row segments per instruction.  Range-checked build: elements outside
            // C get the out-of-range offset and the buffer range check drops the atomic.
            const __amdgpu_buffer_rsrc_t rsrc_c = make_rsrc(c_wave, EDGE ? OOB : ((Cfg::TM - 1) * p.ldc + Cfg::TN) * 4u);
            const uint32_t voff = (4u * g * p.ldc + lrc) * 4u;
            // An atomic takes its data from an ordinary vector register.  Each value is moved out of its accumulation
            // register right where it is used: left to itself the compiler moves all of them first and runs out of
            // registers.  (The moves are opaque to the compiler's hazard pass, hence the explicit wait for the last
            // MFMAs' results.)
            asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
            for (int mi = 0; mi < MI; ++mi) {
#pragma unroll
                for (int ni = 0; ni < NI; ++ni) {
#pragma unroll
                    for (int r = 0; r < NACC; ++r) {
                        const int row = mi * MT + row_of(r);
                        const uint32_t soff = ((uint32_t)row * p.ldc + ni * MT) * 4u;
                        float v;
                        asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(acc[mi][ni][r]));
                        if constexpr (!EDGE) {
                            __builtin_amdgcn_raw_ptr_buffer_atomic_fadd_f32(v, rsrc_c, voff, soff, 0);
                        }
                        else {
                            const bool inside = row < m_left && (int32_t)(ni * MT + lrc) < n_left;
                            __builtin_amdgcn_raw_ptr_buffer_atomic_fadd_f32(v, rsrc_c, inside ? voff + soff : OOB, 0u, 0);
                        }
                    }
                }
                sched_fence();
            }
        }
        else {
            // Buffer stores with a fixed per-lane 32-bit offset; the register-dependent rest is a scalar offset.
            // MT = 32: one dword per lane, two full 128 B row segments per instruction.  MT = 16: four MFMA tiles at a
            // time, 16 B per lane, four 256 B row segments per instruction (see PERM).  Non-temporal, so C does not
            // displace the A/B panels that other tiles are re-reading from the L2.
            constexpr int NT = AUX_NT;
            if constexpr (!EDGE) {
                const __amdgpu_buffer_rsrc_t rsrc_c =
                    make_rsrc(c_wave, ((Cfg::TM - 1) * p.ldc + Cfg::TN) * 4u);
                const uint32_t voff = (4u * g * p.ldc + Cfg::template acc_col<PERM>(0, lrc)) * 4u;
                if constexpr (PERM) {
                    // (a part that another workgroup will add up inside this launch is stored device-coherently as well)
                    if (p.tile_counters != nullptr) {
                        store_wave_tile_16B<AUX_NT_SC1, Cfg>(acc, rsrc_c, voff, p.ldc);
                    }
                    else {
                        store_wave_tile_16B<AUX_NT, Cfg>(acc, rsrc_c, voff, p.ldc);
                    }
                }
                else {
#pragma unroll
                    for (int mi = 0; mi < MI; ++mi) {
#pragma unroll
                        for (int ni = 0; ni < NI; ++ni) {
#pragma unroll
                            for (int r = 0; r < NACC; ++r) {
                                const uint32_t soff = ((mi * MT + row_of(r)) * p.ldc + ni * MT) * 4u;
                                const float v = acc[mi][ni][r];  // (bit_cast straight from a vector element reads element 0)
                                buffer_store_4B<NT>(__builtin_bit_cast(uint32_t, v), rsrc_c, voff, soff);
                            }
                        }
                    }
                }
            }
            else {
                // elements outside C get the out-of-range offset and are dropped by the buffer range check
                const __amdgpu_buffer_rsrc_t rsrc_c = make_rsrc(c_wave, OOB);
                const uint32_t voff = 4u * g * p.ldc * 4u;
                // 16 B per lane when every row of C starts on a 16 B boundary; N is then a multiple of 4, so a lane's
                // four columns are inside or outside together
                const bool vec_ok = PERM && p.ldc % 4u == 0 && ((uintptr_t)cur.c_tile & 15u) == 0;
                if (vec_ok) {
                    if constexpr (PERM) {
#pragma unroll
                        for (int mi = 0; mi < MI; ++mi) {
#pragma unroll
                            for (int nq = 0; nq < NI / 4; ++nq) {
#pragma unroll
                                for (int r = 0; r < NACC; ++r) {
                                    const int row = mi * MT + row_of(r);
                                    const uint32_t col = Cfg::template acc_col<PERM>(4 * nq, lrc);
                                    const uint32_t soff = ((uint32_t)row * p.ldc + col) * 4u;
                                    const bool inside = row < m_left && (int32_t)col < n_left;
                                    const float v0 = acc[mi][4 * nq + 0][r], v1 = acc[mi][4 * nq + 1][r];
                                    const float v2 = acc[mi][4 * nq + 2][r], v3 = acc[mi][4 * nq + 3][r];
                                    const u32x4 bits = {__builtin_bit_cast(uint32_t, v0), __builtin_bit_cast(uint32_t, v1),
                                                        __builtin_bit_cast(uint32_t, v2), __builtin_bit_cast(uint32_t, v3)};
                                    buffer_store_16B<NT>(bits, rsrc_c, inside ? voff + soff : OOB, 0u);
                                    after_wide_store();
                                }
                            }
                        }
                    }
                }
                else {
#pragma unroll
                    for (int mi = 0; mi < MI; ++mi) {
#pragma unroll
                        for (int ni = 0; ni < NI; ++ni) {
#pragma unroll
                            for (int r = 0; r < NACC; ++r) {
                                const int row = mi * MT + row_of(r);
                                const uint32_t col = Cfg::template acc_col<PERM>(ni, lrc);
                                const uint32_t soff = ((uint32_t)row * p.ldc + col) * 4u;
                                const bool inside = row < m_left && (int32_t)col < n_left;
                                const float v = acc[mi][ni][r];
                                buffer_store_4B<NT>(__builtin_bit_cast(uint32_t, v), rsrc_c, inside ? voff + soff : OOB, 0u);
                            }
                        }
                    }
                }
            }
        }

        if constexpr (!ATOMIC && !EDGE) {
            if (p.tile_counters != nullptr) {
                // This was one part of its tile (a K partition's copy, or a stream-K part).  Whoever stores a tile's last
                // part adds them all up, in their fixed order, into the caller's C.
                volatile lds_u32* const flag = (volatile lds_u32*)(lds_char*)smem;  // (the ring is no longer in use)
                // places per thread in flight: fewer for a tile that shares its CU with a second workgroup, which has
                // half of the registers
                constexpr uint32_t SUM_U = 2 * Cfg::LDS_BYTES <= 160 * 1024 ? 4 : 8;
                if constexpr (STREAM) {
                    const uint32_t tiles = p.sk.tiles, S = p.sk.splits, lefts = gridDim.x - tiles * S, t = cur.part_index;
                    uint32_t j_lo, j_hi, left_parts = 0;
                    leftover_runs_of_tile(tiles, sk_kr, lefts, t, j_lo, j_hi);
                    for (uint32_t j = j_lo; j < j_hi; ++j) {
                        left_parts += leftover_run_empty(tiles, sk_kr, lefts, j) ? 0u : 1u;
                    }
                    if (part_stored_is_it_the_last(p.tile_counters + cur.counter, S + left_parts, flag)) {
                        // main partitions' slots t * S ..., then the leftover workgroups' slots tiles * S + j + t
                        auto part = [&](uint32_t i) -> const float* {
                            uint32_t slot = t * S + i;
                            if (i >= S) {
                                uint32_t j = j_lo;
                                for (uint32_t skip = i - S;; ++j) {
                                    if (!leftover_run_empty(tiles, sk_kr, lefts, j)) {
                                        if (skip == 0) {
                                            break;
                                        }
                                        --skip;
                                    }
                                }
                                slot = tiles * S + j + t;
                            }
                            return p.c + (size_t)slot * (BM * BN);
                        };
                        const bool vec = p.ldc_final % 4u == 0 && ((uintptr_t)cur.final_tile & 15u) == 0;
                        if (vec) {
                            sum_tile_parts<BM, BN, Cfg::NTHREADS, f32x4, SUM_U, 3>(part, S + left_parts, BN, cur.final_tile, p.ldc_final, BM, BN);
                        }
                        else {
                            sum_tile_parts<BM, BN, Cfg::NTHREADS, float, 4, 3>(part, S + left_parts, BN, cur.final_tile, p.ldc_final, BM, BN);
                        }
                    }
                }
                else if (part_stored_is_it_the_last(p.tile_counters + cur.counter, cur.parts, flag)) {
                    const char* const part0 = (const char*)cur.c_tile - (size_t)cur.part_index * p.c_split_bytes;
                    auto part = [&](uint32_t i) -> const float* { return (const float*)(part0 + (size_t)i * p.c_split_bytes); };
                    const bool vec = p.ldc % 4u == 0 && p.ldc_final % 4u == 0 && p.c_split_bytes % 16u == 0 &&
                                     (((uintptr_t)part0 | (uintptr_t)cur.final_tile) & 15u) == 0;
                    if (vec) {
                        sum_tile_parts<BM, BN, Cfg::NTHREADS, f32x4, SUM_U, 3>(part, cur.parts, p.ldc, cur.final_tile, p.ldc_final, cur.m_rem, cur.n_rem);
                    }
                    else {
                        sum_tile_parts<BM, BN, Cfg::NTHREADS, float, 4, 3>(part, cur.parts, p.ldc, cur.final_tile, p.ldc_final, cur.m_rem, cur.n_rem);
                    }
                }
            }
        }

        stamp();
        if (p.timeline != nullptr) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            stamp();
        }
    }
    }  // parts
    if (p.timeline != nullptr && threadIdx.x == 0 && p.timeline_slots > 0) {
        // where this workgroup ran: the last slot holds 1 + the hardware id register (CU, shader array, shader engine) and
        // the XCC id, so that a host tool can follow one CU through the launch
        unsigned long long* const dst = p.timeline + ((size_t)blockIdx.x * p.timeline_slots + (p.timeline_slots - 1)) * 2;
        dst[0] = 1ull + __builtin_amdgcn_s_getreg((31 << 11) | 4);
        dst[1] = __builtin_amdgcn_s_getreg((31 << 11) | 20) & 15u;
    }
}

}  // namespace mi_gemm
