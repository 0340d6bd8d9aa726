// Tile family and launcher of the LDS-tiled MFMA GEMM.  Each tile configuration is instantiated in its own translation
// unit (gemm_mfma_inst_*.hip) so that the kernels compile in parallel; gemm_mfma.hip holds the planner and dispatch.
#pragma once

#include <atomic>

#include "gemm_mfma_kernel.hpp"
#include "mi_internal.hpp"

namespace mi_gemm {

// ---- tile family (xgemm_Sm90_n64/_n128/_n256 re-derived for gfx950 MFMA, 64-wide waves, 160 KB LDS).
// All tiles run 4 waves, one per SIMD, so each wave owns the largest register tile the 512-VGPR budget allows and
// LDS fragment traffic per MFMA is minimal (the chip is power-limited: fewer LDS reads means a higher clock).
// BK = 64 makes an LDS row one 128 B cache line (full-line L2 requests) and uses v_mfma_f32_16x16x32, which draws
// less power per flop than the 32x32x16 form; the 256x256 tile cannot fit a third 64 KB slot and runs the split
// ring of five 32 KB units instead.  The BK = 32 twins serve short K with the 32x32x16 form (two k-steps per slot).
//                           BM   BN   BK  WM WN slots swizzle spread MFMA split
using Cfg256x256 = TileCfg<256, 256, 64, 2, 2, 2, 1, 2, 16, true>;  // wave tile 128x128, 160 KB ring
using Cfg256x128 = TileCfg<256, 128, 64, 2, 2, 3, 1, 2, 16>;        // wave tile 128x64, 144 KB ring
using Cfg128x128 = TileCfg<128, 128, 64, 2, 2, 3, 1, 2, 16>;        // wave tile 64x64, 96 KB ring
using Cfg64x128 = TileCfg<64, 128, 64, 2, 2, 4, 1, 2, 16>;          // wave tile 32x64, 96 KB ring
using Cfg192x256 = TileCfg<192, 256, 64, 2, 2, 2, 1, 2, 16, true>;  // wave tile 96x128, 160 KB ring
// In-between heights: a problem whose tile count would leave a round of CUs part empty (or spill a few tiles into
// another round) gets a tile of 5/8 or 7/8 of the height instead.  64-deep only.
using Cfg224x256 = TileCfg<224, 256, 64, 2, 2, 2, 1, 2, 16, true>;  // wave tile 112x128, 160 KB ring
using Cfg160x256 = TileCfg<160, 256, 64, 2, 2, 2, 1, 2, 16, true>;  // wave tile 80x128, 160 KB ring
using Cfg224x128 = TileCfg<224, 128, 64, 2, 2, 3, 1, 2, 16>;        // wave tile 112x64, 132 KB ring
using Cfg160x128 = TileCfg<160, 128, 64, 2, 2, 3, 1, 2, 16>;        // wave tile 80x64, 108 KB ring
// Three quarters of the largest tile along N (N = 6144, 3072, 12288 ...): four waves stacked along M, so that a wave's
// 192 columns are three whole blocks of the 16-byte store permutation.
using Cfg256x192 = TileCfg<256, 192, 64, 4, 1, 2, 1, 2, 16, true>;  // wave tile 64x192, 160 KB ring
// 9/16 of the largest tile, same wave arrangement: 3000 x 6144 is 288 (1.1 rounds of 256 CUs), 384 or 456 tiles of
// the tiles above and 512 of this one.
using Cfg192x192 = TileCfg<192, 192, 64, 4, 1, 3, 1, 2, 16>;        // wave tile 48x192, 144 KB ring
// The one tile whose ring takes half of the LDS: two workgroups share a CU (two waves per SIMD), each with
// four waves; the DMA latency that a two-slot ring cannot hide and the epilogue are covered by the
// other workgroup's MFMAs.  Pays on many rounds of tiles with a short K, where the other tiles spend a third or more of
// a workgroup's life outside the main loop (7072 x 7352 x 1024: 139 -> 126 us); a CU that holds one such workgroup
// alone is slow (2048^3: 34 us against 22).
using Cfg192x128 = TileCfg<192, 128, 64, 2, 2, 2, 1, 2, 16>;        // wave tile 96x64, 80 KB ring
// Three quarters of the 128x128 tile (wave tile 48x64): 768 x 3072 is 144 tiles of 128x128 (56 % of 256 CUs), 288 of
// 64x128 (a round and an eighth) and 192 of this one.
using Cfg96x128 = TileCfg<96, 128, 64, 2, 2, 3, 1, 2, 16>;          // 84 KB ring
using Cfg256x256k32 = TileCfg<256, 256, 32, 2, 2, 4, 1, 2>;         // 128 KB ring
using Cfg256x128k32 = TileCfg<256, 128, 32, 2, 2, 5, 1, 2>;         // 120 KB ring
using Cfg128x128k32 = TileCfg<128, 128, 32, 2, 2, 6, 1, 2>;         // 96 KB ring
using Cfg64x128k32 = TileCfg<64, 128, 32, 2, 2, 8, 1, 2>;           // 96 KB ring
using Cfg192x256k32 = TileCfg<192, 256, 32, 2, 2, 4, 1, 2>;         // 112 KB ring

// Problem as the kernel sees it: C[M,N] row-major = A[M,K] * B[N,K]^T, both operands K-contiguous.
struct Canonical {
    const void* a;
    const void* b;
    float* c;
    uint32_t M, N, K;
    uint32_t lda, ldb;  // row pitches of A and B in elements (K, or K rounded up to 8 for a re-packed operand)
    uint32_t ldc = 0;   // row pitch of C in floats; 0 = N (a sub-problem of a larger C has the larger one's pitch)
    // independent problems of this shape and the distance in bytes from one to the next (xgemm_Sm90.py:45-48, `L`)
    uint32_t batches = 1;
    uint64_t a_batch_bytes = 0, b_batch_bytes = 0, c_batch_bytes = 0;
    // K partitions: 0 = they meet in C through atomics; otherwise partition s writes its own copy of C at
    // c + s * c_split_bytes (see GemmArgs::c_split_bytes)
    uint64_t c_split_bytes = 0;
    // stream-K: `c` is the parts buffer (see gemm_tn_kernel, STREAM), this is the grid (one workgroup per CU) and `sk`
    // the way the tail tiles' K tiles are dealt to it
    uint32_t stream_k_workgroups = 0;
    GemmArgs::StreamKShape sk{};
    // a plain launch over the first `first_tiles_only` tiles of the raster order only (0: all tiles): the whole rounds
    // of a problem whose last tiles run as a stream-K launch
    uint32_t first_tiles_only = 0;
    // parts summed inside the launch (see GemmArgs::tile_counters): the arrival counters (null: not), the caller's C, its row
    // pitch (0 = N) and its batch stride
    uint32_t* tile_counters = nullptr;
    float* c_final = nullptr;
    uint32_t ldc_final = 0;
    uint64_t c_final_batch_bytes = 0;
    // 1: A, 2: B is read once by the launch and too large to stay cached (see gemm_tn_kernel, ONCE); the launcher
    // ignores it where no such build exists
    int read_once = 0;
    // a sub-problem of a problem whose A (bit 0) or B (bit 1) is larger than the memory-side cache: the launches of one
    // call stream that operand from DRAM between them, whatever the size of this launch's share of it
    int parent_beyond_cache = 0;
    // diagnostic timeline request (see GemmArgs::timeline); null in normal use
    unsigned long long* timeline = nullptr;
    uint32_t timeline_slots = 0;
    uint32_t timeline_workgroups = 0;   // capacity of the stamp buffer in workgroups
    uint32_t* launched_workgroups = nullptr;  // out: grid size of the launch
    // set the kernel's attributes (the dynamic LDS opt-in) and launch nothing: see mi_matmul_mfma_prepare
    bool attributes_only = false;
};

constexpr uint32_t GROUP_M = 4;  // tile-rows per raster group (see map_work)
constexpr uint32_t K_ROTATE_TILES = 37;  // K tiles between the starting points of consecutive XCDs' walks (see launch_cfg)

template <int DTYPE, typename Cfg, bool ATOMIC, bool EDGE, bool STREAM = false, int ONCE = 0>
int launch_kernel(const GemmArgs& args, uint32_t grid, hipStream_t stream, bool attributes_only)
{
    // dynamic LDS above the 64 KB default needs an opt-in once per device (gemm/gemm_sm80.cu:473-475)
    static std::atomic<bool> attr_set[64];  // per kernel instantiation; setting the attribute twice is harmless
    int dev = 0;
    MI_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= 64 || !attr_set[dev].load(std::memory_order_acquire)) {
        MI_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_tn_kernel<DTYPE, Cfg, ATOMIC, EDGE, STREAM, ONCE>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES));
        if (dev >= 0 && dev < 64) {
            attr_set[dev].store(true, std::memory_order_release);
        }
    }
    if (attributes_only) {
        return MI_OK;
    }
    hipLaunchKernelGGL((gemm_tn_kernel<DTYPE, Cfg, ATOMIC, EDGE, STREAM, ONCE>), dim3(grid), dim3(Cfg::NTHREADS),
                       Cfg::LDS_BYTES, stream, args);
    MI_CHECK_LAUNCH();
    return MI_OK;
}

// Launch one tile configuration.  `edge`: M, N or K do not divide the tile (the bounds-checked build is used).
template <int DTYPE, typename Cfg>
int launch_cfg(const Canonical& c, uint32_t k_splits, bool edge, hipStream_t stream)
{
    GemmArgs args;
    args.a = c.a;
    args.b = c.b;
    args.c = c.c;
    args.M = c.M;
    args.N = c.N;
    args.K = c.K;
    args.lda = c.lda;
    args.ldb = c.ldb;
    args.ldc = c.ldc ? c.ldc : c.N;
    args.tiles_m = (c.M + Cfg::BM - 1) / Cfg::BM;
    args.tiles_n = (c.N + Cfg::BN - 1) / Cfg::BN;
    args.k_splits = k_splits;
    const uint32_t k_tiles = (c.K + Cfg::BK - 1) / Cfg::BK;
    args.k_tiles_per_split = (k_tiles + k_splits - 1) / k_splits;
    args.group_m = GROUP_M;
    // K partitions of rows whose stride is a large power of two (the dense layout of a deep power-of-two K) all sit at
    // the same offset of their rows modulo that stride, and every row's bytes at one K offset map to the same few
    // memory channels: when all XCDs walk K from the start of their partition the launch queues up on those channels
    // (2048 x 2048 x 65536 in four partitions: 2660 core cycles per K tile against 2320 with rows padded by 128 B).
    // Starting each XCD's walk 37 K tiles further into its partition spreads them: measured 0.97 of the run time on
    // that problem, 0.88 on 2048 x 1024 x 65536 in eight partitions, 0.92 on 1024 x 1024 x 131072 in sixteen, within
    // 1 % either way on other power-of-two strides; on strides that are not powers of two it can cost up to 6 %.
    const uint64_t row_bytes = (uint64_t)c.lda * 2;
    const bool aliasing_rows = c.lda == c.ldb && row_bytes >= 65536 && (row_bytes & (row_bytes - 1)) == 0;
    args.k_rotate = (k_splits > 1 && !edge && aliasing_rows) ? K_ROTATE_TILES : 0;
    args.timeline = c.timeline;
    args.timeline_slots = c.timeline_slots;
    args.batches = c.batches;
    args.a_batch_bytes = c.a_batch_bytes;
    args.b_batch_bytes = c.b_batch_bytes;
    args.c_batch_bytes = c.c_batch_bytes;
    args.c_split_bytes = k_splits > 1 ? c.c_split_bytes : 0;
    // (K partitions' copies of C, or stream-K parts; a sum inside the launch needs one or the other, and whole tiles: the
    // range-checked build does not carry it, see run_mfma)
    const bool sums_inside = c.tile_counters != nullptr && c.c_final != nullptr && !edge && (args.c_split_bytes != 0 || c.stream_k_workgroups > 0);
    args.tile_counters = sums_inside ? c.tile_counters : nullptr;
    args.c_final = c.c_final;
    args.ldc_final = c.ldc_final ? c.ldc_final : c.N;
    args.c_final_batch_bytes = c.c_final_batch_bytes;
    // every partition must own at least one K tile
    if ((uint64_t)args.k_tiles_per_split * (k_splits - 1) >= k_tiles) {
        return MI_ERR_UNSUPPORTED;
    }
    uint64_t items = (uint64_t)args.tiles_m * args.tiles_n * k_splits * c.batches;
    if (items == 0 || items > 0x7fffffffull) {
        return MI_ERR_UNSUPPORTED;
    }
    if (c.first_tiles_only > 0) {
        if (k_splits != 1 || c.batches != 1 || c.first_tiles_only > items) {
            return MI_ERR_UNSUPPORTED;
        }
        items = c.first_tiles_only;
    }
    const bool stream_k = c.stream_k_workgroups > 0;
    args.sk = c.sk;
    if (stream_k) {
        // whole tiles, one problem; the shape must be one that the host's stream_k_shape() makes: tail tiles inside the
        // tile grid, fewer of them than workgroups, main partitions of at least one K tile each, leftover workgroups
        // exactly when K tiles are left over
        const uint64_t g = c.stream_k_workgroups, tiles = (uint64_t)args.tiles_m * args.tiles_n;
        const GemmArgs::StreamKShape& sk = c.sk;
        if (edge || k_splits != 1 || c.batches != 1 || Cfg::BK != 64 || sk.tiles == 0 || sk.tiles >= g ||
            (uint64_t)sk.first_tile + sk.tiles > tiles || sk.splits != g / sk.tiles || sk.main_k > k_tiles ||
            sk.main_k < sk.splits || ((g - (uint64_t)sk.tiles * sk.splits == 0) != (sk.main_k == k_tiles)) ||
            c.first_tiles_only > 0) {
            return MI_ERR_UNSUPPORTED;
        }
        args.ldc = Cfg::BN;
    }
    const uint32_t grid = stream_k ? c.stream_k_workgroups : (uint32_t)items;
    if (c.timeline != nullptr) {
        if (grid > c.timeline_workgroups) {
            return MI_ERR_WORKSPACE;
        }
        if (c.launched_workgroups != nullptr) {
            *c.launched_workgroups = grid;
        }
    }
    // One workgroup per work item: every ring in the family takes more than half of the LDS, so a CU holds one
    // workgroup at a time and the hardware dispatcher hands it the next one as soon as the previous one has ended.
    if constexpr (Cfg::BK == 64) {
        if (stream_k) {
            return launch_kernel<DTYPE, Cfg, false, false, true>(args, grid, stream, c.attributes_only);
        }
    }
    if (k_splits > 1 && c.c_split_bytes == 0) {
        if constexpr (Cfg::BK == 64) {
            if (!edge && c.read_once == 1 && c.batches == 1) {
                return launch_kernel<DTYPE, Cfg, true, false, false, 1>(args, grid, stream, c.attributes_only);
            }
            if (!edge && c.read_once == 2 && c.batches == 1) {
                return launch_kernel<DTYPE, Cfg, true, false, false, 2>(args, grid, stream, c.attributes_only);
            }
        }
        return edge ? launch_kernel<DTYPE, Cfg, true, true>(args, grid, stream, c.attributes_only)
                    : launch_kernel<DTYPE, Cfg, true, false>(args, grid, stream, c.attributes_only);
    }
    if constexpr (Cfg::BK == 64) {
        // (which launches qualify is the host planner's decision: read_once_operand)
        if (!edge && c.read_once == 1 && c.batches == 1) {
            return launch_kernel<DTYPE, Cfg, false, false, false, 1>(args, grid, stream, c.attributes_only);
        }
        if (!edge && c.read_once == 2 && c.batches == 1) {
            return launch_kernel<DTYPE, Cfg, false, false, false, 2>(args, grid, stream, c.attributes_only);
        }
    }
    return edge ? launch_kernel<DTYPE, Cfg, false, true>(args, grid, stream, c.attributes_only)
                : launch_kernel<DTYPE, Cfg, false, false>(args, grid, stream, c.attributes_only);
}

#define MI_GEMM_DECLARE_CFG(Cfg)                                                                    \
    extern template int launch_cfg<MI_F16, Cfg>(const Canonical&, uint32_t, bool, hipStream_t);    \
    extern template int launch_cfg<MI_BF16, Cfg>(const Canonical&, uint32_t, bool, hipStream_t);
#define MI_GEMM_INSTANTIATE_CFG(Cfg)                                                         \
    template int launch_cfg<MI_F16, Cfg>(const Canonical&, uint32_t, bool, hipStream_t);    \
    template int launch_cfg<MI_BF16, Cfg>(const Canonical&, uint32_t, bool, hipStream_t);

// ---- the one table of the tile family.  Everything that depends on which tiles exist is generated from it: tile
// dimensions, names, the dispatch to a configuration's launcher, the planner's cost constants, the exported
// mi_tile_count / mi_tile_name / mi_tile_shape that bindings, tests and the host driver enumerate.  Adding a tile is a
// `using Cfg... = TileCfg<...>` line above, a row here (plus a line in MI_TILE_TWINS if it has a 32-deep twin), an
// enumerator in mi_gemm.h and a gemm_mfma_inst_*.hip that instantiates it.
//
// Columns: ABI code, name, 64-deep configuration, 32-deep twin (or NoTwin: a K that is only a multiple of 32 then runs
// the range-checked build with a half-empty last slot), then the planner's measured constants on MI355X
// at the clock the chip sustains under MFMA load:
//   us_k64      main-loop time per 64-deep K step with every CU busy (of a pair of workgroups for a tile whose ring
//               lets two share a CU)
//   fixed_us    per-workgroup cost outside the main loop (dispatch, ring fill, epilogue), a whole round ending together
//   short_us    the same for K <= 384 and at least two rounds of the largest tile, where a launch is a stream of C stores
//               (measured on 8192^2 x 64..384, 16384^2 x 128, 32768 x 65536 x 48)
//   per_cu      workgroups that share a CU
//   alone_k64 / alone_us   us_k64 / fixed_us of a workgroup that has its CU to itself (differs for per_cu = 2 only)
//   max_k       the planner leaves the tile to callers that force it above this K (0: no limit).  192x128, two per CU,
//               wins where workgroups are short-lived: ahead by 13 % at K = 512 and 1024, level at 1408, behind by 8
//               to 10 % at 1536 and 2048 (3000 x 11008 x 4096: 253 us against 214 us)
#define MI_TILE_TABLE(ROW)                                                                                          \
    ROW(MI_TILE_256x256, "256x256", Cfg256x256, Cfg256x256k32, 1.33, 15.0, 17.4, 1, 1.33, 15.0, 0)             \
    ROW(MI_TILE_256x128, "256x128", Cfg256x128, Cfg256x128k32, 0.73, 10.0, 7.2, 1, 0.73, 10.0, 0)              \
    ROW(MI_TILE_128x128, "128x128", Cfg128x128, Cfg128x128k32, 0.44, 7.0, 3.0, 1, 0.44, 7.0, 0)                \
    ROW(MI_TILE_64x128, "64x128", Cfg64x128, Cfg64x128k32, 0.25, 6.0, 2.8, 1, 0.25, 6.0, 0)                    \
    ROW(MI_TILE_192x256, "192x256", Cfg192x256, Cfg192x256k32, 1.03, 13.0, 8.5, 1, 1.03, 13.0, 0)              \
    ROW(MI_TILE_224x256, "224x256", Cfg224x256, NoTwin, 1.16, 13.5, 13.0, 1, 1.16, 13.5, 0)                         \
    ROW(MI_TILE_160x256, "160x256", Cfg160x256, NoTwin, 0.86, 12.0, 7.5, 1, 0.86, 12.0, 0)                          \
    ROW(MI_TILE_224x128, "224x128", Cfg224x128, NoTwin, 0.64, 9.5, 6.5, 1, 0.64, 9.5, 0)                            \
    ROW(MI_TILE_160x128, "160x128", Cfg160x128, NoTwin, 0.48, 8.5, 4.0, 1, 0.48, 8.5, 0)                            \
    ROW(MI_TILE_256x192, "256x192", Cfg256x192, NoTwin, 1.02, 13.0, 10.0, 1, 1.02, 13.0, 0)                         \
    ROW(MI_TILE_192x192, "192x192", Cfg192x192, NoTwin, 0.755, 18.5, 8.0, 1, 0.755, 18.5, 0)                        \
    /* two per CU: the times of such a pair, measured on 7072 x 7352 x 1024, 6144 x 4096 x 1024, 8192^2 x 2048 and    \
       8192^2 x 256 (126, 53, 246, 65 us) */                                                                        \
    ROW(MI_TILE_192x128, "192x128", Cfg192x128, NoTwin, 1.0, 9.0, 8.0, 2, 0.85, 12.0, 1536)                         \
    ROW(MI_TILE_96x128, "96x128", Cfg96x128, NoTwin, 0.36, 6.5, 2.9, 1, 0.36, 6.5, 0)
#define MI_TILE_TWINS(X) X(Cfg256x256k32) X(Cfg256x128k32) X(Cfg128x128k32) X(Cfg64x128k32) X(Cfg192x256k32)

using LaunchFn = int (*)(const Canonical&, uint32_t, bool, hipStream_t);

struct NoTwin {};
template <typename Cfg>
struct Launchers {
    static constexpr LaunchFn f16 = &launch_cfg<MI_F16, Cfg>, bf16 = &launch_cfg<MI_BF16, Cfg>;
};
template <>
struct Launchers<NoTwin> {
    static constexpr LaunchFn f16 = nullptr, bf16 = nullptr;
};

struct TileRow {
    int code;
    const char* name;
    uint32_t bm, bn;
    LaunchFn deep[2];  // 64-deep configuration, by element type (MI_F16, MI_BF16)
    LaunchFn twin[2];  // 32-deep twin, or null
    double us_k64, fixed_us, short_us;
    int per_cu;
    double alone_k64, alone_us;
    uint32_t max_k;
};

}  // namespace mi_gemm
