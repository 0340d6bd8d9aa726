// Host side of the LDS-tiled MFMA GEMM: layout canonicalisation, support predicate, tile / K-mode planning and
// launch.  Counterpart of the reference dispatchers and launchers (gemm/gemm_sm80.cu:467-550,
// gemm/gemm_sm90.cu:1200-1360).
#include "gemm_mfma_launch.hpp"

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

namespace mi_gemm {

#define MI_ROW_DECLARE(code, name, Cfg, ...) MI_GEMM_DECLARE_CFG(Cfg)
MI_TILE_TABLE(MI_ROW_DECLARE)
MI_TILE_TWINS(MI_GEMM_DECLARE_CFG)
#undef MI_ROW_DECLARE

// The tile family, indexed by ABI code - 1 (code 0 is MI_TILE_AUTO).
#define MI_ROW_ENTRY(code, name, Cfg, Twin, us_k64, fixed_us, short_us, per_cu, alone_k64, alone_us, max_k) \
    TileRow{code,                                                                                           \
            name,                                                                                           \
            Cfg::BM,                                                                                        \
            Cfg::BN,                                                                                        \
            {Launchers<Cfg>::f16, Launchers<Cfg>::bf16},                                                    \
            {Launchers<Twin>::f16, Launchers<Twin>::bf16},                                                  \
            us_k64,                                                                                         \
            fixed_us,                                                                                       \
            short_us,                                                                                       \
            per_cu,                                                                                         \
            alone_k64,                                                                                      \
            alone_us,                                                                                       \
            max_k},
// (not const: the two leading planner constants of a row can be replaced at run time, see mi_tile_set_planner_constants)
static TileRow TILES[] = {MI_TILE_TABLE(MI_ROW_ENTRY)};
#undef MI_ROW_ENTRY
constexpr int TILE_ROWS = sizeof(TILES) / sizeof(TILES[0]);
static_assert(TILE_ROWS == MI_TILE_COUNT_ - 1, "one table row per tile code of the ABI");
// Counts the replacements of planner constants, so that answers remembered under older ones are not given again.
static std::atomic<uint32_t> planner_constants_generation{0};

// The row of a tile code, or null (MI_TILE_AUTO and unknown codes have none).
static const TileRow* tile_row(int tile)
{
    if (tile < 1 || tile > TILE_ROWS || TILES[tile - 1].code != tile) {
        return nullptr;
    }
    return &TILES[tile - 1];
}

struct TileDims {
    uint32_t bm, bn, bk;
};

// K depth of a ring slot for this problem: 64 (one LDS row = one 128 B cache line) unless K is short and only a
// multiple of 32, where the 32-deep twins avoid a half-empty last slot.
static uint32_t slot_depth(uint32_t K)
{
    if (K % 64 == 0) {
        return 64;
    }
    return (K % 32 == 0 && K < 512) ? 32 : 64;
}

static bool tile_dims(int tile, uint32_t K, TileDims& d)
{
    const TileRow* const row = tile_row(tile);
    if (row == nullptr) {
        return false;
    }
    d = {row->bm, row->bn, row->twin[0] != nullptr ? slot_depth(K) : 64u};
    return true;
}

static uint32_t ceil_div(uint32_t a, uint32_t b)
{
    return (a + b - 1) / b;
}

// One input matrix as `rows` x K: element (r, k) is ptr[r*K + k] when K-contiguous, else ptr[k*rows + r].
struct Operand {
    const void* ptr;
    uint32_t rows;
    bool k_contiguous;
};

// The kernel reads an operand in place if it is K-contiguous with whole, aligned 16 B chunks per row.
static bool usable_in_place(const Operand& op, uint32_t K)
{
    return op.k_contiguous && K % 8 == 0 && (uintptr_t)op.ptr % 16 == 0;
}

static size_t round_up(size_t x, size_t to)
{
    return (x + to - 1) / to * to;
}

// A problem made ready for the kernel: C[M,N] row-major = A[M,K] * B[N,K]^T.
// gemm/gemm_sm80.cu:516-539: a column-major C is a row-major C^T = B^T A^T, i.e. the same kernel with the operands
// (and M, N) swapped.  Operands the kernel cannot read in place are re-packed into the workspace first.
struct Prepared {
    Canonical c;
    Operand a_src, b_src;      // the canonical A and B as the caller stored them
    bool repack_a, repack_b;
    size_t ws_a, ws_b;         // workspace offsets of the re-packed copies
    size_t ws_bytes;           // 0: no workspace needed
};

static Prepared prepare(const mi_gemm_tensors& t)
{
    Prepared p;
    Operand a{t.a, t.M, !t.a_col_major}, b{t.b, t.N, t.b_col_major != 0};
    uint32_t M = t.M, N = t.N;
    if (t.c_col_major) {
        const Operand tmp = a;
        a = b;
        b = tmp;
        M = t.N;
        N = t.M;
    }
    p.a_src = a;
    p.b_src = b;
    p.repack_a = !usable_in_place(a, t.K);
    p.repack_b = !usable_in_place(b, t.K);
    const uint32_t kp = (uint32_t)round_up(t.K, 8);
    p.ws_a = 0;
    p.ws_b = p.repack_a ? round_up((size_t)M * kp * 2, 256) : 0;
    p.ws_bytes = p.ws_b + (p.repack_b ? round_up((size_t)N * kp * 2, 256) : 0);
    p.c = {a.ptr, b.ptr, t.c, M, N, t.K, p.repack_a ? kp : t.K, p.repack_b ? kp : t.K};
    return p;
}

// Limits that hold whatever the tile: a 256-row panel must stay below the 2 GiB reach of a buffer descriptor's
// 32-bit offsets, C must be dword aligned, and the range-checked build counts the rows that are left in 32-bit
// signed integers.  (For a column-major C the canonical M is the caller's N: both sides are covered.)
static bool problem_fits(const Canonical& c)
{
    return (uintptr_t)c.c % 4 == 0 && c.K < (1u << 21) && c.N < (1u << 21) && c.M < (1u << 31);
}

static bool tile_fits(const Canonical& c, int tile, uint32_t k_splits)
{
    TileDims d;
    if (!tile_dims(tile, c.K, d)) {
        return false;
    }
    // every K partition (ceil(k_tiles / k_splits) tiles each, the last one shorter) must own at least one tile
    const uint32_t k_tiles = ceil_div(c.K, d.bk);
    return k_splits >= 1 && (uint64_t)ceil_div(k_tiles, k_splits) * (k_splits - 1) < k_tiles;
}

// The bounds-checked build also takes a C that is not 16-byte aligned (the plain build stores 16 B per lane).
static bool needs_edge(const Canonical& c, const TileDims& d)
{
    return c.M % d.bm || c.N % d.bn || c.K % d.bk || (uintptr_t)c.c % 16 || c.c_batch_bytes % 16 || c.c_split_bytes % 16 ||
           c.ldc % 4;
}

struct Plan {
    int tile;
    int k_mode;  // MI_K_OUTPUT_STATIONARY, MI_K_SPLIT (atomics), MI_K_SPLIT_REDUCE (copies of C, then a sum), MI_K_STREAM
    uint32_t k_splits;
    uint32_t workgroups;  // MI_K_STREAM: the grid
    double cost_us;       // the planner's estimate
};

// Which operand, if any, the launch reads exactly once while it is too large to be found again in the 256 MB
// memory-side cache: B when the problem is one tile high, A when it is one tile wide (0: neither, 1: A, 2: B).
// Such an operand is streamed non-temporal (see gemm_tn_kernel, ONCE) so that it does not evict the other one.
constexpr uint64_t MEMORY_SIDE_CACHE = 256ull << 20;

// Which operands come from DRAM on every launch, also in a loop: bit 0 A, bit 1 B.
static int beyond_cache(const Canonical& c)
{
    return c.parent_beyond_cache | ((uint64_t)c.M * c.lda * 2 > MEMORY_SIDE_CACHE ? 1 : 0) |
           ((uint64_t)c.N * c.ldb * 2 > MEMORY_SIDE_CACHE ? 2 : 0);
}

static int read_once_operand(const Canonical& c, const Plan& plan)
{
    TileDims d;
    if (!tile_dims(plan.tile, c.K, d) || d.bk != 64 || needs_edge(c, d) || c.batches != 1 || plan.k_mode == MI_K_STREAM) {
        return 0;  // builds that have no non-temporal twin
    }
    const int big = beyond_cache(c);
    if (c.M <= d.bm && (big & 2)) {
        return 2;
    }
    if (c.N <= d.bn && (big & 1)) {
        return 1;
    }
    return 0;
}

// Bytes of workspace that the K partitions' private copies of C take.
static size_t partial_bytes(const Canonical& c, uint32_t k_splits)
{
    return (size_t)c.M * c.N * 4 * k_splits * c.batches;
}

// How a stream-K call (MI_K_STREAM) is laid out, the role of gemm/gemm_sm90.cu:1009-1030: the whole rounds of tiles
// (`full_tiles`, a multiple of the workgroups one round holds) run the plain output-stationary kernel and store
// straight into C; the `r` tiles that are left, fewer than a round, run as one stream-K launch of `g` workgroups (see
// gemm_tn_kernel, STREAM) whose parts a last kernel sums into C.
struct StreamKLayout {
    uint32_t g;            // workgroups of the stream-K launch: one round
    uint32_t full_tiles;   // tiles of the raster order's head that run output stationary
    uint32_t r;            // tail tiles, 0 < r < g
    uint32_t splits;       // S = g / r main partitions per tail tile
    uint32_t lefts;        // L = g - r * S leftover workgroups
    uint32_t k_tiles;      // KT
    uint32_t main_k;       // Km: K tiles per tile covered by the main partitions (KT when there are no leftovers)
    uint32_t bm, bn;
    uint32_t slots() const { return r * splits + (lefts ? lefts + r - 1 : 0); }
    size_t bytes() const { return (size_t)slots() * bm * bn * 4; }
    uint32_t main_len() const { return (main_k + splits - 1) / splits; }                               // longest main partition
    uint32_t left_len() const { return lefts ? (uint32_t)(((uint64_t)r * (k_tiles - main_k) + lefts - 1) / lefts) : 0; }
    uint32_t left_parts() const  // most parts one leftover workgroup stores
    {
        const uint32_t kr = k_tiles - main_k;
        return lefts ? (left_len() + kr - 2) / kr + 1 : 0;
    }
};

// Stream-K needs whole tiles, one problem, a C that takes 16-byte stores, and a tile count that does not fill whole
// rounds.  Returns false when the mode does not apply.
static bool stream_k_layout(const Canonical& c, int tile, int cus, StreamKLayout& sk)
{
    TileDims d;
    const TileRow* const row = tile_row(tile);
    if (row == nullptr || !tile_dims(tile, c.K, d) || d.bk != 64 || c.M % d.bm || c.N % d.bn || c.K % 64 || c.batches != 1 ||
        (uintptr_t)c.c % 16 || c.ldc % 4 || c.K == 0) {
        return false;
    }
    const uint64_t tiles = (uint64_t)(c.M / d.bm) * (c.N / d.bn);
    if (tiles == 0 || tiles > 0x7fffffffull) {
        return false;
    }
    sk.g = (uint32_t)cus * (uint32_t)row->per_cu;
    sk.r = (uint32_t)(tiles % sk.g);
    sk.full_tiles = (uint32_t)(tiles - sk.r);
    sk.k_tiles = c.K / 64;
    sk.bm = d.bm;
    sk.bn = d.bn;
    if (sk.r == 0) {
        return false;  // whole rounds only: nothing to stream
    }
    sk.splits = sk.g / sk.r;
    sk.lefts = sk.g - sk.r * sk.splits;
    const uint32_t even_run = (uint32_t)((uint64_t)sk.r * sk.k_tiles / sk.g);  // K tiles per workgroup, rounded down
    sk.main_k = sk.lefts ? sk.splits * even_run : sk.k_tiles;
    // a run of at least four K tiles (less is not worth a launch of its own and a summing pass)
    return sk.main_k / sk.splits >= 4;
}

static GemmArgs::StreamKShape stream_k_shape(const StreamKLayout& sk)
{
    return GemmArgs::StreamKShape{sk.full_tiles, sk.r, sk.splits, sk.main_k};
}

// Estimated run time of a stream-K call in microseconds (constants as in plan_cost).
static double stream_k_cost(const Canonical& c, int tile, const StreamKLayout& sk)
{
    const TileRow& row = *tile_row(tile);
    const double tile_bytes = 4.0 * sk.bm * sk.bn, area = tile_bytes / 262144.0;
    double total = 0.0;
    if (sk.full_tiles > 0) {
        // the whole rounds, as a plain launch of so many rounds is priced, and the gap between two launches
        total += (double)(sk.full_tiles / sk.g) * (sk.k_tiles * row.us_k64 + row.fixed_us) + 3.0;
    }
    // The stream-K launch: every workgroup of the main partitions walks main_len K tiles in step with its
    // neighbours (priced like split K); a leftover workgroup walks as many, in up to left_parts pieces, each with its
    // own ring fill and tile store (7 us per 256 x 256 tile when a round of them ends together, 2 us of ring fill).
    const double longest = sk.main_len() > sk.left_len() ? sk.main_len() : sk.left_len();
    const double extra_parts = sk.left_parts() > 1 ? sk.left_parts() - 1.0 : 0.0;
    // The leftover workgroups sit at unrelated K offsets and share no panel: every K tile of theirs is fetched once per
    // workgroup, through the fabric, at the 3.3 to 3.8 TB/s measured when they are many (1536 x 2816 x 65536: 124 of 256
    // workgroups of 256x128 tiles, 883 us; 160 of 512 of 192x128, 705 us).  With few of them the matrix cores set the pace.
    const double left_fetch_us = (double)sk.lefts * sk.left_len() * (sk.bm + sk.bn) * 128.0 / 3.5e6;
    const double loop_us = longest * row.alone_k64 > left_fetch_us ? longest * row.alone_k64 : left_fetch_us;
    total += loop_us + row.alone_us + extra_parts * (7.0 * area + 2.0);
    // then one pass reads every part and writes the tail tiles of C (2.5 us + 6 TB/s, as for summed K partitions)
    total += 2.5 + ((double)sk.slots() + sk.r) * tile_bytes / 6.0e6;
    // streaming floor, as in plan_cost: every byte of A, B and C crosses HBM at least once
    const double M = (double)c.M, N = (double)c.N, K = (double)c.K;
    const double hbm_us = (2.0 * (M * K + N * K) + 4.0 * M * N) / 5.0e6;
    return (total > hbm_us ? total : hbm_us) * (1.0 + 1e-3);
}

// Estimated run time of a plan in microseconds.  One workgroup per CU for every tile (the rings fill the LDS).
// Per-tile constants are measured main-loop times per 64-deep K step and fixed per-workgroup costs (dispatch, ring
// fill, epilogue) on MI355X at the clock the chip sustains under MFMA load.  Partial edge tiles cost like full ones.
static double plan_cost(const Canonical& c, int tile, uint32_t k_splits, bool reduce, bool versus_reduce, int cus)
{
    TileDims d;
    tile_dims(tile, c.K, d);
    // (two workgroups share a CU when the ring is half of the LDS: a round then has two places per CU and the table
    // holds the times of such a pair; a CU that holds one alone runs at alone_k64)
    const TileRow& row = *tile_row(tile);
    double us_per_k64 = row.us_k64, fixed_us = row.fixed_us;
    const double places = (double)row.per_cu * cus;  // workgroups that run side by side in one round
    if (d.bk == 32) {
        us_per_k64 *= 1.1;  // half-line L2 requests and twice the barriers
    }
    // A row of a K tile is 128 bytes.  When rows of A or B do not start on 128-byte boundaries (K not a multiple of
    // 64, or a misaligned operand), each one straddles two cache lines and the DMA asks the L2 for twice as many
    // lines.  Measured on 7680 x 6144 x 12368 against K = 12352: +15 % for 256x256, +18 / 22 / 24 % for the 224 / 192 /
    // 160-row tiles, +27 to 47 % for the 128-column tiles.
    const bool straddles = (c.lda * 2) % 128 || (c.ldb * 2) % 128 || (uintptr_t)c.a % 128 || (uintptr_t)c.b % 128;
    if (straddles && d.bk == 64) {
        // (narrow tiles: forced plans on five shapes with K = 3432 ... 13720 ran at 1.2 to 1.5 times what a factor of
        // 1.38 gave for 64 x 128 (hence 1.9, also for 96 x 128: 2048 x 856 x 3672 ran 35 us against 31 priced at 1.5), at 1.0 to 1.25 times for 128 x 128 and 160 x 128)
        us_per_k64 *= d.bn >= 192 ? 1.15 + 0.09 * (256 - (int)d.bm) / 96.0 : d.bm <= 96 ? 1.9 : 1.5;
    }
    else if (needs_edge(c, d)) {
        us_per_k64 *= 1.05;  // per-instruction bounds bookkeeping
    }
    // Dense rows three times a power of two apart (K = 49152, 98304 with 16-bit elements; the HBM stacks are twelve dies
    // high, which puts a factor of three into the address map) make the panels that workgroups fetch side by side collide
    // in memory.  Measured against their estimates on twelve such shapes: plans of the 128-column tiles run 1.4 to 1.56
    // times as long and the 192 x 192 tile 1.2 to 1.33 times; the 256- and 192-column tiles of 160 rows and more run
    // 0.9 to 1.29 times as long with no pattern that a constant would capture (pricing the 256 x 256 tile up, which
    // is off most often, only hands its problems to tiles that are hit harder), so those keep their estimates.
    if (c.lda == c.ldb && ((uint64_t)c.lda * 2) % 98304 == 0 && c.K >= 32768) {
        us_per_k64 *= d.bn <= 128 ? 1.45 : (d.bm == 192 && d.bn == 192) ? 1.25 : 1.0;
    }
    const double items = (double)ceil_div(c.M, d.bm) * ceil_div(c.N, d.bn) * k_splits * c.batches;
    double waves = __builtin_ceil(items / places);
    const double k64_steps = __builtin_ceil((double)ceil_div(c.K, d.bk) / k_splits) * (d.bk / 64.0);
    const double big_items = (double)ceil_div(c.M, 256) * ceil_div(c.N, 256) * c.batches;
    if (k64_steps <= 6.0 && big_items >= 2.0 * cus && k_splits == 1) {
        // Short K and at least two rounds of the largest tile: the launch is a stream of C stores (5.4 TB/s at best).
        // Measured per-workgroup cost on 8192 x 8192 x 64..384, 16384 x 16384 x 128 and 32768 x 65536 x 48: the
        // 256 x 256 tile's store burst is overlapped by nothing, smaller tiles interleave stores and loads across
        // the CUs, and rounds blur into each other.
        fixed_us = row.short_us;
        waves = items / places;
    }
    else if (places == cus && waves > 4.0) {
        // Many rounds: the CUs drift out of step and their store bursts no longer collide (a workgroup's epilogue takes
        // 2 us when the memory system is free, 7 us on average when a whole round ends together).  Measured per round
        // with the 256 x 256 tile: 24 steps + 8.7 us over 18 rounds (12288 x 24576 x 1536), 13 steps + 8.6 us over 78
        // rounds (32768 x 40016 x 816), against + 14 to 15 us over four rounds.
        const double drift = (waves - 4.0) / 14.0;
        fixed_us *= 1.0 - 0.4 * (drift < 1.0 ? drift : 1.0);
    }
    double total = waves * (k64_steps * us_per_k64 + fixed_us);
    if (waves == __builtin_ceil(items / places)) {
        // Whole rounds, then a last round that leaves CUs idle.  The chip is power-limited in the main loop, so the
        // fewer CUs are busy the faster each one runs: measured per-K-step time of a single round at 25 / 50 / 75 /
        // 100 % of the CUs, as a fraction of the full-chip time: 0.73 / 0.77 / 0.87 / 1 (every tile within 0.03).
        const double full_rounds = __builtin_floor(items / places);
        const double fill = items / places - full_rounds;
        if (fill > 0.0) {
            const double over = fill > 0.25 ? (fill - 0.25) / 0.75 : 0.0;
            const double speed = 0.73 + 0.27 * over * over;
            total = full_rounds * (k64_steps * us_per_k64 + fixed_us) +
                    k64_steps * us_per_k64 * speed + fixed_us * (0.75 + 0.25 * fill);
        }
    }
    if (k_splits > 1 && reduce) {
        // every partition stores its tile like an output-stationary one (part of fixed_us); then one pass reads the
        // k_splits copies and writes C.  From kernel traces of eight plans (8 to 119 MB through the pass, 4.1 to 21 us):
        // 2.5 us + 6 TB/s; queued behind the GEMM the second launch adds no gap of its own.
        const double c_bytes = 4.0 * c.M * c.N * c.batches;
        total += 2.5 + (k_splits + 1.0) * c_bytes / 6.0e6;
        if (waves > 1.0) {
            total *= 1.05;  // measured: a second round of partitions costs a little more than its share
        }
    } else if (k_splits > 1) {
        // zero fill of C, then every partition adds its tile into C with fp32 atomics: measured 25 us per 256x256
        // tile against 7 us for plain stores
        const double c_bytes = 4.0 * c.M * c.N * c.batches;
        total += 3.0 + c_bytes / 3.0e6 + waves * 18.0 * (d.bm * d.bn) / 65536.0;  // (3 us: the fill kernel's launch)
        if (versus_reduce) {
            // Side by side with a workspace sum of the same partitions the atomics measure 5 to 20 us slower than
            // this estimate says (a round of workgroups ending together drains at 1.0 to 1.7 TB/s of atomic
            // operands).  The estimate is kept as it is where only atomics can be chosen: its constants were fitted
            // there, against output-stationary plans.
            total += 5.0 + 0.25 * items * (4.0 * d.bm * d.bn) / 1.0e6;
        }
        if (waves > 1.0) {
            total *= 1.15;  // measured: a second round of atomic partitions costs more than its share
        }
    }
    // streaming floor: every byte of A, B and C crosses HBM at least once (about 5 TB/s is what a streaming kernel
    // reaches); among plans that sit on the floor the one with the most compute slack wins
    const double bytes = (2.0 * ((double)c.M * c.K + (double)c.N * c.K) + 4.0 * c.M * c.N) * c.batches;
    const int big = c.batches == 1 ? beyond_cache(c) : 0;
    if (big) {
        // An operand larger than the 256 MB memory-side cache comes from DRAM on every launch, also in a benchmark
        // loop, and the launch is a stream of it with the matrix work on top: the two overlap only in part.  Measured
        // on M (or N) = 64 ... 1000 against an 8192 x 28672 or 28672 x 8192 operand of 470 MB, sixty forced plans:
        //  * time = sqrt(stream^2 + compute^2) within 10 %;
        //  * the stream runs at 5.7 TB/s when that operand is read once and issued non-temporal (see gemm_tn_kernel,
        //    ONCE); with ordinary loads it keeps pushing the other operand's panels out of the L2, the more the
        //    larger a K partition's share of that operand is (4.9 TB/s at 1.8 MB, 3.6 TB/s from 3.7 MB on);
        //  * a workgroup alone pulls about 26 GB/s (what its ring keeps in flight over the DRAM latency), so a launch
        //    of 64 workgroups streams at 1.7 TB/s however little else it has to do.
        const Plan probe{tile, k_splits == 1 ? MI_K_OUTPUT_STATIONARY : reduce ? MI_K_SPLIT_REDUCE : MI_K_SPLIT, k_splits, 0, 0.0};
        const double a_bytes = 2.0 * c.M * c.lda, b_bytes = 2.0 * c.N * c.ldb;
        const double shared_mb = (big == 3 ? (a_bytes < b_bytes ? a_bytes : b_bytes) : (big & 2) ? a_bytes : b_bytes) / k_splits / 1.0e6;
        double rate = 5.7e6;
        if (!read_once_operand(c, probe)) {
            rate /= 1.0 + 0.16 * shared_mb;
            rate = rate < 3.6e6 ? 3.6e6 : rate;
        }
        const double in_flight = (items < cus ? items : (double)cus) * 26.0e3;
        rate = rate < in_flight ? rate : in_flight;
        const double stream_us = bytes / rate;
        return __builtin_sqrt(stream_us * stream_us + total * total) + 1e-3 * total;
    }
    const double hbm_us = bytes / 5.0e6;
    return (total > hbm_us ? total : hbm_us) + 1e-3 * total;
}

static bool search_plan(const Canonical& c, int k_mode, int tile, size_t partial_space, int cus, Plan& plan);

// `partial_space`: workspace bytes that private copies of C may take (0 = K partitions can only meet through atomics).
static bool make_plan(const Canonical& c, int k_mode, int tile, size_t partial_space, Plan& plan)
{
    if (!problem_fits(c)) {
        return false;
    }
    const int cus = device_compute_units();
    // A caller in a loop asks the same few questions again and again (the size query, then the call), and the search
    // below costs microseconds, which a 10 us kernel launched back to back would feel: remember this thread's last
    // answers.
    struct Memo {
        uint32_t M, N, K, batches;
        uint64_t c_batch_bytes;
        uint32_t lda, ldb, ab_low_bits;  // (the price of a K step depends on how rows sit on 128-byte lines)
        uint32_t c_low_bits;
        int k_mode, tile, cus;
        size_t partial_space;
        uint32_t constants;  // (planner_constants_generation when the answer was found)
        bool valid, found;
        Plan plan;
    };
    constexpr int MEMOS = 4;
    static thread_local Memo memos[MEMOS]{};
    static thread_local int next_memo = 0;
    const uint32_t c_low_bits = (uint32_t)((uintptr_t)c.c % 16);
    const uint32_t ab_low_bits = (uint32_t)(((uintptr_t)c.a | (uintptr_t)c.b) % 128);
    const uint32_t generation = planner_constants_generation.load(std::memory_order_relaxed);
    for (const Memo& memo : memos) {
        if (memo.valid && memo.M == c.M && memo.N == c.N && memo.K == c.K && memo.batches == c.batches &&
            memo.c_batch_bytes == c.c_batch_bytes && memo.lda == c.lda && memo.ldb == c.ldb && memo.ab_low_bits == ab_low_bits &&
            memo.c_low_bits == c_low_bits && memo.k_mode == k_mode &&
            memo.tile == tile && memo.cus == cus && memo.partial_space == partial_space && memo.constants == generation) {
            plan = memo.plan;
            return memo.found;
        }
    }
    plan = Plan{MI_TILE_AUTO, MI_K_OUTPUT_STATIONARY, 1, 0, 0.0};
    const bool found = search_plan(c, k_mode, tile, partial_space, cus, plan);
    memos[next_memo] = {c.M,        c.N,    c.K,  c.batches, c.c_batch_bytes, c.lda, c.ldb, ab_low_bits,
                        c_low_bits, k_mode, tile, cus,       partial_space,   generation, true,  found, plan};
    next_memo = (next_memo + 1) % MEMOS;
    return found;
}

// Tiles the planner leaves to callers that force them.  The tile that shares a CU between two workgroups wins where
// workgroups are short-lived (measured: ahead by 13 % at K = 512 and 1024, level at 1408, behind by 8 to 10 % at 1536
// and 2048, 3000 x 11008 x 4096 253 us against 214 us).
static bool planner_considers(int tile, uint32_t K)
{
    const TileRow* const row = tile_row(tile);
    return row != nullptr && (row->max_k == 0 || K <= row->max_k);
}

static bool search_plan(const Canonical& c, int k_mode, int tile, size_t partial_space, int cus, Plan& plan)
{
    const int tile_lo = tile == MI_TILE_AUTO ? 1 : tile;
    const int tile_hi = tile == MI_TILE_AUTO ? MI_TILE_COUNT_ - 1 : tile;
    bool found = false;
    double best = 0.0;
    for (int tl = tile_lo; tl <= tile_hi; ++tl) {
        TileDims d;
        if (!tile_dims(tl, c.K, d)) {
            return false;
        }
        if (tile == MI_TILE_AUTO && !planner_considers(tl, c.K)) {
            continue;  // (a caller can still force it)
        }
        // Stream-K when asked for, or when the planner may choose and the workspace holds the parts.
        // (Not by itself when an operand is larger than the memory-side cache: such a launch is a DRAM stream, priced
        // by plan_cost with its read-once builds, which stream-K has none of.)
        if (k_mode == MI_K_STREAM || (k_mode == MI_K_AUTO && partial_space > 0 && beyond_cache(c) == 0)) {
            StreamKLayout sk;
            if (stream_k_layout(c, tl, cus, sk) && sk.bytes() <= partial_space) {
                const double cost = stream_k_cost(c, tl, sk);
                // (left to itself the planner takes it only when it is priced clearly ahead: 3 %)
                const double rank = k_mode == MI_K_AUTO ? cost * 1.03 : cost;
                if (!found || rank < best) {
                    found = true;
                    best = rank;
                    plan = {tl, MI_K_STREAM, 1, sk.g, cost};
                }
            }
        }
        if (k_mode == MI_K_STREAM) {
            continue;
        }
        // any partition count, not only powers of two: 66 tiles on 256 CUs want 3 (198 items), not 4 (264)
        for (uint32_t splits = 1; splits <= 32; ++splits) {
            if (splits == 1 && (k_mode == MI_K_SPLIT || k_mode == MI_K_SPLIT_REDUCE) && ceil_div(c.K, d.bk) >= 2) {
                continue;
            }
            if (splits > 1 && k_mode == MI_K_OUTPUT_STATIONARY) {
                break;
            }
            if (!tile_fits(c, tl, splits)) {
                continue;
            }
            for (int reduce = 0; reduce <= (splits > 1 ? 1 : 0); ++reduce) {
                if (splits > 1 && ((reduce && k_mode == MI_K_SPLIT) || (!reduce && k_mode == MI_K_SPLIT_REDUCE) ||
                                   (reduce && partial_bytes(c, splits) > partial_space))) {
                    continue;
                }
                const double cost = plan_cost(c, tl, splits, reduce != 0, partial_space > 0, cus);
                // The estimates are no finer than a microsecond: left to itself the planner takes partitions summed
                // by a second launch only when they are priced that much ahead (160 x 480 x 816: seven of them were
                // priced 0.2 us under the one launch of 9.4 us and ran 1 us over it).
                const double rank = cost + (k_mode == MI_K_AUTO && splits > 1 && reduce ? 1.0 : 0.0);
                if (!found || rank < best) {
                    found = true;
                    best = rank;
                    plan = {tl, splits == 1 ? MI_K_OUTPUT_STATIONARY : reduce ? MI_K_SPLIT_REDUCE : MI_K_SPLIT, splits, 0, cost};
                }
            }
        }
    }
    return found;
}

// A ragged M or N makes every tile of a launch pay for the range-checked build (about 4 % of the main loop, and one
// more round of workgroups when the extra row of tiles does not fit the last one).  Peeling: the whole tiles run as
// one launch of the plain build, the rows below them and the columns right of them as one small range-checked launch
// each (which may split K through atomics: a strip has few tiles and all of K), all writing the caller's C at its own
// pitch.  (A ragged K touches every tile, so the whole tiles then run the range-checked build too; peeling can
// still pay through the tile count.)
struct Peel {
    bool on = false;
    uint32_t Mi = 0, Ni = 0;            // extent of the whole tiles
    Plan interior_plan{}, bottom_plan{}, right_plan{};
    double cost_us = 0.0;
};

// Sub-problems of a peeled launch.  bottom: rows Mi..M-1, every column; right: rows 0..Mi-1, columns Ni..N-1.
static Canonical peel_interior(const Canonical& c, const Peel& peel)
{
    Canonical s = c;
    s.parent_beyond_cache = beyond_cache(c);
    s.M = peel.Mi;
    s.N = peel.Ni;
    s.ldc = c.N;
    return s;
}

static Canonical peel_bottom(const Canonical& c, const Peel& peel)
{
    Canonical s = c;
    s.parent_beyond_cache = beyond_cache(c);
    s.a = (const char*)c.a + (size_t)peel.Mi * c.lda * 2;
    s.c = c.c + (size_t)peel.Mi * c.N;
    s.M = c.M - peel.Mi;
    s.ldc = c.N;
    return s;
}

static Canonical peel_right(const Canonical& c, const Peel& peel)
{
    Canonical s = c;
    s.parent_beyond_cache = beyond_cache(c);
    s.b = (const char*)c.b + (size_t)peel.Ni * c.ldb * 2;
    s.c = c.c + peel.Ni;
    s.M = peel.Mi;
    s.N = c.N - peel.Ni;
    s.ldc = c.N;
    return s;
}

// The estimate of a launch includes its start-up.  For a small strip that start-up hides behind the launch before it
// (measured: it adds about 4 us less than it costs alone); a large second launch hides nothing and adds the gap
// between two launches.
static double launch_adjust_us(double cost_us)
{
    return cost_us < 20.0 ? -2.0 : 3.0;
}

static Peel plan_peeled(const Canonical& c, int cus, double whole_cost_us)
{
    Peel best;
    if (c.batches != 1 || (uintptr_t)c.c % 16 || c.N % 4 || c.ldc != 0 || c.timeline != nullptr) {
        return best;
    }
    if (c.K < 2048) {
        // With a short K the launches lose more between them than the whole tiles gain (7072 x 7352 x 1024: 147 us
        // peeled against 139 us as one launch); every measured win has K of 4096 or more.
        return best;
    }
    // (the answer depends on the shape only: remember the last one of this thread, as make_plan does)
    struct Memo {
        uint32_t M, N, K;
        int cus;
        double whole_cost_us;
        bool valid;
        Peel peel;
    };
    static thread_local Memo memo{};
    if (memo.valid && memo.M == c.M && memo.N == c.N && memo.K == c.K && memo.cus == cus && memo.whole_cost_us == whole_cost_us) {
        return memo.peel;
    }
    for (int tl = 1; tl < MI_TILE_COUNT_; ++tl) {
        TileDims d;
        if (!tile_dims(tl, c.K, d) || !planner_considers(tl, c.K)) {
            continue;
        }
        // Where to cut: at the last whole tile in M and N; or, when the whole tiles make a round of CUs and a bit,
        // after the tile columns (or tile rows) that fill whole rounds, leaving the rest, full height (or width), to
        // a launch of its own with its own tile and K split.
        const uint32_t tiles_m = c.M / d.bm, tiles_n = c.N / d.bn;
        if (tiles_m == 0 || tiles_n == 0) {
            continue;
        }
        const uint32_t whole_rounds = (uint32_t)((uint64_t)tiles_m * tiles_n / (uint32_t)cus);
        uint32_t cuts[3][2] = {{tiles_m, tiles_n}, {0, 0}, {0, 0}};
        if (whole_rounds >= 1) {
            cuts[1][0] = tiles_m;
            cuts[1][1] = (uint32_t)((uint64_t)whole_rounds * cus / tiles_m);
            cuts[2][0] = (uint32_t)((uint64_t)whole_rounds * cus / tiles_n);
            cuts[2][1] = tiles_n;
        }
        for (const auto& cut : cuts) {
            Peel cand;
            cand.Mi = cut[0] * d.bm;
            cand.Ni = cut[1] * d.bn;
            if (cand.Mi == 0 || cand.Ni == 0 || (cand.Mi == c.M && cand.Ni == c.N)) {
                continue;
            }
            cand.interior_plan = Plan{tl, MI_K_OUTPUT_STATIONARY, 1, 0, plan_cost(peel_interior(c, cand), tl, 1, false, false, cus)};
            double total = cand.interior_plan.cost_us;
            if (cand.Mi < c.M) {
                if (!search_plan(peel_bottom(c, cand), MI_K_AUTO, MI_TILE_AUTO, 0, cus, cand.bottom_plan)) {
                    continue;
                }
                total += cand.bottom_plan.cost_us + launch_adjust_us(cand.bottom_plan.cost_us);
            }
            if (cand.Ni < c.N) {
                if (!search_plan(peel_right(c, cand), MI_K_AUTO, MI_TILE_AUTO, 0, cus, cand.right_plan)) {
                    continue;
                }
                total += cand.right_plan.cost_us + launch_adjust_us(cand.right_plan.cost_us);
            }
            if (&cut != &cuts[0]) {
                total *= 1.03;  // a cut after whole rounds must win by more: its second launch is a large one
            }
            cand.cost_us = total;
            if (!best.on || total < best.cost_us) {
                cand.on = true;
                best = cand;
            }
        }
    }
    // the estimates are good to a few percent: peel only when they say it clearly pays
    if (best.on && best.cost_us > 0.97 * whole_cost_us) {
        best.on = false;
    }
    memo = {c.M, c.N, c.K, cus, whole_cost_us, true, best};
    return best;
}

// The planner's own stream-K plan against the best plan that needs no workspace, peeled: a ragged or round-and-a-bit
// problem may do better as an output-stationary launch plus strips than as whole rounds plus a streamed tail
// (4096 x 4352 x 8192: 222 us peeled, 232 us streamed).  Replaces `plan` when the peeled estimate is the lower one.
static void prefer_peeling_to_stream_k(const Canonical& c, int k_mode, int tile, Plan& plan)
{
    if (k_mode != MI_K_AUTO || tile != MI_TILE_AUTO || plan.k_mode != MI_K_STREAM) {
        return;
    }
    Plan alt;
    if (!make_plan(c, MI_K_OUTPUT_STATIONARY, tile, 0, alt)) {
        return;
    }
    const Peel peel = plan_peeled(c, device_compute_units(), alt.cost_us);
    if (peel.on && peel.cost_us < plan.cost_us) {
        plan = alt;
    }
}

__global__ __launch_bounds__(256) void zero_fill_kernel(float* dst, size_t n)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        dst[i] = 0.f;
    }
}

__global__ __launch_bounds__(256) void zero_fill_2d_kernel(float* dst, uint32_t rows, uint32_t cols, uint32_t pitch)
{
    const size_t n = (size_t)rows * cols;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        dst[i / cols * pitch + i % cols] = 0.f;
    }
}

// C = sum of the K partitions' copies, in partition order (so the result does not depend on timing).  Problem l's
// copies lie at partials + l * splits * n, its C at c + l * c_batch_elems.  VEC: n, C and c_batch_elems are 16-byte
// multiples.
template <bool VEC>
__global__ __launch_bounds__(256) void reduce_partials_kernel(const float* partials, float* c, size_t n, uint32_t splits,
                                                              size_t c_batch_elems)
{
    using T = typename std::conditional<VEC, f32x4, float>::type;
    const size_t count = VEC ? n / 4 : n;
    const T* src = reinterpret_cast<const T*>(partials + (size_t)blockIdx.y * splits * n);
    T* dst = reinterpret_cast<T*>(c + (size_t)blockIdx.y * c_batch_elems);
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x) {
        T acc = __builtin_nontemporal_load(src + i);
        uint32_t s = 1;
        for (; s + 3 < splits; s += 4) {
            const T v0 = __builtin_nontemporal_load(src + (size_t)s * count + i);
            const T v1 = __builtin_nontemporal_load(src + (size_t)(s + 1) * count + i);
            const T v2 = __builtin_nontemporal_load(src + (size_t)(s + 2) * count + i);
            const T v3 = __builtin_nontemporal_load(src + (size_t)(s + 3) * count + i);
            acc = (((acc + v0) + v1) + v2) + v3;
        }
        // the last one to three copies: loaded together, added in the same order
        const uint32_t rest = splits - s;
        if (rest == 3) {
            const T v0 = __builtin_nontemporal_load(src + (size_t)s * count + i);
            const T v1 = __builtin_nontemporal_load(src + (size_t)(s + 1) * count + i);
            const T v2 = __builtin_nontemporal_load(src + (size_t)(s + 2) * count + i);
            acc = ((acc + v0) + v1) + v2;
        }
        else if (rest == 2) {
            const T v0 = __builtin_nontemporal_load(src + (size_t)s * count + i);
            const T v1 = __builtin_nontemporal_load(src + (size_t)(s + 1) * count + i);
            acc = (acc + v0) + v1;
        }
        else if (rest == 1) {
            acc += __builtin_nontemporal_load(src + (size_t)s * count + i);
        }
        dst[i] = acc;
    }
}

static int reduce_partials(const float* partials, const Canonical& c, uint32_t splits, hipStream_t stream)
{
    const size_t n = (size_t)c.M * c.N;
    const bool vec = n % 4 == 0 && (uintptr_t)c.c % 16 == 0 && c.c_batch_bytes % 16 == 0;
    size_t blocks = ((vec ? n / 4 : n) + 255) / 256;
    blocks = blocks > 4096 ? 4096 : blocks;
    if (c.batches > 65535u) {
        return MI_ERR_UNSUPPORTED;
    }
    const dim3 grid((uint32_t)blocks, c.batches, 1);
    if (vec) {
        hipLaunchKernelGGL(reduce_partials_kernel<true>, grid, dim3(256), 0, stream, partials, c.c, n, splits,
                           (size_t)(c.c_batch_bytes / 4));
    } else {
        hipLaunchKernelGGL(reduce_partials_kernel<false>, grid, dim3(256), 0, stream, partials, c.c, n, splits,
                           (size_t)(c.c_batch_bytes / 4));
    }
    MI_CHECK_LAUNCH();
    return MI_OK;
}

// Stream-K second pass: tail tile t of C = its main partitions' parts (slots t * S ... t * S + S - 1), then the parts
// of the leftover workgroups whose runs overlap the tile's leftover K tiles (slot r * S + j + t for workgroup j), added
// in that order (see gemm_tn_kernel, STREAM).  One block per 8 rows of a tile; 16-byte accesses throughout.
__global__ __launch_bounds__(256) void stream_k_sum_kernel(const float* parts, float* c, uint32_t ldc, uint32_t bm, uint32_t bn,
                                                           uint32_t k_tiles, uint32_t workgroups, GemmArgs raster)
{
    const uint32_t chunks = bm / 8;
    const uint32_t t = blockIdx.x / chunks, row0 = (blockIdx.x % chunks) * 8;
    const uint32_t r = raster.sk.tiles, splits = raster.sk.splits, kr = k_tiles - raster.sk.main_k;
    const uint32_t lefts = workgroups - r * splits;
    uint32_t j_lo, j_hi;  // leftover workgroups [j_lo, j_hi) overlap the tile
    leftover_runs_of_tile(r, kr, lefts, t, j_lo, j_hi);
    uint32_t tm, tn;
    raster_tile(raster, raster.sk.first_tile + t, tm, tn);
    const uint32_t quads = bn / 4;
    const size_t tile_elems = (size_t)bm * bn;
    for (uint32_t idx = threadIdx.x; idx < 8 * quads; idx += blockDim.x) {
        const uint32_t row = row0 + idx / quads, col = (idx % quads) * 4;
        const size_t at = (size_t)row * bn + col;
        f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
        for (uint32_t sp = 0; sp < splits; ++sp) {
            acc += __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(parts + (size_t)(t * splits + sp) * tile_elems + at));
        }
        for (uint32_t j = j_lo; j < j_hi; ++j) {
            if (leftover_run_empty(r, kr, lefts, j)) {
                continue;  // (an empty run stores nothing)
            }
            acc += __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(parts + (size_t)(r * splits + j + t) * tile_elems + at));
        }
        *reinterpret_cast<f32x4*>(c + (size_t)(tm * bm + row) * ldc + (size_t)tn * bn + col) = acc;
    }
}

static int stream_k_sum(const float* parts, const Canonical& c, const StreamKLayout& sk, hipStream_t stream)
{
    GemmArgs raster{};
    raster.tiles_m = c.M / sk.bm;
    raster.tiles_n = c.N / sk.bn;
    raster.group_m = GROUP_M;
    raster.sk = stream_k_shape(sk);
    const uint32_t blocks = sk.r * (sk.bm / 8);
    hipLaunchKernelGGL(stream_k_sum_kernel, dim3(blocks), dim3(256), 0, stream, parts, c.c, c.ldc ? c.ldc : c.N, sk.bm, sk.bn,
                       sk.k_tiles, sk.g, raster);
    MI_CHECK_LAUNCH();
    return MI_OK;
}

static int launch_tile(int dtype, const Canonical& problem, const Plan& plan, hipStream_t stream)
{
    TileDims d;
    const TileRow* const row = tile_row(plan.tile);
    if (row == nullptr || !tile_dims(plan.tile, problem.K, d) || (dtype != MI_F16 && dtype != MI_BF16)) {
        return MI_ERR_BAD_ARGUMENT;
    }
    Canonical c = problem;
    c.read_once = problem.stream_k_workgroups ? 0 : read_once_operand(c, plan);
    const LaunchFn launch = d.bk == 64 ? row->deep[dtype] : row->twin[dtype];
    return launch(c, plan.k_splits, needs_edge(c, d), stream);
}

// Re-packs an operand into K-contiguous rows of pitch kp (a multiple of 8), zero-padding columns K..kp-1.
// 64 x 64 element tiles; a transposing copy goes through LDS so that both the read and the write are coalesced.
__global__ __launch_bounds__(256) void repack_kernel(const uint16_t* in, uint16_t* out, uint32_t rows, uint32_t K, uint32_t kp,
                                                     int k_contiguous)
{
    __shared__ uint16_t tile[64][65];
    const uint32_t r0 = blockIdx.y * 64, k0 = blockIdx.x * 64;
    const uint32_t tx = threadIdx.x % 64, ty = threadIdx.x / 64;
    if (k_contiguous) {
        for (uint32_t rr = ty; rr < 64; rr += 4) {
            const uint32_t r = r0 + rr, k = k0 + tx;
            if (r < rows && k < kp) {
                out[(size_t)r * kp + k] = k < K ? in[(size_t)r * K + k] : (uint16_t)0;
            }
        }
        return;
    }
    // (all loads of a lane in flight together: out-of-range lanes read element 0 and drop the value)
    uint16_t v[16];
#pragma unroll
    for (uint32_t i = 0; i < 16; ++i) {
        const uint32_t k = k0 + ty + 4 * i, r = r0 + tx;
        v[i] = in[(k < K && r < rows) ? (size_t)k * rows + r : (size_t)0];
    }
#pragma unroll
    for (uint32_t i = 0; i < 16; ++i) {
        const uint32_t k = k0 + ty + 4 * i, r = r0 + tx;
        tile[ty + 4 * i][tx] = (k < K && r < rows) ? v[i] : (uint16_t)0;
    }
    __syncthreads();
    for (uint32_t rr = ty; rr < 64; rr += 4) {
        const uint32_t r = r0 + rr, k = k0 + tx;
        if (r < rows && k < kp) {
            out[(size_t)r * kp + k] = tile[tx][rr];
        }
    }
}

// The transposing re-pack for an even number of rows and a 4-byte aligned source: 128 x 128 blocks, two elements per
// lane on the way in (256-byte segments of a source row per wave and load, all loads of a lane in flight together),
// eight consecutive K values (16 bytes) per lane on the way out.
__global__ __launch_bounds__(256) void repack_transposed_kernel(const uint16_t* __restrict__ in, uint16_t* __restrict__ out,
                                                                uint32_t rows, uint32_t K, uint32_t kp)
{
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    __shared__ uint32_t tile[128][65];  // [k][pair of rows]
    const uint32_t r0 = blockIdx.x * 128, k0 = blockIdx.y * 128;
    const uint32_t tx = threadIdx.x % 64, ty = threadIdx.x / 64;
    const uint32_t r_in = r0 + 2 * tx;  // rows is even: a pair is inside the matrix or outside it
    uint32_t v[32];
#pragma unroll
    for (uint32_t i = 0; i < 32; ++i) {
        const uint32_t k = k0 + ty + 4 * i;
        v[i] = __builtin_nontemporal_load(
            reinterpret_cast<const uint32_t*>(in + ((k < K && r_in < rows) ? (size_t)k * rows + r_in : (size_t)0)));
    }
#pragma unroll
    for (uint32_t i = 0; i < 32; ++i) {
        const uint32_t k = k0 + ty + 4 * i;
        tile[ty + 4 * i][tx] = (k < K && r_in < rows) ? v[i] : 0u;
    }
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < 128 * 16; i += 256) {
        const uint32_t rr = i / 16, ch = i % 16;
        const uint32_t r = r0 + rr, k = k0 + ch * 8;
        if (r >= rows || k >= kp) {
            continue;
        }
        const uint32_t shift = (rr & 1u) * 16;
        uint32_t w[4];
        for (int j = 0; j < 4; ++j) {
            const uint32_t e0 = tile[ch * 8 + 2 * j][rr / 2] >> shift & 0xffffu;
            const uint32_t e1 = tile[ch * 8 + 2 * j + 1][rr / 2] >> shift & 0xffffu;
            w[j] = e0 | e1 << 16;
        }
        *reinterpret_cast<u32x4*>(out + (size_t)r * kp + k) = u32x4{w[0], w[1], w[2], w[3]};
    }
}

static int repack(const Operand& op, uint32_t K, void* dst, hipStream_t stream)
{
    const uint32_t kp = (uint32_t)round_up(K, 8);
    if (!op.k_contiguous && op.rows % 2 == 0 && (uintptr_t)op.ptr % 4 == 0) {
        hipLaunchKernelGGL(repack_transposed_kernel, dim3((op.rows + 127) / 128, (kp + 127) / 128, 1), dim3(256), 0, stream,
                           (const uint16_t*)op.ptr, (uint16_t*)dst, op.rows, K, kp);
        MI_CHECK_LAUNCH();
        return MI_OK;
    }
    const dim3 grid((kp + 63) / 64, (op.rows + 63) / 64, 1);
    if (grid.y > 65535u) {
        return MI_ERR_UNSUPPORTED;
    }
    hipLaunchKernelGGL(repack_kernel, grid, dim3(256), 0, stream, (const uint16_t*)op.ptr, (uint16_t*)dst, op.rows, K, kp,
                       op.k_contiguous ? 1 : 0);
    MI_CHECK_LAUNCH();
    return MI_OK;
}

// fp32 -> bf16 terms, K-contiguous rows of pitch terms*kp: segment s of a row holds the hi part (bf16 nearest to x)
// or the lo part (bf16 nearest to x - hi) of the row's K values, zero-padded to kp.  `lo_mask` bit s selects lo.
// Three kernels: K-contiguous rows of any K and alignment (this one, element by element), K-contiguous rows with
// K % 8 == 0 and 16-byte alignment, and operands stored K x rows.
__device__ __forceinline__ uint16_t bf16_rne(float x)
{
    uint32_t u = __builtin_bit_cast(uint32_t, x);
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        return (uint16_t)((u >> 16) | 0x40u);  // NaN stays NaN
    }
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

__global__ __launch_bounds__(256) void split_f32_kernel(const float* in, uint16_t* out, uint32_t rows, uint32_t K, uint32_t kp,
                                                        uint32_t terms, uint32_t lo_mask)
{
    const uint32_t r0 = blockIdx.y * 64, k0 = blockIdx.x * 64;
    const uint32_t tx = threadIdx.x % 64, ty = threadIdx.x / 64;
    for (uint32_t rr = ty; rr < 64; rr += 4) {
        const uint32_t r = r0 + rr, k = k0 + tx;
        if (r < rows && k < kp) {
            const float x = k < K ? in[(size_t)r * K + k] : 0.0f;
            const uint16_t hi = bf16_rne(x);
            const uint16_t lo = bf16_rne(x - __builtin_bit_cast(float, (uint32_t)hi << 16));
            uint16_t* const row = out + (size_t)r * terms * kp + k;
            for (uint32_t s = 0; s < terms; ++s) {
                row[(size_t)s * kp] = (lo_mask >> s & 1u) ? lo : hi;
            }
        }
    }
}

// The same split for K-contiguous fp32 rows with K % 8 == 0 and 16-byte aligned rows: a lane takes eight consecutive values
// of a row (two 16-byte loads) and writes one 16-byte store per term, so a wave reads 2 KB and writes 1 KB per term in
// one piece.  `chunks` = rows * K / 8; the row pitch of `out` is terms * K.
__global__ __launch_bounds__(256) void split_f32_rows_kernel(const float* __restrict__ in, uint16_t* __restrict__ out,
                                                             uint64_t chunks, uint32_t chunks_per_row, uint32_t terms,
                                                             uint32_t lo_mask)
{
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    for (uint64_t c = (uint64_t)blockIdx.x * 256 + threadIdx.x; c < chunks; c += (uint64_t)gridDim.x * 256) {
        const f32x4* src = reinterpret_cast<const f32x4*>(in) + c * 2;
        const f32x4 x0 = __builtin_nontemporal_load(src), x1 = __builtin_nontemporal_load(src + 1);
        const float x[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
        uint32_t hi[4], lo[4];
        for (int i = 0; i < 4; ++i) {
            const uint16_t h0 = bf16_rne(x[2 * i]), h1 = bf16_rne(x[2 * i + 1]);
            const uint16_t l0 = bf16_rne(x[2 * i] - __builtin_bit_cast(float, (uint32_t)h0 << 16));
            const uint16_t l1 = bf16_rne(x[2 * i + 1] - __builtin_bit_cast(float, (uint32_t)h1 << 16));
            hi[i] = (uint32_t)h0 | (uint32_t)h1 << 16;
            lo[i] = (uint32_t)l0 | (uint32_t)l1 << 16;
        }
        const uint64_t row = c / chunks_per_row;
        const uint32_t in_row = (uint32_t)(c - row * chunks_per_row);
        u32x4* dst = reinterpret_cast<u32x4*>(out) + (row * terms) * chunks_per_row + in_row;
        for (uint32_t s = 0; s < terms; ++s) {
            dst[(uint64_t)s * chunks_per_row] = (lo_mask >> s & 1u) ? u32x4{lo[0], lo[1], lo[2], lo[3]} : u32x4{hi[0], hi[1], hi[2], hi[3]};
        }
    }
}

// The same split for fp32 operands stored K x rows (rows contiguous): 128 x 64 blocks are turned through LDS, so that
// the reads are 256-byte row segments of the source and every lane writes eight consecutive K values (16 bytes) per
// term.  Values beyond K (up to kp, the pitch of one term) are zeros.
__global__ __launch_bounds__(256) void split_f32_transposed_kernel(const float* __restrict__ in, uint16_t* __restrict__ out,
                                                                   uint32_t rows, uint32_t K, uint32_t kp, uint32_t terms,
                                                                   uint32_t lo_mask)
{
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    __shared__ float tile[128][65];
    // consecutive workgroups take neighbouring segments of the same 128 source rows
    const uint32_t r0 = blockIdx.x * 64, k0 = blockIdx.y * 128;
    const uint32_t tx = threadIdx.x % 64, ty = threadIdx.x / 64;
    // every load is issued before the first is awaited: out-of-range lanes read element 0 and drop the value
    float v[32];
    const uint32_t r_in = r0 + tx;
#pragma unroll
    for (uint32_t i = 0; i < 32; ++i) {
        const uint32_t k = k0 + ty + 4 * i;
        v[i] = __builtin_nontemporal_load(in + ((k < K && r_in < rows) ? (size_t)k * rows + r_in : (size_t)0));
    }
#pragma unroll
    for (uint32_t i = 0; i < 32; ++i) {
        const uint32_t k = k0 + ty + 4 * i;
        tile[ty + 4 * i][tx] = (k < K && r_in < rows) ? v[i] : 0.0f;
    }
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < 64 * 16; i += 256) {
        const uint32_t rr = i / 16, ch = i % 16;
        const uint32_t r = r0 + rr, k = k0 + ch * 8;
        if (r >= rows || k >= kp) {
            continue;
        }
        uint32_t hi[4], lo[4];
        for (int j = 0; j < 4; ++j) {
            const float x0 = tile[ch * 8 + 2 * j][rr], x1 = tile[ch * 8 + 2 * j + 1][rr];
            const uint16_t h0 = bf16_rne(x0), h1 = bf16_rne(x1);
            const uint16_t l0 = bf16_rne(x0 - __builtin_bit_cast(float, (uint32_t)h0 << 16));
            const uint16_t l1 = bf16_rne(x1 - __builtin_bit_cast(float, (uint32_t)h1 << 16));
            hi[j] = (uint32_t)h0 | (uint32_t)h1 << 16;
            lo[j] = (uint32_t)l0 | (uint32_t)l1 << 16;
        }
        uint16_t* const row = out + (size_t)r * terms * kp + k;
        for (uint32_t s = 0; s < terms; ++s) {
            *reinterpret_cast<u32x4*>(row + (size_t)s * kp) =
                (lo_mask >> s & 1u) ? u32x4{lo[0], lo[1], lo[2], lo[3]} : u32x4{hi[0], hi[1], hi[2], hi[3]};
        }
    }
}

static int check_modes(const mi_gemm_tensors* t, int k_mode, int tile)
{
    if (const int st = validate_tensors(t)) {
        return st;
    }
    if (k_mode < 0 || k_mode > MI_K_STREAM || tile < 0 || tile >= MI_TILE_COUNT_) {
        return MI_ERR_BAD_ARGUMENT;
    }
    return MI_OK;
}

// Scratch memory of mi_matmul_mfma_static: a device array that is part of the library's code object, so the entry point
// never allocates.  Every GPU the library runs on holds its own copy, at its own address, until the process ends.  In
// host code `scratch` is only a handle for hipGetSymbolAddress; the address that kernels and copies may use is the one
// that call returns, looked up once per device with that device current.
constexpr size_t STATIC_SCRATCH_BYTES = MI_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

int resolve_static_scratch(void** out)
{
    constexpr int MAX_DEVICES = 64;
    static std::mutex guard;
    static void* address[MAX_DEVICES] = {};
    int dev = 0;
    MI_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= MAX_DEVICES) {
        return MI_ERR_UNSUPPORTED;
    }
    std::lock_guard<std::mutex> lock(guard);
    if (address[dev] == nullptr) {
        void* ptr = nullptr;
        MI_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (ptr == nullptr || (uintptr_t)ptr % 256) {
            return MI_ERR_HIP;
        }
        address[dev] = ptr;
    }
    if (out != nullptr) {
        *out = address[dev];
    }
    return MI_OK;
}

// Arrival counters for launches that sum their K partitions (or stream-K parts) themselves, see GemmArgs::tile_counters.
// They must be zero when a launch starts, and every launch leaves them zero, so they cannot live in a caller's workspace
// (whose bytes are the caller's between calls) without a zero-fill launch per call, which would cost what the in-launch
// sum saves.  They are a device array of the library's code object instead: zero when the code object is loaded, one copy
// per GPU.  The array is dealt out in slabs by workspace: calls that share a workspace are already ordered by their
// caller (they would overwrite each other's parts otherwise), so they can share a slab; calls with different workspaces
// may overlap in time and get different slabs.  A workspace keeps its slab until the process ends (a captured graph may
// replay the call at any time).  When all slabs are taken, or a call needs more counters than a slab holds, the call
// sums with a second launch, as it always could.
constexpr uint32_t COUNTER_SLABS = 256, SLAB_COUNTERS = 4096;
static __device__ __align__(256) uint32_t tile_counter_pool[COUNTER_SLABS * SLAB_COUNTERS];

// Off unless asked for: measured on MI355X the sum inside the launch is the slower way on every shape tried (see
// mi_matmul_mfma_sum_in_launch in mi_gemm.h).
static std::atomic<bool> sum_in_launch{false};
static std::atomic<uint64_t> calls_summed_in_launch{0};

static uint32_t* tile_counters_for(const void* workspace, uint64_t needed)
{
    if (!sum_in_launch.load(std::memory_order_relaxed)) {
        return nullptr;
    }
    constexpr int MAX_DEVICES = 64;
    struct PerDevice {
        uint32_t* pool = nullptr;
        const void* owner[COUNTER_SLABS] = {};
        uint32_t used = 0;
    };
    static std::mutex guard;
    static PerDevice devices[MAX_DEVICES];
    int dev = 0;
    if (workspace == nullptr || needed == 0 || needed > SLAB_COUNTERS || hipGetDevice(&dev) != hipSuccess || dev < 0 ||
        dev >= MAX_DEVICES) {
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(guard);
    PerDevice& d = devices[dev];
    if (d.pool == nullptr) {
        void* ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(tile_counter_pool)) != hipSuccess || ptr == nullptr) {
            (void)hipGetLastError();
            return nullptr;
        }
        d.pool = static_cast<uint32_t*>(ptr);
    }
    for (uint32_t i = 0; i < d.used; ++i) {
        if (d.owner[i] == workspace) {
            return d.pool + (size_t)i * SLAB_COUNTERS;
        }
    }
    if (d.used == COUNTER_SLABS) {
        return nullptr;
    }
    d.owner[d.used] = workspace;
    return d.pool + (size_t)(d.used++) * SLAB_COUNTERS;
}

int resolve_tile_counters()
{
    int dev = 0;
    MI_HIP_TRY(hipGetDevice(&dev));
    // (looks the array's address up for this device; the slab of the library's own scratch array is claimed on the way)
    void* scratch_ptr = nullptr;
    if (const int st = resolve_static_scratch(&scratch_ptr)) {
        return st;
    }
    return !sum_in_launch.load() || tile_counters_for(scratch_ptr, 1) != nullptr ? MI_OK : MI_ERR_HIP;
}

struct TimelineRequest {
    unsigned long long* d_stamps;
    uint32_t slots, max_workgroups;
    uint32_t* out_workgroups;
};

// L problems of one shape, each `*_stride` elements after the previous one (in the caller's A, B, C roles).
struct BatchRequest {
    uint32_t batches;
    uint64_t a_stride, b_stride, c_stride;
};

// `attributes_only`: go through the plan this call would run and set the attributes of every GEMM kernel it would
// launch, launching nothing (mi_matmul_mfma_prepare).  The helper kernels (fill, re-pack, sums) need no attribute.
// `workspace_owner`: the start of the caller's workspace when `workspace` is only what an earlier pass has left of it (the
// arrival counters of a call are dealt out by workspace, see tile_counters_for); null: `workspace` itself.
static int run_mfma(const mi_gemm_tensors* t, int k_mode, int tile, void* workspace, size_t workspace_bytes, void* hip_stream,
                    const TimelineRequest* timeline = nullptr, const BatchRequest* batch = nullptr, bool attributes_only = false,
                    const void* workspace_owner = nullptr)
{
    if (const int st = check_modes(t, k_mode, tile)) {
        return st;
    }
    Prepared p = prepare(*t);
    if (batch != nullptr) {
        // the operand swap for column-major C swaps the batch strides with it; operands must be readable in place
        // (a workspace would have to hold every problem's copy)
        if (p.ws_bytes > 0 || (batch->a_stride * 2) % 16 || (batch->b_stride * 2) % 16) {
            return MI_ERR_UNSUPPORTED;
        }
        p.c.batches = batch->batches;
        p.c.a_batch_bytes = (t->c_col_major ? batch->b_stride : batch->a_stride) * 2;
        p.c.b_batch_bytes = (t->c_col_major ? batch->a_stride : batch->b_stride) * 2;
        p.c.c_batch_bytes = batch->c_stride * 4;
    }
    if (p.ws_bytes > 0) {
        if (!workspace) {
            return MI_ERR_UNSUPPORTED;  // needs re-packing: only mi_matmul_mfma_ws can do it
        }
        if (workspace_bytes < p.ws_bytes || (uintptr_t)workspace % 256) {
            return MI_ERR_WORKSPACE;
        }
    }
    // what the re-packed operands leave of the workspace can hold the K partitions' private copies of C
    const size_t partial_off = round_up(p.ws_bytes, 256);
    const bool ws_usable = workspace && (uintptr_t)workspace % 256 == 0 && workspace_bytes > partial_off;
    const size_t partial_space = ws_usable ? workspace_bytes - partial_off : 0;
    Plan plan;
    if (!make_plan(p.c, k_mode, tile, partial_space, plan)) {
        if ((k_mode == MI_K_SPLIT_REDUCE || k_mode == MI_K_STREAM) && make_plan(p.c, k_mode, tile, SIZE_MAX, plan)) {
            return MI_ERR_WORKSPACE;  // it would run with more room
        }
        return MI_ERR_UNSUPPORTED;
    }
    hipStream_t stream = as_stream(hip_stream);
    p.c.attributes_only = attributes_only;
    if (p.repack_a) {
        p.c.a = (char*)workspace + p.ws_a;
        if (const int st = attributes_only ? MI_OK : repack(p.a_src, t->K, const_cast<void*>(p.c.a), stream)) {
            return st;
        }
    }
    if (p.repack_b) {
        p.c.b = (char*)workspace + p.ws_b;
        if (const int st = attributes_only ? MI_OK : repack(p.b_src, t->K, const_cast<void*>(p.c.b), stream)) {
            return st;
        }
    }
    if (timeline != nullptr) {
        p.c.timeline = timeline->d_stamps;
        p.c.timeline_slots = timeline->slots;
        p.c.timeline_workgroups = timeline->max_workgroups;
        p.c.launched_workgroups = timeline->out_workgroups;
    }
    const Canonical& c = p.c;
    if (batch == nullptr && timeline == nullptr) {
        prefer_peeling_to_stream_k(c, k_mode, tile, plan);
    }
    if (tile == MI_TILE_AUTO && plan.k_mode == MI_K_OUTPUT_STATIONARY && batch == nullptr && timeline == nullptr) {
        const Peel peel = plan_peeled(c, device_compute_units(), plan.cost_us);
        if (peel.on) {
            auto launch = [&](const Canonical& part, const Plan& part_plan) -> int {
                if (part_plan.k_splits > 1 && !attributes_only) {
                    // a strip whose K partitions meet through atomics: its part of C starts at zero
                    size_t blocks = ((size_t)part.M * part.N + 255) / 256;
                    blocks = blocks > 4096 ? 4096 : blocks;
                    hipLaunchKernelGGL(zero_fill_2d_kernel, dim3((uint32_t)blocks), dim3(256), 0, stream, part.c, part.M, part.N,
                                       part.ldc);
                    MI_CHECK_LAUNCH();
                }
                return launch_tile(t->ab_dtype, part, part_plan, stream);
            };
            if (const int st = launch(peel_interior(c, peel), peel.interior_plan)) {
                return st;
            }
            if (peel.Mi < c.M) {
                if (const int st = launch(peel_bottom(c, peel), peel.bottom_plan)) {
                    return st;
                }
            }
            return peel.Ni < c.N ? launch(peel_right(c, peel), peel.right_plan) : MI_OK;
        }
    }
    if (plan.k_mode == MI_K_STREAM) {
        StreamKLayout sk;
        if (!stream_k_layout(c, plan.tile, device_compute_units(), sk) || sk.g != plan.workgroups) {
            return MI_ERR_UNSUPPORTED;
        }
        if (sk.full_tiles > 0) {
            // the whole rounds of tiles: output stationary, stored straight into C
            Canonical head = c;
            head.first_tiles_only = sk.full_tiles;
            const Plan head_plan{plan.tile, MI_K_OUTPUT_STATIONARY, 1, 0, 0.0};
            if (const int st = launch_tile(t->ab_dtype, head, head_plan, stream)) {
                return st;
            }
        }
        Canonical k = c;
        k.c = (float*)((char*)workspace + partial_off);
        k.stream_k_workgroups = sk.g;
        k.sk = stream_k_shape(sk);
        // the workgroup that stores a tail tile's last part sums the tile (one counter per tail tile); without
        // counters a last launch does the summing
        k.tile_counters = attributes_only ? nullptr : tile_counters_for(workspace_owner ? workspace_owner : workspace, sk.r);
        k.c_final = c.c;
        k.ldc_final = c.ldc;
        const int st = launch_tile(t->ab_dtype, k, plan, stream);
        if (st == MI_OK && k.tile_counters != nullptr) {
            calls_summed_in_launch.fetch_add(1, std::memory_order_relaxed);
        }
        return st || attributes_only || k.tile_counters != nullptr ? st : stream_k_sum(k.c, c, sk, stream);
    }
    if (plan.k_mode == MI_K_SPLIT_REDUCE) {
        // partition s of problem l stores its copy of C at partials[l][s]; the sum then writes the caller's C
        Canonical k = c;
        k.c = (float*)((char*)workspace + partial_off);
        k.c_split_bytes = (uint64_t)c.M * c.N * 4;
        k.c_batch_bytes = k.c_split_bytes * plan.k_splits;
        // the workgroup that stores a tile's last copy sums the tile (one counter per tile of every problem); without
        // counters a second launch does the summing
        TileDims d;
        tile_dims(plan.tile, c.K, d);
        const uint64_t tiles = (uint64_t)ceil_div(c.M, d.bm) * ceil_div(c.N, d.bn) * c.batches;
        // (whole tiles only: the range-checked build of the kernel does not carry the sum)
        k.tile_counters = attributes_only || needs_edge(k, d) ? nullptr : tile_counters_for(workspace_owner ? workspace_owner : workspace, tiles);
        k.c_final = c.c;
        k.ldc_final = c.ldc;
        k.c_final_batch_bytes = c.c_batch_bytes;
        const int st = launch_tile(t->ab_dtype, k, plan, stream);
        if (st == MI_OK && k.tile_counters != nullptr) {
            calls_summed_in_launch.fetch_add(1, std::memory_order_relaxed);
        }
        return st || attributes_only || k.tile_counters != nullptr ? st : reduce_partials(k.c, c, plan.k_splits, stream);
    }
    if (plan.k_splits > 1 && !attributes_only) {
        // partial sums are atomically added: C must start at zero (gemm/gemm_sm90.cu:1208-1210).  A fill kernel,
        // not hipMemsetAsync, so the call stays safe to capture into a HIP graph.
        const size_t per_problem = (size_t)c.M * c.N;
        const bool dense = c.batches == 1 || c.c_batch_bytes == per_problem * 4;
        const size_t n = dense ? per_problem * c.batches : per_problem;
        size_t blocks = (n + 255) / 256;
        blocks = blocks > 8192 ? 8192 : blocks;
        for (uint32_t l = 0; l < (dense ? 1u : c.batches); ++l) {
            float* const dst = (float*)((char*)c.c + (size_t)l * c.c_batch_bytes);
            hipLaunchKernelGGL(zero_fill_kernel, dim3((uint32_t)blocks), dim3(256), 0, stream, dst, n);
            MI_CHECK_LAUNCH();
        }
    }
    return launch_tile(t->ab_dtype, c, plan, stream);
}

}  // namespace mi_gemm

using namespace mi_gemm;

// MI_GEMM_PLANNER_CONSTANTS="256x256=1.26/16.1,64x128=0.31/5.4": the line `gemm --calibrate` prints for the machine at
// hand, applied when the library is loaded.  Entries that do not parse or name no tile are reported and skipped.
static int apply_planner_environment()
{
    const char* const text = std::getenv("MI_GEMM_PLANNER_CONSTANTS");
    if (text == nullptr) {
        return 0;
    }
    int applied = 0;
    for (const char* at = text; *at != 0;) {
        const char* end = std::strchr(at, ',');
        end = end ? end : at + std::strlen(at);
        char name[32];
        double k64 = 0, fixed = 0;
        int used = 0;
        bool ok = false;
        if (std::sscanf(at, " %31[0-9x]=%lf/%lf %n", name, &k64, &fixed, &used) == 3 && at + used == end) {
            for (int tile = 1; tile <= TILE_ROWS && !ok; ++tile) {
                ok = std::strcmp(TILES[tile - 1].name, name) == 0 && mi_tile_set_planner_constants(tile, k64, fixed) == MI_OK;
            }
        }
        if (ok) {
            ++applied;
        }
        else {
            std::fprintf(stderr, "mi_gemm: MI_GEMM_PLANNER_CONSTANTS: skipped '%.*s'\n", (int)(end - at), at);
        }
        at = *end ? end + 1 : end;
    }
    return applied;
}
static const int planner_environment_applied = apply_planner_environment();

extern "C" {

int mi_matmul_mfma_plan(const mi_gemm_tensors* t, int k_mode, int tile, int* out_tile, int* out_k_mode, int* out_k_splits)
{
    if (const int st = check_modes(t, k_mode, tile)) {
        return st;
    }
    const Prepared p = prepare(*t);
    Plan plan;
    const bool needs_room = k_mode == MI_K_SPLIT_REDUCE || k_mode == MI_K_STREAM;
    if (p.ws_bytes > 0 || !make_plan(p.c, k_mode, tile, needs_room ? SIZE_MAX : 0, plan)) {
        return MI_ERR_UNSUPPORTED;
    }
    if (out_tile) {
        *out_tile = plan.tile;
    }
    if (out_k_mode) {
        *out_k_mode = plan.k_mode;
    }
    if (out_k_splits) {
        *out_k_splits = (int)plan.k_splits;
    }
    return MI_OK;
}

static int describe_plan(const mi_gemm_tensors* t, int k_mode, int tile, size_t workspace_bytes, char* out, size_t out_size,
                         double* out_us)
{
    out[0] = 0;
    if (const int st = check_modes(t, k_mode, tile)) {
        return st;
    }
    const Prepared p = prepare(*t);
    if (p.ws_bytes > workspace_bytes) {
        return workspace_bytes ? MI_ERR_WORKSPACE : MI_ERR_UNSUPPORTED;
    }
    const size_t partial_off = round_up(p.ws_bytes, 256);
    const size_t partial_space = workspace_bytes > partial_off ? workspace_bytes - partial_off : 0;
    Plan plan;
    if (!make_plan(p.c, k_mode, tile, partial_space, plan)) {
        const bool needs_room = k_mode == MI_K_SPLIT_REDUCE || k_mode == MI_K_STREAM;
        return needs_room && make_plan(p.c, k_mode, tile, SIZE_MAX, plan) ? MI_ERR_WORKSPACE : MI_ERR_UNSUPPORTED;
    }
    auto one = [](char* dst, size_t n, const char* what, const Canonical& c, const Plan& pl) {
        const int once = read_once_operand(c, pl);  // (named in the kernel's terms: after the swap for column-major C)
        const char* const tail = once == 1 ? ", A non-temporal" : once == 2 ? ", B non-temporal" : "";
        if (pl.k_splits > 1) {
            return snprintf(dst, n, "%s%ux%ux%u %s %s x%u%s", what, c.M, c.N, c.K, mi_tile_name(pl.tile),
                            mi_k_mode_name(pl.k_mode), pl.k_splits, tail);
        }
        return snprintf(dst, n, "%s%ux%ux%u %s %s%s", what, c.M, c.N, c.K, mi_tile_name(pl.tile), mi_k_mode_name(pl.k_mode), tail);
    };
    size_t used = 0;
    auto append = [&](const char* what, const Canonical& c, const Plan& pl) {
        if (used < out_size) {
            const int n = one(out + used, out_size - used, what, c, pl);
            used += n > 0 ? (size_t)n : 0;
        }
    };
    if (p.repack_a || p.repack_b) {
        used = (size_t)snprintf(out, out_size, "re-pack %s%s%s, then ", p.repack_a ? "A" : "", p.repack_a && p.repack_b ? " and " : "",
                                p.repack_b ? "B" : "");
    }
    prefer_peeling_to_stream_k(p.c, k_mode, tile, plan);
    if (tile == MI_TILE_AUTO && plan.k_mode == MI_K_OUTPUT_STATIONARY) {
        const Peel peel = plan_peeled(p.c, device_compute_units(), plan.cost_us);
        if (peel.on) {
            append("peeled: ", peel_interior(p.c, peel), peel.interior_plan);
            if (peel.Mi < p.c.M) {
                append(" + bottom ", peel_bottom(p.c, peel), peel.bottom_plan);
            }
            if (peel.Ni < p.c.N) {
                append(" + right ", peel_right(p.c, peel), peel.right_plan);
            }
            *out_us = peel.cost_us;
            return MI_OK;
        }
    }
    append("", p.c, plan);
    *out_us = plan.cost_us;
    return MI_OK;
}

int mi_matmul_mfma_describe(const mi_gemm_tensors* t, int k_mode, int tile, size_t workspace_bytes, char* out, size_t out_size)
{
    if (!out || out_size == 0) {
        return MI_ERR_BAD_ARGUMENT;
    }
    double us = 0.0;
    return describe_plan(t, k_mode, tile, workspace_bytes, out, out_size, &us);
}

int mi_matmul_mfma_estimate_us(const mi_gemm_tensors* t, int k_mode, int tile, size_t workspace_bytes, double* out_us)
{
    if (!out_us) {
        return MI_ERR_BAD_ARGUMENT;
    }
    char text[64];
    *out_us = 0.0;
    return describe_plan(t, k_mode, tile, workspace_bytes, text, sizeof text, out_us);
}

int mi_matmul_mfma_supports(const mi_gemm_tensors* t, int k_mode, int tile)
{
    return mi_matmul_mfma_plan(t, k_mode, tile, nullptr, nullptr, nullptr) == MI_OK ? 1 : 0;
}

int mi_matmul_mfma(const mi_gemm_tensors* t, int k_mode, int tile, void* hip_stream)
{
    return run_mfma(t, k_mode, tile, nullptr, 0, hip_stream);
}

int mi_matmul_mfma_timeline(const mi_gemm_tensors* t, int k_mode, int tile, uint64_t* d_stamps, uint32_t slots_per_workgroup,
                            uint32_t max_workgroups, uint32_t* out_workgroups, void* hip_stream)
{
    if (!d_stamps || slots_per_workgroup == 0 || max_workgroups == 0 || (uintptr_t)d_stamps % 8) {
        return MI_ERR_BAD_ARGUMENT;
    }
    static_assert(sizeof(unsigned long long) == sizeof(uint64_t), "stamp width");
    const TimelineRequest req{reinterpret_cast<unsigned long long*>(d_stamps), slots_per_workgroup, max_workgroups,
                              out_workgroups};
    return run_mfma(t, k_mode, tile, nullptr, 0, hip_stream, &req);
}

int mi_matmul_mfma_batched(const mi_gemm_tensors* t, uint32_t batches, uint64_t a_batch_stride, uint64_t b_batch_stride,
                           uint64_t c_batch_stride, int k_mode, int tile, void* hip_stream)
{
    if (!t || batches == 0) {
        return MI_ERR_BAD_ARGUMENT;
    }
    // 0 = densely packed, the reference's A[L,M,K], B[L,N,K], C[L,...] (xgemm_Sm90.py:45-48)
    const BatchRequest req{batches, a_batch_stride ? a_batch_stride : (uint64_t)t->M * t->K,
                           b_batch_stride ? b_batch_stride : (uint64_t)t->N * t->K,
                           c_batch_stride ? c_batch_stride : (uint64_t)t->M * t->N};
    if (req.c_stride < (uint64_t)t->M * t->N) {
        return MI_ERR_BAD_ARGUMENT;  // the problems' C matrices would overlap
    }
    return run_mfma(t, k_mode, tile, nullptr, 0, hip_stream, nullptr, &req);
}

// fp32 operands: sizes of the converted copies and the equivalent bf16 problem
struct F32Prepared {
    mi_gemm_tensors bf16;      // the bf16 problem the MFMA kernel runs: both operands K-contiguous, depth terms*kp
    uint32_t terms, kp;
    size_t ws_b, ws_bytes;     // A copy at 0, B copy at ws_b
};

// `batches` problems of t's shape whose converted copies lie one after the other
static int prepare_f32(const mi_gemm_tensors* t, int precision, F32Prepared& f, uint32_t batches = 1)
{
    if (!t || t->ab_dtype != MI_F32 || (precision != MI_F32_BF16X1 && precision != MI_F32_BF16X3) || batches == 0) {
        return MI_ERR_BAD_ARGUMENT;
    }
    mi_gemm_tensors probe = *t;
    probe.ab_dtype = MI_BF16;
    if (const int st = validate_tensors(&probe)) {
        return st;
    }
    if ((uintptr_t)t->a % 4 || (uintptr_t)t->b % 4) {
        return MI_ERR_BAD_ARGUMENT;
    }
    f.terms = precision == MI_F32_BF16X3 ? 3 : 1;
    f.kp = (uint32_t)round_up(t->K, 8);
    const uint64_t depth = (uint64_t)f.terms * f.kp;
    if (depth >= (1u << 21)) {
        return MI_ERR_UNSUPPORTED;
    }
    f.ws_b = round_up((size_t)batches * t->M * depth * 2, 256);
    f.ws_bytes = f.ws_b + round_up((size_t)batches * t->N * depth * 2, 256);
    f.bf16 = *t;
    f.bf16.ab_dtype = MI_BF16;
    f.bf16.K = (uint32_t)depth;
    f.bf16.a_col_major = 0;  // the converted copies are M x depth and N x depth, depth contiguous
    f.bf16.b_col_major = 1;
    return MI_OK;
}

int mi_matmul_f32_workspace_bytes(const mi_gemm_tensors* t, int precision, size_t* out_bytes)
{
    F32Prepared f;
    if (!out_bytes) {
        return MI_ERR_BAD_ARGUMENT;
    }
    if (const int st = prepare_f32(t, precision, f)) {
        return st;
    }
    *out_bytes = f.ws_bytes;
    return MI_OK;
}

// `batches` problems, densely packed (A[L,M,K], B[L,N,K] and C[L,..]); more than one only with both operands K-contiguous,
// where the L matrices of an operand read as one matrix of L times the rows.
static int run_f32(const mi_gemm_tensors* t, uint32_t batches, int precision, int k_mode, int tile, void* d_workspace,
                   size_t workspace_bytes, void* hip_stream)
{
    F32Prepared f;
    if (const int st = prepare_f32(t, precision, f, batches)) {
        return st;
    }
    if (batches > 1 && (t->a_col_major || !t->b_col_major)) {
        return MI_ERR_UNSUPPORTED;
    }
    if (!d_workspace || workspace_bytes < f.ws_bytes || (uintptr_t)d_workspace % 256) {
        return MI_ERR_WORKSPACE;
    }
    f.bf16.a = d_workspace;
    f.bf16.b = (char*)d_workspace + f.ws_b;
    if (const int st = check_modes(&f.bf16, k_mode, tile)) {
        return st;
    }
    // Refuse before converting anything if the bf16 problem itself cannot run with what the call will give it: the K
    // partitions' copies of C get what the converted operands leave of the workspace, and nothing when problems are batched.
    const size_t used = round_up(f.ws_bytes, 256);
    const size_t partial_space = batches > 1 || workspace_bytes <= used ? 0 : workspace_bytes - used;
    {
        Prepared p = prepare(f.bf16);
        p.c.batches = batches;
        if (batches > 1) {
            p.c.a_batch_bytes = (uint64_t)t->M * f.bf16.K * 2;
            p.c.b_batch_bytes = (uint64_t)t->N * f.bf16.K * 2;
            p.c.c_batch_bytes = (uint64_t)t->M * t->N * 4;
        }
        Plan plan;
        if (p.ws_bytes > 0) {
            return MI_ERR_UNSUPPORTED;
        }
        if (!make_plan(p.c, k_mode, tile, partial_space, plan)) {
            const bool needs_room = k_mode == MI_K_SPLIT_REDUCE || k_mode == MI_K_STREAM;
            return needs_room && make_plan(p.c, k_mode, tile, SIZE_MAX, plan) ? MI_ERR_WORKSPACE : MI_ERR_UNSUPPORTED;
        }
    }
    hipStream_t stream = as_stream(hip_stream);
    // A as [hi | hi | lo], B as [hi | lo | hi]: the depth-3K product is Ahi*Bhi + Ahi*Blo + Alo*Bhi
    const uint32_t a_lo_mask = f.terms == 3 ? 0b100u : 0u, b_lo_mask = f.terms == 3 ? 0b010u : 0u;
    const struct {
        const void* src;
        void* dst;
        uint32_t rows;
        int k_contiguous;
        uint32_t lo_mask;
    } ops[2] = {{t->a, const_cast<void*>(f.bf16.a), t->M, !t->a_col_major, a_lo_mask},
                {t->b, const_cast<void*>(f.bf16.b), t->N, t->b_col_major != 0, b_lo_mask}};
    auto aligned_rows = [&](const auto& op) { return op.k_contiguous && t->K % 8 == 0 && (uintptr_t)op.src % 16 == 0; };
    for (const auto& op : ops) {
        // (only the element-by-element kernel puts the rows into grid.y; the other two have no such limit)
        if (op.k_contiguous && !aligned_rows(op) && ((uint64_t)batches * op.rows + 63) / 64 > 65535u) {
            return MI_ERR_UNSUPPORTED;
        }
        if ((uint64_t)batches * op.rows > 0xffffffffull) {
            return MI_ERR_UNSUPPORTED;
        }
    }
    for (const auto& op : ops) {
        const uint32_t rows = batches * op.rows;
        if (aligned_rows(op)) {
            const uint64_t chunks = (uint64_t)rows * (t->K / 8);
            const uint64_t blocks = (chunks + 255) / 256;
            hipLaunchKernelGGL(split_f32_rows_kernel, dim3((uint32_t)(blocks < 16384 ? blocks : 16384)), dim3(256), 0, stream,
                               (const float*)op.src, (uint16_t*)op.dst, chunks, t->K / 8, f.terms, op.lo_mask);
            MI_CHECK_LAUNCH();
            continue;
        }
        if (!op.k_contiguous) {
            hipLaunchKernelGGL(split_f32_transposed_kernel, dim3((rows + 63) / 64, (f.kp + 127) / 128, 1), dim3(256), 0, stream,
                               (const float*)op.src, (uint16_t*)op.dst, rows, t->K, f.kp, f.terms, op.lo_mask);
            MI_CHECK_LAUNCH();
            continue;
        }
        const dim3 grid((f.kp + 63) / 64, (rows + 63) / 64, 1);
        hipLaunchKernelGGL(split_f32_kernel, grid, dim3(256), 0, stream, (const float*)op.src, (uint16_t*)op.dst, rows, t->K,
                           f.kp, f.terms, op.lo_mask);
        MI_CHECK_LAUNCH();
    }
    if (batches > 1) {
        const BatchRequest req{batches, (uint64_t)t->M * f.bf16.K, (uint64_t)t->N * f.bf16.K, (uint64_t)t->M * t->N};
        return run_mfma(&f.bf16, k_mode, tile, nullptr, 0, hip_stream, nullptr, &req);
    }
    // what the converted operands leave of the workspace may hold K partitions' copies of C
    if (workspace_bytes > used) {
        return run_mfma(&f.bf16, k_mode, tile, (char*)d_workspace + used, workspace_bytes - used, hip_stream, nullptr, nullptr, false,
                        d_workspace);
    }
    return run_mfma(&f.bf16, k_mode, tile, nullptr, 0, hip_stream);
}

int mi_matmul_f32_ws(const mi_gemm_tensors* t, int precision, int k_mode, int tile, void* d_workspace, size_t workspace_bytes,
                     void* hip_stream)
{
    return run_f32(t, 1, precision, k_mode, tile, d_workspace, workspace_bytes, hip_stream);
}

// The operand bundle of one xgemm problem, or an error for sizes the reference's procs assert away
// (xgemm_Sm80.py:19-21, xgemm_Sm90.py:49-54: every size positive).
static int xgemm_tensors(int64_t M, int64_t N, int64_t K, const float* a, const float* b, float* c, bool b_col_major,
                         bool c_col_major, mi_gemm_tensors& t)
{
    if (M <= 0 || N <= 0 || K <= 0 || M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) {
        return MI_ERR_BAD_ARGUMENT;
    }
    t = mi_gemm_tensors{};
    t.M = (uint32_t)M;
    t.N = (uint32_t)N;
    t.K = (uint32_t)K;
    t.a = a;
    t.b = b;
    t.c = c;
    t.a_col_major = 0;
    t.b_col_major = b_col_major;
    t.c_col_major = c_col_major;
    t.ab_dtype = MI_F32;
    return MI_OK;
}

int mi_xgemm_workspace_bytes(int L, int M, int N, int K, int precision, size_t* out_bytes)
{
    mi_gemm_tensors t;
    F32Prepared f;
    if (!out_bytes || L <= 0) {
        return MI_ERR_BAD_ARGUMENT;
    }
    // (sizes only: the pointers are placeholders that pass the alignment checks)
    alignas(256) static const float placeholder[64] = {};
    if (const int st = xgemm_tensors(M, N, K, placeholder, placeholder, const_cast<float*>(placeholder), true, true, t)) {
        return st;
    }
    if (const int st = prepare_f32(&t, precision, f, (uint32_t)L)) {
        return st;
    }
    *out_bytes = f.ws_bytes;
    return MI_OK;
}

// The reference's harness passes ctxt = nullptr (gemm/gemm_test.cu:326,335) and runs on stream 0.  A null context here
// means the same call form: stream 0, MI_F32_BF16X3, MI_TILE_AUTO, and the library-resident scratch array of
// mi_matmul_mfma_static for the converted operands (MI_ERR_WORKSPACE when they do not fit it).
static int resolve_xgemm_context(const mi_xgemm_context* ctxt, const mi_gemm_tensors& t, uint32_t batches, mi_xgemm_context& out)
{
    if (ctxt != nullptr) {
        out = *ctxt;
        return MI_OK;
    }
    // (sizes first, so that a problem that cannot fit is refused before any device call)
    F32Prepared f;
    if (const int st = prepare_f32(&t, MI_F32_BF16X3, f, batches)) {
        return st;
    }
    if (f.ws_bytes > STATIC_SCRATCH_BYTES) {
        return MI_ERR_WORKSPACE;
    }
    void* ptr = nullptr;
    if (const int st = resolve_static_scratch(&ptr)) {
        return st;
    }
    out = mi_xgemm_context{ptr, STATIC_SCRATCH_BYTES, nullptr, MI_F32_BF16X3, MI_TILE_AUTO};
    return MI_OK;
}

int mi_xgemm_Sm80(const mi_xgemm_context* ctxt, int M, int N, int K, const float* A, const float* B, float* C)
{
    mi_gemm_tensors t;
    mi_xgemm_context cx;
    if (const int st = xgemm_tensors(M, N, K, A, B, C, false, false, t)) {
        return st;
    }
    if (const int st = resolve_xgemm_context(ctxt, t, 1, cx)) {
        return st;
    }
    return run_f32(&t, 1, cx.precision, MI_K_AUTO, cx.tile, cx.d_workspace, cx.workspace_bytes, cx.hip_stream);
}

int mi_xgemm_Sm90_wgmma(const mi_xgemm_context* ctxt, int L, int M, int N, int K_splits, int cluster_k, const float* A,
                        const float* B, float* C)
{
    mi_gemm_tensors t;
    mi_xgemm_context cx;
    if (L <= 0 || K_splits <= 0 || cluster_k <= 0) {
        return MI_ERR_BAD_ARGUMENT;
    }
    if (const int st = xgemm_tensors(M, N, (int64_t)K_splits * cluster_k, A, B, C, true, true, t)) {
        return st;
    }
    if (const int st = resolve_xgemm_context(ctxt, t, (uint32_t)L, cx)) {
        return st;
    }
    // K_splits > 1 is the reference's split-K build, which zero-fills C and lets the K tasks add into it
    // (xgemm_Sm90.py:60-61,65): the same request here, with the number of partitions left to the planner
    return run_f32(&t, (uint32_t)L, cx.precision, K_splits > 1 ? MI_K_SPLIT : MI_K_AUTO, cx.tile, cx.d_workspace,
                   cx.workspace_bytes, cx.hip_stream);
}

int mi_matmul_mfma_workspace_bytes(const mi_gemm_tensors* t, size_t* out_bytes)
{
    if (!out_bytes) {
        return MI_ERR_BAD_ARGUMENT;
    }
    *out_bytes = 0;
    if (const int st = validate_tensors(t)) {
        return st;
    }
    const Prepared p = prepare(*t);
    Plan plan;
    if (!make_plan(p.c, MI_K_AUTO, MI_TILE_AUTO, 0, plan)) {
        return MI_ERR_UNSUPPORTED;
    }
    *out_bytes = p.ws_bytes;
    return MI_OK;
}

int mi_matmul_mfma_workspace_bytes_for(const mi_gemm_tensors* t, int k_mode, int tile, size_t* out_required,
                                       size_t* out_preferred)
{
    if (!out_required || !out_preferred) {
        return MI_ERR_BAD_ARGUMENT;
    }
    *out_required = *out_preferred = 0;
    if (const int st = check_modes(t, k_mode, tile)) {
        return st;
    }
    const Prepared p = prepare(*t);
    Plan plan;
    if (!make_plan(p.c, k_mode, tile, SIZE_MAX, plan)) {
        return MI_ERR_UNSUPPORTED;
    }
    prefer_peeling_to_stream_k(p.c, k_mode, tile, plan);
    const size_t with_partials = round_up(p.ws_bytes, 256) + partial_bytes(p.c, plan.k_splits);
    *out_preferred = plan.k_mode == MI_K_SPLIT_REDUCE ? with_partials : p.ws_bytes;
    *out_required = p.ws_bytes;
    if (plan.k_mode == MI_K_STREAM) {
        const int cus = device_compute_units();
        StreamKLayout sk;
        if (!stream_k_layout(p.c, plan.tile, cus, sk)) {
            return MI_ERR_UNSUPPORTED;
        }
        *out_preferred = round_up(p.ws_bytes, 256) + sk.bytes();
        if (k_mode == MI_K_STREAM) {
            // the forced mode runs with whatever holds the parts of the tile that needs the least room
            size_t least = SIZE_MAX;
            for (int tl = tile == MI_TILE_AUTO ? 1 : tile; tl <= (tile == MI_TILE_AUTO ? MI_TILE_COUNT_ - 1 : tile); ++tl) {
                if (stream_k_layout(p.c, tl, cus, sk) && sk.bytes() < least) {
                    least = sk.bytes();
                }
            }
            *out_required = round_up(p.ws_bytes, 256) + least;
        }
    }
    if (k_mode == MI_K_SPLIT_REDUCE && plan.k_splits > 1) {
        // the forced mode runs with any room that holds the fewest copies some tile can be split into
        const int tile_lo = tile == MI_TILE_AUTO ? 1 : tile;
        const int tile_hi = tile == MI_TILE_AUTO ? MI_TILE_COUNT_ - 1 : tile;
        for (uint32_t splits = 2; splits <= plan.k_splits; ++splits) {
            bool fits = false;
            for (int tl = tile_lo; tl <= tile_hi && !fits; ++tl) {
                fits = tile_fits(p.c, tl, splits);
            }
            if (fits) {
                *out_required = round_up(p.ws_bytes, 256) + partial_bytes(p.c, splits);
                break;
            }
        }
    }
    return MI_OK;
}

int mi_matmul_mfma_ws(const mi_gemm_tensors* t, int k_mode, int tile, void* d_workspace, size_t workspace_bytes,
                      void* hip_stream)
{
    if (const int st = validate_tensors(t)) {
        return st;
    }
    const size_t need = prepare(*t).ws_bytes;
    if (need > 0 && (!d_workspace || workspace_bytes < need)) {
        return MI_ERR_WORKSPACE;
    }
    return run_mfma(t, k_mode, tile, d_workspace, d_workspace ? workspace_bytes : 0, hip_stream);
}

int mi_matmul_mfma_sum_in_launch(int enable, uint64_t* out_calls)
{
    const bool was = enable < 0 ? sum_in_launch.load() : sum_in_launch.exchange(enable != 0);
    if (out_calls) {
        *out_calls = calls_summed_in_launch.load();
    }
    return was ? 1 : 0;
}

int mi_matmul_mfma_prepare(const mi_gemm_tensors* t, int k_mode, int tile, size_t workspace_bytes)
{
    if (const int st = check_modes(t, k_mode, tile)) {
        return st;
    }
    // the plan depends on the workspace's size only (and on its presence): a stand-in address with the alignment the
    // call asks for keeps the planner on the path the real call takes; nothing is read or written through it
    void* const stand_in = workspace_bytes ? reinterpret_cast<void*>(uintptr_t(256)) : nullptr;
    if (workspace_bytes && prepare(*t).ws_bytes > workspace_bytes) {
        return MI_ERR_WORKSPACE;
    }
    if (workspace_bytes) {
        (void)resolve_tile_counters();  // (an address look-up that the captured call then need not make)
    }
    return run_mfma(t, k_mode, tile, stand_in, workspace_bytes, nullptr, nullptr, nullptr, true);
}

int mi_matmul_mfma_static(const mi_gemm_tensors* t, int k_mode, int tile, void* hip_stream)
{
    if (const int st = check_modes(t, k_mode, tile)) {
        return st;
    }
    // what must fit: the re-packed operands (the K partitions' copies of C take what is left, or K splits by atomics)
    if (prepare(*t).ws_bytes > STATIC_SCRATCH_BYTES) {
        return MI_ERR_WORKSPACE;
    }
    void* ptr = nullptr;
    if (const int st = resolve_static_scratch(&ptr)) {
        return st;
    }
    return run_mfma(t, k_mode, tile, ptr, STATIC_SCRATCH_BYTES, hip_stream);
}

int mi_tile_count(void)
{
    return MI_TILE_COUNT_;
}

const char* mi_tile_name(int tile)
{
    if (tile == MI_TILE_AUTO) {
        return "auto";
    }
    const TileRow* const row = tile_row(tile);
    return row != nullptr ? row->name : "unknown";
}

int mi_tile_shape(int tile, uint32_t* out_bm, uint32_t* out_bn, int* out_workgroups_per_cu, int* out_has_32_deep_twin)
{
    const TileRow* const row = tile_row(tile);
    if (row == nullptr) {
        return MI_ERR_BAD_ARGUMENT;
    }
    if (out_bm) {
        *out_bm = row->bm;
    }
    if (out_bn) {
        *out_bn = row->bn;
    }
    if (out_workgroups_per_cu) {
        *out_workgroups_per_cu = row->per_cu;
    }
    if (out_has_32_deep_twin) {
        *out_has_32_deep_twin = row->twin[0] != nullptr ? 1 : 0;
    }
    return MI_OK;
}

int mi_tile_planner_constants(int tile, double* out_us_per_k64, double* out_fixed_us)
{
    const TileRow* const row = tile_row(tile);
    if (row == nullptr) {
        return MI_ERR_BAD_ARGUMENT;
    }
    if (out_us_per_k64) {
        *out_us_per_k64 = row->us_k64;
    }
    if (out_fixed_us) {
        *out_fixed_us = row->fixed_us;
    }
    return MI_OK;
}

int mi_tile_set_planner_constants(int tile, double us_per_k64, double fixed_us)
{
    if (tile_row(tile) == nullptr || !(us_per_k64 > 0.0) || !(fixed_us > 0.0) || us_per_k64 > 1e3 || fixed_us > 1e3) {
        return MI_ERR_BAD_ARGUMENT;
    }
    TileRow& row = TILES[tile - 1];
    // a tile that has a CU to itself has one pair of constants; the tile that shares a CU keeps its figures for a
    // workgroup running alone, scaled as the pair's are
    if (row.per_cu == 1) {
        row.alone_k64 = us_per_k64;
        row.alone_us = fixed_us;
    }
    else {
        row.alone_k64 *= us_per_k64 / row.us_k64;
        row.alone_us *= fixed_us / row.fixed_us;
    }
    row.short_us *= fixed_us / row.fixed_us;
    row.us_k64 = us_per_k64;
    row.fixed_us = fixed_us;
    planner_constants_generation.fetch_add(1, std::memory_order_relaxed);
    return MI_OK;
}

const char* mi_k_mode_name(int k_mode)
{
    switch (k_mode) {
    case MI_K_OUTPUT_STATIONARY: return "output stationary";
    case MI_K_SPLIT: return "split k";
    case MI_K_SPLIT_REDUCE: return "split k (workspace sum)";
    case MI_K_STREAM: return "stream k";
    case MI_K_AUTO: return "auto";
    }
    return "unknown";
}

}  // extern "C"
