/*
 * mi_gemm.h — C ABI of the MI355X (gfx950) dense GEMM library, libmi_gemm.so.
 *
 * This is the drop-in boundary for the GEMM entry points of the akeley98/spork testbed: plain C, plain
 * pointers and sizes, no C++ or framework types.  Every entry point names the reference interface it
 * replaces (paths relative to the reference repository).  All device pointers are owned by the caller; every
 * call enqueues asynchronously on the caller's HIP stream and never synchronises it (the reference harness
 * records events between launches, gemm/gemm_test.cu:282,388).  The reference returns void and asserts; a C
 * ABI cannot, so every call returns an int status (MI_OK == 0).
 */
#ifndef MI_GEMM_H
#define MI_GEMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---------------------------------------------------------------------------------------------- status */
enum {
    MI_OK = 0,
    MI_ERR_UNSUPPORTED = 1, /* shape / layout / dtype not handled by the requested algorithm            */
    MI_ERR_BAD_ARGUMENT = 2, /* null pointer, zero size, unknown enum, misaligned pointer                */
    MI_ERR_WORKSPACE = 3,    /* caller-provided workspace too small                                      */
    MI_ERR_HIP = 4,          /* a HIP runtime call failed; see mi_last_hip_error()                       */
    MI_ERR_NO_DEVICE = 5,    /* no gfx950 device visible                                                  */
};
/* Not every misuse has a status: two calls that use the same scratch memory while they overlap in time on one GPU - the same
 * workspace given to mi_matmul_mfma_ws on two streams, or any two overlapping calls of mi_matmul_mfma_static or of the Exo
 * entry points with a null context, which all share the library's one scratch array per GPU - are undefined (wrong results),
 * and are not detected. */
const char* mi_status_string(int status);
/* hipError_t of the most recent failing HIP call made by this library on the calling thread (0 if none). */
int mi_last_hip_error(void);
const char* mi_last_hip_error_string(void);

/* --------------------------------------------------------------------------------------------- tensors */
/* Element type of A and B.  C and the accumulator are always fp32. */
enum {
    MI_F16 = 0,
    MI_BF16 = 1,
    MI_F32 = 2 /* a and b are float, the reference's own element type; accepted by mi_matmul_f32_* only */
};

/* Replaces `struct GPU_Tensors` (gemm/gpu_tensor.h:9-21) — same fields, same meaning, with 16-bit A/B and a
 * dtype tag.  Index rules (gemm/gemm_baseline.cu:47-52,63-68,94-99):
 *   A[m,k] = a_col_major ? a[k*M+m] : a[m*K+k]
 *   B[k,n] = b_col_major ? b[n*K+k] : b[k*N+n]
 *   C[m,n] -> c_col_major ? c[n*M+m] : c[m*N+n]
 * The testbed's canonical call is {a_col_major=0, b_col_major=1, c_col_major=0} (gemm/gemm_test.cu:305,365). */
typedef struct mi_gemm_tensors {
    uint32_t M, N, K;
    const void* a; /* device memory, 2-byte elements */
    const void* b; /* device memory, 2-byte elements */
    float* c;      /* device memory */
    uint8_t a_col_major;
    uint8_t b_col_major;
    uint8_t c_col_major;
    uint8_t ab_dtype; /* MI_F16 | MI_BF16 (| MI_F32 for the mi_matmul_f32_* entry points) */
} mi_gemm_tensors;

/* ------------------------------------------------------------------------------------------ algorithms */
/* K scheduling modes; replaces `enum class gemm_sm90_k_mode` (gemm/gemm_sm90.h:5-12). */
enum {
    MI_K_OUTPUT_STATIONARY = 0, /* one workgroup owns an output tile for all of K                        */
    MI_K_SPLIT = 1,             /* K split across workgroups; C zero-filled by the callee, partials are
                                   reduced with fp32 atomic adds (gemm/gemm_sm90.cu:1096-1115,1208-1210)  */
    MI_K_AUTO = 2,              /* library picks by shape (and by the workspace it is given)              */
    MI_K_SPLIT_REDUCE = 3,      /* K split across workgroups; every partition stores its own copy of its tile of C in
                                   the caller's workspace and the copies are added in partition order into C: no zero
                                   fill, no floating-point atomics, the same bits on every run.  By a second kernel, or
                                   (mi_matmul_mfma_sum_in_launch) inside the one launch by the workgroup that stores a
                                   tile's last copy, as the reference's partitions meet in its epilogue
                                   (gemm/gemm_sm90.cu:944-963).  Only through mi_matmul_mfma_ws / mi_matmul_mfma_static /
                                   mi_matmul_f32_ws                                                                   */
    MI_K_STREAM = 4,            /* stream-K (the role of gemm_sm90_k_mode::stream_k_*, gemm/gemm_sm90.h:10-11), laid out
                                   as gemm/gemm_sm90.cu:1009-1030 lays it out: the tiles that fill whole rounds of CUs run
                                   output stationary; the tail tiles, fewer than a round, are split along K over one
                                   round of workgroups (as many equal partitions per tile as fit, the K tiles left over
                                   dealt in equal runs to the workgroups left over), so the chip is full whatever the
                                   tile count.  Every part goes to the workspace and each tail tile's parts are added in
                                   a fixed order into C, by a last kernel or (mi_matmul_mfma_sum_in_launch) by the
                                   workgroup that stores the tile's last part: the same bits on every run.  For problems
                                   of whole tiles (M, N multiples of the tile, K of 64), any tile count that is not a
                                   whole number of rounds; only through mi_matmul_mfma_ws / mi_matmul_mfma_static /
                                   mi_matmul_f32_ws                                                                   */
};

/* Workgroup tile family; replaces the n64/n128/n256 tile constructors (xgemm_Sm90.py:11-21,
 * xgemm_Sm90_n64.py:3, _n128.py:3, _n256.py:3), re-derived for gfx950 MFMA (16x16x32) and 64-wide waves. */
enum {
    MI_TILE_AUTO = 0,
    MI_TILE_256x256 = 1, /* 4 waves, wave tile 128x128 */
    MI_TILE_256x128 = 2, /* 4 waves, wave tile 128x64  */
    MI_TILE_128x128 = 3, /* 4 waves, wave tile 64x64   */
    MI_TILE_64x128 = 4,  /* 4 waves, wave tile 32x64 (tall-skinny, bandwidth-bound shapes) */
    MI_TILE_192x256 = 5, /* 4 waves, wave tile 96x128: three quarters of the largest tile, for tile counts that would
                            leave most of a last round of 256x256 tiles idle */
    MI_TILE_224x256 = 6, /* in-between heights (wave tiles 112x128, 80x128, 112x64, 80x64) for tile counts that */
    MI_TILE_160x256 = 7, /* would leave the last round of CUs part empty with the tiles above                   */
    MI_TILE_224x128 = 8,
    MI_TILE_160x128 = 9,
    MI_TILE_256x192 = 10, /* wave tile 64x192 (four waves along M): three quarters of the largest tile along N */
    MI_TILE_192x192 = 11, /* wave tile 48x192: 9/16 of the largest tile, for tile counts the others round badly */
    MI_TILE_192x128 = 12, /* wave tile 96x64 with a two-slot ring of 80 KB, so that two workgroups share a CU and one's
                             epilogue overlaps the other's main loop: for many rounds of tiles with a short K */
    MI_TILE_96x128 = 13,  /* wave tile 48x64: three quarters of the 128x128 tile, for small problems whose 128x128 tiles
                             fill 55 to 75 % of the CUs */
    MI_TILE_COUNT_
};

/* Replaces `void matmul_baseline(GPU_Tensors, cudaStream_t)` (gemm/gemm_baseline.h:5, .cu:129-168): slow,
 * obviously-correct fp32-FMA GEMM on the widened inputs, any shape, all 8 layout combinations.  It is the
 * on-device checker of the host driver, exactly the role it has in gemm/gemm_test.cu:264-268. */
int mi_matmul_baseline(const mi_gemm_tensors* t, void* hip_stream);

/* One 32x32 MFMA tile per wave, operands fetched straight from global memory (no LDS).  Needs the canonical
 * layout, M%32==0, N%32==0, K%16==0.  Exists to pin the MFMA lane<->element mapping on its own. */
int mi_matmul_mfma_direct(const mi_gemm_tensors* t, void* hip_stream);

/* Replaces `bool matmul_sm80_supports(GPU_Tensors)` (gemm/gemm_sm80.h:6, .cu:541-550): 1 if
 * mi_matmul_mfma(t, k_mode, tile, ...) can run this problem, else 0. */
int mi_matmul_mfma_supports(const mi_gemm_tensors* t, int k_mode, int tile);

/* Replaces `void matmul_sm80(GPU_Tensors, cudaStream_t)` (gemm/gemm_sm80.h:5) and
 * `void matmul_sm90(GPU_Tensors, gemm_sm90_k_mode, cudaStream_t)` (gemm/gemm_sm90.h:14): the LDS-tiled MFMA
 * GEMM.  Layout canonicalisation follows gemm/gemm_sm80.cu:516-539 (swap A/B and M/N so the kernel always
 * sees both operands K-contiguous).  Any M and N; K a multiple of 8; A and B 16-byte aligned and K-contiguous
 * (a_col_major = 0, b_col_major = 1); C row- or column-major.  MI_K_SPLIT zero-fills C on the stream first.  Uses no
 * scratch memory: problems that need re-packing (see mi_matmul_mfma_ws) are MI_ERR_UNSUPPORTED here. */
int mi_matmul_mfma(const mi_gemm_tensors* t, int k_mode, int tile, void* hip_stream);

/* Any layout, any K, through caller-provided scratch memory.  An operand that is not K-contiguous (a_col_major=1,
 * b_col_major=0), whose K is not a multiple of 8, or that is not 16-byte aligned is first re-packed (transposed and
 * zero-padded to a row pitch of K rounded up to 8) into the workspace, then the same MFMA kernel runs.  This is how
 * the reference's dispatchers accept every GPU_Tensors layout (gemm/gemm_sm80.cu:516-539, gemm/gemm_sm90.cu:1344-1360);
 * the workspace plays the role of StreamWorkspace::alloc_at_least (gemm/gpu_tensor.h:48-67) as matmul_cutlass uses it
 * (gemm/cutlass_gemm.cu:124-125).  mi_matmul_mfma_workspace_bytes gives the size (0 when nothing needs re-packing);
 * the workspace must be 256-byte aligned and is free for reuse once the stream has passed the call. */
int mi_matmul_mfma_workspace_bytes(const mi_gemm_tensors* t, size_t* out_bytes);
/* The same question for a given K mode and tile, with two answers.  `out_required`: below this mi_matmul_mfma_ws
 * returns MI_ERR_WORKSPACE (the re-packed operands; for MI_K_SPLIT_REDUCE also two copies of C, the fewest
 * partitions there can be).  `out_preferred`: the room the plan the library likes best would use
 * (k_splits * M * N * 4 bytes after the re-packed operands, rounded up to 256, when that plan is MI_K_SPLIT_REDUCE).
 * Between the two the planner works with what it gets: MI_K_SPLIT_REDUCE takes fewer partitions, MI_K_AUTO falls
 * back to MI_K_SPLIT, so the result's rounding, not its accuracy bound, depends on the workspace given. */
int mi_matmul_mfma_workspace_bytes_for(const mi_gemm_tensors* t, int k_mode, int tile, size_t* out_required,
                                       size_t* out_preferred);
int mi_matmul_mfma_ws(const mi_gemm_tensors* t, int k_mode, int tile, void* d_workspace, size_t workspace_bytes,
                      void* hip_stream);

/* mi_matmul_mfma_ws without the workspace argument, for callers that cannot allocate device memory: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference (its callers
 * bring a StreamWorkspace that allocates on demand, gemm/gpu_tensor.h:48-67).  The workspace is an array of
 * MI_STATIC_SCRATCH_BYTES inside the library's own code object; the call allocates and frees nothing.  Everything
 * mi_matmul_mfma_ws accepts is accepted as long as the re-packed operands fit (MI_ERR_WORKSPACE otherwise); K partitions
 * are summed from copies of C in what is left of the array, or fall back to atomics.  Each GPU the library runs on holds
 * its own copy of the array until the process ends.  All calls on one GPU share it: calls that overlap in time on one GPU
 * (two streams, two threads) race and must be serialised by the caller; calls on one stream are ordered.  Nothing in the
 * array needs clearing between calls (every byte a call reads was written by that call).  The array's address is looked
 * up at mi_rt_set_device, else on the first call on a device: make that first call outside a graph capture. */
#define MI_STATIC_SCRATCH_BYTES ((size_t)64 << 20)
int mi_matmul_mfma_static(const mi_gemm_tensors* t, int k_mode, int tile, void* hip_stream);

/* Where the parts of MI_K_SPLIT_REDUCE and MI_K_STREAM are summed: by a kernel launch of its own behind the GEMM (0, the
 * default), or inside the GEMM launch (1), where the workgroup that stores a tile's last part adds the tile's parts - the
 * reference's scheme (gemm/gemm_sm90.cu:944-963,1004-1095), with plain loads and stores in a fixed order in place of its
 * reduce-adds.  The results are the same bits either way.  The default is the faster way on MI355X on almost every shape
 * measured (2048 x 2048 x 65536 in four partitions: 412 against 425 us; 160 x 480 x 816 in seven: 7.7 against 12 us; level on
 * 16384 x 128 x 8192 in two): only one workgroup per tile sums where the extra launch puts every CU to it.  Inside the
 * launch the parts are stored and read back with device-coherent accesses (`sc1`), so no cache is written back or invalidated
 * as a whole.  Problems of whole tiles only: a ragged problem sums with the extra launch whatever the setting.
 * The sum inside the launch takes one arrival counter per tile, zero when the launch starts; the counters are an array in
 * the library's own code object (zero when it is loaded, left zero by every launch), dealt out in slabs of 4096 by
 * workspace address: calls that share a workspace are ordered by their caller anyway and share a slab, calls on different
 * workspaces may overlap and get slabs of their own.  A call that needs more counters than a slab holds, or finds all 256
 * slabs of the GPU taken by other workspaces, sums with the extra launch.
 * `enable` < 0 leaves the setting alone; returns the setting as it was.  *out_calls (may be NULL): how many calls of this
 * process have summed inside their launch so far.  The host driver's `--kmodes` prints both ways. */
int mi_matmul_mfma_sum_in_launch(int enable, uint64_t* out_calls);

/* Sets up, once per device, what the first launch of a kernel would otherwise set up on the fly (the opt-in to more
 * than 64 KB of dynamic LDS, gemm/gemm_sm80.cu:473-475; the reference does it under std::call_once,
 * gemm/gemm_sm90.cu:1218-1219): every GEMM kernel that mi_matmul_mfma (workspace_bytes = 0) or mi_matmul_mfma_ws /
 * mi_matmul_mfma_static (workspace_bytes = the size that call will be given) would launch for this problem, mode and tile.
 * Launches nothing and touches no operand.  For callers that capture the call into a HIP graph without a warm-up call:
 * a kernel's attributes cannot be set while its stream is capturing, so either call this first or make one eager call. */
int mi_matmul_mfma_prepare(const mi_gemm_tensors* t, int k_mode, int tile, size_t workspace_bytes);

/* `batches` independent problems of one shape in one launch: problem l reads a + l*a_batch_stride and
 * b + l*b_batch_stride (16-bit elements) and writes c + l*c_batch_stride (floats); a stride of 0 means densely packed
 * (M*K, N*K, M*N).  This is the leading `L` dimension of the reference's generated kernels,
 * `xgemm_Sm90_wgmma(L, M, N, K_splits, cluster_k, A[L,M,..], B[L,N,..], C[L,N,M])` (xgemm_Sm90.py:43-48, called with
 * L = 1 at gemm/gemm_test.cu:335); its C[L,N,M] is c_col_major = 1 here.  All problems share one grid, so small
 * problems fill the chip together.  Same operand constraints as mi_matmul_mfma, plus batch strides of A and B that are
 * multiples of 8 elements.  MI_K_SPLIT zero-fills every problem's C. */
int mi_matmul_mfma_batched(const mi_gemm_tensors* t, uint32_t batches, uint64_t a_batch_stride,
                           uint64_t b_batch_stride, uint64_t c_batch_stride, int k_mode, int tile, void* hip_stream);

/* fp32 A and B - what the reference's GPU_Tensors carries (gemm/gpu_tensor.h:14-16) and its kernels feed to TF32
 * tensor-core instructions (gemm/gemm_sm80.cu:92-101).  gfx950 has no TF32 MFMA, so the operands are converted on the
 * device into the caller's workspace and run through the bf16 kernel:
 *   MI_F32_BF16X1  each value rounded to one bf16 (8 significant bits; TF32 keeps 11), 1x the bf16 work;
 *   MI_F32_BF16X3  each value split into hi + lo bf16 (16 significant bits) and
 *                  C = Ahi*Bhi + Ahi*Blo + Alo*Bhi computed as ONE GEMM of depth 3K on the operands
 *                  [Ahi|Ahi|Alo] and [Bhi|Blo|Bhi], 3x the bf16 work, more accurate than TF32.
 * t->ab_dtype must be MI_F32; every layout flag and any K are accepted (the conversion pass re-packs anyway).
 * The workspace must be 256-byte aligned; mi_matmul_f32_workspace_bytes gives its size. */
enum { MI_F32_BF16X1 = 0, MI_F32_BF16X3 = 1 };
int mi_matmul_f32_workspace_bytes(const mi_gemm_tensors* t, int precision, size_t* out_bytes);
int mi_matmul_f32_ws(const mi_gemm_tensors* t, int precision, int k_mode, int tile, void* d_workspace,
                     size_t workspace_bytes, void* hip_stream);

/* The C entry points that the reference's Exo procs compile to, with their argument lists:
 *   xgemm_Sm80_fence / xgemm_Sm80_mbarrier (ctxt, M, N, K, A f32[M,K], B f32[K,N], C f32[M,N])      xgemm_Sm80.py:18-21
 *   xgemm_Sm90_wgmma_n{64,128,256}[_tma_to_gmem|_split_k]
 *       (ctxt, L, M, N, K_splits, cluster_k, A f32[L,M,K_splits,cluster_k], B f32[L,N,K_splits,cluster_k],
 *        C f32[L,N,M])                                                                           xgemm_Sm90.py:43-48
 * called at gemm/gemm_test.cu:288-294,326-362 (the Sm90 ones with the operands swapped, so that C[L,N,M] comes out as
 * the harness's row-major M x N).  All tensors are dense and row-major in the order written; K = K_splits * cluster_k.
 * The reference passes ctxt = nullptr, its generated code needing nothing from the caller, and runs these on stream 0
 * only (gemm/gemm_test.cu:289,325).  This library never allocates, so ctxt brings the scratch memory the fp32 operands
 * are converted into, and the stream.  ctxt = NULL is the reference's call form: stream 0, MI_F32_BF16X3, MI_TILE_AUTO,
 * and the scratch array of mi_matmul_mfma_static (MI_STATIC_SCRATCH_BYTES, shared by every such call on a GPU: calls that
 * overlap in time race); MI_ERR_WORKSPACE when mi_xgemm_workspace_bytes(...) exceeds it (1024^3 takes 12 MiB, 8192^3 768).  K_splits > 1 selects what the reference's
 * split-K build does - C zero-filled, K partitions added into it (xgemm_Sm90.py:60-61) - with the number of
 * partitions chosen by the planner; the sum is the same.  The procs' divisibility assertions (M % 192, N % 256,
 * K % 16, cluster_k % 4) are limits of those kernels, not of the interface: every positive size is accepted.
 * L problems run in one launch after one conversion pass over each operand. */
typedef struct mi_xgemm_context {
    void* d_workspace;      /* 256-byte aligned device memory, at least mi_xgemm_workspace_bytes(...) */
    size_t workspace_bytes;
    void* hip_stream;
    int precision;          /* MI_F32_BF16X1 | MI_F32_BF16X3 */
    int tile;               /* MI_TILE_AUTO, or the tile that stands for an n64 / n128 / n256 variant */
} mi_xgemm_context;
int mi_xgemm_workspace_bytes(int L, int M, int N, int K, int precision, size_t* out_bytes);
int mi_xgemm_Sm80(const mi_xgemm_context* ctxt, int M, int N, int K, const float* A, const float* B, float* C);
int mi_xgemm_Sm90_wgmma(const mi_xgemm_context* ctxt, int L, int M, int N, int K_splits, int cluster_k, const float* A,
                        const float* B, float* C);

/* Diagnostic: the launch mi_matmul_mfma would make, with every workgroup recording time stamps so that a host tool
 * can show where a launch spends its time (per phase, per workgroup, per XCD).  Complements the whole-launch event
 * timing of the reference harness (gemm/gemm_test.cu:392-404), which has no in-kernel view.  Workgroup g writes
 * stamp i to d_stamps[(g * slots_per_workgroup + i) * 2] (the constant 100 MHz clock) and [... + 1] (the core clock
 * counter): stamp 0 at kernel entry, then for each work item of the workgroup one stamp when its first K tile has
 * landed in LDS, one at the end of its K loop and one when its stores have been issued, and a last one when all stores
 * have landed.  The last slot is not a stamp: [0] = 1 + the wave's hardware id register (CU, shader array and shader
 * engine in bits 8..15), [1] = the XCC (XCD) id, so that a tool can follow one CU through the launch.  Stamps beyond
 * slots_per_workgroup - 1 are dropped.  The caller zero-fills d_stamps (2 * 8 bytes * slots * max_workgroups);
 * *out_workgroups receives the grid size; MI_ERR_WORKSPACE if that exceeds max_workgroups.  C is computed as usual. */
int mi_matmul_mfma_timeline(const mi_gemm_tensors* t, int k_mode, int tile, uint64_t* d_stamps,
                            uint32_t slots_per_workgroup, uint32_t max_workgroups, uint32_t* out_workgroups,
                            void* hip_stream);

/* Measurement tool, no reference counterpart: a register-only loop of dense MFMA instructions (mfma_tile 32:
 * v_mfma_f32_32x32x16, 16: v_mfma_f32_16x16x32), one wave per SIMD on every CU, with the register footprint of the
 * GEMM's 128x128 wave tile, on operand values read from d_operands (at least CUs x 256 x 512 bytes, 16-byte aligned;
 * e.g. the benchmark's A matrix, or zeros).  Shows what the matrix cores sustain on given data: they are power-limited
 * and reach the published peak only on zeros.  d_clocks receives per workgroup the core-clock cycles and the ticks
 * of the constant 100 MHz clock the loop took (2 x uint64 each); *out_flop the flop the launch performs; time the
 * launch with events.  d_sink is one float of device memory (keeps the result alive). */
int mi_mfma_ceiling(const void* d_operands, size_t operand_bytes, int ab_dtype, int mfma_tile, uint32_t iterations,
                    uint64_t* d_clocks, float* d_sink, uint32_t* out_workgroups, double* out_flop, void* hip_stream);

/* Measurement tool, no reference counterpart: what a kernel that only streams `bytes` of d_src sustains, the yardstick for
 * the GEMM shapes that memory bounds (mi_mfma_ceiling is the one for the shapes the matrix cores bound).
 *   MI_STREAM_READ  16-byte non-temporal vector loads into registers (d_sink: one dword of device memory that the kernel
 *                   scribbles on, to keep the loads alive);
 *   MI_STREAM_DMA   `buffer_load_dwordx4 ... lds`, the GEMM kernel's own producer, into a ring in LDS that is never read:
 *                   72 KB in flight per workgroup, what the 64x128 tile's four-slot ring holds ahead of the slot in use
 *                   (bytes < 4 GiB, workgroups_per_cu <= 2);
 *   MI_STREAM_COPY  read d_src, write d_dst (`bytes` each way): the usual copy figure.
 * workgroups_per_cu (1..8) workgroups of 256 threads per CU; time the launch with events; rate = bytes / time (twice the
 * bytes for MI_STREAM_COPY). */
enum { MI_STREAM_READ = 0, MI_STREAM_DMA = 1, MI_STREAM_COPY = 2 };
int mi_hbm_stream_ceiling(const void* d_src, void* d_dst, size_t bytes, int mode, uint32_t workgroups_per_cu,
                          uint32_t* d_sink, void* hip_stream);
/* The same LDS DMA with the access pattern of the GEMM's tall-skinny tile on its large operand: a row-major matrix of
 * `rows` x `row_bytes` (a multiple of 128), every workgroup walking `rows_per_workgroup` (a multiple of 8) consecutive rows
 * 128 bytes at a time, 72 KB in flight: what the memory system gives a kernel that reads an operand panel by panel and
 * nothing else.  One workgroup per `rows_per_workgroup` rows; rate = rows * row_bytes / time. */
int mi_hbm_stream_rows_ceiling(const void* d_src, uint32_t rows, uint32_t row_bytes, uint32_t rows_per_workgroup,
                               void* hip_stream);

/* What MI_*_AUTO resolves to for this problem when no workspace is given (for logging): fills tile, k_mode and the
 * number of K splits (1 for MI_K_STREAM, whose partitions per tail tile follow from the tile count and the CUs). */
int mi_matmul_mfma_plan(const mi_gemm_tensors* t, int k_mode, int tile, int* out_tile, int* out_k_mode,
                        int* out_k_splits);
/* The same as text, for a call of mi_matmul_mfma_ws with `workspace_bytes` of (aligned) workspace, 0 for
 * mi_matmul_mfma: every launch the call would make, e.g. "256x256 output stationary" or
 * "peeled: 39936x32768 256x256 output stationary + bottom 80x32768 64x128 + right ...".  A ragged M or N under
 * MI_TILE_AUTO may be peeled: the whole tiles run the plain kernel, the leftover rows and columns one small
 * range-checked launch each.  ", A non-temporal" / ", B non-temporal" after a launch: that operand (in the kernel's
 * terms, i.e. after the swap a column-major C implies) is read once by the launch and larger than the 256 MB
 * memory-side cache, and is streamed past the L2 so that it does not evict the other one.  Writes at most out_size
 * bytes including the terminating 0. */
int mi_matmul_mfma_describe(const mi_gemm_tensors* t, int k_mode, int tile, size_t workspace_bytes, char* out,
                            size_t out_size);
/* The planner's own estimate, in microseconds on MI355X, of the launches mi_matmul_mfma_describe names (the figure it
 * ranks plans by: measured per-K-step and per-workgroup times, not a promise).  Repacking passes are not included. */
int mi_matmul_mfma_estimate_us(const mi_gemm_tensors* t, int k_mode, int tile, size_t workspace_bytes, double* out_us);

/* The tile family as data, so that bindings, tests and drivers enumerate it instead of restating it: tile codes run from
 * 1 to mi_tile_count() - 1 (0 is MI_TILE_AUTO); mi_tile_shape gives a tile's rows and columns, how many workgroups of it
 * share a CU and whether it has a 32-deep twin (any out pointer may be NULL; MI_ERR_BAD_ARGUMENT for an unknown code). */
int mi_tile_count(void);
const char* mi_tile_name(int tile);
int mi_tile_shape(int tile, uint32_t* out_bm, uint32_t* out_bn, int* out_workgroups_per_cu, int* out_has_32_deep_twin);
const char* mi_k_mode_name(int k_mode);
/* The two constants MI_K_AUTO prices a tile with: microseconds per 64-deep K step of one round of workgroups, and
 * microseconds per workgroup besides its K loop (ring fill, stores, dispatch).  They were measured on MI355X; on another
 * board, power limit or ROCm release `gemm --calibrate` measures them again in a minute and prints them beside these and
 * as one line for the environment variable MI_GEMM_PLANNER_CONSTANTS ("256x256=1.26/16.1,64x128=0.31/5.4", read when
 * the library is loaded).  mi_tile_set_planner_constants replaces a tile's pair for the rest of the process (the figures
 * derived from it - a lone workgroup of a tile that shares its CU, short launches - are scaled with it); it is not
 * synchronised with calls that are planning at the same time, so set the constants before the first GEMM call.  No
 * counterpart in the reference, whose schedule is chosen by the caller (gemm/gemm_sm90.h:5-12).
 * MI_ERR_BAD_ARGUMENT: unknown tile, or a constant that is not in (0, 1000]. */
int mi_tile_planner_constants(int tile, double* out_us_per_k64, double* out_fixed_us);
int mi_tile_set_planner_constants(int tile, double us_per_k64, double fixed_us);

/* ------------------------------------------------------------------------------- harness device helpers */
/* Test-data styles; 0..2 replace `enum class TestDataCode` (gemm/gemm_test.h:6-11); 3,4 are the seeded
 * benchmark distributions uniform[-param,param] and normal(0,1)*param. */
enum { MI_DATA_RANDOM = 0, MI_DATA_IDENTITY = 1, MI_DATA_TILED_NUMBERS = 2, MI_DATA_UNIFORM = 3, MI_DATA_NORMAL = 4 };

/* Replaces `device_init_test_data<T>` (gemm/gemm_test.cu:55-96): fills a rows x cols row-major 16-bit tensor.
 * transpose_rule as in the reference (gemm_test.cu:64-65).  seed is used by styles 3 and 4 only. */
int mi_init_test_data(void* d_tensor, uint32_t rows, uint32_t cols, int data_code, int transpose_rule,
                      int ab_dtype, double param, uint32_t seed, void* hip_stream);

/* 16-bit elements widened to fp32, exactly: lets the fp32 entry points run on the values of a 16-bit test tensor, so
 * that their results can be held against the same baseline (the reference's harness keeps every tensor in fp32,
 * gemm/gemm_test.cu:218-226). */
int mi_widen_to_f32(const void* d_src, int ab_dtype, float* d_dst, size_t count, void* hip_stream);

/* Replaces `launch_device_compare_tensor` (gemm/gemm_test.cu:177-187): compares two rows x cols fp32 tensors
 * with the reference's rule (same sign, ratio < 1+1/32, gemm_test.cu:138-147) and additionally accumulates
 * max|a-b| and max|a|.  Results land in the 4 x uint64 device block `d_result`:
 *   [0] packed (row<<32|col) of the first failing element in row-major order, UINT64_MAX if none
 *   [1] bits of (double) max|a-b| ; [2] bits of (double) max|a| ; [3] count of failing elements. */
int mi_compare_tensors(const float* d_a, const float* d_b, uint32_t rows, uint32_t cols, uint64_t* d_result,
                       void* hip_stream);

/* ------------------------------------------------------------------------------------ thin HIP runtime */
/* The host driver is plain C++ and never includes HIP headers; these wrap what gemm/gemm_test.cu uses of the
 * CUDA runtime (cudaMallocAsync/cudaFreeAsync :218-226,466-471, cudaMemsetAsync :246, events :275-284,
 * cudaStreamSynchronize :392, cudaSetDevice gemm/gemm_main.cpp:10). */
int mi_rt_device_count(int* count);
int mi_rt_set_device(int device);
/* name: at least 256 bytes.  Any out pointer may be NULL. */
int mi_rt_device_info(int device, char* name, char* gcn_arch, int* compute_units, int* clock_khz,
                      size_t* lds_bytes_per_block, size_t* global_mem_bytes);
int mi_rt_malloc(void** d_ptr, size_t bytes);
int mi_rt_free(void* d_ptr);
int mi_rt_memset_async(void* d_ptr, int byte_value, size_t bytes, void* hip_stream);
int mi_rt_memcpy_h2d(void* d_dst, const void* h_src, size_t bytes);
int mi_rt_memcpy_d2h(void* h_dst, const void* d_src, size_t bytes);
int mi_rt_stream_create(void** hip_stream);
int mi_rt_stream_destroy(void* hip_stream);
int mi_rt_stream_synchronize(void* hip_stream);
int mi_rt_device_synchronize(void);
int mi_rt_event_create(void** event);
int mi_rt_event_record(void* event, void* hip_stream);
int mi_rt_event_synchronize(void* event);
int mi_rt_event_elapsed_ms(float* ms, void* start_event, void* stop_event);
int mi_rt_event_destroy(void* event);

#ifdef __cplusplus
}
#endif
#endif
