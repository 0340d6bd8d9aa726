// Test harness interface, counterpart of gemm/gemm_test.h.
#pragma once

#include <stdint.h>
#include <stdio.h>

#include "gpu_tensor.h"

// gemm/gemm_test.h:6-11, plus the two seeded distributions of the benchmark configurations.
enum class TestDataCode
{
    random = MI_DATA_RANDOM,
    identity = MI_DATA_IDENTITY,
    tiled_numbers = MI_DATA_TILED_NUMBERS,
    uniform = MI_DATA_UNIFORM,  // uniform[-data_param, data_param]
    normal = MI_DATA_NORMAL,    // normal(0,1) * data_param
};

// gemm/gemm_test.h:13-38: one bit per algorithm raced against the baseline.  The fixed algorithms come first; after
// them one "this tile, output stationary" algorithm per tile of the library's family (index algorithm_fixed_count +
// tile code - 1): the list is whatever mi_tile_count() / mi_tile_name() report, so a new tile shows up here by itself.
enum class AlgorithmCode
{
    mfma_direct,          // one MFMA tile per wave straight from global memory
    mi355_auto,           // planner picks tile and K mode
    mi355_split_k,        // planner picks the tile, K split forced
    mi355_row_major_b,    // B given K x N row-major (the baseline's own call): re-packed through the workspace
    mi355_auto_ws,        // planner with a workspace at hand: K partitions may be summed from copies of C
    mi355_split_k_sum,    // K split forced, partitions summed from copies of C in the workspace (no atomics)
    mi355_stream_k,       // stream-K forced: equal runs of (tile, K tile) pairs, parts summed from the workspace
    mi355_split_k_sum_in,  // the two rows above with the parts summed inside the GEMM launch instead of by a launch of its
    mi355_stream_k_in,     //   own (mi_matmul_mfma_sum_in_launch(1)): only where asked for (--kmodes)
    hipblaslt,            // vendor comparator (the cuBLAS / CUTLASS rows of gemm/gemm_test.h:19-20)
    exo_sm_80_fence,      // the reference's Exo entry points by name (gemm/gemm_test.h:21-31), on the test data widened
    exo_sm_90_n256,       //   to fp32: three bf16 terms per product, so about 3.3x the 16-bit time
    exo_sm_90_n256_K2,
    exo_sm_90_n128,
    exo_sm_90_n64,
    first_forced_tile,    // + (tile code - 1)
};

constexpr uint32_t algorithm_fixed_count = static_cast<uint32_t>(AlgorithmCode::first_forced_tile);
constexpr uint32_t algorithm_max_count = 64;  // bits of the selection mask

inline uint32_t algorithm_count()
{
    return algorithm_fixed_count + static_cast<uint32_t>(mi_tile_count() - 1);
}

inline uint64_t algorithm_code_bit(AlgorithmCode code)
{
    return uint64_t(1) << static_cast<uint32_t>(code);
}

// the algorithm that forces tile `tile` (an MI_TILE_* code other than MI_TILE_AUTO), output stationary
inline AlgorithmCode forced_tile_algorithm(int tile)
{
    return static_cast<AlgorithmCode>(algorithm_fixed_count + static_cast<uint32_t>(tile - 1));
}

// 0 for the fixed algorithms, else the tile code the algorithm forces
inline int forced_tile_of(AlgorithmCode code)
{
    const uint32_t index = static_cast<uint32_t>(code);
    return index < algorithm_fixed_count ? 0 : static_cast<int>(index - algorithm_fixed_count) + 1;
}

// (the returned pointer is valid until the next call from the same thread)
inline const char* algorithm_name(AlgorithmCode code)
{
    switch (code) {
      case AlgorithmCode::mfma_direct:
        return "mfma_direct";
      case AlgorithmCode::mi355_auto:
        return "mi355 (auto)";
      case AlgorithmCode::mi355_split_k:
        return "mi355 (split k)";
      case AlgorithmCode::mi355_row_major_b:
        return "mi355 (row-major B via workspace)";
      case AlgorithmCode::mi355_auto_ws:
        return "mi355 (auto, workspace)";
      case AlgorithmCode::mi355_split_k_sum:
        return "mi355 (split k, workspace sum)";
      case AlgorithmCode::mi355_stream_k:
        return "mi355 (stream k)";
      case AlgorithmCode::mi355_split_k_sum_in:
        return "mi355 (split k, workspace sum inside the launch)";
      case AlgorithmCode::mi355_stream_k_in:
        return "mi355 (stream k, sum inside the tail launch)";
      case AlgorithmCode::hipblaslt:
        return "hipBLASLt";
      case AlgorithmCode::exo_sm_80_fence:
        return "exo_sm_80_fence (fp32 in, bf16x3)";
      case AlgorithmCode::exo_sm_90_n256:
        return "exo_sm_90_n256 (fp32 in, bf16x3)";
      case AlgorithmCode::exo_sm_90_n256_K2:
        return "exo_sm_90_n256_K2 (fp32 in, bf16x3)";
      case AlgorithmCode::exo_sm_90_n128:
        return "exo_sm_90_n128 (fp32 in, bf16x3)";
      case AlgorithmCode::exo_sm_90_n64:
        return "exo_sm_90_n64 (fp32 in, bf16x3)";
      default:
        break;
    }
    const int tile = forced_tile_of(code);
    int per_cu = 1;
    if (tile < 1 || mi_tile_shape(tile, nullptr, nullptr, &per_cu, nullptr) != MI_OK) {
        return "unknown";
    }
    static thread_local char text[64];
    snprintf(text, sizeof text, "mi355 %s%s (output stationary)", mi_tile_name(tile), per_cu == 2 ? ", two per CU" : "");
    return text;
}

// gemm/gemm_test.h:100-105, with the element type and the distribution parameter added.
struct TestParams
{
    uint32_t M, N, K;
    TestDataCode test_data_code_A, test_data_code_B;
    uint64_t algorithm_code_bits;
    int ab_dtype;        // MI_F16 | MI_BF16
    double data_param;   // for TestDataCode::uniform / normal
    double* out_ms = nullptr;  // optional, algorithm_count() entries: the reported time of each algorithm that ran
};

// Runs every selected algorithm 25 times, compares each against the baseline kernel on the device and prints one line
// per algorithm.  Returns the number of algorithms whose normalised max error exceeded 1e-3.
int gemm_test(TestParams params, gpu_stream_t stream);

struct TimelineParams
{
    uint32_t M, N, K;
    int ab_dtype;     // MI_F16 | MI_BF16
    int tile;         // MI_TILE_*
    uint32_t warmup;  // launches before the one that is reported
};

// Prints what a register-only MFMA loop sustains (TFLOP/s and core clock) for both dense 16-bit MFMA shapes on the
// benchmark's operand distributions and on zeros: the ceiling a GEMM kernel on this power-limited part works under.
int mfma_ceiling_report(gpu_stream_t stream);

// Measures, tile by tile, the two constants the library's planner prices a tile with (main-loop time per 64-deep K step,
// per-workgroup cost outside it) and prints them beside what the planner's estimates imply: `gemm --calibrate`.
int planner_calibration(gpu_stream_t stream);

// Launches the planner's kernel for A MxK, B NxK with in-kernel time stamps and prints, per phase of a workgroup's
// life (K loop and store issue of each output tile), the min/mean/max duration and the core clock, and per XCD the
// time its workgroups finish.  Returns non-zero if nothing was recorded.
int gemm_timeline(TimelineParams params, gpu_stream_t stream);
