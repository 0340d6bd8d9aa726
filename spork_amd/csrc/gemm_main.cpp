// Host driver, counterpart of gemm/gemm_main.cpp: picks sizes x data styles x an algorithm bitmask and hands each
// to gemm_test().  Plain C++; the GPU is reached only through the C ABI of libmi_gemm.so.
//
//   gemm            the reference's size list plus the five benchmark configurations
//   gemm --quick    small shapes only (seconds)
//   gemm --sweep    the reference's round-boundary and large ragged shapes (its H100 list) only
//   gemm --rounds   the same idea re-derived for this chip: tile counts around multiples of its CU count
//   gemm --versus llm|random    the planner against hipBLASLt over many shapes, with a summary table
//   gemm --one M N K [f16|bf16] [data style 1..5] [param]    the planner (without and with workspace) and hipBLASLt on one shape
//   gemm --kmodes M N K [f16|bf16] [style] [param]  one size: the planner, each K mode forced, hipBLASLt
//   gemm --exo M N K [f16|bf16] [style] [param]     one size: the planner and every Exo-named fp32 entry point
//   gemm --timeline M N K [f16|bf16] [tile code]    in-kernel timeline of one launch
//   gemm --ceiling  what a register-only MFMA loop sustains on the benchmark's operand values
//   gemm --calibrate  the planner's two constants per tile, measured on this machine, beside the planner's own
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "gemm_test.h"

#include <initializer_list>

int main(int argc, char** argv)
{
    const bool quick = argc > 1 && strcmp(argv[1], "--quick") == 0;
    const bool sweep = argc > 1 && strcmp(argv[1], "--sweep") == 0;
    const bool rounds = argc > 1 && strcmp(argv[1], "--rounds") == 0;
    const bool versus = argc > 2 && strcmp(argv[1], "--versus") == 0;
    const bool kmodes = argc > 1 && strcmp(argv[1], "--kmodes") == 0;  // --one with every K mode as a row of its own
    const bool exo = argc > 1 && strcmp(argv[1], "--exo") == 0;  // --one with the Exo-named entry points as rows
    const bool one = kmodes || exo || (argc > 1 && strcmp(argv[1], "--one") == 0);
    int device_count = 0;
    if (mi_rt_device_count(&device_count) != MI_OK || device_count == 0) {
        fprintf(stderr, "no GPU visible\n");
        return 1;
    }
    gpu_check(mi_rt_set_device(0), "set device");

    char name[256], arch[256];
    int cus = 0, clock_khz = 0;
    gpu_check(mi_rt_device_info(0, name, arch, &cus, &clock_khz, nullptr, nullptr), "device info");
    const bool is_gfx950 = strncmp(arch, "gfx950", 6) == 0;
    fprintf(stderr, "device: %s (%s), %i CUs, %i MHz; is_gfx950: %i\n", name, arch, cus, clock_khz / 1000, is_gfx950);
    {
        char vendor_path[512] = "?";
        mi_vendor_library(vendor_path, sizeof vendor_path);
        fprintf(stderr, "hipBLASLt: %s (version %i)\n", vendor_path, mi_vendor_version());
    }
    if (!is_gfx950) {
        fprintf(stderr, "the MFMA kernels are built for gfx950 only\n");
        return 1;
    }

    if (argc > 1 && strcmp(argv[1], "--ceiling") == 0) {
        return mfma_ceiling_report({});
    }
    if (argc > 1 && strcmp(argv[1], "--calibrate") == 0) {
        return planner_calibration({});
    }
    if (argc > 1 && strcmp(argv[1], "--timeline") == 0) {
        if (argc < 5) {
            fprintf(stderr, "usage: gemm --timeline M N K [f16|bf16] [tile code, 0 = auto]\n");
            return 2;
        }
        TimelineParams tp{};
        tp.M = uint32_t(strtoul(argv[2], nullptr, 10));
        tp.N = uint32_t(strtoul(argv[3], nullptr, 10));
        tp.K = uint32_t(strtoul(argv[4], nullptr, 10));
        tp.ab_dtype = argc > 5 && strcmp(argv[5], "f16") == 0 ? MI_F16 : MI_BF16;
        tp.tile = argc > 6 ? atoi(argv[6]) : MI_TILE_AUTO;
        tp.warmup = 30;
        return gemm_timeline(tp, {});
    }

    int failures = 0;
    uint64_t keep_bits = ~uint64_t(0);  // --versus times three algorithms only
    double* out_ms = nullptr;

    // data_style 0: all three reference styles; 1: tiled x identity; 2: identity x tiled; 3: reference random;
    // 4: uniform[-param, param]; 5: normal(0,1)/sqrt(K)
    auto sized_tests = [&failures, &keep_bits, &out_ms, exo_rows = exo, kmode_rows = kmodes](uint32_t M, uint32_t N, uint32_t K, int data_style, int ab_dtype, double param = 1.0) {
        TestParams params{};
        params.M = M;
        params.N = N;
        params.K = K;
        params.ab_dtype = ab_dtype;
        params.data_param = param;

        params.algorithm_code_bits = 0;
        {
            GPU_Tensors t{};
            t.M = M;
            t.N = N;
            t.K = K;
            t.a = t.b = reinterpret_cast<const void*>(uintptr_t(256));  // only shapes and alignment are inspected
            t.c = reinterpret_cast<float*>(uintptr_t(256));
            t.b_col_major = true;
            t.ab_dtype = ab_dtype;
            if (matmul_mi355_supports(t, MI_K_AUTO, MI_TILE_AUTO)) {
                params.algorithm_code_bits |= algorithm_code_bit(AlgorithmCode::mi355_auto);
            }
            for (int tile = 1; tile < mi_tile_count(); ++tile) {  // every tile of the family, forced
                if (matmul_mi355_supports(t, MI_K_OUTPUT_STATIONARY, tile)) {
                    params.algorithm_code_bits |= algorithm_code_bit(forced_tile_algorithm(tile));
                }
            }
            if (matmul_mi355_supports(t, MI_K_SPLIT, MI_TILE_AUTO)) {
                params.algorithm_code_bits |= algorithm_code_bit(AlgorithmCode::mi355_split_k);
                params.algorithm_code_bits |= algorithm_code_bit(AlgorithmCode::mi355_split_k_sum);
                if (kmode_rows) {
                    params.algorithm_code_bits |= algorithm_code_bit(AlgorithmCode::mi355_split_k_sum_in);
                }
            }
            if (matmul_mi355_supports(t, MI_K_AUTO, MI_TILE_AUTO)) {
                params.algorithm_code_bits |= algorithm_code_bit(AlgorithmCode::mi355_auto_ws);
            }
            if (matmul_mi355_supports(t, MI_K_STREAM, MI_TILE_AUTO)) {
                params.algorithm_code_bits |= algorithm_code_bit(AlgorithmCode::mi355_stream_k);
                if (kmode_rows) {
                    params.algorithm_code_bits |= algorithm_code_bit(AlgorithmCode::mi355_stream_k_in);
                }
            }
        }
        params.algorithm_code_bits |= algorithm_code_bit(AlgorithmCode::mi355_row_major_b);  // any shape, any layout
        // fp32 operands are re-packed anyway: any shape; the n128 / n64 / K2 rows only where asked for (--exo)
        params.algorithm_code_bits |= algorithm_code_bit(AlgorithmCode::exo_sm_80_fence) | algorithm_code_bit(AlgorithmCode::exo_sm_90_n256);
        if (exo_rows) {
            params.algorithm_code_bits |= algorithm_code_bit(AlgorithmCode::exo_sm_90_n128) | algorithm_code_bit(AlgorithmCode::exo_sm_90_n64);
            if (K % 2 == 0) {
                params.algorithm_code_bits |= algorithm_code_bit(AlgorithmCode::exo_sm_90_n256_K2);
            }
        }
        if (hipblaslt_enabled()) {
            params.algorithm_code_bits |= algorithm_code_bit(AlgorithmCode::hipblaslt);
        }
        if (M % 32 == 0 && N % 32 == 0 && K % 16 == 0 && double(M) * N * K <= 7e10) {
            params.algorithm_code_bits |= algorithm_code_bit(AlgorithmCode::mfma_direct);
        }

        params.algorithm_code_bits &= keep_bits;
        params.out_ms = out_ms;

        if (data_style == 0 || data_style == 1) {
            params.test_data_code_A = TestDataCode::tiled_numbers;
            params.test_data_code_B = TestDataCode::identity;
            failures += gemm_test(params, {});
        }
        if (data_style == 0 || data_style == 2) {
            params.test_data_code_A = TestDataCode::identity;
            params.test_data_code_B = TestDataCode::tiled_numbers;
            failures += gemm_test(params, {});
        }
        if (data_style == 0 || data_style == 3) {
            params.test_data_code_A = TestDataCode::random;
            params.test_data_code_B = TestDataCode::random;
            failures += gemm_test(params, {});
        }
        if (data_style == 4) {
            params.test_data_code_A = TestDataCode::uniform;
            params.test_data_code_B = TestDataCode::uniform;
            failures += gemm_test(params, {});
        }
        if (data_style == 5) {
            params.test_data_code_A = TestDataCode::normal;
            params.test_data_code_B = TestDataCode::normal;
            params.data_param = 1.0 / sqrt(double(K));
            failures += gemm_test(params, {});
        }
    };

    if (quick) {
        sized_tests(512, 512, 512, 0, MI_F16);
        sized_tests(512, 512, 512, 4, MI_F16, 1.0);
        sized_tests(768, 768, 32, 2, MI_BF16);
        sized_tests(160, 480, 816, 0, MI_F16);
        sized_tests(1024, 1024, 1024, 5, MI_BF16);
    }
    else if (sweep) {
        // The reference's H100 list (gemm/gemm_main.cpp:106-117): large ragged shapes and deep-K tile counts that
        // straddle a round of its 132 SMs.  The same tile counts (60, 66, 72, 33, 99, 44 tiles of 256x256) straddle
        // nothing on 256 CUs by themselves; what they test here is the planner's choice of K partitions.
        sized_tests(32768, 65536, 48, 3, MI_BF16);
        sized_tests(40016, 32768, 6400, 3, MI_BF16);
        sized_tests(12288, 24576, 1536, 3, MI_F16);
        sized_tests(6 * 256, 3 * 256, 65536, 3, MI_F16);
        sized_tests(6 * 256, 10 * 256, 65536, 3, MI_F16);
        sized_tests(6 * 256, 11 * 256, 65536, 3, MI_F16);
        sized_tests(6 * 256, 12 * 256, 65536, 3, MI_F16);
        sized_tests(3 * 256, 11 * 256, 65536, 3, MI_F16);
        sized_tests(9 * 256, 11 * 256, 65536, 3, MI_F16);
        sized_tests(4 * 256, 11 * 256, 16384 * 3, 3, MI_F16);
    }
    else if (one) {
        if (argc < 5) {
            fprintf(stderr, "usage: gemm --one M N K [f16|bf16] [data style: 1 tiled x identity, 2 identity x tiled, 3 sparse "
                            "random, 4 uniform[-param,param], 5 normal/sqrt(K) (default)] [param, default 1]\n");
            return 2;
        }
        keep_bits = algorithm_code_bit(AlgorithmCode::mi355_auto) | algorithm_code_bit(AlgorithmCode::mi355_auto_ws) |
                    algorithm_code_bit(AlgorithmCode::hipblaslt);
        if (exo) {
            keep_bits = algorithm_code_bit(AlgorithmCode::mi355_auto) | algorithm_code_bit(AlgorithmCode::exo_sm_80_fence) |
                        algorithm_code_bit(AlgorithmCode::exo_sm_90_n256) | algorithm_code_bit(AlgorithmCode::exo_sm_90_n256_K2) |
                        algorithm_code_bit(AlgorithmCode::exo_sm_90_n128) | algorithm_code_bit(AlgorithmCode::exo_sm_90_n64);
        }
        if (kmodes) {
            keep_bits |= algorithm_code_bit(AlgorithmCode::mi355_split_k) | algorithm_code_bit(AlgorithmCode::mi355_split_k_sum) |
                         algorithm_code_bit(AlgorithmCode::mi355_stream_k) | algorithm_code_bit(AlgorithmCode::mi355_split_k_sum_in) |
                         algorithm_code_bit(AlgorithmCode::mi355_stream_k_in);
        }
        const int style = argc > 6 ? atoi(argv[6]) : 5;
        if (style < 1 || style > 5) {
            fprintf(stderr, "data style must be 1..5\n");
            return 2;
        }
        sized_tests(uint32_t(strtoul(argv[2], nullptr, 10)), uint32_t(strtoul(argv[3], nullptr, 10)),
                    uint32_t(strtoul(argv[4], nullptr, 10)), style, argc > 5 && strcmp(argv[5], "f16") == 0 ? MI_F16 : MI_BF16,
                    argc > 7 ? atof(argv[7]) : 1.0);
    }
    else if (versus) {
        // The planner (without and with the workspace it prefers) against hipBLASLt on bf16 normal(0,1)/sqrt(K) data:
        // "llm": 8 token counts x 7 weight shapes; "random": 60 shapes, M, N in 256..8192, K in 256..16384, all
        // multiples of 8, half of the draws powers of two (a fixed list).
        struct Shape {
            uint32_t M, N, K;
        };
        static const Shape random_shapes[] = {
        {8192, 3952, 8192}, {5408, 4096, 2576}, {4096, 5608, 10464}, {736, 7456, 4096}, {3864, 1024, 8440},
        {2048, 512, 1024}, {496, 512, 6584}, {7192, 512, 16384}, {3688, 2048, 2048}, {376, 1352, 512},
        {6784, 5840, 7584}, {1024, 5528, 6720}, {2048, 7504, 3320}, {600, 3872, 8192}, {2048, 856, 3672},
        {8192, 8192, 8192}, {7072, 7352, 1024}, {7696, 6192, 12368}, {4096, 512, 1032}, {8192, 4096, 8192},
        {2656, 7864, 3992}, {2544, 6384, 4096}, {2296, 2048, 8952}, {1008, 4096, 11016}, {5088, 2048, 16024},
        {512, 2048, 2488}, {8192, 6288, 2048}, {944, 7392, 14400}, {4096, 5024, 1568}, {4096, 8192, 7472},
        {4504, 2792, 8128}, {512, 8192, 512}, {2720, 1024, 4096}, {1024, 3568, 10640}, {1024, 8192, 3688},
        {4320, 512, 13720}, {4096, 1024, 16384}, {2048, 2880, 4808}, {2048, 2784, 1024}, {3976, 6552, 13016},
        {512, 8192, 15952}, {4096, 512, 9016}, {1024, 6632, 6696}, {4096, 4096, 3480}, {8192, 4048, 1872},
        {1024, 2048, 4544}, {3104, 4096, 4096}, {4248, 512, 13360}, {4616, 1024, 15744}, {1024, 8192, 13872},
        {8192, 2808, 1024}, {4944, 3616, 512}, {480, 4480, 8296}, {8192, 4096, 4096}, {2048, 4096, 1024},
        {512, 1312, 3432}, {2048, 6176, 10408}, {4344, 8192, 1024}, {4096, 7008, 9072}, {4592, 2160, 8192},
        };
        Shape shapes[64];
        uint32_t shape_count = 0;
        if (strcmp(argv[2], "llm") == 0) {
            const uint32_t tokens[] = {256, 1000, 2048, 3000, 4096, 5000, 8192, 16384};
            const Shape weights[] = {{0, 4096, 4096}, {0, 11008, 4096}, {0, 4096, 11008}, {0, 6144, 4096},
                                     {0, 28672, 8192}, {0, 8192, 28672}, {0, 1024, 8192}};
            for (const uint32_t m : tokens) {
                for (const Shape& w : weights) {
                    shapes[shape_count++] = Shape{m, w.N, w.K};
                }
            }
        }
        else if (strcmp(argv[2], "random") == 0) {
            for (const Shape& s : random_shapes) {
                shapes[shape_count++] = s;
            }
        }
        else {
            fprintf(stderr, "usage: gemm --versus llm|random\n");
            return 2;
        }
        keep_bits = algorithm_code_bit(AlgorithmCode::mi355_auto) | algorithm_code_bit(AlgorithmCode::mi355_auto_ws) |
                    algorithm_code_bit(AlgorithmCode::hipblaslt);
        static double ms[64][algorithm_max_count] = {};
        for (uint32_t i = 0; i < shape_count; ++i) {
            out_ms = ms[i];
            sized_tests(shapes[i].M, shapes[i].N, shapes[i].K, 5, MI_BF16);
        }
        out_ms = nullptr;
        printf("| M,N,K | ours us | ours with workspace us | hipBLASLt us | ratio | ratio with workspace |\n|---|---|---|---|---|---|\n");
        double log_sum = 0, log_sum_ws = 0, worst = 1e9, best = 0;
        uint32_t counted = 0, below = 0;
        for (uint32_t i = 0; i < shape_count; ++i) {
            const double ours = ms[i][static_cast<uint32_t>(AlgorithmCode::mi355_auto)];
            const double ours_ws = ms[i][static_cast<uint32_t>(AlgorithmCode::mi355_auto_ws)];
            const double vendor = ms[i][static_cast<uint32_t>(AlgorithmCode::hipblaslt)];
            if (!(ours > 0) || !(ours_ws > 0) || !(vendor > 0)) {
                continue;
            }
            printf("| %u,%u,%u | %.1f | %.1f | %.1f | %.2f | %.2f |\n", shapes[i].M, shapes[i].N, shapes[i].K, ours * 1e3,
                   ours_ws * 1e3, vendor * 1e3, vendor / ours, vendor / ours_ws);
            log_sum += log(vendor / ours);
            log_sum_ws += log(vendor / ours_ws);
            worst = fmin(worst, vendor / ours_ws);
            best = fmax(best, vendor / ours_ws);
            below += vendor / ours_ws < 0.97;
            ++counted;
        }
        if (counted) {
            printf("\n%u shapes: geometric mean of hipBLASLt time / ours %.3f, with workspace %.3f (worst %.2f, best %.2f, "
                   "%u below 0.97)\n", counted, exp(log_sum / counted), exp(log_sum_ws / counted), worst, best, below);
        }
    }
    else if (rounds) {
        // What gemm/gemm_main.cpp:111-117 does for the H100's 132 SMs (tile counts just under, at and just over a
        // round), for this chip: the number of 256x256 tiles against the CU count (256 on MI355X).
        const uint32_t side = 4096, k = 8192;                                  // 16 tiles along M
        const uint32_t per_round = (uint32_t)cus / (side / 256);               // tile columns that fill one round
        for (const int delta : {-8, -1, 0, 1, 4, 8}) {
            sized_tests(side, (per_round + delta) * 256, k, 3, MI_BF16);       // 0.5 .. 1.5 rounds
        }
        for (const int delta : {-1, 0, 1}) {
            sized_tests(side, (2 * per_round + delta) * 256, k, 3, MI_BF16);   // around two rounds
            sized_tests(side - 256, (per_round + delta) * 256, 65536, 3, MI_F16);  // deep K, around one round
        }
    }
    else {
        // the reference's size list (gemm/gemm_main.cpp:98-104,119-121)
        sized_tests(2048, 2048, 2048, 2, MI_F16);
        sized_tests(4096, 4096, 4096, 2, MI_F16);
        sized_tests(8192, 8192, 8192, 2, MI_BF16);
        sized_tests(768, 768, 32, 2, MI_F16);
        sized_tests(7680, 1536, 4096, 0, MI_F16);
        sized_tests(15360, 1536, 8192, 3, MI_BF16);
        sized_tests(6 * 256, 9 * 256, 65536, 3, MI_F16);
        sized_tests(7680, 3072, 16384, 3, MI_BF16);
        sized_tests(768, 3072, 3072, 3, MI_F16);
        // ragged sizes from the reference's H100 list (gemm/gemm_main.cpp:106-109)
        sized_tests(160, 480, 816, 0, MI_F16);
        sized_tests(32768, 40016, 816, 3, MI_BF16);
        // the five benchmark configurations
        sized_tests(512, 512, 512, 4, MI_F16, 1.0);
        sized_tests(4096, 4096, 4096, 4, MI_F16, 1.0);
        sized_tests(8192, 8192, 8192, 5, MI_BF16);
        sized_tests(16384, 128, 8192, 4, MI_F16, 1.0);
        sized_tests(2048, 2048, 65536, 4, MI_F16, 0.5);
    }

    gpu_check(mi_rt_device_synchronize(), "device sync");
    if (failures) {
        fprintf(stderr, "%i algorithm runs FAILED the error check\n", failures);
    }
    return failures ? 1 : 0;
}
