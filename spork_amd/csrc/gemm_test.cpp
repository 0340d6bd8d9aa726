// Test harness, counterpart of gemm/gemm_test.cu: allocate, seeded on-device init, baseline run, 25 timed runs per
// algorithm with an event between each, on-device compare, one printed line per (size, data, algorithm).
#include "gemm_test.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <string>
#include <vector>

namespace gemm_test_impl {

constexpr uint32_t SEED_A = 20010106u;  // gemm/gemm_test.cu:76
constexpr uint32_t SEED_B = 19980724u;  // gemm/gemm_test.cu:87

static void* device_alloc(size_t bytes)
{
    void* p = nullptr;
    if (mi_rt_malloc(&p, bytes) != MI_OK || !p) {
        fprintf(stderr, "Error on device malloc of %zu bytes: %i (%s)\n", bytes, mi_last_hip_error(),
                mi_last_hip_error_string());
        exit(1);
    }
    return p;
}

// What the harness shows of a wrong element: [baseline, tested] pairs of the 5 x 5 elements around it, the wrong one in
// bold (gemm/gemm_test.cu:98-120, which prints from the device; here the rows are copied back and printed by the host).
static void print_tensor_neighborhood(const float* d_a, const float* d_b, uint32_t rows, uint32_t cols, uint32_t y, uint32_t x)
{
    if (y >= rows || x >= cols) {
        return;
    }
    const uint32_t y_min = y < 2 ? 0u : y - 2, y_max = y + 2 >= rows ? rows - 1u : y + 2;
    const uint32_t x_min = x < 2 ? 0u : x - 2, x_max = x + 2 >= cols ? cols - 1u : x + 2;
    const uint32_t width = x_max - x_min + 1;
    float a[5], b[5];
    for (uint32_t cy = y_min; cy <= y_max; ++cy) {
        const size_t first = size_t(cy) * cols + x_min;
        gpu_check(mi_rt_memcpy_d2h(a, d_a + first, sizeof(float) * width), "read baseline row");
        gpu_check(mi_rt_memcpy_d2h(b, d_b + first, sizeof(float) * width), "read tested row");
        for (uint32_t cx = x_min; cx <= x_max; ++cx) {
            const bool it = cy == y && cx == x;
            printf("%s[%6g, %5g]%s  ", it ? "\x1b[1m" : "", a[cx - x_min], b[cx - x_min], it ? "\x1b[0m" : "");
        }
        printf("\n");
    }
}

int gemm_test(TestParams params, gpu_stream_t stream)
{
    StreamWorkspace stream_ws{stream};
    const size_t M = params.M, N = params.N, K = params.K;
    uint64_t* d_result = static_cast<uint64_t*>(device_alloc(4 * sizeof(uint64_t)));
    void* d_a = device_alloc(2 * M * K);
    void* d_b = device_alloc(2 * N * K);     // K x N row-major
    void* d_bCol = device_alloc(2 * N * K);  // same matrix stored N x K
    float* d_c_baseline = static_cast<float*>(device_alloc(sizeof(float) * M * N));
    float* d_c_tested = static_cast<float*>(device_alloc(sizeof(float) * M * N));

    // Initialize test data (gemm/gemm_test.cu:236-241).  For the seeded distributions A and B use different seeds.
    {
        const int code_a = static_cast<int>(params.test_data_code_A), code_b = static_cast<int>(params.test_data_code_B);
        gpu_check(mi_init_test_data(d_a, params.M, params.K, code_a, false, params.ab_dtype, params.data_param, SEED_A, stream), "init a");
        gpu_check(mi_init_test_data(d_b, params.K, params.N, code_b, false, params.ab_dtype, params.data_param, SEED_B, stream), "init b");
        gpu_check(mi_init_test_data(d_bCol, params.N, params.K, code_b, true, params.ab_dtype, params.data_param, SEED_B, stream), "init bCol");
    }

    auto fill_garbage = [params, stream](float* d_c) {
        gpu_check(mi_rt_memset_async(d_c, 0x7D, sizeof(*d_c) * params.M * params.N, stream), "memset");
    };

    // Initialize baseline data (gemm/gemm_test.cu:264-268): row-major B, so the tested algorithms (which get the
    // N x K copy) are also checked against a different storage of the same matrix.
    {
        GPU_Tensors t{params.M, params.N, params.K, d_a, d_b, d_c_baseline, 0, 0, 0, params.ab_dtype};
        fill_garbage(t.c);
        matmul_baseline(t, stream);
    }

    // The Exo entry points take fp32 tensors (gemm/gemm_test.cu:218-226 keeps everything in fp32): the same values,
    // widened, so that their results are held against the same baseline.
    const uint64_t exo_bits = algorithm_code_bit(AlgorithmCode::exo_sm_80_fence) | algorithm_code_bit(AlgorithmCode::exo_sm_90_n256) |
                              algorithm_code_bit(AlgorithmCode::exo_sm_90_n256_K2) | algorithm_code_bit(AlgorithmCode::exo_sm_90_n128) |
                              algorithm_code_bit(AlgorithmCode::exo_sm_90_n64);
    float *d_a32 = nullptr, *d_b32 = nullptr, *d_bCol32 = nullptr;
    if (params.algorithm_code_bits & exo_bits) {
        d_a32 = static_cast<float*>(device_alloc(4 * M * K));
        d_b32 = static_cast<float*>(device_alloc(4 * N * K));
        d_bCol32 = static_cast<float*>(device_alloc(4 * N * K));
        gpu_check(mi_widen_to_f32(d_a, params.ab_dtype, d_a32, M * K, stream), "widen a");
        gpu_check(mi_widen_to_f32(d_b, params.ab_dtype, d_b32, N * K, stream), "widen b");
        gpu_check(mi_widen_to_f32(d_bCol, params.ab_dtype, d_bCol32, N * K, stream), "widen bCol");
    }

    int failures = 0;

    // Test loop
    auto run_tests = [&](AlgorithmCode algo, uint32_t test_count) {
        std::vector<float> test_times(test_count);
        std::vector<void*> test_events(test_count + 1);
        auto new_event = [stream] {
            void* event{};
            gpu_check(mi_rt_event_create(&event), "event create");
            gpu_check(mi_rt_event_record(event, stream), "event record");
            return event;
        };
        fill_garbage(d_c_tested);

        GPU_Tensors t{params.M, params.N, params.K, d_a, d_bCol, d_c_tested, 0, 1, 0, params.ab_dtype};
        // About thirty milliseconds of untimed launches first (the reference has none).  Measured on MI355X: after an idle
        // spell or a kernel of low intensity (the direct kernel before the first algorithm of the list), the same
        // launch runs 8 to 20 % slower for 25 to 30 ms before it settles; the 25 timed launches of a small problem span
        // a millisecond or two, so that whole window would be charged to whichever algorithm happens to run next.
        const double est_us = std::max(8.0, 2.0 * params.M * params.N * params.K / 1.0e9);  // at about 1 PFLOP/s
        const uint32_t warmup_count = (uint32_t)std::min(1000.0, std::max(3.0, std::ceil(30000.0 / est_us)));
        for (uint32_t launch_i = 0; launch_i < warmup_count + test_count; ++launch_i) {
            const uint32_t test_i = launch_i < warmup_count ? 0 : launch_i - warmup_count;
            if (launch_i == warmup_count) {
                test_events[0] = new_event();
            }
            switch (algo) {
              case AlgorithmCode::mfma_direct:
                matmul_mfma_direct(t, stream);
                break;
              case AlgorithmCode::mi355_auto:
                matmul_mi355(t, MI_K_AUTO, MI_TILE_AUTO, stream);
                break;
              case AlgorithmCode::mi355_split_k:
                matmul_mi355(t, MI_K_SPLIT, MI_TILE_AUTO, stream);
                break;
              case AlgorithmCode::hipblaslt:
                matmul_hipblaslt(t, stream_ws);
                break;
              case AlgorithmCode::mi355_auto_ws:
                matmul_mi355_any_layout(t, stream_ws);
                break;
              case AlgorithmCode::mi355_split_k_sum:
                matmul_mi355_any_layout(t, stream_ws, MI_K_SPLIT_REDUCE, MI_TILE_AUTO);
                break;
              case AlgorithmCode::mi355_stream_k:
                matmul_mi355_any_layout(t, stream_ws, MI_K_STREAM, MI_TILE_AUTO);
                break;
              case AlgorithmCode::mi355_split_k_sum_in:
              case AlgorithmCode::mi355_stream_k_in: {
                const int was = mi_matmul_mfma_sum_in_launch(1, nullptr);
                matmul_mi355_any_layout(t, stream_ws, algo == AlgorithmCode::mi355_stream_k_in ? MI_K_STREAM : MI_K_SPLIT_REDUCE,
                                        MI_TILE_AUTO);
                mi_matmul_mfma_sum_in_launch(was, nullptr);
                break;
              }
              // gemm/gemm_test.cu:326,335,358,362 and :288-294: the Sm90 ones with the operands swapped, so that their
              // C[L,N,M] is the row-major M x N of the harness
              case AlgorithmCode::exo_sm_80_fence: {
                mi_xgemm_context ctxt = xgemm_context(stream_ws, 1, int(params.M), int(params.N), int(params.K));
                xgemm_Sm80_fence(&ctxt, int(params.M), int(params.N), int(params.K), d_a32, d_b32, d_c_tested);
                break;
              }
              case AlgorithmCode::exo_sm_90_n256: {
                mi_xgemm_context ctxt = xgemm_context(stream_ws, 1, int(params.N), int(params.M), int(params.K));
                xgemm_Sm90_wgmma_n256(&ctxt, 1, int(params.N), int(params.M), 1, int(params.K), d_bCol32, d_a32, d_c_tested);
                break;
              }
              case AlgorithmCode::exo_sm_90_n256_K2: {
                mi_xgemm_context ctxt = xgemm_context(stream_ws, 1, int(params.N), int(params.M), int(params.K));
                xgemm_Sm90_wgmma_n256_split_k(&ctxt, 1, int(params.N), int(params.M), 2, int(params.K / 2), d_bCol32, d_a32, d_c_tested);
                break;
              }
              case AlgorithmCode::exo_sm_90_n128: {
                mi_xgemm_context ctxt = xgemm_context(stream_ws, 1, int(params.N), int(params.M), int(params.K));
                xgemm_Sm90_wgmma_n128(&ctxt, 1, int(params.N), int(params.M), 1, int(params.K), d_bCol32, d_a32, d_c_tested);
                break;
              }
              case AlgorithmCode::exo_sm_90_n64: {
                mi_xgemm_context ctxt = xgemm_context(stream_ws, 1, int(params.N), int(params.M), int(params.K));
                xgemm_Sm90_wgmma_n64(&ctxt, 1, int(params.N), int(params.M), 1, int(params.K), d_bCol32, d_a32, d_c_tested);
                break;
              }
              case AlgorithmCode::mi355_row_major_b: {
                GPU_Tensors t_row{params.M, params.N, params.K, d_a, d_b, d_c_tested, 0, 0, 0, params.ab_dtype};
                matmul_mi355_any_layout(t_row, stream_ws);
                break;
              }
              default:  // one of the library's tiles, forced
                matmul_mi355(t, MI_K_OUTPUT_STATIONARY, forced_tile_of(algo), stream);
                break;
            }
            if (launch_i >= warmup_count) {
                test_events[test_i + 1] = new_event();
            }
            else if (launch_i % 32 == 31 || launch_i + 1 == warmup_count) {
                // keep the warm-up from piling up a deep queue: the timed launches start from an empty one, as they
                // do in the reference's loop (a library with a costly host side would otherwise be timed host-bound)
                gpu_check(mi_rt_stream_synchronize(stream), "stream sync");
            }
        }
        gpu_check(mi_compare_tensors(d_c_baseline, d_c_tested, params.M, params.N, d_result, stream), "compare");
        gpu_check(mi_rt_stream_synchronize(stream), "stream sync");

        uint64_t result[4];
        gpu_check(mi_rt_memcpy_d2h(result, d_result, sizeof(result)), "read compare result");
        double max_diff, max_ref;
        memcpy(&max_diff, &result[1], 8);
        memcpy(&max_ref, &result[2], 8);
        const double rel_err = max_ref > 0 ? max_diff / max_ref : max_diff;
        const bool nonneg_data = params.test_data_code_A <= TestDataCode::tiled_numbers && params.test_data_code_B <= TestDataCode::tiled_numbers;
        const bool failed = !(rel_err <= 1e-3) || (nonneg_data && result[0] != UINT64_MAX);
        if (result[0] != UINT64_MAX) {
            // the reference's ratio rule (gemm/gemm_test.cu:138-147); informative for signed data, where elements
            // near zero fail it through cancellation alone
            const uint32_t y = static_cast<uint32_t>(result[0] >> 32), x = static_cast<uint32_t>(result[0]);
            printf("TestParams{%u,%u,%u, %i,%i} \x1b[1m[%u,%u]\x1b[0m first of %llu elements outside ratio 1+1/32\n", params.M,
                   params.N, params.K, static_cast<int>(params.test_data_code_A), static_cast<int>(params.test_data_code_B), y, x,
                   static_cast<unsigned long long>(result[3]));
            if (failed) {
                print_tensor_neighborhood(d_c_baseline, d_c_tested, params.M, params.N, y, x);
            }
        }
        failures += failed;

        for (uint32_t test_i = 0; test_i < test_count; ++test_i) {
            gpu_check(mi_rt_event_elapsed_ms(&test_times[test_i], test_events[test_i], test_events[test_i + 1]), "elapsed");
            mi_rt_event_destroy(test_events[test_i]);
        }
        mi_rt_event_destroy(test_events[test_count]);
        std::sort(&test_times[0], &test_times[test_count]);
        double samples_ms = 0.0;
        const int sample_count = (test_count + 1) / 2;
        for (int i = 0; i < sample_count; ++i) {
            samples_ms += test_times[test_count / 4 + i];  // the middle half of the sorted samples (gemm/gemm_test.cu:399-404)
        }
        const double flops = sample_count * double(params.M) * params.N * params.K * 2.0 * 1000.0 / samples_ms;
        if (params.out_ms) {
            params.out_ms[static_cast<uint32_t>(algo)] = samples_ms / sample_count;
        }
        const bool bold = double(params.M) * params.N * params.K >= 1e11 && params.test_data_code_A >= TestDataCode::uniform;
        printf("TestParams{%u,%u,%u, %i,%i %s} %.3g ms %.4g \x1b[%imTFLOPS\x1b[0m max_rel_err %.2e %s(%s)\n", params.M, params.N,
               params.K, static_cast<int>(params.test_data_code_A), static_cast<int>(params.test_data_code_B),
               params.ab_dtype == MI_BF16 ? "bf16" : "f16", samples_ms / sample_count, flops * 1e-12, bold ? 1 : 0, rel_err,
               failed ? "\x1b[31mFAILED\x1b[0m " : "", algorithm_name(algo));
        fflush(stdout);
    };

    for (uint32_t bit_index = 0; bit_index < algorithm_count() && bit_index < algorithm_max_count; ++bit_index) {
        if ((params.algorithm_code_bits >> bit_index & 1) == 0) {
            continue;
        }
        run_tests(static_cast<AlgorithmCode>(bit_index), 25);
    }

    printf("\n");

    gpu_check(mi_rt_stream_synchronize(stream), "stream sync");
    mi_rt_free(d_a);
    mi_rt_free(d_b);
    mi_rt_free(d_bCol);
    if (d_a32) {
        mi_rt_free(d_a32);
        mi_rt_free(d_b32);
        mi_rt_free(d_bCol32);
    }
    mi_rt_free(d_c_baseline);
    mi_rt_free(d_c_tested);
    mi_rt_free(d_result);
    return failures;
}

// One launch seen from inside: per-workgroup stamps of the constant 100 MHz clock and of the core clock counter.
int gemm_timeline(TimelineParams params, gpu_stream_t stream)
{
    const size_t M = params.M, N = params.N, K = params.K;
    void* d_a = device_alloc(2 * M * K);
    void* d_b = device_alloc(2 * N * K);
    float* d_c = static_cast<float*>(device_alloc(sizeof(float) * M * N));
    const bool bf16 = params.ab_dtype == MI_BF16;
    // the benchmark distributions: normal(0,1)/sqrt(K) for bf16, uniform[-1,1] for fp16
    const int code = static_cast<int>(bf16 ? TestDataCode::normal : TestDataCode::uniform);
    const double param = bf16 ? 1.0 / sqrt(double(K)) : 1.0;
    gpu_check(mi_init_test_data(d_a, params.M, params.K, code, false, params.ab_dtype, param, SEED_A, stream), "init a");
    gpu_check(mi_init_test_data(d_b, params.N, params.K, code, true, params.ab_dtype, param, SEED_B, stream), "init b");
    GPU_Tensors t{params.M, params.N, params.K, d_a, d_b, d_c, 0, 1, 0, params.ab_dtype};
    const mi_gemm_tensors abi = t.abi();
    int tile = params.tile, k_mode = MI_K_AUTO, k_splits = 0;
    gpu_check(mi_matmul_mfma_plan(&abi, MI_K_AUTO, params.tile, &tile, &k_mode, &k_splits), "plan");

    // The stamp buffer is sized to the grid (found by growing it until the launch accepts it) and kept small: clearing
    // a large buffer between launches would itself disturb the caches the kernel runs from.
    constexpr uint32_t SLOTS = 32;
    uint32_t max_wg = 1024, wgs = 0;
    uint64_t* d_stamps = nullptr;
    size_t stamp_bytes = 0;
    for (;; max_wg *= 4) {
        stamp_bytes = sizeof(uint64_t) * 2 * SLOTS * max_wg;
        d_stamps = static_cast<uint64_t*>(device_alloc(stamp_bytes));
        gpu_check(mi_rt_memset_async(d_stamps, 0, stamp_bytes, stream), "memset stamps");
        const int st = mi_matmul_mfma_timeline(&abi, MI_K_AUTO, params.tile, d_stamps, SLOTS, max_wg, &wgs, stream);
        if (st == MI_OK) {
            break;
        }
        gpu_check(mi_rt_stream_synchronize(stream), "stream sync");
        mi_rt_free(d_stamps);
        if (st != MI_ERR_WORKSPACE || max_wg >= (1u << 22)) {
            gpu_check(st, "timeline launch");
        }
    }
    // The clocks take 25 to 30 ms of load to settle: warm up with plain launches for at least `warmup` launches and
    // 60 ms (a 100 us problem needs hundreds of them), then report one stamped launch.
    {
        void *w0 = nullptr, *w1 = nullptr;
        gpu_check(mi_rt_event_create(&w0), "event create");
        gpu_check(mi_rt_event_create(&w1), "event create");
        gpu_check(mi_rt_event_record(w0, stream), "event record");
        float ms = 0.0f;
        for (uint32_t done = 0; done < 20000 && (done < params.warmup || ms < 60.0f);) {
            for (uint32_t i = 0; i < 8; ++i, ++done) {
                gpu_check(mi_matmul_mfma(&abi, MI_K_AUTO, params.tile, stream), "warm-up launch");
            }
            gpu_check(mi_rt_event_record(w1, stream), "event record");
            gpu_check(mi_rt_event_synchronize(w1), "event sync");
            gpu_check(mi_rt_event_elapsed_ms(&ms, w0, w1), "elapsed");
        }
        mi_rt_event_destroy(w0);
        mi_rt_event_destroy(w1);
    }
    gpu_check(mi_rt_memset_async(d_stamps, 0, sizeof(uint64_t) * 2 * SLOTS * wgs, stream), "memset stamps");
    gpu_check(mi_matmul_mfma_timeline(&abi, MI_K_AUTO, params.tile, d_stamps, SLOTS, max_wg, &wgs, stream), "timeline launch");
    gpu_check(mi_rt_stream_synchronize(stream), "stream sync");
    std::vector<uint64_t> h(size_t(2) * SLOTS * wgs);
    gpu_check(mi_rt_memcpy_d2h(h.data(), d_stamps, sizeof(uint64_t) * h.size()), "read stamps");

    auto wall = [&](uint32_t g, uint32_t i) { return h[(size_t(g) * SLOTS + i) * 2]; };
    auto core = [&](uint32_t g, uint32_t i) { return h[(size_t(g) * SLOTS + i) * 2 + 1]; };
    // the last slot names the CU: hardware id register + 1 (CU, shader array, shader engine in bits 8..15) and XCC id
    auto xcc_of = [&](uint32_t g) { return uint32_t(core(g, SLOTS - 1)); };
    auto cu_key = [&](uint32_t g) { return xcc_of(g) << 8 | (uint32_t(wall(g, SLOTS - 1) - 1) >> 8 & 0xffu); };
    uint64_t t0 = ~uint64_t(0), t1 = 0;
    uint32_t max_stamps = 0;
    std::vector<uint32_t> count(wgs, 0);
    for (uint32_t g = 0; g < wgs; ++g) {
        while (count[g] < SLOTS - 1 && wall(g, count[g]) != 0) {
            ++count[g];
        }
        max_stamps = std::max(max_stamps, count[g]);
        if (count[g]) {
            t0 = std::min(t0, wall(g, 0));
            t1 = std::max(t1, wall(g, count[g] - 1));
        }
    }
    const double span_us = double(t1 - t0) * 0.01;
    printf("timeline %ux%ux%u %s, tile %s, %s, %i K split(s): %u workgroups, up to %u stamps each\n", params.M, params.N,
           params.K, bf16 ? "bf16" : "f16", mi_tile_name(tile), mi_k_mode_name(k_mode), k_splits, wgs, max_stamps);
    printf("first entry to last store landed: %.2f us = %.1f TFLOP/s\n", span_us, 2.0 * M * N * K / span_us * 1e-6);
    if (max_stamps < 5) {
        printf("no stamps recorded\n");
        return 1;
    }
    struct Stat {
        double mn = 1e30, mx = 0, sum = 0, mhz = 0;
        uint32_t n = 0;
        void add(double us, double cycles)
        {
            mn = std::min(mn, us);
            mx = std::max(mx, us);
            sum += us;
            mhz += us > 0 ? cycles / us : 0;
            ++n;
        }
        void print(const char* label) const
        {
            if (n) {
                printf("%-34s %10.2f %10.2f %10.2f %10.0f %8u\n", label, mn, sum / n, mx, mhz / n, n);
            }
        }
    };
    // stamps: 0 entry | per item: K tile 0 landed, K loop end, stores issued | last: stores landed
    static const char* const phase_name[3] = {"wait for K tile 0", "K loop", "store issue"};
    printf("%-34s %10s %10s %10s %10s %8s\n", "phase (us)", "min", "mean", "max", "core MHz", "count");
    for (uint32_t i = 1; i < max_stamps; ++i) {
        Stat st;
        for (uint32_t g = 0; g < wgs; ++g) {
            if (count[g] == max_stamps) {  // workgroups with fewer items are left out of the per-phase rows
                st.add(double(wall(g, i) - wall(g, i - 1)) * 0.01, double(core(g, i) - core(g, i - 1)));
            }
        }
        char label[64];
        if (i + 1 == max_stamps) {
            snprintf(label, sizeof label, "stores landed");
        }
        else {
            snprintf(label, sizeof label, "item %u %s", (i - 1) / 3, phase_name[(i - 1) % 3]);
        }
        st.print(label);
    }
    // One CU through the launch: its workgroups in order of entry.  `turn` = how many workgroups the CU ran before.
    std::vector<uint32_t> order(wgs);
    for (uint32_t g = 0; g < wgs; ++g) {
        order[g] = g;
    }
    std::sort(order.begin(), order.end(), [&](uint32_t x, uint32_t y) {
        return cu_key(x) != cu_key(y) ? cu_key(x) < cu_key(y) : wall(x, 0) < wall(y, 0);
    });
    constexpr uint32_t TURNS = 8;
    Stat gap_landed[TURNS], gap_issued[TURNS], fill[TURNS], loop[TURNS], store[TURNS], life[TURNS];
    uint32_t cus_seen = 0, overlapped = 0;
    for (uint32_t i = 0, turn = 0; i < wgs; ++i) {
        const uint32_t g = order[i];
        if (count[g] < 5) {
            continue;
        }
        const bool same_cu = i > 0 && cu_key(order[i - 1]) == cu_key(g) && count[order[i - 1]] >= 5;
        turn = same_cu ? turn + 1 : 0;
        cus_seen += same_cu ? 0 : 1;
        const uint32_t tr = std::min(turn, TURNS - 1);
        if (same_cu) {
            const uint32_t q = order[i - 1];
            const double from_landed = (double(wall(g, 0)) - double(wall(q, count[q] - 1))) * 0.01;
            const double from_issued = (double(wall(g, 0)) - double(wall(q, count[q] - 2))) * 0.01;
            overlapped += from_issued < 0 ? 1 : 0;  // (two workgroups at once on the CU: tiles with a half-LDS ring)
            gap_landed[tr].add(from_landed, 0);
            gap_issued[tr].add(from_issued, 0);
        }
        fill[tr].add(double(wall(g, 1) - wall(g, 0)) * 0.01, double(core(g, 1) - core(g, 0)));
        loop[tr].add(double(wall(g, 2) - wall(g, 1)) * 0.01, double(core(g, 2) - core(g, 1)));
        store[tr].add(double(wall(g, 3) - wall(g, 2)) * 0.01, double(core(g, 3) - core(g, 2)));
        life[tr].add(double(wall(g, count[g] - 1) - wall(g, 0)) * 0.01, double(core(g, count[g] - 1) - core(g, 0)));
    }
    printf("%u CUs seen; by the workgroup's turn on its CU (first item of each workgroup)%s\n", cus_seen,
           overlapped ? "; workgroups overlap on a CU" : "");
    for (uint32_t tr = 0; tr < TURNS; ++tr) {
        char label[64];
        snprintf(label, sizeof label, "turn %u%s: previous landed -> entry", tr, tr + 1 == TURNS ? "+" : "");
        gap_landed[tr].print(label);
        snprintf(label, sizeof label, "turn %u%s: previous issued -> entry", tr, tr + 1 == TURNS ? "+" : "");
        gap_issued[tr].print(label);
        snprintf(label, sizeof label, "turn %u%s: wait for K tile 0", tr, tr + 1 == TURNS ? "+" : "");
        fill[tr].print(label);
        snprintf(label, sizeof label, "turn %u%s: K loop", tr, tr + 1 == TURNS ? "+" : "");
        loop[tr].print(label);
        snprintf(label, sizeof label, "turn %u%s: store issue", tr, tr + 1 == TURNS ? "+" : "");
        store[tr].print(label);
        snprintf(label, sizeof label, "turn %u%s: entry -> landed", tr, tr + 1 == TURNS ? "+" : "");
        life[tr].print(label);
    }
    printf("%-34s %10s %10s %10s %8s\n", "workgroups end, by XCD (us)", "first", "last", "K-loop MHz", "count");
    for (uint32_t x = 0; x < 8; ++x) {
        double mn = 1e30, mx = 0, mhz = 0;
        uint32_t n = 0;
        for (uint32_t g = 0; g < wgs; ++g) {
            if (count[g] < 5 || xcc_of(g) != x) {
                continue;
            }
            const double fin = double(wall(g, count[g] - 1) - t0) * 0.01;
            mn = std::min(mn, fin);
            mx = std::max(mx, fin);
            const double us = double(wall(g, 2) - wall(g, 1)) * 0.01;  // first K loop of the workgroup
            mhz += us > 0 ? double(core(g, 2) - core(g, 1)) / us : 0;
            ++n;
        }
        if (n) {
            printf("xcd %-30u %10.2f %10.2f %10.0f %8u\n", x, mn, mx, mhz / n, n);
        }
    }
    fflush(stdout);
    mi_rt_free(d_a);
    mi_rt_free(d_b);
    mi_rt_free(d_c);
    mi_rt_free(d_stamps);
    return 0;
}

int mfma_ceiling_report(gpu_stream_t stream)
{
    constexpr uint32_t ROWS = 4096, COLS = 4096;  // 32 MiB of 16-bit operands: 512 B per lane of 256 CUs x 256 lanes
    const size_t bytes = size_t(2) * ROWS * COLS;
    void* d_ops = device_alloc(bytes);
    uint64_t* d_clocks = static_cast<uint64_t*>(device_alloc(sizeof(uint64_t) * 2 * 1024));
    float* d_sink = static_cast<float*>(device_alloc(sizeof(float)));
    void *ev0 = nullptr, *ev1 = nullptr;
    gpu_check(mi_rt_event_create(&ev0), "event create");
    gpu_check(mi_rt_event_create(&ev1), "event create");
    struct Data {
        const char* name;
        int dtype, code;
        double param;
    };
    const Data data[] = {{"bf16 normal(0,1)/sqrt(8192) (headline operands)", MI_BF16, int(TestDataCode::normal), 1.0 / sqrt(8192.0)},
                         {"f16 uniform[-1,1]", MI_F16, int(TestDataCode::uniform), 1.0},
                         {"bf16 zeros", MI_BF16, -1, 0.0}};
    printf("%-50s %-12s %10s %10s %14s\n", "operands", "MFMA", "TFLOP/s", "core MHz", "cycles / MFMA");
    for (const Data& d : data) {
        if (d.code < 0) {
            gpu_check(mi_rt_memset_async(d_ops, 0, bytes, stream), "memset");
        }
        else {
            gpu_check(mi_init_test_data(d_ops, ROWS, COLS, d.code, false, d.dtype, d.param, SEED_A, stream), "init");
        }
        for (int tile : {32, 16}) {
            const uint32_t iters = 4000;
            uint32_t wgs = 0;
            double flop = 0;
            for (int rep = 0; rep < 6; ++rep) {  // the clocks settle over a few milliseconds of load
                if (rep == 5) {
                    gpu_check(mi_rt_event_record(ev0, stream), "event record");
                }
                gpu_check(mi_mfma_ceiling(d_ops, bytes, d.dtype, tile, iters, d_clocks, d_sink, &wgs, &flop, stream), "ceiling");
            }
            gpu_check(mi_rt_event_record(ev1, stream), "event record");
            gpu_check(mi_rt_stream_synchronize(stream), "stream sync");
            float ms = 0;
            gpu_check(mi_rt_event_elapsed_ms(&ms, ev0, ev1), "elapsed");
            std::vector<uint64_t> h(size_t(2) * wgs);
            gpu_check(mi_rt_memcpy_d2h(h.data(), d_clocks, sizeof(uint64_t) * h.size()), "read clocks");
            double mhz = 0, cyc = 0;
            for (uint32_t g = 0; g < wgs; ++g) {
                mhz += 100.0 * double(h[2 * g]) / double(h[2 * g + 1]);
                cyc += double(h[2 * g]);
            }
            const double mfmas = double(iters) * 2.0 * (tile == 32 ? 16.0 : 64.0);
            printf("%-50s %-12s %10.1f %10.0f %14.1f\n", d.name, tile == 32 ? "32x32x16" : "16x16x32", flop / (ms * 1e-3) * 1e-12,
                   mhz / wgs, cyc / wgs / mfmas);
            fflush(stdout);
        }
    }
    mi_rt_event_destroy(ev0);
    mi_rt_event_destroy(ev1);
    mi_rt_free(d_ops);
    mi_rt_free(d_clocks);
    mi_rt_free(d_sink);
    return 0;
}

// The planner ranks plans by two measured constants per tile: the main-loop time per 64-deep K step with every CU busy, and
// the cost of a workgroup outside the main loop.  This measures both on the machine at hand, tile by tile, from two
// one-round problems that differ only in K (bf16 normal data, output stationary, the reference's statistic over 25
// launches after 30 ms of the same launch), and prints them beside what the planner's own estimate implies for the same two
// problems: the way to see whether the table still fits a new box or toolchain, and the figures to put into it if not.
int planner_calibration(gpu_stream_t stream)
{
    char name[256], arch[256];
    int cus = 0;
    gpu_check(mi_rt_device_info(0, name, arch, &cus, nullptr, nullptr, nullptr), "device info");
    constexpr uint32_t K1 = 2048, K2 = 6144;
    printf("one round of each tile on %i CUs, bf16 normal(0,1)/sqrt(K), K = %u and %u\n", cus, K1, K2);
    printf("%-10s %8s %10s %10s | %12s %12s | %12s %12s\n", "tile", "M x N", "us @K1", "us @K2", "us per K64", "(planner)",
           "fixed us", "(planner)");
    void *ev0 = nullptr, *ev1 = nullptr;
    gpu_check(mi_rt_event_create(&ev0), "event create");
    gpu_check(mi_rt_event_create(&ev1), "event create");
    std::string environment;
    for (int tile = 1; tile < mi_tile_count(); ++tile) {
        uint32_t bm = 0, bn = 0;
        int per_cu = 1;
        gpu_check(mi_tile_shape(tile, &bm, &bn, &per_cu, nullptr), "tile shape");
        // a grid of tiles that fills every place of one round exactly: 16 x (CUs / 16) tiles, twice that for two per CU
        if (cus % 16) {
            continue;
        }
        const uint32_t M = bm * 16, N = bn * uint32_t(cus / 16) * uint32_t(per_cu);
        void* d_a = device_alloc(size_t(2) * M * K2);
        void* d_b = device_alloc(size_t(2) * N * K2);
        float* d_c = static_cast<float*>(device_alloc(sizeof(float) * M * N));
        gpu_check(mi_init_test_data(d_a, M, K2, int(TestDataCode::normal), false, MI_BF16, 1.0 / sqrt(double(K2)), SEED_A, stream), "init");
        gpu_check(mi_init_test_data(d_b, N, K2, int(TestDataCode::normal), true, MI_BF16, 1.0 / sqrt(double(K2)), SEED_B, stream), "init");
        double us[2] = {0, 0}, est[2] = {0, 0};
        bool ok = true;
        for (int which = 0; which < 2 && ok; ++which) {
            const uint32_t K = which ? K2 : K1;  // (the same buffers read as M x K and N x K: the values do not matter)
            const mi_gemm_tensors t{M, N, K, d_a, d_b, d_c, 0, 1, 0, MI_BF16};
            if (!mi_matmul_mfma_supports(&t, MI_K_OUTPUT_STATIONARY, tile) ||
                mi_matmul_mfma_estimate_us(&t, MI_K_OUTPUT_STATIONARY, tile, 0, &est[which]) != MI_OK) {
                ok = false;
                break;
            }
            const int settle = int(30000.0 / std::max(5.0, est[which])) + 1;
            for (int i = 0; i < settle; ++i) {
                gpu_check(mi_matmul_mfma(&t, MI_K_OUTPUT_STATIONARY, tile, stream), "matmul");
                if (i % 32 == 31) {
                    gpu_check(mi_rt_stream_synchronize(stream), "stream sync");
                }
            }
            float times[25];
            for (float& ms : times) {
                gpu_check(mi_rt_event_record(ev0, stream), "event record");
                gpu_check(mi_matmul_mfma(&t, MI_K_OUTPUT_STATIONARY, tile, stream), "matmul");
                gpu_check(mi_rt_event_record(ev1, stream), "event record");
                gpu_check(mi_rt_stream_synchronize(stream), "stream sync");
                gpu_check(mi_rt_event_elapsed_ms(&ms, ev0, ev1), "elapsed");
            }
            std::sort(&times[0], &times[25]);
            double sum = 0;
            for (int i = 6; i < 19; ++i) {
                sum += times[i];  // the middle half (gemm/gemm_test.cu:399-404)
            }
            us[which] = sum / 13.0 * 1e3;
        }
        if (ok) {
            const double steps1 = K1 / 64.0, steps2 = K2 / 64.0;
            const double per_k64 = (us[1] - us[0]) / (steps2 - steps1), fixed = us[0] - steps1 * per_k64;
            const double est_k64 = (est[1] - est[0]) / (steps2 - steps1), est_fixed = est[0] - steps1 * est_k64;
            printf("%-10s %4ux%-5u %9.1f %10.1f | %12.3f %12.3f | %12.1f %12.1f\n", mi_tile_name(tile), M, N, us[0], us[1], per_k64,
                   est_k64, fixed, est_fixed);
            fflush(stdout);
            if (per_k64 > 0 && fixed > 0) {
                char entry[64];
                snprintf(entry, sizeof(entry), "%s%s=%.3f/%.1f", environment.empty() ? "" : ",", mi_tile_name(tile), per_k64, fixed);
                environment += entry;
            }
        }
        mi_rt_free(d_a);
        mi_rt_free(d_b);
        mi_rt_free(d_c);
    }
    mi_rt_event_destroy(ev0);
    mi_rt_event_destroy(ev1);
    // (what the library reads when it is loaded; mi_tile_set_planner_constants does the same from code)
    printf("to plan with the measured figures:\nMI_GEMM_PLANNER_CONSTANTS=%s\n", environment.c_str());
    return 0;
}

}  // namespace gemm_test_impl

int mfma_ceiling_report(gpu_stream_t stream)
{
    return gemm_test_impl::mfma_ceiling_report(stream);
}

int gemm_timeline(TimelineParams params, gpu_stream_t stream)
{
    return gemm_test_impl::gemm_timeline(params, stream);
}

int planner_calibration(gpu_stream_t stream)
{
    return gemm_test_impl::planner_calibration(stream);
}

int gemm_test(TestParams params, gpu_stream_t stream)
{
    return gemm_test_impl::gemm_test(params, stream);
}
