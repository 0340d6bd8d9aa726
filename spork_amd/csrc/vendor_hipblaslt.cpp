// hipBLASLt comparator behind the mi_gemm_tensors bundle (role of gemm/cutlass_gemm.cu:97-127 and of the cuBLAS row
// gemm/gemm_test.cu:249-261).  Host-only code; built into libmi_gemm_vendor.so.
#include <hipblaslt/hipblaslt.h>
#include <hip/hip_runtime_api.h>

#include <dlfcn.h>

#include <cstring>
#include <map>
#include <mutex>
#include <tuple>

#include "mi_gemm_vendor.h"

namespace {

thread_local int g_last_status = 0;

struct Key {
    uint32_t M, N, K;
    uint8_t ac, bc, cc, dt;
    size_t ws;
    bool operator<(const Key& o) const
    {
        return std::tie(M, N, K, ac, bc, cc, dt, ws) < std::tie(o.M, o.N, o.K, o.ac, o.bc, o.cc, o.dt, o.ws);
    }
};

struct Prepared {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t first = nullptr, second = nullptr, out = nullptr;
    hipblasLtMatmulAlgo_t algo;
    bool first_is_b = false;  // which caller buffer is hipBLASLt's "A"

    // (entries of the plan cache live until the process ends; a plan that is not kept is destroyed by its maker)
    void destroy()
    {
        if (desc) {
            hipblasLtMatmulDescDestroy(desc);
        }
        for (hipblasLtMatrixLayout_t l : {first, second, out}) {
            if (l) {
                hipblasLtMatrixLayoutDestroy(l);
            }
        }
        desc = nullptr;
        first = second = out = nullptr;
    }
};

std::mutex g_mutex;
hipblasLtHandle_t g_handle = nullptr;
bool g_tried = false;
std::map<Key, Prepared> g_cache;

bool ensure_handle()
{
    if (!g_tried) {
        g_tried = true;
        if (hipblasLtCreate(&g_handle) != HIPBLAS_STATUS_SUCCESS) {
            g_handle = nullptr;
        }
    }
    return g_handle != nullptr;
}

#define LT_TRY(expr)                            \
    do {                                        \
        const hipblasStatus_t st_ = (expr);     \
        if (st_ != HIPBLAS_STATUS_SUCCESS) {    \
            g_last_status = (int)st_;           \
            return MI_ERR_HIP;                  \
        }                                       \
    } while (0)

// hipBLASLt is column-major.  A row-major R x C buffer is a column-major C x R matrix with leading dimension C.
// Row-major C[M,N] is the column-major N x M product  B_op (N x K) * A_op (K x M);
// column-major C[M,N] is the product                 A_op (M x K) * B_op (K x N).
int fill_plan(const mi_gemm_tensors& t, size_t ws_bytes, Prepared& p);

// Builds the plan for one problem; on any failure everything created so far is destroyed again.
int prepare(const mi_gemm_tensors& t, size_t ws_bytes, Prepared& p)
{
    const int st = fill_plan(t, ws_bytes, p);
    if (st != MI_OK) {
        p.destroy();
    }
    return st;
}

int fill_plan(const mi_gemm_tensors& t, size_t ws_bytes, Prepared& p)
{
    const hipDataType in_type = t.ab_dtype == MI_BF16 ? HIP_R_16BF : HIP_R_16F;
    LT_TRY(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F));
    const uint64_t M = t.M, N = t.N, K = t.K;
    // each operand as a column-major matrix: (rows, cols, ld) and whether it must be transposed to become op(X)
    // A wanted as K x M (row-major C) or M x K (column-major C); stored M x K row-major = K x M column-major.
    // B wanted as N x K (row-major C) or K x N (column-major C); stored N x K row-major (b_col_major) = K x N column-major.
    hipblasOperation_t op_first, op_second;
    if (!t.c_col_major) {
        p.first_is_b = true;
        // first = B as N x K
        if (t.b_col_major) {
            LT_TRY(hipblasLtMatrixLayoutCreate(&p.first, in_type, K, N, K));
            op_first = HIPBLAS_OP_T;
        }
        else {
            LT_TRY(hipblasLtMatrixLayoutCreate(&p.first, in_type, N, K, N));
            op_first = HIPBLAS_OP_N;
        }
        // second = A as K x M
        if (!t.a_col_major) {
            LT_TRY(hipblasLtMatrixLayoutCreate(&p.second, in_type, K, M, K));
            op_second = HIPBLAS_OP_N;
        }
        else {
            LT_TRY(hipblasLtMatrixLayoutCreate(&p.second, in_type, M, K, M));
            op_second = HIPBLAS_OP_T;
        }
        LT_TRY(hipblasLtMatrixLayoutCreate(&p.out, HIP_R_32F, N, M, N));
    }
    else {
        p.first_is_b = false;
        // first = A as M x K
        if (!t.a_col_major) {
            LT_TRY(hipblasLtMatrixLayoutCreate(&p.first, in_type, K, M, K));
            op_first = HIPBLAS_OP_T;
        }
        else {
            LT_TRY(hipblasLtMatrixLayoutCreate(&p.first, in_type, M, K, M));
            op_first = HIPBLAS_OP_N;
        }
        // second = B as K x N
        if (t.b_col_major) {
            LT_TRY(hipblasLtMatrixLayoutCreate(&p.second, in_type, K, N, K));
            op_second = HIPBLAS_OP_N;
        }
        else {
            LT_TRY(hipblasLtMatrixLayoutCreate(&p.second, in_type, N, K, N));
            op_second = HIPBLAS_OP_T;
        }
        LT_TRY(hipblasLtMatrixLayoutCreate(&p.out, HIP_R_32F, M, N, M));
    }
    LT_TRY(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &op_first, sizeof(op_first)));
    LT_TRY(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &op_second, sizeof(op_second)));

    hipblasLtMatmulPreference_t pref = nullptr;
    LT_TRY(hipblasLtMatmulPreferenceCreate(&pref));
    const uint64_t max_ws = ws_bytes;
    hipblasStatus_t st = hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &max_ws, sizeof(max_ws));
    hipblasLtMatmulHeuristicResult_t result{};
    int found = 0;
    if (st == HIPBLAS_STATUS_SUCCESS) {
        st = hipblasLtMatmulAlgoGetHeuristic(g_handle, p.desc, p.first, p.second, p.out, p.out, pref, 1, &result, &found);
    }
    hipblasLtMatmulPreferenceDestroy(pref);
    if (st != HIPBLAS_STATUS_SUCCESS || found < 1) {
        g_last_status = (int)st;
        return st != HIPBLAS_STATUS_SUCCESS ? MI_ERR_HIP : MI_ERR_UNSUPPORTED;
    }
    // The algorithm is run with the caller's workspace pointer and size on every later call: one that was not reported
    // usable, or that wants more room than the caller has, must never be cached.
    if (const int verdict = mi_vendor_accepts_algorithm((int)result.state, result.workspaceSize, ws_bytes)) {
        g_last_status = (int)result.state;
        return verdict;
    }
    p.algo = result.algo;
    return MI_OK;
}

}  // namespace

extern "C" {

int mi_vendor_enabled(void)
{
    std::lock_guard<std::mutex> lock(g_mutex);
    return ensure_handle() ? 1 : 0;
}

int mi_vendor_library(char* out, size_t out_size)
{
    if (!out || out_size == 0) {
        return MI_ERR_BAD_ARGUMENT;
    }
    out[0] = 0;
    Dl_info info{};
    if (!dladdr(reinterpret_cast<void*>(&hipblasLtMatmul), &info) || !info.dli_fname) {
        return MI_ERR_UNSUPPORTED;
    }
    std::strncpy(out, info.dli_fname, out_size - 1);
    out[out_size - 1] = 0;
    return MI_OK;
}

int mi_vendor_version(void)
{
    std::lock_guard<std::mutex> lock(g_mutex);
    if (!ensure_handle()) {
        return -1;
    }
    int version = 0;
    if (hipblasLtGetVersion(g_handle, &version) != HIPBLAS_STATUS_SUCCESS) {
        return -1;
    }
    return version;
}

int mi_vendor_accepts_algorithm(int heuristic_state, size_t algorithm_workspace_bytes, size_t given_workspace_bytes)
{
    if (heuristic_state != (int)HIPBLAS_STATUS_SUCCESS) {
        return MI_ERR_UNSUPPORTED;
    }
    if (algorithm_workspace_bytes > given_workspace_bytes) {
        return MI_ERR_WORKSPACE;
    }
    return MI_OK;
}

int mi_vendor_last_status(void)
{
    return g_last_status;
}

int mi_vendor_matmul(const mi_gemm_tensors* t, void* d_workspace, size_t workspace_bytes, void* hip_stream)
{
    if (!t || !t->a || !t->b || !t->c || t->M == 0 || t->N == 0 || t->K == 0 ||
        (t->ab_dtype != MI_F16 && t->ab_dtype != MI_BF16)) {
        return MI_ERR_BAD_ARGUMENT;
    }
    if (!d_workspace || workspace_bytes < MI_VENDOR_MIN_WORKSPACE) {
        return MI_ERR_WORKSPACE;
    }
    std::lock_guard<std::mutex> lock(g_mutex);
    if (!ensure_handle()) {
        return MI_ERR_NO_DEVICE;
    }
    const size_t ws = workspace_bytes;
    const Key key{t->M, t->N, t->K, t->a_col_major, t->b_col_major, t->c_col_major, t->ab_dtype, ws};
    auto it = g_cache.find(key);
    if (it == g_cache.end()) {
        Prepared p;
        if (const int st = prepare(*t, ws, p)) {
            return st;
        }
        it = g_cache.emplace(key, p).first;
    }
    const Prepared& p = it->second;
    const float alpha = 1.0f, beta = 0.0f;
    const void* first = p.first_is_b ? t->b : t->a;
    const void* second = p.first_is_b ? t->a : t->b;
    LT_TRY(hipblasLtMatmul(g_handle, p.desc, &alpha, first, p.first, second, p.second, &beta, t->c, p.out, t->c, p.out,
                           &p.algo, d_workspace, ws, static_cast<hipStream_t>(hip_stream)));
    return MI_OK;
}

}  // extern "C"
