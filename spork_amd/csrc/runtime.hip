// Thin HIP runtime layer of the C ABI: status strings, error bookkeeping and the handful of runtime calls the
// plain-C++ host driver needs (it never includes HIP headers).  Wraps what gemm/gemm_test.cu uses of the CUDA
// runtime: stream-ordered alloc/free (:218-226,466-471), memset (:246), events (:275-284,394-398), stream sync (:392).
#include <atomic>
#include <string.h>

#include "mi_internal.hpp"

namespace mi_gemm {

static thread_local hipError_t g_last_hip_error = hipSuccess;

void record_hip_error(hipError_t err)
{
    g_last_hip_error = err;
}

int device_compute_units()
{
    static std::atomic<int> cached[64];  // zero-initialised; threads may race to store the same value
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        return 256;
    }
    if (cached[dev].load(std::memory_order_relaxed) == 0) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
            cus = 256;
        }
        cached[dev].store(cus, std::memory_order_relaxed);
    }
    return cached[dev].load(std::memory_order_relaxed);
}

int validate_tensors(const mi_gemm_tensors* t)
{
    if (!t || !t->a || !t->b || !t->c) {
        return MI_ERR_BAD_ARGUMENT;
    }
    if (t->M == 0 || t->N == 0 || t->K == 0) {
        return MI_ERR_BAD_ARGUMENT;
    }
    if (t->ab_dtype != MI_F16 && t->ab_dtype != MI_BF16) {
        return MI_ERR_BAD_ARGUMENT;
    }
    if (t->a_col_major > 1 || t->b_col_major > 1 || t->c_col_major > 1) {
        return MI_ERR_BAD_ARGUMENT;
    }
    return MI_OK;
}

}  // namespace mi_gemm

using namespace mi_gemm;

extern "C" {

const char* mi_status_string(int status)
{
    switch (status) {
    case MI_OK: return "ok";
    case MI_ERR_UNSUPPORTED: return "unsupported shape, layout or dtype for this algorithm";
    case MI_ERR_BAD_ARGUMENT: return "bad argument";
    case MI_ERR_WORKSPACE: return "workspace too small";
    case MI_ERR_HIP: return "HIP runtime error";
    case MI_ERR_NO_DEVICE: return "no gfx950 device";
    }
    return "unknown status";
}

int mi_last_hip_error(void)
{
    return (int)g_last_hip_error;
}

const char* mi_last_hip_error_string(void)
{
    return hipGetErrorString(g_last_hip_error);
}

int mi_rt_device_count(int* count)
{
    if (!count) {
        return MI_ERR_BAD_ARGUMENT;
    }
    *count = 0;
    MI_HIP_TRY(hipGetDeviceCount(count));
    return MI_OK;
}

int mi_rt_set_device(int device)
{
    MI_HIP_TRY(hipSetDevice(device));
    // the set-up call of a process that uses this device: look up the address of the library's scratch array here, so
    // that mi_matmul_mfma_static finds it ready (it looks it up itself, and reports a failure, when this did not)
    (void)resolve_static_scratch(nullptr);
    (void)resolve_tile_counters();
    return MI_OK;
}

int mi_rt_device_info(int device, char* name, char* gcn_arch, int* compute_units, int* clock_khz,
                      size_t* lds_bytes_per_block, size_t* global_mem_bytes)
{
    hipDeviceProp_t prop;
    MI_HIP_TRY(hipGetDeviceProperties(&prop, device));
    if (name) {
        strncpy(name, prop.name, 255);
        name[255] = 0;
    }
    if (gcn_arch) {
        strncpy(gcn_arch, prop.gcnArchName, 255);
        gcn_arch[255] = 0;
    }
    if (compute_units) {
        *compute_units = prop.multiProcessorCount;
    }
    if (clock_khz) {
        *clock_khz = prop.clockRate;
    }
    if (lds_bytes_per_block) {
        *lds_bytes_per_block = prop.sharedMemPerBlock;
    }
    if (global_mem_bytes) {
        *global_mem_bytes = prop.totalGlobalMem;
    }
    return MI_OK;
}

int mi_rt_malloc(void** d_ptr, size_t bytes)
{
    if (!d_ptr) {
        return MI_ERR_BAD_ARGUMENT;
    }
    *d_ptr = nullptr;
    MI_HIP_TRY(hipMalloc(d_ptr, bytes));
    return MI_OK;
}

int mi_rt_free(void* d_ptr)
{
    MI_HIP_TRY(hipFree(d_ptr));
    return MI_OK;
}

int mi_rt_memset_async(void* d_ptr, int byte_value, size_t bytes, void* hip_stream)
{
    MI_HIP_TRY(hipMemsetAsync(d_ptr, byte_value, bytes, as_stream(hip_stream)));
    return MI_OK;
}

int mi_rt_memcpy_h2d(void* d_dst, const void* h_src, size_t bytes)
{
    MI_HIP_TRY(hipMemcpy(d_dst, h_src, bytes, hipMemcpyHostToDevice));
    return MI_OK;
}

int mi_rt_memcpy_d2h(void* h_dst, const void* d_src, size_t bytes)
{
    MI_HIP_TRY(hipMemcpy(h_dst, d_src, bytes, hipMemcpyDeviceToHost));
    return MI_OK;
}

int mi_rt_stream_create(void** hip_stream)
{
    if (!hip_stream) {
        return MI_ERR_BAD_ARGUMENT;
    }
    hipStream_t s = nullptr;
    MI_HIP_TRY(hipStreamCreate(&s));  // default priority on purpose
    *hip_stream = s;
    return MI_OK;
}

int mi_rt_stream_destroy(void* hip_stream)
{
    MI_HIP_TRY(hipStreamDestroy(as_stream(hip_stream)));
    return MI_OK;
}

int mi_rt_stream_synchronize(void* hip_stream)
{
    MI_HIP_TRY(hipStreamSynchronize(as_stream(hip_stream)));
    return MI_OK;
}

int mi_rt_device_synchronize(void)
{
    MI_HIP_TRY(hipDeviceSynchronize());
    return MI_OK;
}

int mi_rt_event_create(void** event)
{
    if (!event) {
        return MI_ERR_BAD_ARGUMENT;
    }
    hipEvent_t e = nullptr;
    MI_HIP_TRY(hipEventCreate(&e));
    *event = e;
    return MI_OK;
}

int mi_rt_event_record(void* event, void* hip_stream)
{
    MI_HIP_TRY(hipEventRecord(reinterpret_cast<hipEvent_t>(event), as_stream(hip_stream)));
    return MI_OK;
}

int mi_rt_event_synchronize(void* event)
{
    MI_HIP_TRY(hipEventSynchronize(reinterpret_cast<hipEvent_t>(event)));
    return MI_OK;
}

int mi_rt_event_elapsed_ms(float* ms, void* start_event, void* stop_event)
{
    if (!ms) {
        return MI_ERR_BAD_ARGUMENT;
    }
    MI_HIP_TRY(hipEventElapsedTime(ms, reinterpret_cast<hipEvent_t>(start_event), reinterpret_cast<hipEvent_t>(stop_event)));
    return MI_OK;
}

int mi_rt_event_destroy(void* event)
{
    MI_HIP_TRY(hipEventDestroy(reinterpret_cast<hipEvent_t>(event)));
    return MI_OK;
}

}  // extern "C"
