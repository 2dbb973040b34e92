// Device runtime shim: allocation, copies, streams, events, device queries.
// Stands in for the allocator library of the reference
// (minit/cuda/allocator.py:30-50) with explicit streams and error codes.
#include "common.h"

#include <cstdarg>
#include <cstdio>
#include <cstring>

namespace mh {

static thread_local char g_error[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

int compute_units() {
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
        cached[dev] = cus;
    }
    return cached[dev];
}

__global__ void copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n) {
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}

}  // namespace mh

using namespace mh;

extern "C" {

int mh_abi_version(void) { return 1; }

const char* mh_last_error(void) { return g_error; }

int mh_device_count(int* count) {
    MH_REQUIRE(count != nullptr, "mh_device_count: null output");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        *count = 0;
        return fail(MH_ERR_HIP, "hipGetDeviceCount: %s", hipGetErrorString(e));
    }
    *count = n;
    return MH_OK;
}

int mh_device_info(int* compute_units_out, int* wavefront_size, size_t* total_mem,
                   size_t* lds_per_block, int* clock_khz, char* name, size_t name_len) {
    int dev = 0;
    MH_CHECK_HIP(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    MH_CHECK_HIP(hipGetDeviceProperties(&prop, dev));
    if (compute_units_out) *compute_units_out = prop.multiProcessorCount;
    if (wavefront_size) *wavefront_size = prop.warpSize;
    if (total_mem) *total_mem = prop.totalGlobalMem;
    if (lds_per_block) *lds_per_block = prop.sharedMemPerBlock;
    if (clock_khz) *clock_khz = prop.clockRate;
    if (name && name_len) {
        snprintf(name, name_len, "%s (%s)", prop.name, prop.gcnArchName);
    }
    return MH_OK;
}

int mh_malloc(void** ptr, size_t bytes) {
    MH_REQUIRE(ptr != nullptr, "mh_malloc: null output");
    *ptr = nullptr;
    if (bytes == 0) return MH_OK;
    MH_CHECK_HIP(hipMalloc(ptr, bytes));
    return MH_OK;
}

int mh_free(void* ptr) {
    if (ptr) MH_CHECK_HIP(hipFree(ptr));
    return MH_OK;
}

int mh_host_malloc(void** ptr, size_t bytes) {
    MH_REQUIRE(ptr != nullptr, "mh_host_malloc: null output");
    *ptr = nullptr;
    if (bytes == 0) return MH_OK;
    MH_CHECK_HIP(hipHostMalloc(ptr, bytes, hipHostMallocDefault));
    return MH_OK;
}

int mh_host_free(void* ptr) {
    if (ptr) MH_CHECK_HIP(hipHostFree(ptr));
    return MH_OK;
}

int mh_memcpy(void* dst, const void* src, size_t bytes, mh_stream_t stream) {
    if (bytes == 0) return MH_OK;
    MH_REQUIRE(dst && src, "mh_memcpy: null pointer");
    MH_CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDefault, as_stream(stream)));
    return MH_OK;
}

int mh_memset(void* dst, int value, size_t bytes, mh_stream_t stream) {
    if (bytes == 0) return MH_OK;
    MH_REQUIRE(dst != nullptr, "mh_memset: null pointer");
    MH_CHECK_HIP(hipMemsetAsync(dst, value, bytes, as_stream(stream)));
    return MH_OK;
}

int mh_stream_create(mh_stream_t* stream) {
    MH_REQUIRE(stream != nullptr, "mh_stream_create: null output");
    hipStream_t s;
    MH_CHECK_HIP(hipStreamCreate(&s));  // default priority on purpose
    *stream = s;
    return MH_OK;
}

int mh_stream_destroy(mh_stream_t stream) {
    if (stream) MH_CHECK_HIP(hipStreamDestroy(as_stream(stream)));
    return MH_OK;
}

int mh_stream_synchronize(mh_stream_t stream) {
    MH_CHECK_HIP(hipStreamSynchronize(as_stream(stream)));
    return MH_OK;
}

int mh_device_synchronize(void) {
    MH_CHECK_HIP(hipDeviceSynchronize());
    return MH_OK;
}

int mh_event_create(mh_event_t* event) {
    MH_REQUIRE(event != nullptr, "mh_event_create: null output");
    hipEvent_t e;
    MH_CHECK_HIP(hipEventCreate(&e));
    *event = e;
    return MH_OK;
}

int mh_event_destroy(mh_event_t event) {
    if (event) MH_CHECK_HIP(hipEventDestroy(reinterpret_cast<hipEvent_t>(event)));
    return MH_OK;
}

int mh_event_record(mh_event_t event, mh_stream_t stream) {
    MH_REQUIRE(event != nullptr, "mh_event_record: null event");
    MH_CHECK_HIP(hipEventRecord(reinterpret_cast<hipEvent_t>(event), as_stream(stream)));
    return MH_OK;
}

int mh_event_synchronize(mh_event_t event) {
    MH_REQUIRE(event != nullptr, "mh_event_synchronize: null event");
    MH_CHECK_HIP(hipEventSynchronize(reinterpret_cast<hipEvent_t>(event)));
    return MH_OK;
}

int mh_event_elapsed_ms(float* ms, mh_event_t start, mh_event_t stop) {
    MH_REQUIRE(ms && start && stop, "mh_event_elapsed_ms: null argument");
    MH_CHECK_HIP(hipEventElapsedTime(ms, reinterpret_cast<hipEvent_t>(start),
                                     reinterpret_cast<hipEvent_t>(stop)));
    return MH_OK;
}

int mh_copy_kernel(mh_stream_t stream, const void* src, void* dst, size_t bytes) {
    if (bytes == 0) return MH_OK;
    MH_REQUIRE(src && dst, "mh_copy_kernel: null pointer");
    MH_REQUIRE(bytes % 16 == 0, "mh_copy_kernel: bytes must be a multiple of 16");
    MH_REQUIRE(((uintptr_t)src | (uintptr_t)dst) % 16 == 0, "mh_copy_kernel: pointers must be 16-byte aligned");
    size_t n = bytes / 16;
    size_t blocks = (n + 255) / 256;
    size_t cap = (size_t)compute_units() * 32;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(copy_kernel, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                       (const uint4*)src, (uint4*)dst, n);
    MH_CHECK_LAUNCH();
    return MH_OK;
}

}  // extern "C"
