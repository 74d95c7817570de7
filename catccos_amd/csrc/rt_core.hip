// Error reporting and the small device-runtime shim behind the C ABI.
#include "mx_common.h"

namespace cmx {
namespace {
thread_local std::string g_last_error;
}
void set_error(const std::string& msg) { g_last_error = msg; }
}  // namespace cmx

extern "C" {

int cmx_version(void) { return 100; }

const char* cmx_last_error(void) { return cmx::g_last_error.c_str(); }

int cmx_rt_device_count(int* count) {
    CMX_REQUIRE(count, "null pointer");
    CMX_HIP(hipGetDeviceCount(count));
    return CMX_OK;
}

int cmx_rt_set_device(int device) {
    CMX_HIP(hipSetDevice(device));
    return CMX_OK;
}

int cmx_rt_malloc(void** ptr, size_t bytes) {
    CMX_REQUIRE(ptr, "null pointer");
    CMX_HIP(hipMalloc(ptr, bytes ? bytes : 1));
    return CMX_OK;
}

int cmx_rt_free(void* ptr) {
    if (ptr) CMX_HIP(hipFree(ptr));
    return CMX_OK;
}

int cmx_rt_malloc_host(void** ptr, size_t bytes) {
    CMX_REQUIRE(ptr, "null pointer");
    CMX_HIP(hipHostMalloc(ptr, bytes ? bytes : 1, hipHostMallocDefault));
    return CMX_OK;
}

int cmx_rt_free_host(void* ptr) {
    if (ptr) CMX_HIP(hipHostFree(ptr));
    return CMX_OK;
}

int cmx_rt_memcpy_h2d(void* dst, const void* host_src, size_t bytes) {
    if (bytes == 0) return CMX_OK;
    CMX_REQUIRE(dst && host_src, "null pointer");
    CMX_HIP(hipMemcpy(dst, host_src, bytes, hipMemcpyHostToDevice));
    return CMX_OK;
}

int cmx_rt_memcpy_d2h(void* host_dst, const void* src, size_t bytes) {
    if (bytes == 0) return CMX_OK;
    CMX_REQUIRE(host_dst && src, "null pointer");
    CMX_HIP(hipMemcpy(host_dst, src, bytes, hipMemcpyDeviceToHost));
    return CMX_OK;
}

int cmx_rt_memset(void* dst, int value, size_t bytes) {
    if (bytes == 0) return CMX_OK;
    CMX_REQUIRE(dst, "null pointer");
    CMX_HIP(hipMemset(dst, value, bytes));
    return CMX_OK;
}

int cmx_rt_stream_create(cmx_stream_t* stream) {
    CMX_REQUIRE(stream, "null pointer");
    hipStream_t s;
    CMX_HIP(hipStreamCreate(&s));
    *stream = s;
    return CMX_OK;
}

int cmx_rt_stream_destroy(cmx_stream_t stream) {
    if (stream) CMX_HIP(hipStreamDestroy(static_cast<hipStream_t>(stream)));
    return CMX_OK;
}

int cmx_rt_stream_sync(cmx_stream_t stream) {
    CMX_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    return CMX_OK;
}

}  // extern "C"
