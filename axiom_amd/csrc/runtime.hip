// Device discovery, the backend stream, allocation and explicit transfers.
// Takes the place of Axiom's MetalContext / MetalExecutionStream / MetalStorage
// trio: one process-wide stream, every transfer an explicit hipMemcpyAsync.
#include "common.hpp"

#include <chrono>
#include <cstring>
#include <mutex>

namespace axhip {

namespace {
thread_local char g_last_error[512] = "";
std::mutex g_init_mutex;
bool g_initialised = false;
int g_device = -1;
hipStream_t g_stream = nullptr;
} // namespace

void set_last_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
}

int ensure_init() {
    {
        std::lock_guard<std::mutex> lock(g_init_mutex);
        if (g_initialised) return AXHIP_OK;
    }
    return axhip_init(0);
}

hipStream_t resolve_stream(void *stream) {
    return stream ? static_cast<hipStream_t>(stream) : g_stream;
}

} // namespace axhip

using namespace axhip;

extern "C" {

const char *axhip_version(void) { return "axhip 0.1 (gfx950)"; }

const char *axhip_last_error(void) { return g_last_error; }

size_t axhip_sizeof(int which) {
    switch (which) {
    case 0: return sizeof(AxhipSdpaParams);
    case 1: return sizeof(AxhipRowsProgram);
    case 2: return sizeof(AxhipGemmParams);
    case 3: return sizeof(AxhipOperand);
    case 4: return sizeof(AxhipChainOp);
    default: return 0;
    }
}

int axhip_device_count(int *count) {
    AXHIP_REQUIRE(count != nullptr, AXHIP_ERR_INVALID_ARG, "axhip_device_count: count is NULL");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        n = 0;
    }
    *count = n;
    return AXHIP_OK;
}

int axhip_init(int device) {
    std::lock_guard<std::mutex> lock(g_init_mutex);
    if (g_initialised && device == g_device) return AXHIP_OK;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n == 0) {
        (void)hipGetLastError();
        set_last_error("axhip_init: no HIP device available");
        return AXHIP_ERR_NO_DEVICE;
    }
    AXHIP_REQUIRE(device >= 0 && device < n, AXHIP_ERR_INVALID_ARG, "axhip_init: device %d out of range (%d present)", device, n);
    AXHIP_CHECK_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    AXHIP_CHECK_HIP(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        set_last_error("axhip_init: device %d is %s; this library holds gfx950 code only", device, prop.gcnArchName);
        return AXHIP_ERR_UNSUPPORTED;
    }
    if (!g_stream) AXHIP_CHECK_HIP(hipStreamCreateWithFlags(&g_stream, hipStreamNonBlocking));
    int rc = rows_setup_device();
    if (rc) return rc;
    g_device = device;
    g_initialised = true;
    return AXHIP_OK;
}

void *axhip_default_stream(void) { return g_stream; }

int axhip_malloc(void **ptr, size_t bytes) {
    AXHIP_REQUIRE(ptr != nullptr, AXHIP_ERR_INVALID_ARG, "axhip_malloc: ptr is NULL");
    int rc = ensure_init();
    if (rc) return rc;
    *ptr = nullptr;
    if (bytes == 0) return AXHIP_OK;
    AXHIP_CHECK_HIP(hipMalloc(ptr, bytes));
    return AXHIP_OK;
}

int axhip_free(void *ptr) {
    if (!ptr) return AXHIP_OK;
    AXHIP_CHECK_HIP(hipFree(ptr));
    return AXHIP_OK;
}

int axhip_memcpy_h2d_async(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes == 0) return AXHIP_OK;
    AXHIP_REQUIRE(dst && src, AXHIP_ERR_INVALID_ARG, "axhip_memcpy_h2d_async: NULL buffer");
    int rc = ensure_init();
    if (rc) return rc;
    AXHIP_CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, resolve_stream(stream)));
    return AXHIP_OK;
}

int axhip_memcpy_d2h_async(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes == 0) return AXHIP_OK;
    AXHIP_REQUIRE(dst && src, AXHIP_ERR_INVALID_ARG, "axhip_memcpy_d2h_async: NULL buffer");
    int rc = ensure_init();
    if (rc) return rc;
    AXHIP_CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, resolve_stream(stream)));
    return AXHIP_OK;
}

int axhip_memcpy_d2d_async(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes == 0) return AXHIP_OK;
    AXHIP_REQUIRE(dst && src, AXHIP_ERR_INVALID_ARG, "axhip_memcpy_d2d_async: NULL buffer");
    int rc = ensure_init();
    if (rc) return rc;
    AXHIP_CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, resolve_stream(stream)));
    return AXHIP_OK;
}

int axhip_stream_sync(void *stream) {
    int rc = ensure_init();
    if (rc) return rc;
    hipStream_t s = resolve_stream(stream);
    // Most waits here are for a kernel of tens of microseconds, and a blocking wait adds an interrupt round trip of
    // the same order.  Poll for up to a millisecond first; longer work then blocks without burning the core.
    const auto t0 = std::chrono::steady_clock::now();
    for (;;) {
        const hipError_t e = hipStreamQuery(s);
        if (e == hipSuccess) return AXHIP_OK;
        if (e != hipErrorNotReady) {
            AXHIP_CHECK_HIP(e);
        }
        (void)hipGetLastError(); // hipErrorNotReady is sticky in the runtime's last-error slot
        if (std::chrono::steady_clock::now() - t0 > std::chrono::microseconds(1000)) break;
    }
    AXHIP_CHECK_HIP(hipStreamSynchronize(s));
    return AXHIP_OK;
}

} // extern "C"
