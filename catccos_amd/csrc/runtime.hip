// Runtime shims of the C ABI: device selection, memory, streams, error text.
#include <cstring>

#include "common.h"

namespace cch {
int routing_scratch_setup(int32_t **out);   // routing.hip: device address of its built-in histogram area

static thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

void clear_error() { g_err[0] = '\0'; }
}  // namespace cch

using cch::fail;

extern "C" {

const char *cch_last_error(void) { return cch::g_err; }

int cch_init(int device)
{
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n == 0) return fail(CCH_ENODEV, "no HIP device visible");
    CCH_REQUIRE(device >= 0 && device < n, "device %d out of range (0..%d)", device, n - 1);
    hipDeviceProp_t prop;
    CCH_HIP(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(CCH_ENODEV, "device %d is %s; this library holds gfx950 code only", device, prop.gcnArchName);
    CCH_HIP(hipSetDevice(device));
    // set-up for cch_moe_init_routing_noalloc, so that its calls look nothing up
    return cch::routing_scratch_setup(nullptr);
}

int cch_device_info(char *name, size_t name_len, int *compute_units, int *clock_mhz, uint64_t *hbm_bytes)
{
    int dev = 0;
    CCH_HIP(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    CCH_HIP(hipGetDeviceProperties(&prop, dev));
    if (name && name_len) {
        snprintf(name, name_len, "%s (%s)", prop.name, prop.gcnArchName);
    }
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (clock_mhz) *clock_mhz = prop.clockRate / 1000;
    if (hbm_bytes) *hbm_bytes = prop.totalGlobalMem;
    return CCH_OK;
}

int cch_malloc(void **ptr, size_t bytes)
{
    CCH_REQUIRE(ptr != nullptr, "cch_malloc: null result pointer");
    *ptr = nullptr;
    if (bytes == 0) return CCH_OK;
    CCH_HIP(hipMalloc(ptr, bytes));
    return CCH_OK;
}

int cch_free(void *ptr)
{
    if (ptr) CCH_HIP(hipFree(ptr));
    return CCH_OK;
}

int cch_malloc_host(void **ptr, size_t bytes)
{
    CCH_REQUIRE(ptr != nullptr, "cch_malloc_host: null result pointer");
    *ptr = nullptr;
    if (bytes == 0) return CCH_OK;
    CCH_HIP(hipHostMalloc(ptr, bytes, hipHostMallocDefault));
    return CCH_OK;
}

int cch_free_host(void *ptr)
{
    if (ptr) CCH_HIP(hipHostFree(ptr));
    return CCH_OK;
}

int cch_memcpy_h2d(void *dst, const void *src, size_t bytes)
{
    if (bytes) CCH_HIP(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
    return CCH_OK;
}

int cch_memcpy_d2h(void *dst, const void *src, size_t bytes)
{
    if (bytes) CCH_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
    return CCH_OK;
}

int cch_memset(void *dst, int value, size_t bytes)
{
    if (bytes) CCH_HIP(hipMemset(dst, value, bytes));
    return CCH_OK;
}

int cch_stream_create(void **stream)
{
    CCH_REQUIRE(stream != nullptr, "cch_stream_create: null result pointer");
    hipStream_t s;
    CCH_HIP(hipStreamCreate(&s));
    *stream = s;
    return CCH_OK;
}

int cch_stream_sync(void *stream)
{
    CCH_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    return CCH_OK;
}

int cch_stream_destroy(void *stream)
{
    if (stream) CCH_HIP(hipStreamDestroy(static_cast<hipStream_t>(stream)));
    return CCH_OK;
}

}  // extern "C"
