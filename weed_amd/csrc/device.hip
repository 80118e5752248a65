// Device, stream, memory and error plumbing of libweed_hip.
//
// Takes the place of Weed's OCLEngine singleton and GpuDevice queue (include/common/oclengine.hpp,
// include/devices/gpu_device.hpp): one HIP stream, stream-ordered launches, no callbacks, no JIT.
#include "common.h"

#include <map>
#include <mutex>
#include <string>
#include <vector>

namespace weedhip {

namespace {
thread_local std::string g_last_error;
std::mutex g_mutex;
bool g_initialised = false;
int g_device = 0;
hipStream_t g_own_stream = nullptr;
hipStream_t g_stream = nullptr;
bool g_profile = false;

struct ProfileEntry {
    std::vector<std::pair<hipEvent_t, hipEvent_t>> pending;
    double total_ms = 0.0;
    uint64_t launches = 0;
};
std::map<std::string, ProfileEntry> g_profiles;

void resolve_pending(ProfileEntry &e)
{
    for (auto &p : e.pending) {
        float ms = 0.0f;
        if (hipEventSynchronize(p.second) == hipSuccess && hipEventElapsedTime(&ms, p.first, p.second) == hipSuccess) {
            e.total_ms += (double)ms;
            ++e.launches;
        }
        (void)hipEventDestroy(p.first);
        (void)hipEventDestroy(p.second);
    }
    e.pending.clear();
}
} // namespace

void set_error(const char *fmt, ...)
{
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
}

int fail(int code, const char *fmt, ...)
{
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

hipStream_t stream() { return g_stream; }

int ensure_init()
{
    if (g_initialised) {
        return WEED_HIP_OK;
    }
    return weed_hip_init(0);
}

ProfileScope::ProfileScope(const char *name)
    : name_(name)
{
    if (!g_profile) {
        return;
    }
    if (hipEventCreate(&start_) != hipSuccess || hipEventCreate(&stop_) != hipSuccess) {
        start_ = stop_ = nullptr;
        return;
    }
    (void)hipEventRecord(start_, g_stream);
}

ProfileScope::~ProfileScope()
{
    if (!start_) {
        return;
    }
    (void)hipEventRecord(stop_, g_stream);
    std::lock_guard<std::mutex> lock(g_mutex);
    ProfileEntry &e = g_profiles[name_];
    e.pending.emplace_back(start_, stop_);
    if (e.pending.size() >= 2048) {
        resolve_pending(e);
    }
}

} // namespace weedhip

using namespace weedhip;

extern "C" {

int weed_hip_init(int device_id)
{
    std::lock_guard<std::mutex> lock(g_mutex);
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0) {
        return fail(WEED_HIP_EDEVICE, "weed_hip_init: no HIP device available (%s)",
                    e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
    }
    if (device_id < 0 || device_id >= count) {
        return fail(WEED_HIP_EINVAL, "weed_hip_init: device %d out of range [0, %d)", device_id, count);
    }
    WEED_HIP_CHECK(hipSetDevice(device_id));
    if (g_initialised && g_device == device_id) {
        return WEED_HIP_OK;
    }
    g_device = device_id;
    if (!g_own_stream) {
        WEED_HIP_CHECK(hipStreamCreateWithFlags(&g_own_stream, hipStreamNonBlocking));
    }
    if (!g_stream) {
        g_stream = g_own_stream;
    }
    g_initialised = true;
    return WEED_HIP_OK;
}

int weed_hip_device_count(int *count)
{
    WEED_HIP_REQUIRE(count, "weed_hip_device_count: null pointer");
    int c = 0;
    hipError_t e = hipGetDeviceCount(&c);
    *count = (e == hipSuccess) ? c : 0;
    return WEED_HIP_OK;
}

int weed_hip_device_name(char *buf, size_t buf_len)
{
    WEED_HIP_REQUIRE(buf && buf_len, "weed_hip_device_name: null buffer");
    WEED_HIP_TRY(ensure_init());
    hipDeviceProp_t prop;
    WEED_HIP_CHECK(hipGetDeviceProperties(&prop, g_device));
    snprintf(buf, buf_len, "%s (%s, %d CUs)", prop.name, prop.gcnArchName, prop.multiProcessorCount);
    return WEED_HIP_OK;
}

int weed_hip_set_stream(void *hip_stream)
{
    WEED_HIP_TRY(ensure_init());
    g_stream = hip_stream ? (hipStream_t)hip_stream : g_own_stream;
    return WEED_HIP_OK;
}

void *weed_hip_stream(void) { return (void *)g_stream; }

int weed_hip_sync(void)
{
    WEED_HIP_TRY(ensure_init());
    WEED_HIP_CHECK(hipStreamSynchronize(g_stream));
    return WEED_HIP_OK;
}

const char *weed_hip_last_error(void) { return g_last_error.c_str(); }

const char *weed_hip_version(void) { return "weed_hip 0.1 (gfx950)"; }

int weed_hip_malloc(void **ptr_dev, size_t bytes)
{
    WEED_HIP_REQUIRE(ptr_dev, "weed_hip_malloc: null pointer");
    WEED_HIP_TRY(ensure_init());
    *ptr_dev = nullptr;
    if (!bytes) {
        return WEED_HIP_OK;
    }
    hipError_t e = hipMalloc(ptr_dev, bytes);
    if (e != hipSuccess) {
        *ptr_dev = nullptr;
        return fail(WEED_HIP_ENOMEM, "weed_hip_malloc: %zu bytes: %s", bytes, hipGetErrorString(e));
    }
    return WEED_HIP_OK;
}

int weed_hip_free(void *ptr_dev)
{
    if (!ptr_dev) {
        return WEED_HIP_OK;
    }
    WEED_HIP_TRY(ensure_init());
    WEED_HIP_CHECK(hipStreamSynchronize(g_stream));
    WEED_HIP_CHECK(hipFree(ptr_dev));
    return WEED_HIP_OK;
}

int weed_hip_memset(void *ptr_dev, int byte_value, size_t bytes)
{
    WEED_HIP_TRY(ensure_init());
    if (!bytes) {
        return WEED_HIP_OK;
    }
    WEED_HIP_REQUIRE(ptr_dev, "weed_hip_memset: null pointer");
    WEED_HIP_CHECK(hipMemsetAsync(ptr_dev, byte_value, bytes, g_stream));
    return WEED_HIP_OK;
}

int weed_hip_memcpy_h2d(void *dst_dev, const void *src, size_t bytes)
{
    WEED_HIP_TRY(ensure_init());
    if (!bytes) {
        return WEED_HIP_OK;
    }
    WEED_HIP_REQUIRE(dst_dev && src, "weed_hip_memcpy_h2d: null pointer");
    WEED_HIP_CHECK(hipMemcpyAsync(dst_dev, src, bytes, hipMemcpyHostToDevice, g_stream));
    WEED_HIP_CHECK(hipStreamSynchronize(g_stream));
    return WEED_HIP_OK;
}

int weed_hip_memcpy_d2h(void *dst, const void *src_dev, size_t bytes)
{
    WEED_HIP_TRY(ensure_init());
    if (!bytes) {
        return WEED_HIP_OK;
    }
    WEED_HIP_REQUIRE(dst && src_dev, "weed_hip_memcpy_d2h: null pointer");
    WEED_HIP_CHECK(hipMemcpyAsync(dst, src_dev, bytes, hipMemcpyDeviceToHost, g_stream));
    WEED_HIP_CHECK(hipStreamSynchronize(g_stream));
    return WEED_HIP_OK;
}

int weed_hip_memcpy_d2d(void *dst_dev, const void *src_dev, size_t bytes)
{
    WEED_HIP_TRY(ensure_init());
    if (!bytes) {
        return WEED_HIP_OK;
    }
    WEED_HIP_REQUIRE(dst_dev && src_dev, "weed_hip_memcpy_d2d: null pointer");
    WEED_HIP_CHECK(hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, g_stream));
    return WEED_HIP_OK;
}

int weed_hip_profile_enable(int on)
{
    WEED_HIP_TRY(ensure_init());
    g_profile = on != 0;
    return WEED_HIP_OK;
}

int weed_hip_profile_reset(void)
{
    WEED_HIP_TRY(ensure_init());
    WEED_HIP_CHECK(hipStreamSynchronize(g_stream));
    std::lock_guard<std::mutex> lock(g_mutex);
    for (auto &kv : g_profiles) {
        resolve_pending(kv.second);
    }
    g_profiles.clear();
    return WEED_HIP_OK;
}

int weed_hip_profile_read(const char *name, double *total_ms, uint64_t *launches)
{
    WEED_HIP_REQUIRE(name && total_ms && launches, "weed_hip_profile_read: null pointer");
    WEED_HIP_TRY(ensure_init());
    std::lock_guard<std::mutex> lock(g_mutex);
    auto it = g_profiles.find(name);
    if (it == g_profiles.end()) {
        *total_ms = 0.0;
        *launches = 0;
        return WEED_HIP_OK;
    }
    resolve_pending(it->second);
    *total_ms = it->second.total_ms;
    *launches = it->second.launches;
    return WEED_HIP_OK;
}

} // extern "C"
