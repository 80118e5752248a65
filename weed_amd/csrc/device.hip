// Device, stream, memory and error plumbing of libweed_hip.
//
// Takes the place of Weed's OCLEngine singleton and GpuDevice queue (include/common/oclengine.hpp,
// include/devices/gpu_device.hpp): one HIP stream, stream-ordered launches, no callbacks, no JIT.
#include "common.h"

#include <cstdlib>
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

// Stream-ordered block cache behind weed_hip_malloc / weed_hip_free.  Every launch of the library goes to ONE stream,
// so a freed block may be handed out again without waiting: whatever still reads it was enqueued before whatever
// will write it.  hipMalloc and hipFree (which waits for the device) then only run while the working set grows, not
// once per intermediate tensor of every module call.  Sizes are rounded up (512 B, 2 MiB above 1 MiB); a request takes
// the smallest cached block that is large enough and at most half again as large.  When the stream is replaced the old
// one is drained first.  Cached bytes are capped (kPoolCapBytes, or WEED_HIP_POOL_MAX_MB; 0 turns the cache off).
std::mutex g_pool_mutex;
std::map<void *, size_t> g_pool_sizes;       // every live or cached block of the pool -> rounded size
std::multimap<size_t, void *> g_pool_free;   // cached blocks by size
size_t g_pool_cached = 0;
constexpr size_t kPoolCapBytes = 64ull << 30;

size_t pool_cap()
{
    static const size_t cap = [] {
        const char *env = std::getenv("WEED_HIP_POOL_MAX_MB");
        return env ? (size_t)std::strtoull(env, nullptr, 10) << 20 : kPoolCapBytes;
    }();
    return cap;
}

size_t pool_round(size_t bytes)
{
    const size_t unit = bytes > (1u << 20) ? (2u << 20) : 512u;
    return (bytes + unit - 1) / unit * unit;
}

// Give every cached block back to the driver (the caller holds g_pool_mutex and has drained the stream).
void pool_release_locked()
{
    for (auto &kv : g_pool_free) {
        (void)hipFree(kv.second);
        g_pool_sizes.erase(kv.second);
    }
    g_pool_free.clear();
    g_pool_cached = 0;
}

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

int current_device() { return g_initialised ? g_device : -1; }

int ensure_init()
{
    if (g_initialised) {
        return WEED_HIP_OK;
    }
    return weed_hip_init(0);
}

ProfileScope::ProfileScope(const char *name, bool enabled)
    : name_(name)
{
    if (!g_profile || !enabled) {
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
    WEED_HIP_TRY(decode_scratch_setup(device_id));
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
    hipStream_t next = hip_stream ? (hipStream_t)hip_stream : g_own_stream;
    if (next != g_stream) {
        // cached blocks are reused without waiting, which is only in order on one stream
        WEED_HIP_CHECK(hipStreamSynchronize(g_stream));
        g_stream = next;
    }
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
    const size_t want = pool_round(bytes);
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    auto it = g_pool_free.lower_bound(want);
    if (it != g_pool_free.end() && it->first <= want + want / 2) {
        *ptr_dev = it->second;
        g_pool_cached -= it->first;
        g_pool_free.erase(it);
        return WEED_HIP_OK;
    }
    hipError_t e = hipMalloc(ptr_dev, want);
    if (e != hipSuccess && !g_pool_free.empty()) {
        // out of memory with blocks in the cache: drain, give them back, try once more
        (void)hipGetLastError();
        WEED_HIP_CHECK(hipStreamSynchronize(g_stream));
        pool_release_locked();
        e = hipMalloc(ptr_dev, want);
    }
    if (e != hipSuccess) {
        (void)hipGetLastError();
        *ptr_dev = nullptr;
        return fail(WEED_HIP_ENOMEM, "weed_hip_malloc: %zu bytes: %s", bytes, hipGetErrorString(e));
    }
    g_pool_sizes[*ptr_dev] = want;
    return WEED_HIP_OK;
}

int weed_hip_free(void *ptr_dev)
{
    if (!ptr_dev) {
        return WEED_HIP_OK;
    }
    WEED_HIP_TRY(ensure_init());
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    auto it = g_pool_sizes.find(ptr_dev);
    if (it != g_pool_sizes.end()) {
        // a block that is already in the cache must not enter it twice (two later allocations would share it)
        auto range = g_pool_free.equal_range(it->second);
        for (auto f = range.first; f != range.second; ++f) {
            if (f->second == ptr_dev) {
                return fail(WEED_HIP_EINVAL, "weed_hip_free: %p was freed already", ptr_dev);
            }
        }
    }
    if (it != g_pool_sizes.end() && g_pool_cached + it->second <= pool_cap()) {
        g_pool_free.emplace(it->second, ptr_dev);
        g_pool_cached += it->second;
        return WEED_HIP_OK;
    }
    // not one of the pool's blocks, or the cache is full: wait for whatever still uses it, then give it back
    if (it != g_pool_sizes.end()) {
        g_pool_sizes.erase(it);
    }
    WEED_HIP_CHECK(hipStreamSynchronize(g_stream));
    WEED_HIP_CHECK(hipFree(ptr_dev));
    return WEED_HIP_OK;
}

int weed_hip_release_cached(void)
{
    WEED_HIP_TRY(ensure_init());
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    WEED_HIP_CHECK(hipStreamSynchronize(g_stream));
    pool_release_locked();
    return WEED_HIP_OK;
}

int weed_hip_shutdown(void)
{
    std::lock_guard<std::mutex> lock(g_mutex);
    if (!g_initialised) {
        return WEED_HIP_OK;
    }
    WEED_HIP_CHECK(hipSetDevice(g_device));
    // (the static decode scratch outlives the library's state: leave its arrival counters at zero for a later start)
    WEED_HIP_TRY(decode_scratch_clear_counters());
    WEED_HIP_CHECK(hipStreamSynchronize(g_stream));
    if (g_own_stream && g_stream != g_own_stream) {
        WEED_HIP_CHECK(hipStreamSynchronize(g_own_stream));
    }
    for (auto &kv : g_profiles) {
        resolve_pending(kv.second);
    }
    g_profiles.clear();
    g_profile = false;
    {
        std::lock_guard<std::mutex> pool_lock(g_pool_mutex);
        pool_release_locked();
    }
    release_split_scratch();
    if (g_own_stream) {
        (void)hipStreamDestroy(g_own_stream);
        g_own_stream = nullptr;
    }
    g_stream = nullptr;
    g_initialised = false;
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
