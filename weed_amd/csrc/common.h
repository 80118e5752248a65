// Shared internals of libweed_hip: error latch, stream, per-kernel timing.  Not part of the C ABI.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>

#include "../../include/weed_hip.h"

namespace weedhip {

// Thread-local message behind weed_hip_last_error().
void set_error(const char *fmt, ...);
int fail(int code, const char *fmt, ...);

// The stream every launch goes to.
hipStream_t stream();

// Ensures weed_hip_init() ran (device 0 by default).  Returns a WEED_HIP_* status.
int ensure_init();

// Device weed_hip_init() selected last (-1 before the first call).
int current_device();

// Looks up this device's copy of the decode entry point's static scratch array (kv_decode.hip); weed_hip_init calls
// it once per device with that device current.
int decode_scratch_setup(int device_id);

// Puts the arrival counters at the start of the current device's static decode scratch back to zero (a fill kernel
// on the library's stream).  Every launch that completes leaves them at zero; this is for a launch that the device
// aborted midway.  weed_hip_kv_cache_reset and weed_hip_shutdown call it.
int decode_scratch_clear_counters();

// Frees the scratch of the split products (matmul.hip); weed_hip_shutdown calls it after draining the stream.
void release_split_scratch();

// RAII timing scope: when profiling is on, records events around the enclosed launches.
struct ProfileScope {
    explicit ProfileScope(const char *name, bool enabled = true);
    ~ProfileScope();
    ProfileScope(const ProfileScope &) = delete;
    ProfileScope &operator=(const ProfileScope &) = delete;

private:
    const char *name_;
    hipEvent_t start_ = nullptr;
    hipEvent_t stop_ = nullptr;
};

} // namespace weedhip

#define WEED_HIP_CHECK(expr)                                                                                           \
    do {                                                                                                               \
        hipError_t _e = (expr);                                                                                        \
        if (_e != hipSuccess) {                                                                                        \
            return weedhip::fail(WEED_HIP_EDEVICE, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__,    \
                                 __LINE__);                                                                            \
        }                                                                                                              \
    } while (0)

#define WEED_HIP_LAUNCH_CHECK()                                                                                        \
    do {                                                                                                               \
        hipError_t _e = hipGetLastError();                                                                             \
        if (_e != hipSuccess) {                                                                                        \
            return weedhip::fail(WEED_HIP_EDEVICE, "kernel launch failed: %s (%s:%d)", hipGetErrorString(_e),          \
                                 __FILE__, __LINE__);                                                                  \
        }                                                                                                              \
    } while (0)

#define WEED_HIP_REQUIRE(cond, ...)                                                                                    \
    do {                                                                                                               \
        if (!(cond)) {                                                                                                 \
            return weedhip::fail(WEED_HIP_EINVAL, __VA_ARGS__);                                                        \
        }                                                                                                              \
    } while (0)

#define WEED_HIP_TRY(expr)                                                                                             \
    do {                                                                                                               \
        int _s = (expr);                                                                                               \
        if (_s != WEED_HIP_OK) {                                                                                       \
            return _s;                                                                                                 \
        }                                                                                                              \
    } while (0)
