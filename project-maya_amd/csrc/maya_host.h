// maya_host.h - host-side helpers shared by the library's translation units: status codes with a thread-local
// message, HIP error checks, the per-device state (codebooks in device memory).
#pragma once

#include <hip/hip_runtime.h>
#include <mutex>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/maya_moe.h"
#include "maya_dev.hpp"

namespace maya {

extern thread_local char g_err[512];
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int hip_fail(hipError_t e, const char* what);
#define MAYA_HIP(call)                                         \
    do {                                                       \
        const hipError_t e_ = (call);                          \
        if (e_ != hipSuccess) return hip_fail(e_, #call);      \
    } while (0)
#define MAYA_LAUNCHED(name)                                    \
    do {                                                       \
        const hipError_t e_ = hipGetLastError();               \
        if (e_ != hipSuccess) return hip_fail(e_, name);       \
    } while (0)

struct DeviceState {
    bool ready = false;
    Codebooks cb{};
    int lds_limit = 65536;
    int n_cu = 0;
    void* static_scratch = nullptr;   // this device's copy of the file-scope scratch array (maya_moe_layer_decode_static)
    // maya_moe_layer_decode_shared: the stream the shared expert's launches run on beside the caller's, and the two events
    // that fork it from the caller's stream and join it back (default priority; one call at a time a device: side_mu)
    hipStream_t side = nullptr;
    hipEvent_t side_fork = nullptr, side_join = nullptr;
    std::mutex side_mu;
};
// the current device's state, initialised on first use (gfx950 only); MAYA_OK or a status
int current_state(DeviceState** out);
inline hipStream_t as_stream(void* s) { return (hipStream_t) s; }

}  // namespace maya
