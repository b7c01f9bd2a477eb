// Host-side helpers shared by the library's source files.
#ifndef BITNET_AMD_HOST_UTIL_H
#define BITNET_AMD_HOST_UTIL_H

#include <hip/hip_runtime.h>

#include <mutex>

namespace bitnet_host {

// Runs a set-up step (a hipFuncSetAttribute call: kernel attributes are per device) once per device
// and keeps its result, so every later call on that device reports the same outcome.  Safe to call
// from several host threads.
constexpr int kMaxDevices = 16;
struct OncePerDevice {
    std::once_flag flag[kMaxDevices];
    hipError_t result[kMaxDevices];
    template <class F>
    hipError_t run(F&& f) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return f();
        std::call_once(flag[dev], [&] { result[dev] = f(); });
        return result[dev];
    }
};

}  // namespace bitnet_host

#endif
