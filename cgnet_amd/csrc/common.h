// Shared helpers of libcgnet_hip: error reporting, argument checks, small device utilities.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

#include "../../include/cgnet_hip.h"

namespace cgnet {

// Records a printf-style message for cgnet_last_error() of the calling thread.
void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
void clear_error();

#define CGNET_HIP(expr)                                                                       \
    do {                                                                                      \
        hipError_t e__ = (expr);                                                              \
        if (e__ != hipSuccess) {                                                              \
            ::cgnet::set_error("%s: %s (%s:%d)", #expr, hipGetErrorString(e__), __FILE__,     \
                               __LINE__);                                                     \
            return CGNET_ERR_HIP;                                                             \
        }                                                                                     \
    } while (0)

#define CGNET_REQUIRE(cond, code, ...)                                                        \
    do {                                                                                      \
        if (!(cond)) {                                                                        \
            ::cgnet::set_error(__VA_ARGS__);                                                  \
            return (code);                                                                    \
        }                                                                                     \
    } while (0)

constexpr int kMaxL = 47;          // 2L+1 <= 96 complex columns per sample in the mixing kernel; CG table (2L+1)^2 floats in LDS
constexpr int kMaxTau = 1024;      // channels of one degree

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// Optional per-kernel timing (cgnet_profile_*): when enabled, every launch is bracketed by a
// pair of HIP events recorded on the launch stream.
class KernelTimer {
public:
    KernelTimer(const char* name, hipStream_t stream);
    ~KernelTimer();
private:
    const char* name_;
    hipStream_t stream_;
    hipEvent_t start_ = nullptr, stop_ = nullptr;
};

#define CGNET_LAUNCH(kernel, grid, block, lds, stream, ...)                                   \
    do {                                                                                      \
        ::cgnet::KernelTimer timer__(#kernel, stream);                                        \
        hipLaunchKernelGGL(kernel, grid, block, lds, stream, __VA_ARGS__);                    \
    } while (0)

}  // namespace cgnet
