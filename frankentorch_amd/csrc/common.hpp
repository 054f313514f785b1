// Shared host-side plumbing of the gfx950 backend: error slots, stream resolution, launch checks.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>

#include "ft_kernel_hip.h"

namespace fth {

// Thread-local payload of the last failing call (read back through fth_last_error).
fth_error_info &last_error();
// Records `code` with a printf-style message and returns `code`.
int32_t set_error(int32_t code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
// Records a HIP runtime failure as FTH_ERR_KERNEL (or FTH_ERR_BUFFER_TOO_LARGE for OOM).
int32_t hip_fail(hipError_t e, const char *what);
// True when a gfx950 device is usable. The probe runs once per process.
bool available();
// NULL selects the library's own stream (created on first use, default priority).
hipStream_t resolve_stream(fth_stream s);
// Number of compute units of device 0 (cached).
int compute_units();

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace fth

#define FTH_HIP(expr)                                             \
    do {                                                          \
        hipError_t _fth_e = (expr);                               \
        if (_fth_e != hipSuccess) return fth::hip_fail(_fth_e, #expr); \
    } while (0)

#define FTH_REQUIRE_DEVICE()                                                                  \
    do {                                                                                      \
        if (!fth::available())                                                                \
            return fth::set_error(FTH_ERR_UNAVAILABLE, "no usable gfx950 HIP device in this process"); \
    } while (0)

#define FTH_CHECK_LAUNCH(name)                                    \
    do {                                                          \
        hipError_t _fth_e = hipGetLastError();                    \
        if (_fth_e != hipSuccess) return fth::hip_fail(_fth_e, name); \
    } while (0)

#define FTH_ARG(cond, ...)                                                       \
    do {                                                                         \
        if (!(cond)) return fth::set_error(FTH_ERR_INVALID_ARGUMENT, __VA_ARGS__); \
    } while (0)
