// Shared host-side plumbing of the gfx950 backend: error slots, stream resolution, launch checks.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <vector>

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

// Softmax over contiguous rows too long or too ragged for the 128-bit row kernels (any length up to 65 536 floats /
// 32 768 doubles, any 4- / 8-byte alignment): the register-resident row kernel of the loss unit. Returns false, with
// nothing launched, when a row does not fit.
bool softmax_resident_rows(const float *x, float *y, int64_t rows, int64_t cols, hipStream_t st);
bool softmax_resident_rows(const double *x, double *y, int64_t rows, int64_t cols, hipStream_t st);

// logits = x . w^T (x [m, k], w [n, k], contiguous) with, as a by-product of the product's epilogue, the maximum of every
// row over each group of 64 columns: rowmax[group * m + row], gemm_rowmax_groups(n) groups, NaN where a group's maximum is
// not known (the group holds a NaN). Returns false, nothing launched, for shapes
// the large-tile direct kernel does not take. argmax_from_group_max then finds each row's argmax (first strict maximum, the
// first NaN wins: the rule of the argmax kernel, bit for bit) from those maxima and at most a few 64-column pieces of the
// stored logits, instead of reading every row again.
int64_t gemm_rowmax_groups(int64_t n);
bool gemm_f32_nt_rowmax(int64_t m, int64_t n, int64_t k, const float *a, const float *b, float *c, float *rowmax, hipStream_t st,
                        int32_t *rc);
int32_t argmax_from_group_max(const float *logits, int64_t rows, int64_t cols, const float *rowmax, int64_t groups, float *out,
                              hipStream_t st);

// Causal attention launches whose workgroups are ALL resident at once (grid <= workgroups per compute unit x compute
// units) cannot rely on heaviest-first issue to balance: nothing is left to hand out when a light workgroup ends. The
// hardware deals workgroup ids round-robin over the 8 XCDs and, inside an XCD, over its compute units in id order, so a
// compute unit holds ids j, j + P, j + 2 P, ... of its XCD (P = compute units per XCD). Walking every other pass
// backwards pairs the heavy end of one pass with the light end of the next; a compute unit's workgroups then add up to
// about the same work. Returns the pass length P when the launch qualifies, else 0.
template <typename K> int snake_pass_length(K kernel, int threads, size_t smem, int64_t grid, bool causal) {
    if (!causal) return 0;
    // The occupancy of a (kernel, block size, LDS size) never changes: asked once, kept (a handful of entries).
    struct Seen { const void *k; int threads; size_t smem; int per_cu; };
    static std::mutex mu;
    static std::vector<Seen> seen;
    int per_cu = -1;
    {
        std::lock_guard<std::mutex> lock(mu);
        for (const Seen &e : seen)
            if (e.k == reinterpret_cast<const void *>(kernel) && e.threads == threads && e.smem == smem) per_cu = e.per_cu;
        if (per_cu < 0) {
            if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, smem) != hipSuccess) per_cu = 0;
            seen.push_back({reinterpret_cast<const void *>(kernel), threads, smem, per_cu});
        }
    }
    if (per_cu <= 0) return 0;
    const int cus = compute_units() > 0 ? compute_units() : 256;
    return (cus % 8 == 0 && grid <= (int64_t)per_cu * cus && grid > cus) ? cus / 8 : 0;
}

// Position i of an XCD's id sequence of `total` entries -> the position whose work it takes (see snake_pass_length).
__host__ __device__ inline int64_t snake_order(int64_t i, int pass_len, int64_t total) {
    if (pass_len <= 0) return i;
    const int64_t pass = i / pass_len, j = i % pass_len, lo = pass * pass_len;
    const int64_t hi = lo + pass_len < total ? lo + pass_len : total;
    return (pass & 1) ? hi - 1 - j : i;
}

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
