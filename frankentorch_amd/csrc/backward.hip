// Backward kernels of the transformer forward ops: LayerNorm, RMSNorm, linear and scaled-dot-product
// attention. Every reduction has a fixed order (no atomics), so results are bitwise repeatable.
//
// replaces layer_norm_backward_f32 / _f64 (crates/ft-kernel-cpu/src/lib.rs:6189-6322, 6052-6183),
// rms_norm_backward_f32 / _f64 (:6574-6646, 6503-6570), linear_backward_f64 (:17226-17302) and its
// f32 use through the same formulas, sdpa_backward_f32 / _f64 (:5539-5650, 5300-5414).
//
// Norm backward. One workgroup owns a run of consecutive rows. A row's x and dy are loaded once
// into registers (128-bit loads), the row statistics and the two dot products are reduced with a
// fixed butterfly per wavefront and a fixed left-to-right fold across the four wavefronts, dx is
// stored once, and the column sums (dweight, dbias) of the workgroup's rows are accumulated in
// registers in row order. Each workgroup then writes one row of partial column sums; a second
// kernel adds the partials in workgroup order. The reference sums the rows serially in one chain;
// this is the same sum re-associated into (rows of a workgroup) then (workgroups), which the
// 1e-5 / 1e-12 parity tolerances cover. Row lengths that do not fit the register layout take a
// streaming kernel (x and dy re-read from cache per pass) plus a separate column-sum pass.
//
// Linear backward is two MFMA GEMMs (dx = dy.W as stored, dweight = dy^T.x with dy read as stored
// through the [k, m] operand path) and a column sum of dy. SDPA backward follows the reference's
// own structure on the device: P = softmax(scale * Q.K^T) and dU are materialised per
// (batch*head) in a caller-provided workspace (2 * num_bh * seq_q * seq_k elements), the five
// products are batched MFMA GEMMs and the two row passes are HBM-bound row kernels. Long causal
// square problems cut every product into blocks along the sequence and leave out what lies above
// the block diagonal.

#include <algorithm>
#include <mutex>
#include <type_traits>

#include "common.hpp"
#include "sdpa_bwd.hpp"

namespace {

#ifndef FTH_BWD_BLOCKS_PER_CU
#define FTH_BWD_BLOCKS_PER_CU 1
#endif
constexpr int kWave = 64;
constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;

template <typename T> struct Vec16;
template <> struct Vec16<float> {
    using type = float4;
    static constexpr int N = 4;
};
template <> struct Vec16<double> {
    using type = double2;
    static constexpr int N = 2;
};
__device__ __forceinline__ float vget(const float4 &v, int i) { return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w; }
__device__ __forceinline__ double vget(const double2 &v, int i) { return i == 0 ? v.x : v.y; }
__device__ __forceinline__ void vset(float4 &v, int i, float x) {
    if (i == 0) v.x = x;
    else if (i == 1) v.y = x;
    else if (i == 2) v.z = x;
    else v.w = x;
}
__device__ __forceinline__ void vset(double2 &v, int i, double x) {
    if (i == 0) v.x = x;
    else v.y = x;
}

// Streaming (non-temporal) 16-byte loads and stores: rows are read once and outputs never re-read.
typedef float nat_f4 __attribute__((ext_vector_type(4)));
typedef double nat_d2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void stream_store(float4 *p, const float4 &v) {
    nat_f4 n = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(n, reinterpret_cast<nat_f4 *>(p));
}
__device__ __forceinline__ void stream_store(double2 *p, const double2 &v) {
    nat_d2 n = {v.x, v.y};
    __builtin_nontemporal_store(n, reinterpret_cast<nat_d2 *>(p));
}

__device__ __forceinline__ float4 stream_load(const float4 *p) {
    nat_f4 v = __builtin_nontemporal_load(reinterpret_cast<const nat_f4 *>(p));
    return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ double2 stream_load(const double2 *p) {
    nat_d2 v = __builtin_nontemporal_load(reinterpret_cast<const nat_d2 *>(p));
    return make_double2(v.x, v.y);
}

template <typename T> __device__ __forceinline__ T wave_sum(T v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

// Sum of NV values per thread over the workgroup: butterfly inside each wavefront, then wavefront 0..3
// added left to right by every thread (same result in all threads). `red` holds 2 * kWaves * 2
// values: consecutive calls alternate between its halves (`phase`), so one barrier per call is
// enough -- a wavefront can only reach the write of call n + 2 after passing the barrier of call
// n + 1, which every wavefront reaches only after its reads of call n.
template <typename T, int NV, int NW = kWaves> __device__ __forceinline__ void block_sum(T (&v)[NV], T *red, int &phase) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    T *buf = red + phase * (NW * 2);
    phase ^= 1;
#pragma unroll
    for (int i = 0; i < NV; ++i) v[i] = wave_sum(v[i]);
    if (lane == 0) {
#pragma unroll
        for (int i = 0; i < NV; ++i) buf[wave * NV + i] = v[i];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        T s = buf[i];
#pragma unroll
        for (int w = 1; w < NW; ++w) s += buf[w * NV + i];
        v[i] = s;
    }
}

template <typename T> __device__ __forceinline__ T t_rsqrt_of(T v) { return T(1) / sqrt(v); }

// ---- register-resident norm backward ----
// RMS = false: LayerNorm (weight required, partial dbias written); RMS = true: RMSNorm (weight optional).
// NT threads own a row; VPT: 16-byte vectors per thread; cols <= NT * VPT * N and cols % N == 0.
// DEPTH: rows requested ahead of the one being reduced (0, 1 or 2 register sets). The kernel waits for rows far more
// than it computes, and what limits the rows in flight per compute unit is registers: a thread holds the row in hand,
// the sets in flight, the weight and two column accumulators. Rows of up to 1024 vectors use 512 threads with two
// vectors each and two sets in flight (two such workgroups per compute unit: four rows of 32 KiB in flight, twice what
// 256 threads with four vectors and one set could hold).
template <typename T, int VPT, bool RMS, int NT = kThreads, int DEPTH = (VPT * Vec16<T>::N <= 16 ? 1 : 0)>
__global__ __launch_bounds__(NT) void norm_backward_kernel(const T *__restrict__ dy, const T *__restrict__ x,
                                                           const T *__restrict__ w, int64_t rows, int cols, T eps,
                                                           T *__restrict__ dx, T *__restrict__ part_w,
                                                           T *__restrict__ part_b, int rows_per_block) {
    using V = typename Vec16<T>::type;
    constexpr int N = Vec16<T>::N;
    constexpr int NW = NT / kWave;
    __shared__ T red[2 * NW * 2];
    int phase = 0;
    const int tid = threadIdx.x;
    const int nvec = cols / N;
    const T inv_n = T(1) / (T)cols;
    V wv[VPT];
    T aw[VPT][N], ab[VPT][N];
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int v = tid + i * NT;
#pragma unroll
        for (int e = 0; e < N; ++e) {
            aw[i][e] = T(0);
            ab[i][e] = T(0);
            vset(wv[i], e, T(1));
        }
        if (w != nullptr && v < nvec) wv[i] = reinterpret_cast<const V *>(w)[v];
    }
    // Workgroup b takes rows b, b + G, b + 2 G, ... (G workgroups): at any moment the workgroups together read one
    // contiguous band of rows, as a launch of fresh blocks would, instead of G separate streams (measured at fp32
    // [8192,4096], whole entry point: 0.60 -> 0.66 of the HBM peak with two workgroups per compute unit, 0.71 with one,
    // whose partial sums are half as many). The caller sizes the partial sums for ceil(rows / rows_per_block)
    // workgroups and launches exactly that many.
    (void)rows_per_block;
    const int64_t rstep = gridDim.x;
    const int64_t r0 = blockIdx.x, r1 = rows;
    auto load_row = [&](int64_t r, V *xd, V *gd) __attribute__((always_inline)) {
        if (r >= r1) return;  // workgroup-uniform: nothing left to request
        const V *xr = reinterpret_cast<const V *>(x + r * cols);
        const V *dyr = reinterpret_cast<const V *>(dy + r * cols);
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int v = tid + i * NT;
            if (v < nvec) {
                xd[i] = stream_load(xr + v);
                gd[i] = stream_load(dyr + v);
            } else {
#pragma unroll
                for (int e = 0; e < N; ++e) {
                    vset(xd[i], e, T(0));
                    vset(gd[i], e, T(0));
                }
            }
        }
    };
    // One row: xs / gs hold it on entry (DEPTH > 0) and are handed the row DEPTH ahead as soon as they have been copied.
    auto do_row = [&](int64_t r, V *xs, V *gs) __attribute__((always_inline)) {
        V xv[VPT], gv[VPT];
        if constexpr (DEPTH > 0) {
#pragma unroll
            for (int i = 0; i < VPT; ++i) {
                xv[i] = xs[i];
                gv[i] = gs[i];
            }
            load_row(r + DEPTH * rstep, xs, gs);
        } else {
            load_row(r, xv, gv);
        }
        if constexpr (!RMS) {
            // Two block reductions per row instead of the reference's four serial sums: neither sum(dy w) nor
            // sum(dy w (x - mean)) needs rstd, so the first rides with sum(x) and the second with sum((x - mean)^2);
            // c1 = rstd * sum(dy w (x - mean)) is the reference's sum(dy w xhat) with rstd factored out.
            T s[2] = {T(0), T(0)};
#pragma unroll
            for (int i = 0; i < VPT; ++i)
#pragma unroll
                for (int e = 0; e < N; ++e) {
                    s[0] += vget(xv[i], e);
                    s[1] += vget(gv[i], e) * vget(wv[i], e);  // padding lanes hold dy = 0
                }
            block_sum<T, 2, NW>(s, red, phase);
            const T mean = s[0] * inv_n;
            T q[2] = {T(0), T(0)};
#pragma unroll
            for (int i = 0; i < VPT; ++i) {
                const bool live = tid + i * NT < nvec;
#pragma unroll
                for (int e = 0; e < N; ++e) {
                    const T d = vget(xv[i], e) - mean;
                    if (live) {
                        q[0] += d * d;
                        q[1] += (vget(gv[i], e) * vget(wv[i], e)) * d;
                    }
                }
            }
            block_sum<T, 2, NW>(q, red, phase);
            const T rstd = t_rsqrt_of(q[0] * inv_n + eps);
            const T c[2] = {s[1], rstd * q[1]};
            V *dxr = reinterpret_cast<V *>(dx + r * cols);
#pragma unroll
            for (int i = 0; i < VPT; ++i) {
                const int v = tid + i * NT;
                V o;
#pragma unroll
                for (int e = 0; e < N; ++e) {
                    const T xhat = (vget(xv[i], e) - mean) * rstd;
                    const T dxhat = vget(gv[i], e) * vget(wv[i], e);
                    vset(o, e, rstd * (dxhat - (c[0] + xhat * c[1]) * inv_n));
                    aw[i][e] += vget(gv[i], e) * xhat;
                    ab[i][e] += vget(gv[i], e);
                }
                if (v < nvec) stream_store(dxr + v, o);
            }
        } else {
            // one block reduction per row: sum(x^2) and sum(dy w x) do not depend on each other
            T s[2] = {T(0), T(0)};
#pragma unroll
            for (int i = 0; i < VPT; ++i)
#pragma unroll
                for (int e = 0; e < N; ++e) {
                    s[0] += vget(xv[i], e) * vget(xv[i], e);
                    s[1] += (vget(gv[i], e) * vget(wv[i], e)) * vget(xv[i], e);
                }
            block_sum<T, 2, NW>(s, red, phase);
            const T rstd = t_rsqrt_of(s[0] * inv_n + eps);
            const T coef = rstd * rstd * rstd * s[1] * inv_n;
            V *dxr = reinterpret_cast<V *>(dx + r * cols);
#pragma unroll
            for (int i = 0; i < VPT; ++i) {
                const int v = tid + i * NT;
                V o;
#pragma unroll
                for (int e = 0; e < N; ++e) {
                    const T g = vget(gv[i], e) * vget(wv[i], e);
                    vset(o, e, rstd * g - coef * vget(xv[i], e));
                    aw[i][e] += vget(gv[i], e) * vget(xv[i], e) * rstd;
                }
                if (v < nvec) stream_store(dxr + v, o);
            }
        }
    };
    V xa[DEPTH > 0 ? VPT : 1], ga[DEPTH > 0 ? VPT : 1], xb[DEPTH > 1 ? VPT : 1], gb[DEPTH > 1 ? VPT : 1];
    if constexpr (DEPTH > 0) load_row(r0, xa, ga);
    if constexpr (DEPTH > 1) load_row(r0 + rstep, xb, gb);
    if constexpr (DEPTH > 1) {
        for (int64_t r = r0; r < r1; r += 2 * rstep) {  // the two register sets take alternate rows
            do_row(r, xa, ga);
            if (r + rstep < r1) do_row(r + rstep, xb, gb);
        }
    } else {
        for (int64_t r = r0; r < r1; r += rstep) do_row(r, xa, ga);
    }
    // one row of partial column sums per workgroup
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int v = tid + i * NT;
        if (v < nvec) {
            V ow, ob;
#pragma unroll
            for (int e = 0; e < N; ++e) {
                vset(ow, e, aw[i][e]);
                vset(ob, e, ab[i][e]);
            }
            if (part_w) reinterpret_cast<V *>(part_w + (int64_t)blockIdx.x * cols)[v] = ow;
            if (part_b) reinterpret_cast<V *>(part_b + (int64_t)blockIdx.x * cols)[v] = ob;
        }
    }
}

// ---- streaming norm backward (any row length): one workgroup per row, x / dy re-read per pass ----
// Writes dx and the row statistics (mean, rstd; mean = 0 for RMSNorm) for the column-sum pass.
template <typename T, bool RMS>
__global__ __launch_bounds__(kThreads) void norm_backward_stream_kernel(const T *__restrict__ dy, const T *__restrict__ x,
                                                                        const T *__restrict__ w, int64_t cols, T eps,
                                                                        T *__restrict__ dx, T *__restrict__ stats) {
    __shared__ T red[2 * kWaves * 2];
    int phase = 0;
    const int64_t r = blockIdx.x;
    const T *xr = x + r * cols, *dyr = dy + r * cols;
    T *dxr = dx + r * cols;
    const T inv_n = T(1) / (T)cols;
    T mean = T(0), rstd;
    if constexpr (!RMS) {
        T s[1] = {T(0)};
        for (int64_t j = threadIdx.x; j < cols; j += kThreads) s[0] += xr[j];
        block_sum<T, 1>(s, red, phase);
        mean = s[0] * inv_n;
        T q[1] = {T(0)};
        for (int64_t j = threadIdx.x; j < cols; j += kThreads) {
            const T d = xr[j] - mean;
            q[0] += d * d;
        }
        block_sum<T, 1>(q, red, phase);
        rstd = t_rsqrt_of(q[0] * inv_n + eps);
        T c[2] = {T(0), T(0)};
        for (int64_t j = threadIdx.x; j < cols; j += kThreads) {
            const T xhat = (xr[j] - mean) * rstd;
            const T dxhat = dyr[j] * w[j];
            c[0] += dxhat;
            c[1] += dxhat * xhat;
        }
        block_sum<T, 2>(c, red, phase);
        for (int64_t j = threadIdx.x; j < cols; j += kThreads) {
            const T xhat = (xr[j] - mean) * rstd;
            const T dxhat = dyr[j] * w[j];
            dxr[j] = rstd * (dxhat - (c[0] + xhat * c[1]) * inv_n);
        }
    } else {
        T s[1] = {T(0)};
        for (int64_t j = threadIdx.x; j < cols; j += kThreads) s[0] += xr[j] * xr[j];
        block_sum<T, 1>(s, red, phase);
        rstd = t_rsqrt_of(s[0] * inv_n + eps);
        T c[1] = {T(0)};
        for (int64_t j = threadIdx.x; j < cols; j += kThreads) c[0] += (dyr[j] * (w ? w[j] : T(1))) * xr[j];
        block_sum<T, 1>(c, red, phase);
        const T coef = rstd * rstd * rstd * c[0] * inv_n;
        for (int64_t j = threadIdx.x; j < cols; j += kThreads) dxr[j] = rstd * (dyr[j] * (w ? w[j] : T(1))) - coef * xr[j];
    }
    if (threadIdx.x == 0 && stats) {
        stats[2 * r] = mean;
        stats[2 * r + 1] = rstd;
    }
}

// Partial column sums over a run of rows, one thread per column (coalesced), rows in order.
// MODE 0: sum of src; MODE 1: LayerNorm dweight, sum of dy * (x - mean) * rstd; MODE 2: RMSNorm
// dweight, sum of dy * x * rstd. part[blockIdx.y][col].
template <typename T, int MODE>
__global__ __launch_bounds__(kThreads) void col_partial_kernel(const T *__restrict__ src, const T *__restrict__ x,
                                                               const T *__restrict__ stats, int64_t rows, int64_t cols,
                                                               int64_t ld, int rows_per_block, T *__restrict__ part) {
    const int64_t col = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (col >= cols) return;
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_block;
    const int64_t r1 = r0 + rows_per_block < rows ? r0 + rows_per_block : rows;
    T acc = T(0);
    for (int64_t r = r0; r < r1; ++r) {
        const T g = src[r * ld + col];
        if constexpr (MODE == 0) acc += g;
        else if constexpr (MODE == 1) acc += g * ((x[r * ld + col] - stats[2 * r]) * stats[2 * r + 1]);
        else acc += g * x[r * ld + col] * stats[2 * r + 1];
    }
    part[(int64_t)blockIdx.y * cols + col] = acc;
}

// out[col] = sum over the parts. A workgroup owns 32 columns; its 8 part-lanes each add every 8th
// part in ascending order (loads eight deep, independent of the adds), then the 8 lane sums are
// added lane 0..7. The order is a function of (nparts) only.
template <typename T>
__global__ __launch_bounds__(kThreads) void col_final_kernel(const T *__restrict__ part, int nparts, int64_t cols, T *__restrict__ out,
                                                             const T *__restrict__ part2, T *__restrict__ out2) {
    // blockIdx.y == 1: the second array of partial sums (dbias beside dweight), summed in the same launch
    if (blockIdx.y == 1) {
        part = part2;
        out = out2;
    }
    constexpr int CW = 32, PL = kThreads / CW;
    __shared__ T red[PL][CW];
    const int c = threadIdx.x % CW, pl = threadIdx.x / CW;
    const int64_t col = (int64_t)blockIdx.x * CW + c;
    T acc = T(0);
    if (col < cols) {
        int b = pl;
        for (; b + 7 * PL < nparts; b += 8 * PL) {
            T v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = part[(int64_t)(b + u * PL) * cols + col];
#pragma unroll
            for (int u = 0; u < 8; ++u) acc += v[u];
        }
        for (; b < nparts; b += PL) acc += part[(int64_t)b * cols + col];
    }
    red[pl][c] = acc;
    __syncthreads();
    if (pl == 0 && col < cols) {
        T s = red[0][c];
#pragma unroll
        for (int l = 1; l < PL; ++l) s += red[l][c];
        out[col] = s;
    }
}

// Zero fill as a kernel (memset nodes are avoided so that callers can capture these entry points).
template <typename T> __global__ __launch_bounds__(kThreads) void fill_kernel(T *dst, int64_t n, T value) {
    const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (i < n) dst[i] = value;
}
template <typename T> int32_t value_fill(T *dst, int64_t n, T value, hipStream_t st) {
    if (n <= 0) return FTH_OK;
    FTH_ARG(fth::ceil_div(n, kThreads) <= 2147483647LL, "fill: extent too large");
    fill_kernel<T><<<dim3((unsigned)fth::ceil_div(n, kThreads)), dim3(kThreads), 0, st>>>(dst, n, value);
    FTH_CHECK_LAUNCH("fill");
    return FTH_OK;
}
template <typename T> int32_t zero_fill(T *dst, int64_t n, hipStream_t st) { return value_fill<T>(dst, n, T(0), st); }

inline int pick_rows_per_block(int64_t rows) {
    // one workgroup per compute unit (FTH_BWD_BLOCKS_PER_CU), at most 64 rows each
    const int cus = fth::compute_units() > 0 ? fth::compute_units() : 256;
    int64_t r = rows / ((int64_t)cus * FTH_BWD_BLOCKS_PER_CU);
    if (r < 1) r = 1;
    if (r > 64) r = 64;
    return (int)r;
}

template <typename T> bool norm_fast_path(int64_t cols, const void *a, const void *b, const void *c, const void *d) {
    constexpr int N = Vec16<T>::N;
    auto al = [](const void *q) { return q == nullptr || (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
    return cols % N == 0 && cols <= (int64_t)kThreads * 16 * N && al(a) && al(b) && al(c) && al(d);
}

template <typename T> size_t norm_backward_workspace(int64_t rows, int64_t cols) {
    // fast path: 2 partial arrays of [blocks, cols]; streaming path: stats [rows, 2] + 2 partial arrays
    const int rpb = pick_rows_per_block(rows);
    const int64_t blocks = fth::ceil_div(rows, rpb);
    return (size_t)(2 * blocks * cols + 2 * rows + 64) * sizeof(T);
}

template <typename T, bool RMS>
int32_t norm_backward_entry(const T *dy, const T *x, const T *w, int64_t rows, int64_t cols, T eps, T *dx, T *dw, T *db,
                            void *workspace, size_t workspace_bytes, fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(rows >= 0 && cols >= 0, "norm backward: negative extent");
    FTH_ARG(RMS || w != nullptr, "layer_norm backward: weight is required");
    FTH_ARG(RMS || (dw != nullptr && db != nullptr), "layer_norm backward: dweight and dbias are required");
    FTH_ARG(!(RMS && w == nullptr && dw != nullptr), "rms_norm backward: dweight without a weight");
    hipStream_t st = fth::resolve_stream(s);
    if (cols == 0) return FTH_OK;
    const bool want_w = dw != nullptr;
    if (rows == 0) {
        if (want_w) if (int32_t rc = zero_fill<T>(dw, cols, st)) return rc;
        if (db) if (int32_t rc = zero_fill<T>(db, cols, st)) return rc;
        return FTH_OK;
    }
    FTH_ARG(dy && x && dx, "norm backward: NULL operand");
    FTH_ARG(cols <= 2147483647LL && rows <= 2147483647LL, "norm backward: extent too large");
    FTH_ARG(workspace_bytes >= norm_backward_workspace<T>(rows, cols) && (workspace != nullptr),
            "norm backward: workspace of %zu bytes needed, %zu given", norm_backward_workspace<T>(rows, cols), workspace_bytes);
    const int rpb = pick_rows_per_block(rows);
    const int64_t blocks = fth::ceil_div(rows, rpb);
    T *part_w = static_cast<T *>(workspace);
    T *part_b = part_w + blocks * cols;
    T *stats = part_b + blocks * cols;
    const int64_t col_blocks = fth::ceil_div(cols, kThreads);
    if (norm_fast_path<T>(cols, dy, x, w, dx)) {
        constexpr int N = Vec16<T>::N;
        const int64_t nvec = cols / N;
        const int vpt = (int)fth::ceil_div(nvec, kThreads);
        T *pw = want_w ? part_w : nullptr, *pb = db ? part_b : nullptr;
#define FTH_NORM_BWD(V) \
    norm_backward_kernel<T, V, RMS><<<dim3((unsigned)blocks), dim3(kThreads), 0, st>>>(dy, x, w, rows, (int)cols, eps, dx, pw, pb, rpb)
#define FTH_NORM_BWD_DEEP(V, NT_) \
    norm_backward_kernel<T, V, RMS, NT_, 2><<<dim3((unsigned)blocks), dim3(NT_), 0, st>>>(dy, x, w, rows, (int)cols, eps, dx, pw, pb, rpb)
        if (nvec <= kThreads) FTH_NORM_BWD_DEEP(1, kThreads);
        else if (nvec <= 2 * kThreads) FTH_NORM_BWD_DEEP(1, 2 * kThreads);
        else if (nvec <= 4 * kThreads) FTH_NORM_BWD_DEEP(2, 2 * kThreads);
        else if (vpt <= 8) FTH_NORM_BWD(8);
        else FTH_NORM_BWD(16);
#undef FTH_NORM_BWD_DEEP
#undef FTH_NORM_BWD
        FTH_CHECK_LAUNCH("norm_backward");
    } else {
        norm_backward_stream_kernel<T, RMS><<<dim3((unsigned)rows), dim3(kThreads), 0, st>>>(dy, x, w, cols, eps, dx, stats);
        FTH_CHECK_LAUNCH("norm_backward_stream");
        if (want_w) {
            col_partial_kernel<T, RMS ? 2 : 1><<<dim3((unsigned)col_blocks, (unsigned)blocks), dim3(kThreads), 0, st>>>(
                dy, x, stats, rows, cols, cols, rpb, part_w);
            FTH_CHECK_LAUNCH("norm_backward_dweight");
        }
        if (db) {
            col_partial_kernel<T, 0><<<dim3((unsigned)col_blocks, (unsigned)blocks), dim3(kThreads), 0, st>>>(
                dy, nullptr, nullptr, rows, cols, cols, rpb, part_b);
            FTH_CHECK_LAUNCH("norm_backward_dbias");
        }
    }
    if (want_w && db) {
        col_final_kernel<T><<<dim3((unsigned)fth::ceil_div(cols, 32), 2), dim3(kThreads), 0, st>>>(part_w, (int)blocks, cols, dw, part_b, db);
        FTH_CHECK_LAUNCH("norm_backward_dweight_dbias_sum");
    } else if (want_w) {
        col_final_kernel<T><<<dim3((unsigned)fth::ceil_div(cols, 32)), dim3(kThreads), 0, st>>>(part_w, (int)blocks, cols, dw, nullptr, nullptr);
        FTH_CHECK_LAUNCH("norm_backward_dweight_sum");
    } else if (db) {
        col_final_kernel<T><<<dim3((unsigned)fth::ceil_div(cols, 32)), dim3(kThreads), 0, st>>>(part_b, (int)blocks, cols, db, nullptr, nullptr);
        FTH_CHECK_LAUNCH("norm_backward_dbias_sum");
    }
    return FTH_OK;
}

// ---- linear backward ----
template <typename T> size_t linear_backward_workspace(int64_t batch, int64_t out_f) {
    const int rpb = pick_rows_per_block(batch);
    return (size_t)(fth::ceil_div(batch > 0 ? batch : 1, rpb) * out_f + 64) * sizeof(T);
}

template <typename T> int32_t dev_gemm(const fth_gemm_desc *d, T alpha, const T *a, const T *b, T *c, fth_stream s);
template <> int32_t dev_gemm<float>(const fth_gemm_desc *d, float alpha, const float *a, const float *b, float *c, fth_stream s) {
    return fth_dev_gemm_f32(d, alpha, a, b, c, nullptr, nullptr, s);
}
template <> int32_t dev_gemm<double>(const fth_gemm_desc *d, double alpha, const double *a, const double *b, double *c, fth_stream s) {
    return fth_dev_gemm_f64(d, alpha, a, b, c, nullptr, nullptr, s);
}

inline fth_gemm_desc make_desc(int64_t m, int64_t n, int64_t k, int trans_a, int trans_b, int64_t batch) {
    fth_gemm_desc d{};
    d.m = m; d.n = n; d.k = k;
    d.lda = trans_a ? m : k;
    d.ldb = trans_b ? k : n;
    d.ldc = n;
    d.batch = batch;
    d.stride_a = m * k; d.stride_b = k * n; d.stride_c = m * n;
    d.trans_a = trans_a; d.trans_b = trans_b;
    return d;
}

template <typename T>
int32_t linear_backward_entry(const T *dy, const T *x, const T *w, int64_t batch, int64_t in_f, int64_t out_f, T *dx, T *dw,
                              T *db, void *workspace, size_t workspace_bytes, fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(batch >= 0 && in_f >= 0 && out_f >= 0, "linear backward: negative extent");
    hipStream_t st = fth::resolve_stream(s);
    fth_stream fs = reinterpret_cast<fth_stream>(st);
    // dx = dy . W : [batch, out] . [out, in]
    if (batch > 0 && in_f > 0) {
        FTH_ARG(dx != nullptr, "linear backward: dx is NULL");
        fth_gemm_desc d = make_desc(batch, in_f, out_f, 0, 0, 1);
        if (int32_t rc = dev_gemm<T>(&d, T(1), dy, w, dx, fs)) return rc;
    }
    // dweight = dy^T . x : dy [batch, out] read as the [k, m] operand
    if (out_f > 0 && in_f > 0) {
        FTH_ARG(dw != nullptr, "linear backward: dweight is NULL");
        fth_gemm_desc d = make_desc(out_f, in_f, batch, 1, 0, 1);
        if (int32_t rc = dev_gemm<T>(&d, T(1), dy, x, dw, fs)) return rc;
    }
    if (db && out_f > 0) {
        if (batch == 0) {
            if (int32_t rc = zero_fill<T>(db, out_f, st)) return rc;
            return FTH_OK;
        }
        FTH_ARG(workspace != nullptr && workspace_bytes >= linear_backward_workspace<T>(batch, out_f),
                "linear backward: workspace of %zu bytes needed, %zu given", linear_backward_workspace<T>(batch, out_f), workspace_bytes);
        const int rpb = pick_rows_per_block(batch);
        const int64_t blocks = fth::ceil_div(batch, rpb), col_blocks = fth::ceil_div(out_f, kThreads);
        T *part = static_cast<T *>(workspace);
        col_partial_kernel<T, 0><<<dim3((unsigned)col_blocks, (unsigned)blocks), dim3(kThreads), 0, st>>>(dy, nullptr, nullptr, batch,
                                                                                                         out_f, out_f, rpb, part);
        FTH_CHECK_LAUNCH("linear_backward_dbias");
        col_final_kernel<T><<<dim3((unsigned)fth::ceil_div(out_f, 32)), dim3(kThreads), 0, st>>>(part, (int)blocks, out_f, db, nullptr, nullptr);
        FTH_CHECK_LAUNCH("linear_backward_dbias_sum");
    }
    return FTH_OK;
}

// ---- SDPA backward row passes ----
// In place on the score rows: scale, strict-max scan over the first `limit` entries, exp, sum,
// divide, zero tail (the forward's row loop, crates/ft-kernel-cpu/src/lib.rs:5594-5616). One
// wavefront per row; limit = min(i + 1, seq_k) when causal, i = row % seq_q.
template <typename T> __device__ __forceinline__ T dev_exp_t(T v);
template <> __device__ __forceinline__ float dev_exp_t<float>(float v) { return expf(v); }
template <> __device__ __forceinline__ double dev_exp_t<double>(double v) { return exp(v); }

template <typename T>
__global__ __launch_bounds__(kThreads) void sdpa_softmax_rows_kernel(T *__restrict__ p, int64_t rows, int64_t seq_q, int64_t seq_k,
                                                                    T scale, int causal, const T *__restrict__ mask,
                                                                    int64_t mask_bh_stride) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t r = (int64_t)blockIdx.x * kWaves + threadIdx.x / kWave;
    if (r >= rows) return;
    const int64_t i = r % seq_q;
    const int64_t limit = causal ? (i + 1 < seq_k ? i + 1 : seq_k) : seq_k;
    T *row = p + r * seq_k;
    // additive mask row (sdpa_backward_masked_f64, :5466-5475): the score becomes s * scale + mask
    const T *mrow = mask ? mask + (r / seq_q) * mask_bh_stride + i * seq_k : nullptr;
    T m = -__builtin_inf();
    for (int64_t j = lane; j < limit; j += kWave) {
        T v = row[j] * scale;
        if (mrow) v = v + mrow[j];
        row[j] = v;
        m = v > m ? v : m;
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const T o = __shfl_xor(m, off, kWave);
        m = o > m ? o : m;
    }
    T sum = T(0);
    for (int64_t j = lane; j < limit; j += kWave) {  // each lane re-reads only what it wrote above
        const T e = dev_exp_t<T>(row[j] - m);
        row[j] = e;
        sum += e;
    }
    sum = wave_sum(sum);
    for (int64_t j = lane; j < limit; j += kWave) row[j] = row[j] / sum;
    for (int64_t j = limit + lane; j < seq_k; j += kWave) row[j] = T(0);
}

// dU_ij = P_ij * (dU_ij - sum_j P_ij dU_ij), in place on dU (:5637-5647).
template <typename T>
__global__ __launch_bounds__(kThreads) void sdpa_softmax_backward_rows_kernel(const T *__restrict__ p, T *__restrict__ du, int64_t rows,
                                                                             int64_t seq_k) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t r = (int64_t)blockIdx.x * kWaves + threadIdx.x / kWave;
    if (r >= rows) return;
    const T *pr = p + r * seq_k;
    T *dr = du + r * seq_k;
    T dot = T(0);
    for (int64_t j = lane; j < seq_k; j += kWave) dot += pr[j] * dr[j];
    dot = wave_sum(dot);
    for (int64_t j = lane; j < seq_k; j += kWave) dr[j] = pr[j] * (dr[j] - dot);
}

// Columns of query row i that the block-causal products compute and read: whole key blocks up to the one holding i.
__device__ __forceinline__ int sdpa_block_limit(int64_t i, int blk, int seq_k) {
    const int64_t l = (i / blk + 1) * blk;
    return (int)(l < seq_k ? l : seq_k);
}

// Register-resident forms of the two row passes for rows of up to 64 * VPL 16-byte vectors: the row is
// read once (only its first `limit` entries matter for the softmax; the rest is written as zeros)
// and written once. Same arithmetic as the streaming kernels above, lane-strided partial sums.
template <typename T, int VPL>
__global__ __launch_bounds__(kThreads) void sdpa_softmax_rows_vec_kernel(T *__restrict__ p, int64_t rows, int64_t seq_q, int seq_k,
                                                                        T scale, int causal, int blk, const T *__restrict__ mask,
                                                                        int64_t mask_bh_stride) {
    using V = typename Vec16<T>::type;
    constexpr int N = Vec16<T>::N;
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t r = (int64_t)blockIdx.x * kWaves + threadIdx.x / kWave;
    if (r >= rows) return;
    const int64_t i = r % seq_q;
    const int limit = causal ? (int)(i + 1 < seq_k ? i + 1 : seq_k) : seq_k;
    // blk > 0: only the first (i / blk + 1) * blk columns of the row exist downstream (block-causal products)
    const int nvec = (blk > 0 ? sdpa_block_limit(i, blk, seq_k) : seq_k) / N;
    V *row = reinterpret_cast<V *>(p + r * seq_k);
    // additive mask row, 16-byte aligned like the score row (the launcher checks)
    const V *mrow = mask ? reinterpret_cast<const V *>(mask + (r / seq_q) * mask_bh_stride + i * seq_k) : nullptr;
    T e[VPL][N];
    T m = -__builtin_inf();
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
        const int v = lane + u * kWave;
        if (v < nvec && v * N < limit) {
            const V x = row[v];
            V mv;
            if (mrow) mv = mrow[v];
#pragma unroll
            for (int c = 0; c < N; ++c) {
                e[u][c] = vget(x, c) * scale;
                if (mrow) e[u][c] = e[u][c] + vget(mv, c);
                if (v * N + c < limit) m = e[u][c] > m ? e[u][c] : m;
            }
        } else {
#pragma unroll
            for (int c = 0; c < N; ++c) e[u][c] = T(0);
        }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const T o = __shfl_xor(m, off, kWave);
        m = o > m ? o : m;
    }
    T sum = T(0);
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
        const int v = lane + u * kWave;
#pragma unroll
        for (int c = 0; c < N; ++c) {
            if (v * N + c < limit) {
                e[u][c] = dev_exp_t<T>(e[u][c] - m);
                sum += e[u][c];
            } else {
                e[u][c] = T(0);
            }
        }
    }
    sum = wave_sum(sum);
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
        const int v = lane + u * kWave;
        if (v < nvec) {
            V o;
#pragma unroll
            for (int c = 0; c < N; ++c) vset(o, c, (v * N + c < limit) ? e[u][c] / sum : T(0));
            row[v] = o;
        }
    }
}

template <typename T, int VPL>
__global__ __launch_bounds__(kThreads) void sdpa_softmax_backward_rows_vec_kernel(const T *__restrict__ p, T *__restrict__ du, int64_t rows,
                                                                                 int64_t seq_q, int seq_k, int blk) {
    using V = typename Vec16<T>::type;
    constexpr int N = Vec16<T>::N;
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t r = (int64_t)blockIdx.x * kWaves + threadIdx.x / kWave;
    if (r >= rows) return;
    const int nvec = (blk > 0 ? sdpa_block_limit(r % seq_q, blk, seq_k) : seq_k) / N;
    const V *pr = reinterpret_cast<const V *>(p + r * seq_k);
    V *dr = reinterpret_cast<V *>(du + r * seq_k);
    V pv[VPL], dv[VPL];
    T dot = T(0);
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
        const int v = lane + u * kWave;
        if (v < nvec) {
            pv[u] = pr[v];
            dv[u] = dr[v];
#pragma unroll
            for (int c = 0; c < N; ++c) dot += vget(pv[u], c) * vget(dv[u], c);
        }
    }
    dot = wave_sum(dot);
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
        const int v = lane + u * kWave;
        if (v < nvec) {
            V o;
#pragma unroll
            for (int c = 0; c < N; ++c) vset(o, c, vget(pv[u], c) * (vget(dv[u], c) - dot));
            dr[v] = o;
        }
    }
}

// 0 when the rows do not fit the register-resident kernels, else the vectors per lane to use.
template <typename T> int sdpa_row_vpl(int64_t seq_k, const void *a, const void *b) {
    constexpr int N = Vec16<T>::N;
    auto al = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
    if (seq_k % N != 0 || seq_k > (int64_t)kWave * 16 * N || !al(a) || !al(b)) return 0;
    const int64_t per = fth::ceil_div(seq_k / N, kWave);
    return per <= 1 ? 1 : per <= 2 ? 2 : per <= 4 ? 4 : per <= 8 ? 8 : 16;
}

// Two score-shaped matrices (P and dU; on the fused fp32 path S and dP / dS in whole 32 x 32 tiles with one spare tile
// row, which is what the size allows for), 64 elements of slack, and two per-row vectors (log-sum-exp and delta of the
// fused path).
template <typename T> int64_t sdpa_backward_score_elems(int64_t num_bh, int64_t seq_q, int64_t seq_k) {
    if (std::is_same<T, float>::value) {
        int64_t s_floats, d_floats;
        fth::sdpa_backward_fused_workspace(num_bh, seq_q, seq_k, &s_floats, &d_floats);
        return s_floats + d_floats;  // >= 2 * num_bh * seq_q * seq_k
    }
    return 2 * num_bh * seq_q * seq_k;
}
template <typename T> size_t sdpa_backward_workspace(int64_t num_bh, int64_t seq_q, int64_t seq_k) {
    return (size_t)(sdpa_backward_score_elems<T>(num_bh, seq_q, seq_k) + 64 + 2 * num_bh * seq_q + 32) * sizeof(T);
}

template <typename T>
int32_t sdpa_backward_entry(const T *q, const T *k, const T *v, const T *dout, int64_t num_bh, int64_t seq_q, int64_t seq_k,
                            int64_t d_k, int64_t d_v, T scale, int causal, T *dq, T *dk, T *dv, void *workspace,
                            size_t workspace_bytes, fth_stream s, const T *mask = nullptr, int64_t mask_bh_stride = 0,
                            bool unit_dout = false) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(num_bh >= 0 && seq_q >= 0 && seq_k >= 0 && d_k >= 0 && d_v >= 0, "sdpa backward: negative extent");
    hipStream_t st = fth::resolve_stream(s);
    fth_stream fs = reinterpret_cast<fth_stream>(st);
    if (num_bh == 0) return FTH_OK;
    // Degenerate extents: the gradients that exist are all zero (crates/ft-kernel-cpu/src/lib.rs:5552-5554).
    if (seq_q == 0 || seq_k == 0 || (d_k == 0 && d_v == 0)) {
        if (dq && num_bh * seq_q * d_k > 0) if (int32_t rc = zero_fill<T>(dq, num_bh * seq_q * d_k, st)) return rc;
        if (dk && num_bh * seq_k * d_k > 0) if (int32_t rc = zero_fill<T>(dk, num_bh * seq_k * d_k, st)) return rc;
        if (dv && num_bh * seq_k * d_v > 0) if (int32_t rc = zero_fill<T>(dv, num_bh * seq_k * d_v, st)) return rc;
        return FTH_OK;
    }
    FTH_ARG(q && k && v && (dout || unit_dout) && dq && dk && dv, "sdpa backward: NULL operand");
    int64_t pe;
    FTH_ARG(!__builtin_mul_overflow(num_bh, seq_q, &pe) && !__builtin_mul_overflow(pe, seq_k, &pe) && pe < ((int64_t)1 << 40),
            "sdpa backward: score matrix too large");
    const size_t ws_need = sdpa_backward_workspace<T>(num_bh, seq_q, seq_k) + (unit_dout ? (size_t)(seq_q * d_v + 4) * sizeof(T) : 0);
    FTH_ARG(workspace != nullptr && workspace_bytes >= ws_need, "sdpa backward: workspace of %zu bytes needed, %zu given", ws_need,
            workspace_bytes);
    T *p = static_cast<T *>(workspace);
    T *du = p + pe;
    const int64_t score_elems = sdpa_backward_score_elems<T>(num_bh, seq_q, seq_k);
    // dOut = ones (sdpa_backward_f32_unit_dout, :5662-5770): one [seq_q, d_v] plane of ones shared by every (batch, head)
    // through a zero batch stride stands in for the gradient; nothing of size num_bh is materialised.
    int64_t dout_bs = seq_q * d_v;
    if (unit_dout) {
        T *ones = p + ((score_elems + 64 + 3) & ~(int64_t)3);  // keeps the 16-byte alignment of the workspace base
        if (int32_t rc = value_fill<T>(ones, seq_q * d_v, T(1), st)) return rc;
        dout = ones;
        dout_bs = 0;
    }
    const int64_t rows = num_bh * seq_q;
    FTH_ARG(fth::ceil_div(rows, kWaves) <= 2147483647LL, "sdpa backward: too many rows");
    if constexpr (std::is_same<T, float>::value) {
        // Fused path: a statistics pass (scores, dP, log-sum-exp, delta), one key-owned kernel for dS, dK and dV, and
        // the dQ product. P and dU are never materialised.
        auto al = [](const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; };
        if (!mask && fth::sdpa_backward_fused_applies(num_bh, seq_q, seq_k, d_k, d_v, scale) && al(q) && al(k) && al(v) && al(dout) &&
            al(dq) && al(dk) && al(dv) && al(workspace)) {
            float *lse = p + ((score_elems + 64 + 3) & ~(int64_t)3) + (unit_dout ? ((seq_q * d_v + 4 + 3) & ~(int64_t)3) : 0);  // behind the ones plane
            lse = reinterpret_cast<float *>((reinterpret_cast<uintptr_t>(lse) + 15u) & ~(uintptr_t)15u);
            float *delta = lse + ((rows + 3) & ~(int64_t)3);
            int64_t s_floats, d_floats;
            fth::sdpa_backward_fused_workspace(num_bh, seq_q, seq_k, &s_floats, &d_floats);
            float *dpds = p + s_floats;
            if (int32_t rc = fth::sdpa_backward_stats_f32(q, k, v, dout, dout_bs, num_bh, seq_q, seq_k, d_k, scale, causal, p, dpds, lse, delta, st))
                return rc;
            if (int32_t rc = fth::sdpa_backward_keys_f32(q, dout, dout_bs, p, lse, delta, num_bh, seq_q, seq_k, d_k, scale, causal, 128, dpds, dk,
                                                        dv, st))
                return rc;
            return fth::sdpa_backward_dq_f32(dpds, k, num_bh, seq_q, seq_k, d_k, scale, causal, dq, st);
        }
    }
    int vpl = sdpa_row_vpl<T>(seq_k, p, du);
    if (mask && ((reinterpret_cast<uintptr_t>(mask) & 15u) != 0 || mask_bh_stride % Vec16<T>::N != 0)) vpl = 0;  // unaligned mask rows
    const dim3 row_grid((unsigned)fth::ceil_div(rows, kWaves));
    // Causal square problems: the five products are cut into key / query blocks of `blk` rows so that nothing above the
    // block diagonal is computed, stored or read (a little over half of the full work at eight blocks). Each block is one
    // batched launch over all (batch, head) pairs; the choice depends on the shape only.
    int64_t blk = 0;
    if (causal && seq_q == seq_k && vpl > 0 && seq_k >= 512 && seq_k % 128 == 0 && d_k > 0 && d_v > 0) {
        blk = (seq_k / 8 + 127) / 128 * 128;
        if (blk < 256) blk = 256;  // measured: blocks of 128 rows cost more in launches than they save in work
    }
    const int64_t nblk = blk > 0 ? fth::ceil_div(seq_q, blk) : 1;
    auto strided = [&](int64_t m, int64_t n, int64_t kk, int ta, int tb, int64_t lda, int64_t ldb, int64_t ldc, int64_t sa, int64_t sb,
                       int64_t sc) {
        fth_gemm_desc d{};
        d.m = m; d.n = n; d.k = kk;
        d.lda = lda; d.ldb = ldb; d.ldc = ldc;
        d.batch = num_bh;
        d.stride_a = sa; d.stride_b = sb; d.stride_c = sc;
        d.trans_a = ta; d.trans_b = tb;
        return d;
    };
    // P = Q . K^T  (scores; scaled inside the row pass)
    if (blk > 0) {
        for (int64_t ib = 0; ib < nblk; ++ib) {
            const int64_t i0 = ib * blk, i1 = std::min(seq_q, i0 + blk);
            fth_gemm_desc d = strided(i1 - i0, i1, d_k, 0, 1, d_k, d_k, seq_k, seq_q * d_k, seq_k * d_k, seq_q * seq_k);
            if (int32_t rc = dev_gemm<T>(&d, T(1), q + i0 * d_k, k, p + i0 * seq_k, fs)) return rc;
        }
    } else if (d_k > 0) {
        fth_gemm_desc d = make_desc(seq_q, seq_k, d_k, 0, 1, num_bh);
        if (int32_t rc = dev_gemm<T>(&d, T(1), q, k, p, fs)) return rc;
    } else {
        if (int32_t rc = zero_fill<T>(p, pe, st)) return rc;
    }
#define FTH_ROWS_VEC(KERN, ...)                                                         \
    switch (vpl) {                                                                      \
        case 1: KERN<T, 1><<<row_grid, dim3(kThreads), 0, st>>>(__VA_ARGS__); break;     \
        case 2: KERN<T, 2><<<row_grid, dim3(kThreads), 0, st>>>(__VA_ARGS__); break;     \
        case 4: KERN<T, 4><<<row_grid, dim3(kThreads), 0, st>>>(__VA_ARGS__); break;     \
        case 8: KERN<T, 8><<<row_grid, dim3(kThreads), 0, st>>>(__VA_ARGS__); break;     \
        default: KERN<T, 16><<<row_grid, dim3(kThreads), 0, st>>>(__VA_ARGS__); break;   \
    }
    if (vpl > 0) {
        FTH_ROWS_VEC(sdpa_softmax_rows_vec_kernel, p, rows, seq_q, (int)seq_k, scale, causal, (int)blk, mask, mask_bh_stride)
    } else {
        sdpa_softmax_rows_kernel<T><<<row_grid, dim3(kThreads), 0, st>>>(p, rows, seq_q, seq_k, scale, causal, mask, mask_bh_stride);
    }
    FTH_CHECK_LAUNCH("sdpa_backward_softmax");
    // dU = dOut . V^T
    if (blk > 0) {
        for (int64_t ib = 0; ib < nblk; ++ib) {
            const int64_t i0 = ib * blk, i1 = std::min(seq_q, i0 + blk);
            fth_gemm_desc d = strided(i1 - i0, i1, d_v, 0, 1, d_v, d_v, seq_k, dout_bs, seq_k * d_v, seq_q * seq_k);
            if (int32_t rc = dev_gemm<T>(&d, T(1), dout + i0 * d_v, v, du + i0 * seq_k, fs)) return rc;
        }
    } else if (d_v > 0) {
        fth_gemm_desc d = make_desc(seq_q, seq_k, d_v, 0, 1, num_bh);
        d.stride_a = dout_bs;
        if (int32_t rc = dev_gemm<T>(&d, T(1), dout, v, du, fs)) return rc;
    } else {
        if (int32_t rc = zero_fill<T>(du, pe, st)) return rc;
    }
    // dV = P^T . dOut  (P read as the [k, m] operand); key block j only sees the queries from its first row on
    if (blk > 0) {
        for (int64_t jb = 0; jb < nblk; ++jb) {
            const int64_t j0 = jb * blk, j1 = std::min(seq_k, j0 + blk);
            fth_gemm_desc d = strided(j1 - j0, d_v, seq_q - j0, 1, 0, seq_k, d_v, d_v, seq_q * seq_k, dout_bs, seq_k * d_v);
            if (int32_t rc = dev_gemm<T>(&d, T(1), p + j0 * seq_k + j0, dout + j0 * d_v, dv + j0 * d_v, fs)) return rc;
        }
    } else if (d_v > 0) {
        fth_gemm_desc d = make_desc(seq_k, d_v, seq_q, 1, 0, num_bh);
        d.stride_b = dout_bs;
        if (int32_t rc = dev_gemm<T>(&d, T(1), p, dout, dv, fs)) return rc;
    }
    if (vpl > 0) {
        FTH_ROWS_VEC(sdpa_softmax_backward_rows_vec_kernel, p, du, rows, seq_q, (int)seq_k, (int)blk)
    } else {
        sdpa_softmax_backward_rows_kernel<T><<<row_grid, dim3(kThreads), 0, st>>>(p, du, rows, seq_k);
    }
#undef FTH_ROWS_VEC
    FTH_CHECK_LAUNCH("sdpa_backward_softmax_grad");
    if (blk > 0) {
        // dQ = scale * dU . K over the keys up to the query block's end; dK = scale * dU^T . Q over the queries from the key block on
        for (int64_t ib = 0; ib < nblk; ++ib) {
            const int64_t i0 = ib * blk, i1 = std::min(seq_q, i0 + blk);
            fth_gemm_desc d = strided(i1 - i0, d_k, i1, 0, 0, seq_k, d_k, d_k, seq_q * seq_k, seq_k * d_k, seq_q * d_k);
            if (int32_t rc = dev_gemm<T>(&d, scale, du + i0 * seq_k, k, dq + i0 * d_k, fs)) return rc;
        }
        for (int64_t jb = 0; jb < nblk; ++jb) {
            const int64_t j0 = jb * blk, j1 = std::min(seq_k, j0 + blk);
            fth_gemm_desc d = strided(j1 - j0, d_k, seq_q - j0, 1, 0, seq_k, d_k, d_k, seq_q * seq_k, seq_q * d_k, seq_k * d_k);
            if (int32_t rc = dev_gemm<T>(&d, scale, du + j0 * seq_k + j0, q + j0 * d_k, dk + j0 * d_k, fs)) return rc;
        }
    } else if (d_k > 0) {
        // dQ = scale * dU . K ; dK = scale * dU^T . Q
        fth_gemm_desc dqd = make_desc(seq_q, d_k, seq_k, 0, 0, num_bh);
        if (int32_t rc = dev_gemm<T>(&dqd, scale, du, k, dq, fs)) return rc;
        fth_gemm_desc dkd = make_desc(seq_k, d_k, seq_q, 1, 0, num_bh);
        if (int32_t rc = dev_gemm<T>(&dkd, scale, du, q, dk, fs)) return rc;
    }
    return FTH_OK;
}

// ---- the allocation-free LayerNorm backward ----
// Partial column sums live in a file-scope device array instead of a caller workspace. Every GPU
// the library is loaded on holds its own copy at its own address, so the address is looked up once
// per device (with that device current) and only that pointer is ever given to kernels.
constexpr size_t kStaticScratchBytes = (size_t)24 << 20;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

int32_t static_scratch(void **out) {
    static std::mutex mu;
    static void *per_device[kMaxDevices] = {};
    int dev = 0;
    FTH_HIP(hipGetDevice(&dev));
    FTH_ARG(dev >= 0 && dev < kMaxDevices, "static scratch: device ordinal %d out of range", dev);
    std::lock_guard<std::mutex> lock(mu);
    if (!per_device[dev]) {
        void *ptr = nullptr;
        FTH_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        FTH_ARG(ptr != nullptr, "static scratch: the device array has no address on device %d", dev);
        per_device[dev] = ptr;
    }
    *out = per_device[dev];
    return FTH_OK;
}

}  // namespace

extern "C" {

size_t fth_dev_layer_norm_backward_noalloc_max_bytes(void) { return kStaticScratchBytes; }

int32_t fth_dev_layer_norm_backward_f32_noalloc(const float *dy, const float *x, const float *weight, int64_t rows, int64_t cols, float eps,
                                                float *dx, float *dweight, float *dbias, fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(rows >= 0 && cols >= 0, "layer_norm backward (no allocation): negative extent");
    FTH_ARG(cols <= 2147483647LL && rows <= 2147483647LL, "layer_norm backward (no allocation): extent too large");
    const size_t need = norm_backward_workspace<float>(rows, cols);
    if (need > kStaticScratchBytes)
        return fth::set_error(FTH_ERR_BUFFER_TOO_LARGE,
                              "layer_norm backward (no allocation): [%lld, %lld] needs %zu bytes of partial sums, the built-in scratch holds %zu; "
                              "use fth_dev_layer_norm_backward_f32 with a workspace",
                              (long long)rows, (long long)cols, need, kStaticScratchBytes);
    void *ptr = nullptr;
    if (int32_t rc = static_scratch(&ptr)) return rc;
    // Nothing in the scratch has to start at zero: every partial row and statistic that the second
    // pass reads is written by the first pass of the same call.
    return norm_backward_entry<float, false>(dy, x, weight, rows, cols, eps, dx, dweight, dbias, ptr, kStaticScratchBytes, s);
}

size_t fth_dev_norm_backward_workspace_bytes(int64_t rows, int64_t cols, int32_t dtype) {
    if (rows < 0 || cols < 0) return 0;
    return dtype == FTH_DTYPE_F64 ? norm_backward_workspace<double>(rows, cols) : norm_backward_workspace<float>(rows, cols);
}
int32_t fth_dev_layer_norm_backward_f32(const float *dy, const float *x, const float *weight, int64_t rows, int64_t cols, float eps,
                                        float *dx, float *dweight, float *dbias, void *workspace, size_t workspace_bytes,
                                        fth_stream s) {
    return norm_backward_entry<float, false>(dy, x, weight, rows, cols, eps, dx, dweight, dbias, workspace, workspace_bytes, s);
}
int32_t fth_dev_layer_norm_backward_f64(const double *dy, const double *x, const double *weight, int64_t rows, int64_t cols, double eps,
                                        double *dx, double *dweight, double *dbias, void *workspace, size_t workspace_bytes,
                                        fth_stream s) {
    return norm_backward_entry<double, false>(dy, x, weight, rows, cols, eps, dx, dweight, dbias, workspace, workspace_bytes, s);
}
int32_t fth_dev_rms_norm_backward_f32(const float *dy, const float *x, const float *weight, int64_t rows, int64_t cols, float eps,
                                      float *dx, float *dweight, void *workspace, size_t workspace_bytes, fth_stream s) {
    return norm_backward_entry<float, true>(dy, x, weight, rows, cols, eps, dx, dweight, nullptr, workspace, workspace_bytes, s);
}
int32_t fth_dev_rms_norm_backward_f64(const double *dy, const double *x, const double *weight, int64_t rows, int64_t cols, double eps,
                                      double *dx, double *dweight, void *workspace, size_t workspace_bytes, fth_stream s) {
    return norm_backward_entry<double, true>(dy, x, weight, rows, cols, eps, dx, dweight, nullptr, workspace, workspace_bytes, s);
}

size_t fth_dev_linear_backward_workspace_bytes(int64_t batch, int64_t out_features, int32_t dtype) {
    if (batch < 0 || out_features < 0) return 0;
    return dtype == FTH_DTYPE_F64 ? linear_backward_workspace<double>(batch, out_features) : linear_backward_workspace<float>(batch, out_features);
}
int32_t fth_dev_linear_backward_f32(const float *dy, const float *x, const float *weight, int64_t batch, int64_t in_features,
                                    int64_t out_features, float *dx, float *dweight, float *dbias, void *workspace,
                                    size_t workspace_bytes, fth_stream s) {
    return linear_backward_entry<float>(dy, x, weight, batch, in_features, out_features, dx, dweight, dbias, workspace, workspace_bytes, s);
}
int32_t fth_dev_linear_backward_f64(const double *dy, const double *x, const double *weight, int64_t batch, int64_t in_features,
                                    int64_t out_features, double *dx, double *dweight, double *dbias, void *workspace,
                                    size_t workspace_bytes, fth_stream s) {
    return linear_backward_entry<double>(dy, x, weight, batch, in_features, out_features, dx, dweight, dbias, workspace, workspace_bytes, s);
}

size_t fth_dev_sdpa_backward_workspace_bytes(int64_t num_bh, int64_t seq_q, int64_t seq_k, int32_t dtype) {
    if (num_bh < 0 || seq_q < 0 || seq_k < 0) return 0;
    return dtype == FTH_DTYPE_F64 ? sdpa_backward_workspace<double>(num_bh, seq_q, seq_k) : sdpa_backward_workspace<float>(num_bh, seq_q, seq_k);
}
int32_t fth_dev_sdpa_backward_f32(const float *q, const float *k, const float *v, const float *dout, int64_t num_bh, int64_t seq_q,
                                  int64_t seq_k, int64_t d_k, int64_t d_v, float scale, int32_t causal, float *dq, float *dk,
                                  float *dv, void *workspace, size_t workspace_bytes, fth_stream s) {
    return sdpa_backward_entry<float>(q, k, v, dout, num_bh, seq_q, seq_k, d_k, d_v, scale, causal, dq, dk, dv, workspace, workspace_bytes, s);
}
int32_t fth_dev_sdpa_backward_f64(const double *q, const double *k, const double *v, const double *dout, int64_t num_bh, int64_t seq_q,
                                  int64_t seq_k, int64_t d_k, int64_t d_v, double scale, int32_t causal, double *dq, double *dk,
                                  double *dv, void *workspace, size_t workspace_bytes, fth_stream s) {
    return sdpa_backward_entry<double>(q, k, v, dout, num_bh, seq_q, seq_k, d_k, d_v, scale, causal, dq, dk, dv, workspace, workspace_bytes, s);
}
size_t fth_dev_sdpa_backward_unit_dout_workspace_bytes(int64_t num_bh, int64_t seq_q, int64_t seq_k, int64_t d_v, int32_t dtype) {
    if (num_bh < 0 || seq_q < 0 || seq_k < 0 || d_v < 0) return 0;
    const size_t el = dtype == FTH_DTYPE_F64 ? sizeof(double) : sizeof(float);
    return fth_dev_sdpa_backward_workspace_bytes(num_bh, seq_q, seq_k, dtype) + (size_t)(seq_q * d_v + 4) * el;
}
int32_t fth_dev_sdpa_backward_unit_dout_f32(const float *q, const float *k, const float *v, int64_t num_bh, int64_t seq_q, int64_t seq_k,
                                            int64_t d_k, int64_t d_v, float scale, int32_t causal, float *dq, float *dk, float *dv,
                                            void *workspace, size_t workspace_bytes, fth_stream s) {
    return sdpa_backward_entry<float>(q, k, v, nullptr, num_bh, seq_q, seq_k, d_k, d_v, scale, causal, dq, dk, dv, workspace, workspace_bytes, s,
                                      nullptr, 0, true);
}
int32_t fth_dev_sdpa_backward_unit_dout_f64(const double *q, const double *k, const double *v, int64_t num_bh, int64_t seq_q, int64_t seq_k,
                                            int64_t d_k, int64_t d_v, double scale, int32_t causal, double *dq, double *dk, double *dv,
                                            void *workspace, size_t workspace_bytes, fth_stream s) {
    return sdpa_backward_entry<double>(q, k, v, nullptr, num_bh, seq_q, seq_k, d_k, d_v, scale, causal, dq, dk, dv, workspace, workspace_bytes, s,
                                       nullptr, 0, true);
}
int32_t fth_dev_sdpa_backward_masked_f32(const float *q, const float *k, const float *v, const float *dout, int64_t num_bh, int64_t seq_q,
                                         int64_t seq_k, int64_t d_k, int64_t d_v, float scale, const float *mask, int64_t mask_bh_stride,
                                         float *dq, float *dk, float *dv, void *workspace, size_t workspace_bytes, fth_stream s) {
    FTH_ARG(mask != nullptr || num_bh == 0 || seq_q == 0 || seq_k == 0, "sdpa backward: NULL mask");
    FTH_ARG(mask_bh_stride == 0 || mask_bh_stride >= seq_q * seq_k, "sdpa backward: mask_bh_stride %lld is neither 0 nor >= seq_q * seq_k",
            (long long)mask_bh_stride);
    return sdpa_backward_entry<float>(q, k, v, dout, num_bh, seq_q, seq_k, d_k, d_v, scale, 0, dq, dk, dv, workspace, workspace_bytes, s, mask,
                                      mask_bh_stride);
}
int32_t fth_dev_sdpa_backward_masked_f64(const double *q, const double *k, const double *v, const double *dout, int64_t num_bh, int64_t seq_q,
                                         int64_t seq_k, int64_t d_k, int64_t d_v, double scale, const double *mask, int64_t mask_bh_stride,
                                         double *dq, double *dk, double *dv, void *workspace, size_t workspace_bytes, fth_stream s) {
    FTH_ARG(mask != nullptr || num_bh == 0 || seq_q == 0 || seq_k == 0, "sdpa backward: NULL mask");
    FTH_ARG(mask_bh_stride == 0 || mask_bh_stride >= seq_q * seq_k, "sdpa backward: mask_bh_stride %lld is neither 0 nor >= seq_q * seq_k",
            (long long)mask_bh_stride);
    return sdpa_backward_entry<double>(q, k, v, dout, num_bh, seq_q, seq_k, d_k, d_v, scale, 0, dq, dk, dv, workspace, workspace_bytes, s, mask,
                                       mask_bh_stride);
}

}  // extern "C"
